"""The colour-spec part of the format API against the reference's own known-answer tests
(tests/nvcv_types/system/TestColorSpec.cpp: the tables at :45-50, the name strings at :128-154 and :543-655,
the field-by-field get/set loops at :310-535, the predefined specs' ranges and transfer functions at :166-238).
CPU only."""
import ctypes as C

import pytest


@pytest.fixture(scope="module")
def nv(cv):
    import cvcuda_amd._capi as capi
    lib = capi.nvcv
    for f in ("nvcvChromaSubsamplingGetName", "nvcvColorSpecGetName", "nvcvColorModelGetName", "nvcvColorSpaceGetName",
              "nvcvWhitePointGetName", "nvcvYCbCrEncodingGetName", "nvcvColorTransferFunctionGetName",
              "nvcvColorRangeGetName", "nvcvChromaLocationGetName", "nvcvRawPatternGetName"):
        getattr(lib, f).restype = C.c_char_p
        getattr(lib, f).argtypes = [C.c_int]
    return lib


def spec_word(space, enc, xfer, rng, loch, locv):
    """NVCV_MAKE_COLOR_SPEC as the test file's loops use it, with out-of-range arguments truncated per field."""
    return (space & 7) | (xfer & 15) << 3 | (enc & 7) << 7 | (loch & 3) << 10 | (locv & 3) << 12 | (rng & 1) << 14


CSS = [("444", 0, 4, 4, "4:4:4"), ("422", 1, 2, 4, "4:2:2"), ("422R", 2, 4, 2, "4:2:2R"), ("411R", 4, 4, 1, "4:1:1R"),
       ("411", 3, 1, 4, "4:1:1"), ("420", 5, 2, 2, "4:2:0"), ("410", 6, 1, 2, "4:1:0"), ("410R", 7, 2, 1, "4:1:0R")]


@pytest.mark.parametrize("name,code,h,v,text", CSS)
def test_chroma_subsampling_table(nv, K, name, code, h, v, text):
    assert getattr(K, "CSS_" + name) == code
    sh, sv = C.c_int32(), C.c_int32()
    assert nv.nvcvChromaSubsamplingGetNumSamples(code, C.byref(sh), C.byref(sv)) == 0 and (sh.value, sv.value) == (h, v)
    out = C.c_int(-1)
    assert nv.nvcvMakeChromaSubsampling(C.byref(out), h, v) == 0 and out.value == code
    assert nv.nvcvChromaSubsamplingGetName(code) == text.encode()


def test_chroma_subsampling_edges(nv, K):
    out = C.c_int(-1)
    assert nv.nvcvMakeChromaSubsampling(C.byref(out), 1, 1) == 0 and out.value == K.CSS_444
    for h, v in ((5, 5), (4, 5), (2, 5), (1, 5)):
        assert nv.nvcvMakeChromaSubsampling(C.byref(out), h, v) == 2
    assert nv.nvcvMakeChromaSubsampling(None, 2, 4) == 2
    assert nv.nvcvChromaSubsamplingGetNumSamples(K.CSS_444, None, None) == 2
    sh = C.c_int32()
    assert nv.nvcvChromaSubsamplingGetNumSamples(255, C.byref(sh), None) == 2


def test_color_spec_names(nv, K):
    assert nv.nvcvColorSpecGetName(K.COLOR_SPEC_MPEG2_SMPTE240M) == b"NVCV_COLOR_SPEC_MPEG2_SMPTE240M"
    spec = C.c_int()
    assert nv.nvcvMakeColorSpec(C.byref(spec), K.COLOR_SPACE_DCIP3, K.YCbCr_ENC_BT2020c, K.COLOR_XFER_sYCC,
                                K.COLOR_RANGE_LIMITED, K.CHROMA_LOC_ODD, K.CHROMA_LOC_CENTER) == 0
    assert nv.nvcvColorSpecGetName(spec.value) == b"NVCVColorSpec(SPACE_DCIP3,ENC_BT2020c,XFER_sYCC,RANGE_LIMITED,LOC_ODD,LOC_CENTER)"
    assert nv.nvcvColorSpecGetName(0x7FFFFFFF) == (b"NVCVColorSpec(invalid)NVCVColorSpec(NVCVColorSpace(7),NVCVYCbCrEncoding(7),"
                                                    b"NVCVColorTransferFunction(15),RANGE_LIMITED,LOC_ODD,LOC_ODD)")
    assert nv.nvcvMakeColorSpec(None, 0, 0, 0, 0, 0, 0) == 2


def test_predefined_specs_decode(nv, K):
    rng = C.c_int()
    full = ["UNDEFINED", "BT601_ER", "BT709_ER", "BT2020_ER", "BT2020c_ER", "BT2020_PQ_ER", "sRGB", "DISPLAYP3_LINEAR",
            "DISPLAYP3", "sYCC", "MPEG2_BT601", "MPEG2_BT709", "MPEG2_SMPTE240M"]
    limited = ["BT601", "BT709", "BT709_LINEAR", "BT2020", "BT2020c", "BT2020_PQ", "BT2020_LINEAR", "SMPTE240M"]
    for names, want in ((full, K.COLOR_RANGE_FULL), (limited, K.COLOR_RANGE_LIMITED)):
        for n in names:
            assert nv.nvcvColorSpecGetRange(getattr(K, "COLOR_SPEC_" + n), C.byref(rng)) == 0 and rng.value == want, n
    xfer = C.c_int()
    table = {"LINEAR": ["UNDEFINED", "BT709_LINEAR", "BT2020_LINEAR", "DISPLAYP3_LINEAR"], "PQ": ["BT2020_PQ", "BT2020_PQ_ER"],
             "sRGB": ["sRGB", "DISPLAYP3"], "BT709": ["BT601", "BT601_ER", "MPEG2_BT601", "MPEG2_BT709", "BT709", "BT709_ER"],
             "BT2020": ["BT2020", "BT2020c", "BT2020c_ER", "BT2020_ER"], "SMPTE240M": ["SMPTE240M", "MPEG2_SMPTE240M"],
             "sYCC": ["sYCC"]}
    for x, names in table.items():
        for n in names:
            assert nv.nvcvColorSpecGetColorTransferFunction(getattr(K, "COLOR_SPEC_" + n), C.byref(xfer)) == 0
            assert xfer.value == getattr(K, "COLOR_XFER_" + x), n


FIELDS = [  # setter, getter, position of the field among NVCV_MAKE_COLOR_SPEC's arguments, bits
    ("nvcvColorSpecSetColorSpace", "nvcvColorSpecGetColorSpace", 0, 3),
    ("nvcvColorSpecSetYCbCrEncoding", "nvcvColorSpecGetYCbCrEncoding", 1, 3),
    ("nvcvColorSpecSetColorTransferFunction", "nvcvColorSpecGetColorTransferFunction", 2, 3),
    ("nvcvColorSpecSetRange", "nvcvColorSpecGetRange", 3, 1),
]


@pytest.mark.parametrize("setter,getter,pos,bits", FIELDS)
def test_each_field_is_set_and_read_without_touching_the_others(nv, setter, getter, pos, bits):
    # the reference's loops: every other field all ones, the field under test 0, 1, 2, 4 ...
    values = [0] + [1 << i for i in range(bits)]
    for val in values:
        args = [0xFFFFFFFF] * 6
        args[pos] = 1 if val == 0 else 0
        spec = C.c_int32(spec_word(*args))
        args[pos] = val
        gold = spec_word(*args)
        assert getattr(nv, setter)(C.byref(spec), val) == 0
        assert spec.value & 0xFFFFFFFF == gold
        out = C.c_int(-1)
        assert getattr(nv, getter)(gold, C.byref(out)) == 0 and out.value == val
        assert getattr(nv, getter)(gold, None) == 2
    assert getattr(nv, setter)(None, 0) == 2


def test_chroma_locations(nv):
    ones = 0xFFFFFFFF
    for loc in (0, 1, 2):
        spec = C.c_int32(spec_word(ones, ones, ones, ones, 1 if loc == 0 else 0, ones))
        assert nv.nvcvColorSpecSetChromaLoc(C.byref(spec), loc, 3) == 0
        assert spec.value & 0xFFFFFFFF == spec_word(ones, ones, ones, ones, loc, ones)
        spec = C.c_int32(spec_word(ones, ones, ones, ones, ones, 1 if loc == 0 else 0))
        assert nv.nvcvColorSpecSetChromaLoc(C.byref(spec), 3, loc) == 0
        assert spec.value & 0xFFFFFFFF == spec_word(ones, ones, ones, ones, ones, loc)
        h, v = C.c_int(-1), C.c_int(-1)
        word = spec_word(ones, ones, ones, ones, loc & 3, ~loc & 3)
        assert nv.nvcvColorSpecGetChromaLoc(word, C.byref(h), C.byref(v)) == 0 and (h.value, v.value) == (loc & 3, ~loc & 3)
        assert nv.nvcvColorSpecGetChromaLoc(word, C.byref(h), None) == 0 and nv.nvcvColorSpecGetChromaLoc(word, None, C.byref(v)) == 0
    assert nv.nvcvColorSpecGetChromaLoc(0, None, None) == 2
    assert nv.nvcvColorSpecSetChromaLoc(None, 1, 3) == 2


def test_color_model_needs_colorspec(nv, K):
    out = C.c_int8(-1)
    for name, want in (("YCbCr", 1), ("RGB", 1), ("UNDEFINED", 0), ("RAW", 0), ("XYZ", 0), ("HSV", 0), ("CMYK", 0), ("YCCK", 0)):
        assert nv.nvcvColorModelNeedsColorspec(getattr(K, "COLOR_MODEL_" + name), C.byref(out)) == 0 and out.value == want
    out = C.c_int8(7)
    assert nv.nvcvColorModelNeedsColorspec(419, C.byref(out)) == 2 and out.value == 7  # output untouched
    assert nv.nvcvColorModelNeedsColorspec(K.COLOR_MODEL_RGB, None) == 2


def test_enumerator_names(nv, K):
    assert nv.nvcvColorModelGetName(K.COLOR_MODEL_YCbCr) == b"NVCV_COLOR_MODEL_YCbCr"
    assert nv.nvcvColorModelGetName(-1) == b"NVCVColorModel(-1)"
    for n in ("UNDEFINED", "BT601", "BT709", "BT2020", "BT2020c", "SMPTE240M"):
        assert nv.nvcvYCbCrEncodingGetName(getattr(K, "YCbCr_ENC_" + n)) == b"NVCV_YCbCr_ENC_" + n.encode()
    assert nv.nvcvYCbCrEncodingGetName(-1) == b"NVCVYCbCrEncoding(-1)"
    assert nv.nvcvChromaLocationGetName(K.CHROMA_LOC_EVEN) == b"NVCV_CHROMA_LOC_EVEN"
    assert nv.nvcvChromaLocationGetName(K.CHROMA_LOC_BOTH) == b"NVCV_CHROMA_LOC_BOTH"
    assert nv.nvcvChromaLocationGetName(-1) == b"NVCVChromaLocation(-1)"
    for i, n in enumerate(("RGGB", "BGGR", "GRBG", "GBRG", "RCCB", "BCCR", "CRBC", "CBRC", "RCCC", "CRCC", "CCRC", "CCCR", "CCCC")):
        assert getattr(K, "RAW_BAYER_" + n) == i
        assert nv.nvcvRawPatternGetName(i) == b"NVCV_RAW_BAYER_" + n.encode()
    assert nv.nvcvRawPatternGetName(255) == b"NVCVRawPattern(255)" and nv.nvcvRawPatternGetName(-1) == b"NVCVRawPattern(-1)"
    for n in ("BT601", "BT709", "BT2020", "DCIP3"):
        assert nv.nvcvColorSpaceGetName(getattr(K, "COLOR_SPACE_" + n)) == b"NVCV_COLOR_SPACE_" + n.encode()
    assert nv.nvcvColorSpaceGetName(-1) == b"NVCVColorSpace(-1)"
    assert nv.nvcvWhitePointGetName(0) == b"NVCV_WHITE_POINT_D65"
    assert nv.nvcvWhitePointGetName(255) == b"NVCVWhitePoint(255)" and nv.nvcvWhitePointGetName(-1) == b"NVCVWhitePoint(-1)"
    assert nv.nvcvColorTransferFunctionGetName(K.COLOR_XFER_PQ) == b"NVCV_COLOR_XFER_PQ"
    assert nv.nvcvColorTransferFunctionGetName(-1) == b"NVCVColorTransferFunction(-1)"
    assert nv.nvcvColorRangeGetName(K.COLOR_RANGE_FULL) == b"NVCV_COLOR_RANGE_FULL"
    assert nv.nvcvColorRangeGetName(-1) == b"NVCVColorRange(-1)"
