"""Image-format, packing and data-layout functions against the expectations the reference's own unit tests hold,
restated as data (tests/nvcv_types/system/TestImageFormat.cpp and TestDataLayout.cpp; line ranges at each table).
The per-format table is the fixture tests/golden/image_format_vectors.json. CPU only."""
import ctypes as C
import json
import os

import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
INVALID = 2
INVALID_IMAGE_FORMAT = 3


class ExtraInfo(C.Structure):
    _fields_ = [("numChannels", C.c_int32), ("bitsPerPixel", C.c_int32), ("datakind", C.c_int), ("channelType", C.c_int)]


class PackingParams(C.Structure):
    _fields_ = [("byteOrder", C.c_int), ("alignment", C.c_int32), ("swizzle", C.c_int), ("bits", C.c_int32 * 4)]


@pytest.fixture(scope="module")
def nv(cv):
    import cvcuda_amd._capi as capi
    lib = capi.nvcv
    for f in ("nvcvImageFormatGetName", "nvcvPackingGetName", "nvcvChannelGetName", "nvcvByteOrderGetName", "nvcvSwizzleGetName",
              "nvcvMemLayoutGetName", "nvcvDataKindGetName"):
        getattr(lib, f).restype = C.c_char_p
    lib.nvcvImageFormatGetName.argtypes = [C.c_uint64]
    u64, i32, p = C.c_uint64, C.c_int32, C.c_void_p
    lib.nvcvMakeColorImageFormat.argtypes = [p] + [C.c_int] * 10 + [p]
    lib.nvcvMakeYCbCrImageFormat.argtypes = [p] + [C.c_int] * 10 + [p]
    lib.nvcvMakeNonColorImageFormat.argtypes = [p] + [C.c_int] * 8 + [p]
    lib.nvcvMakeRawImageFormat.argtypes = [p] + [C.c_int] * 9 + [p]
    lib.nvcvMakeImageFormatFromPlanes.argtypes = [p, u64, u64, u64, u64]
    lib.nvcvMakeImageFormatFromFourCC.argtypes = [p, C.c_uint32, C.c_int, C.c_int]
    for f in ("nvcvImageFormatGetPlaneFormat", "nvcvImageFormatGetPlaneSwizzle", "nvcvImageFormatGetPlanePacking",
              "nvcvImageFormatGetPlaneBitsPerPixel", "nvcvImageFormatGetPlaneNumChannels", "nvcvImageFormatGetPlaneDataType",
              "nvcvImageFormatGetPlanePixelStrideBytes"):
        getattr(lib, f).argtypes = [u64, i32, p]
    for f in ("nvcvImageFormatToFourCC", "nvcvImageFormatGetExtraChannelInfo", "nvcvImageFormatGetRawPattern",
              "nvcvImageFormatGetSwizzle", "nvcvImageFormatGetColorModel", "nvcvImageFormatGetColorSpec", "nvcvImageFormatGetMemLayout",
              "nvcvImageFormatGetChromaSubsampling", "nvcvImageFormatGetAlphaType", "nvcvImageFormatGetDataKind",
              "nvcvImageFormatGetNumPlanes", "nvcvImageFormatGetNumChannels", "nvcvImageFormatGetBitsPerChannel"):
        getattr(lib, f).argtypes = [u64, p]
    lib.nvcvImageFormatGetPlaneSize.argtypes = [u64, i32, i32, i32, p, p]
    lib.nvcvImageFormatHasSameDataLayout.argtypes = [u64, u64, p]
    lib.nvcvImageFormatSetSwizzleAndPacking.argtypes = [p] + [C.c_int] * 5
    return lib


def const(K, name):
    return getattr(K, name[5:] if name.startswith("NVCV_") else name)


def make_color(nv, K, model, spec, layout, kind, sw, packs, alpha="ASSOCIATED", ex=None):
    f = C.c_uint64(0x1234)
    pk = [const(K, "PACKING_" + x) for x in packs] + [0] * (4 - len(packs))
    st = nv.nvcvMakeColorImageFormat(C.byref(f), const(K, "COLOR_MODEL_" + model), const(K, "COLOR_SPEC_" + spec),
                                     const(K, "MEM_LAYOUT_" + layout), const(K, "DATA_KIND_" + kind), const(K, "SWIZZLE_" + sw),
                                     *pk, const(K, "ALPHA_" + alpha), C.byref(ex) if ex is not None else None)
    return st, f.value


def make_ycbcr(nv, K, spec, css, layout, kind, sw, packs, ex=None):
    f = C.c_uint64(0)
    pk = [const(K, "PACKING_" + x) for x in packs] + [0] * (4 - len(packs))
    spec = const(K, "COLOR_SPEC_" + spec) if isinstance(spec, str) else spec
    sw = const(K, "SWIZZLE_" + sw) if isinstance(sw, str) else sw
    st = nv.nvcvMakeYCbCrImageFormat(C.byref(f), spec, const(K, "CSS_" + css), const(K, "MEM_LAYOUT_" + layout),
                                     const(K, "DATA_KIND_" + kind), sw, *pk, K.ALPHA_ASSOCIATED, C.byref(ex) if ex is not None else None)
    return st, f.value


def make_noncolor(nv, K, layout, kind, sw, packs, ex=None):
    f = C.c_uint64(0)
    pk = [const(K, "PACKING_" + x) for x in packs] + [0] * (4 - len(packs))
    st = nv.nvcvMakeNonColorImageFormat(C.byref(f), const(K, "MEM_LAYOUT_" + layout), const(K, "DATA_KIND_" + kind),
                                        const(K, "SWIZZLE_" + sw), *pk, K.ALPHA_ASSOCIATED, C.byref(ex) if ex is not None else None)
    return st, f.value


def make_raw(nv, K, raw, layout, kind, sw, packs, ex=None):
    f = C.c_uint64(0)
    pk = [const(K, "PACKING_" + x) for x in packs] + [0] * (4 - len(packs))
    st = nv.nvcvMakeRawImageFormat(C.byref(f), const(K, "RAW_" + raw), const(K, "MEM_LAYOUT_" + layout), const(K, "DATA_KIND_" + kind),
                                   const(K, "SWIZZLE_" + sw), *pk, K.ALPHA_ASSOCIATED, C.byref(ex) if ex is not None else None)
    return st, f.value


VECTORS = json.load(open(os.path.join(GOLD, "image_format_vectors.json")))


@pytest.mark.parametrize("v", VECTORS, ids=[v["format"][18:] for v in VECTORS])
def test_named_format_properties(nv, K, v):
    # TestImageFormat.cpp:93-308 (table), :309-337, :529-730 (the checks made on every row)
    fmt = const(K, v["format"])
    ex = None
    if v["extra"]["numChannels"]:
        ex = ExtraInfo(v["extra"]["numChannels"], v["extra"]["bitsPerPixel"], const(K, v["extra"]["dataKind"]), const(K, v["extra"]["channelType"]))
    packs = [x for x in v["packings"]]
    if v["colorModel"] == "YCbCr":
        st, made = make_ycbcr(nv, K, v["colorSpec"], v["css"], v["memLayout"], v["dataKind"], v["swizzle"], packs, ex)
    else:
        st, made = make_color(nv, K, v["colorModel"], v["colorSpec"], v["memLayout"], v["dataKind"], v["swizzle"], packs, v["alphaType"], ex)
    assert st == 0 and made == fmt

    out, o64 = C.c_int(-7), C.c_uint64()
    for p in range(4):
        assert nv.nvcvImageFormatGetPlanePacking(fmt, p, C.byref(out)) == 0 and out.value == const(K, "PACKING_" + v["packings"][p])
        want = v["planes"][p] if p < len(v["planes"]) else {"bpp": 0, "channels": 0, "dataType": "NVCV_DATA_TYPE_NONE", "swizzle": "NVCV_SWIZZLE_0000"}
        assert nv.nvcvImageFormatGetPlaneBitsPerPixel(fmt, p, C.byref(out)) == 0 and out.value == want["bpp"]
        assert nv.nvcvImageFormatGetPlaneNumChannels(fmt, p, C.byref(out)) == 0 and out.value == want["channels"]
        assert nv.nvcvImageFormatGetPlaneDataType(fmt, p, C.byref(o64)) == 0 and o64.value == const(K, want["dataType"])
        assert nv.nvcvImageFormatGetPlaneSwizzle(fmt, p, C.byref(out)) == 0 and out.value == const(K, want["swizzle"])
    assert nv.nvcvImageFormatGetDataKind(fmt, C.byref(out)) == 0 and out.value == const(K, "DATA_KIND_" + v["dataKind"])
    assert nv.nvcvImageFormatGetSwizzle(fmt, C.byref(out)) == 0 and out.value == const(K, "SWIZZLE_" + v["swizzle"])
    assert nv.nvcvImageFormatGetMemLayout(fmt, C.byref(out)) == 0 and out.value == const(K, "MEM_LAYOUT_" + v["memLayout"])
    assert nv.nvcvImageFormatGetColorSpec(fmt, C.byref(out)) == 0 and out.value == const(K, "COLOR_SPEC_" + v["colorSpec"])
    assert nv.nvcvImageFormatGetColorModel(fmt, C.byref(out)) == 0 and out.value == const(K, "COLOR_MODEL_" + v["colorModel"])
    assert nv.nvcvImageFormatGetChromaSubsampling(fmt, C.byref(out)) == 0 and out.value == const(K, "CSS_" + v["css"])
    assert nv.nvcvImageFormatGetNumPlanes(fmt, C.byref(out)) == 0 and out.value == v["planeCount"]
    nch = sum(1 for b in v["bitsPerChannel"] if b)
    assert nv.nvcvImageFormatGetNumChannels(fmt, C.byref(out)) == 0 and out.value == nch
    bits = (C.c_int32 * 4)()
    assert nv.nvcvImageFormatGetBitsPerChannel(fmt, bits) == 0 and list(bits) == v["bitsPerChannel"]
    info = ExtraInfo()
    assert nv.nvcvImageFormatGetExtraChannelInfo(fmt, C.byref(info)) == 0
    assert (info.numChannels, info.bitsPerPixel, info.datakind, info.channelType) == (
        v["extra"]["numChannels"], v["extra"]["bitsPerPixel"], const(K, v["extra"]["dataKind"]), const(K, v["extra"]["channelType"]))


def test_the_none_format_and_out_of_range_planes(nv, K):
    # TestImageFormat.cpp:339-527
    out, o64 = C.c_int(-7), C.c_uint64(K.IMAGE_FORMAT_NV12)
    assert nv.nvcvMakeColorImageFormat(C.byref(o64), K.COLOR_MODEL_RGB, K.COLOR_SPEC_BT601, K.MEM_LAYOUT_PL, K.DATA_KIND_UNSIGNED,
                                       K.SWIZZLE_XYZW, K.PACKING_X8, K.PACKING_X8, K.PACKING_X8, K.PACKING_X128, 0, None) == INVALID
    assert o64.value == K.IMAGE_FORMAT_NV12  # output untouched
    for p in range(4):
        assert nv.nvcvImageFormatGetPlanePacking(0, p, C.byref(out)) == 0 and out.value == 0
        assert nv.nvcvImageFormatGetPlaneBitsPerPixel(0, p, C.byref(out)) == 0 and out.value == 0
    assert nv.nvcvImageFormatGetDataKind(0, C.byref(out)) == 0 and out.value == K.DATA_KIND_UNSIGNED
    assert nv.nvcvImageFormatGetSwizzle(0, C.byref(out)) == 0 and out.value == K.SWIZZLE_0000
    assert nv.nvcvImageFormatGetColorModel(0, C.byref(out)) == 0 and out.value == K.COLOR_MODEL_UNDEFINED
    assert nv.nvcvImageFormatGetAlphaType(0, C.byref(out)) == 0 and out.value == K.ALPHA_ASSOCIATED
    assert nv.nvcvImageFormatGetMemLayout(0, C.byref(out)) == 0 and out.value == K.MEM_LAYOUT_PITCH_LINEAR
    assert nv.nvcvImageFormatGetColorSpec(0, C.byref(out)) == 0 and out.value == K.COLOR_SPEC_UNDEFINED
    assert nv.nvcvImageFormatGetChromaSubsampling(0, C.byref(out)) == 0 and out.value == K.CSS_NONE
    assert nv.nvcvImageFormatGetRawPattern(0, C.byref(out)) == INVALID
    info = ExtraInfo(9, 9, 9, 9)
    assert nv.nvcvImageFormatGetExtraChannelInfo(0, C.byref(info)) == 0
    assert (info.numChannels, info.bitsPerPixel, info.datakind, info.channelType) == (0, 0, K.DATA_KIND_UNSPECIFIED, K.EXTRA_CHANNEL_U)
    assert nv.nvcvImageFormatGetExtraChannelInfo(0, None) == INVALID
    none = C.c_uint64(0)
    ex = ExtraInfo(2, 8, K.DATA_KIND_UNSIGNED, K.EXTRA_CHANNEL_POS3D)
    assert nv.nvcvImageFormatSetExtraChannelInfo(C.byref(none), C.byref(ex)) == INVALID
    assert nv.nvcvImageFormatSetExtraChannelInfo(None, C.byref(ex)) == INVALID
    assert nv.nvcvImageFormatSetDataKind(C.byref(none), K.DATA_KIND_SIGNED) == INVALID
    assert nv.nvcvImageFormatSetMemLayout(C.byref(none), K.MEM_LAYOUT_BL) == INVALID
    assert nv.nvcvImageFormatSetColorSpec(C.byref(none), K.COLOR_SPEC_BT601) == INVALID
    assert nv.nvcvImageFormatSetRawPattern(C.byref(none), K.RAW_BAYER_BGGR) == INVALID
    assert nv.nvcvImageFormatSetChromaSubsampling(C.byref(none), K.CSS_420) == INVALID
    assert nv.nvcvImageFormatSetAlphaType(C.byref(none), K.ALPHA_UNASSOCIATED) == INVALID
    assert nv.nvcvImageFormatSetSwizzleAndPacking(C.byref(none), K.SWIZZLE_X000, K.PACKING_X8, 0, 0, 0) == INVALID
    out = C.c_int(K.PACKING_X8_Y8__X8_Z8)
    assert nv.nvcvImageFormatGetPlanePacking(K.IMAGE_FORMAT_NV12, 342, C.byref(out)) == 0 and out.value == 0
    out = C.c_int32(123)
    assert nv.nvcvImageFormatGetPlaneBitsPerPixel(K.IMAGE_FORMAT_NV12, 342, C.byref(out)) == 0 and out.value == 0


def test_extra_channel_info_limits_and_round_trip(nv, K):
    # TestImageFormat.cpp:440-462, :1108-1126
    f = C.c_uint64(K.IMAGE_FORMAT_BGRf32)
    for bad in (ExtraInfo(8, 8, K.DATA_KIND_UNSIGNED, K.EXTRA_CHANNEL_POS3D), ExtraInfo(-1, 8, K.DATA_KIND_UNSIGNED, K.EXTRA_CHANNEL_POS3D),
                ExtraInfo(2, 256, K.DATA_KIND_UNSIGNED, K.EXTRA_CHANNEL_POS3D)):
        assert nv.nvcvImageFormatSetExtraChannelInfo(C.byref(f), C.byref(bad)) == INVALID
    planar = C.c_uint64(K.IMAGE_FORMAT_BGRf32p)
    ok = ExtraInfo(2, 8, K.DATA_KIND_UNSIGNED, K.EXTRA_CHANNEL_POS3D)
    assert nv.nvcvImageFormatSetExtraChannelInfo(C.byref(planar), C.byref(ok)) == INVALID
    st, a = make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8_Y8_Z8_W8"], ex=ExtraInfo(2, 8, K.DATA_KIND_UNSIGNED, K.EXTRA_CHANNEL_U))
    new = ExtraInfo(3, 16, K.DATA_KIND_SIGNED, K.EXTRA_CHANNEL_D)
    st2, gold = make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8_Y8_Z8_W8"], ex=new)
    assert st == 0 and st2 == 0
    f = C.c_uint64(a)
    assert nv.nvcvImageFormatSetExtraChannelInfo(C.byref(f), C.byref(new)) == 0 and f.value == gold
    # every width the word can hold reads back as it was set, also on a format that had none before
    for bpp in (8, 16, 24, 32, 64, 128):
        f = C.c_uint64(K.IMAGE_FORMAT_RGB8)
        ex = ExtraInfo(5, bpp, K.DATA_KIND_FLOAT, K.EXTRA_CHANNEL_D)
        got = ExtraInfo()
        n = C.c_int()
        assert nv.nvcvImageFormatSetExtraChannelInfo(C.byref(f), C.byref(ex)) == 0
        assert nv.nvcvImageFormatGetExtraChannelInfo(f.value, C.byref(got)) == 0
        assert (got.numChannels, got.bitsPerPixel, got.datakind, got.channelType) == (5, bpp, K.DATA_KIND_FLOAT, K.EXTRA_CHANNEL_D)
        assert nv.nvcvImageFormatGetNumPlanes(f.value, C.byref(n)) == 0 and n.value == 1
        assert nv.nvcvImageFormatGetPlanePacking(f.value, 0, C.byref(n)) == 0 and n.value == K.PACKING_X8_Y8_Z8


def test_setters(nv, K):
    # TestImageFormat.cpp:1072-1232, :1943-1992
    _, rgba = make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8_Y8_Z8_W8"])
    f = C.c_uint64(rgba)
    _, gold = make_color(nv, K, "RGB", "UNDEFINED", "PL", "FLOAT", "XYZW", ["X8_Y8_Z8_W8"])
    assert nv.nvcvImageFormatSetDataKind(C.byref(f), K.DATA_KIND_FLOAT) == 0 and f.value == gold
    f = C.c_uint64(rgba)
    _, gold = make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8_Y8_Z8_W8"], alpha="UNASSOCIATED")
    assert nv.nvcvImageFormatSetAlphaType(C.byref(f), K.ALPHA_UNASSOCIATED) == 0 and f.value == gold
    f = C.c_uint64(rgba)
    _, gold = make_color(nv, K, "RGB", "UNDEFINED", "BLOCK4_LINEAR", "UNSIGNED", "XYZW", ["X8_Y8_Z8_W8"])
    assert nv.nvcvImageFormatSetMemLayout(C.byref(f), K.MEM_LAYOUT_BLOCK4_LINEAR) == 0 and f.value == gold
    _, raw = make_raw(nv, K, "BAYER_RGGB", "PL", "UNSIGNED", "X000", ["X8"])
    _, gold = make_raw(nv, K, "BAYER_CCCR", "PL", "UNSIGNED", "X000", ["X8"])
    f = C.c_uint64(raw)
    out = C.c_int()
    assert nv.nvcvImageFormatSetRawPattern(C.byref(f), K.RAW_BAYER_CCCR) == 0 and f.value == gold
    assert nv.nvcvImageFormatGetRawPattern(f.value, C.byref(out)) == 0 and out.value == K.RAW_BAYER_CCCR
    f = C.c_uint64(rgba)
    assert nv.nvcvImageFormatSetRawPattern(C.byref(f), K.RAW_BAYER_CCCR) == INVALID
    assert nv.nvcvImageFormatGetRawPattern(rgba, C.byref(out)) == INVALID
    # colour spec: YCbCr keeps it whole, RGB drops the YCbCr encoding
    _, y = make_ycbcr(nv, K, "BT601", "420", "PL", "UNSIGNED", "XYZ0", ["X8", "X8_Y8"])
    _, gold = make_ycbcr(nv, K, "BT709_ER", "420", "PL", "UNSIGNED", "XYZ0", ["X8", "X8_Y8"])
    f = C.c_uint64(y)
    assert nv.nvcvImageFormatSetColorSpec(C.byref(f), K.COLOR_SPEC_BT709_ER) == 0 and f.value == gold
    f = C.c_uint64(K.IMAGE_FORMAT_RGB8)
    assert nv.nvcvImageFormatSetColorSpec(C.byref(f), K.COLOR_SPEC_BT601) == 0
    spec, enc = C.c_int(), C.c_int()
    assert nv.nvcvImageFormatGetColorSpec(f.value, C.byref(spec)) == 0
    assert nv.nvcvColorSpecGetYCbCrEncoding(spec.value, C.byref(enc)) == 0 and enc.value == K.YCbCr_ENC_UNDEFINED
    want = C.c_int(K.COLOR_SPEC_BT601)
    assert nv.nvcvColorSpecSetYCbCrEncoding(C.byref(want), K.YCbCr_ENC_UNDEFINED) == 0 and spec.value == want.value
    # setting the undefined spec
    for start, gold in ((K.IMAGE_FORMAT_U8, K.IMAGE_FORMAT_U8), (raw, raw)):
        f = C.c_uint64(start)
        assert nv.nvcvImageFormatSetColorSpec(C.byref(f), K.COLOR_SPEC_UNDEFINED) == 0 and f.value == gold
    f = C.c_uint64(K.IMAGE_FORMAT_RGB8)
    assert nv.nvcvImageFormatSetColorSpec(C.byref(f), K.COLOR_SPEC_UNDEFINED) == 0 and f.value == K.IMAGE_FORMAT_RGB8
    f = C.c_uint64(K.IMAGE_FORMAT_NV12)
    assert nv.nvcvImageFormatSetColorSpec(C.byref(f), K.COLOR_SPEC_UNDEFINED) == 0
    assert nv.nvcvImageFormatGetColorSpec(f.value, C.byref(spec)) == 0 and spec.value == K.COLOR_SPEC_UNDEFINED
    # chroma subsampling
    _, gold = make_ycbcr(nv, K, "BT601", "422", "PL", "UNSIGNED", "XYZ0", ["X8", "X8_Y8"])
    f = C.c_uint64(y)
    assert nv.nvcvImageFormatSetChromaSubsampling(C.byref(f), K.CSS_422) == 0 and f.value == gold
    f = C.c_uint64(K.IMAGE_FORMAT_RGB8)
    assert nv.nvcvImageFormatSetChromaSubsampling(C.byref(f), K.CSS_NONE) == 0 and f.value == K.IMAGE_FORMAT_RGB8
    assert nv.nvcvImageFormatSetChromaSubsampling(C.byref(f), K.CSS_422) == INVALID


def macro_color(K, spec, layout, sw, packs):
    """What NVCV_MAKE_COLOR_IMAGE_FORMAT gives for the RGB model, unsigned, associated alpha (no validation)."""
    w = 0
    put = lambda v, off, n: (v & ((1 << n) - 1)) << off
    slot = lambda p, nsub, nch, nbpp: (put(0x7FF if (nsub == 0 and (p >> 6) & 15 == 0 and p & 15 == 4) else (p >> 6) & 15, nsub + nch, nbpp)
                                        | put((p >> 4) & 3, nsub, nch) | put(p & 15, 0, nsub))
    pk = [const(K, "PACKING_" + x) for x in packs] + [0] * (4 - len(packs))
    w |= put(const(K, "SWIZZLE_" + sw), 0, 6) | put(const(K, "MEM_LAYOUT_" + layout), 12, 3)
    w |= put(1, 16, 1) | put(const(K, "COLOR_SPEC_" + spec), 20, 15) | put(K.COLOR_MODEL_RGB - 2, 17, 3)
    w |= put(slot(pk[0], 3, 2, 4), 35, 9) | put(1, 7, 1) | put(slot(pk[1], 3, 1, 3), 44, 7) | put(slot(pk[2], 3, 1, 3), 51, 7)
    w |= put(slot(pk[3], 0, 0, 3), 58, 3)
    return w


def test_set_swizzle_and_packing(nv, K):
    # TestImageFormat.cpp:2037-2122
    ok = [(("XYZ1", ["X64", "X16", "X32"]), ("ZYX1", ["X16", "X32", "X64"])),
          (("XYZ1", ["X64", "X16", "X32"]), ("ZYX0", ["X16", "X32", "X64"])),
          (("XYZ1", ["X64", "X16", "X32"]), ("YX00", ["X8_Y8"])),
          (("XYZW", ["X16", "X32", "X8", "X16"]), ("XYZW", ["X16", "X32", "X8", "X16"]))]
    for (sw0, pk0), (sw1, pk1) in ok:
        f = C.c_uint64(macro_color(K, "BT601", "PL", sw0, pk0))
        pk = [const(K, "PACKING_" + x) for x in pk1] + [0] * (4 - len(pk1))
        assert nv.nvcvImageFormatSetSwizzleAndPacking(C.byref(f), const(K, "SWIZZLE_" + sw1), *pk) == 0
        assert f.value == macro_color(K, "BT601", "PL", sw1, pk1)
        st, made = make_color(nv, K, "RGB", "BT601", "PL", "UNSIGNED", sw1, pk1)
        assert st == 0 and made == f.value
    bad = [(("XYZW", ["X16", "X32", "X8", "X16"]), ("XYZ1", ["X16", "X32", "X8", "X16"])),
           (("XYZW", ["X16", "X32", "X8"]), ("XYZW", ["X16", "X32", "X8"])),
           (("XYZW", ["X16", "X32", "X8_Y8"]), ("XYZW", ["X16", "X32", "X8"])),
           (("XYZW", ["X16", "X32", "X8", "X16"]), ("XYZW", ["X16", "X32", "X8"])),
           (("XYZW", ["X16", "X32", "X8", "X16"]), ("XYZW", ["X16", "X32", "X8", "X128"]))]
    for (sw0, pk0), (sw1, pk1) in bad:
        start = macro_color(K, "BT601", "PL", sw0, pk0)
        f = C.c_uint64(start)
        pk = [const(K, "PACKING_" + x) for x in pk1] + [0] * (4 - len(pk1))
        assert nv.nvcvImageFormatSetSwizzleAndPacking(C.byref(f), const(K, "SWIZZLE_" + sw1), *pk) == INVALID
        assert f.value == start


PLANE_SWIZZLES = [  # TestImageFormat.cpp:1355-1373: swizzle, packings, swizzle of each plane
    ("XYZ1", ["X8", "X8", "X8"], ["X001", "0X01", "00X1", "0000"]), ("XYZ1", ["X8_Y8", "X8"], ["XY01", "00X1", "0000", "0000"]),
    ("XYZ1", ["X8", "X8_Y8"], ["X001", "0XY1", "0000", "0000"]), ("ZYX1", ["X8", "X8", "X8"], ["00X1", "0X01", "X001", "0000"]),
    ("ZYX1", ["X8_Y8", "X8"], ["0YX1", "X001", "0000", "0000"]), ("ZYX1", ["X8", "X8_Y8"], ["00X1", "YX01", "0000", "0000"]),
    ("XYZ1", ["X8_Y8__X8_Z8"], ["XYZ1", "0000", "0000", "0000"]), ("XYZ1", ["Y8_X8__Z8_X8"], ["XYZ1", "0000", "0000", "0000"]),
    ("XZY1", ["X8_Y8__X8_Z8"], ["XZY1", "0000", "0000", "0000"]), ("XXX1", ["X8"], ["XXX1", "0000", "0000", "0000"]),
    ("XXXY", ["X8_Y8"], ["XXXY", "0000", "0000", "0000"]), ("ZYX0", ["X8_Y8_Z8"], ["ZYX0", "0000", "0000", "0000"]),
    ("XY01", ["X8", "X8"], ["X001", "0X01", "0000", "0000"]), ("YX01", ["X8", "X8"], ["0X01", "X001", "0000", "0000"]),
]


@pytest.mark.parametrize("sw,packs,plane_sw", PLANE_SWIZZLES)
def test_plane_swizzles_plane_formats_and_the_merge_back(nv, K, sw, packs, plane_sw):
    # TestImageFormat.cpp:1375-1479
    st, fmt = make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", sw, packs)
    assert st == 0
    out, planes = C.c_int(), []
    for p in range(4):
        assert nv.nvcvImageFormatGetPlaneSwizzle(fmt, p, C.byref(out)) == 0 and out.value == const(K, "SWIZZLE_" + plane_sw[p]), p
        f = C.c_uint64(77)
        assert nv.nvcvImageFormatGetPlaneFormat(fmt, p, C.byref(f)) == 0
        if p < len(packs):
            st, gold = make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", plane_sw[p], [packs[p]])
            assert st == 0 and f.value == gold
        else:
            assert f.value == 0
        planes.append(f.value)
    merged = C.c_uint64()
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(merged), *planes) == 0 and merged.value == fmt


def test_invalid_from_planes_and_plane_swizzle(nv, K):
    # TestImageFormat.cpp:731-748, :1481-1540
    f = C.c_uint64()
    assert nv.nvcvMakeImageFormatFromPlanes(None, 0, 0, 0, 0) == INVALID
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), 0, 0, 0, 0) == INVALID
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), K.IMAGE_FORMAT_RGB8p, 0, 0, 0) == INVALID
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), K.IMAGE_FORMAT_2S16, K.IMAGE_FORMAT_2S16, K.IMAGE_FORMAT_U8, K.IMAGE_FORMAT_U8) == INVALID
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), K.IMAGE_FORMAT_Y8_BL, K.IMAGE_FORMAT_Y8_ER, 0, 0) == INVALID
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), K.IMAGE_FORMAT_U8, K.IMAGE_FORMAT_U8_BL, 0, 0) == INVALID
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), K.IMAGE_FORMAT_U8, K.IMAGE_FORMAT_S8, 0, 0) == INVALID
    _, r1 = make_raw(nv, K, "BAYER_RGGB", "PL", "UNSIGNED", "X000", ["X8"])
    _, r2 = make_raw(nv, K, "BAYER_BGGR", "PL", "UNSIGNED", "X000", ["X8"])
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), r1, r2, 0, 0) == INVALID
    _, y1 = make_ycbcr(nv, K, "BT601", "422", "PL", "UNSIGNED", "X000", ["X8"])
    _, y2 = make_ycbcr(nv, K, "BT601", "422R", "PL", "UNSIGNED", "X000", ["X8"])
    assert nv.nvcvMakeImageFormatFromPlanes(C.byref(f), y2, y1, 0, 0) == INVALID
    assert nv.nvcvImageFormatGetPlaneSwizzle(K.IMAGE_FORMAT_NV12, 0, None) == INVALID
    assert nv.nvcvImageFormatGetPlaneFormat(K.IMAGE_FORMAT_NV12, 0, None) == INVALID


BAD_SWIZZLE_PACKING = [  # TestImageFormat.cpp:1563-1582
    ("XY00", ["X8"]), ("X000", ["X8", "X8"]), ("X000", ["X8_Y8"]), ("X000", ["X16_Y16"]), ("XY00", ["X8", "X8_Y8"]),
    ("XY00", ["X8", "X16_Y16"]), ("XYZ0", ["X8_Y8", "X8_Y8"]), ("XYZ0", ["X16_Y16", "X8_Y8"]), ("XYZ0", ["X8_Y8", "X16_Y16"]),
    ("XYZ0", ["X16_Y16", "X16_Y16"]), ("XYZW", ["X8_Y8", "X8", "X8_Y8"]), ("XYZW", ["X16_Y16", "X8", "X8_Y8"]),
    ("XYZW", ["X8_Y8", "X8", "X16_Y16"]), ("XYZW", ["X16_Y16", "X8", "X16_Y16"]), ("XYZ1", ["X8_Y8_Z8_W8"]),
    ("XYZ1", ["X8_Y8", "X8", "X8_Y8"]), ("XYZ1", ["X8_Y8", "X8", "X16_Y16"])]


@pytest.mark.parametrize("sw,packs", BAD_SWIZZLE_PACKING)
def test_swizzle_and_packings_must_name_the_same_number_of_channels(nv, K, sw, packs):
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", sw, packs)[0] == INVALID


def test_constructor_limits(nv, K):
    # TestImageFormat.cpp:1041-1070, :2220-2337
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "0000", ["0"])[0] == INVALID
    assert make_ycbcr(nv, K, "BT601", "420", "PL", "UNSIGNED", "0000", ["0"])[0] == INVALID
    assert make_noncolor(nv, K, "PL", "UNSIGNED", "0000", ["0"])[0] == INVALID
    assert make_raw(nv, K, "BAYER_RGGB", "PL", "UNSIGNED", "0000", ["0"])[0] == INVALID
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XY00", ["X8", "X256"])[0] == INVALID
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZ0", ["X8", "X8", "X256"])[0] == INVALID
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8", "X8", "X8", "X256"])[0] == INVALID
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8", "X8", "X8", "X128"])[0] == INVALID
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8", "X8", "X8", "X64"])[0] == 0
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZW", ["X8", "X8_Y8_Z8"])[0] == INVALID  # plane 1: 2 channels at most
    # a plane slot keeps 3 bits of a packing's sub-code (none for plane 3): values beyond cannot be stored. The reference
    # probes this with made-up packing values of the 16-bit one-channel family.
    base = K.PACKING_X16
    mk = lambda sw, pk: nv.nvcvMakeColorImageFormat(C.byref(C.c_uint64()), K.COLOR_MODEL_RGB, K.COLOR_SPEC_BT601, K.MEM_LAYOUT_PL,
                                                    K.DATA_KIND_UNSIGNED, const(K, "SWIZZLE_" + sw), *pk, K.ALPHA_ASSOCIATED, None)
    assert mk("X000", [base + 7, 0, 0, 0]) == 0 and mk("X000", [base + 8, 0, 0, 0]) == INVALID
    assert mk("XY00", [K.PACKING_X8, base + 7, 0, 0]) == 0 and mk("XY00", [K.PACKING_X8, base + 8, 0, 0]) == INVALID
    assert mk("XYZ0", [K.PACKING_X8, K.PACKING_X8, base + 7, 0]) == 0 and mk("XYZ0", [K.PACKING_X8, K.PACKING_X8, base + 8, 0]) == INVALID
    assert mk("XYZW", [K.PACKING_X8, K.PACKING_X8, K.PACKING_X8, base]) == 0 and mk("XYZW", [K.PACKING_X8, K.PACKING_X8, K.PACKING_X8, base + 1]) == INVALID
    assert mk("XY00", [K.PACKING_X8, K.PACKING_X128, 0, 0]) == 0 and mk("XY00", [K.PACKING_X8, K.PACKING_X192, 0, 0]) == INVALID
    assert mk("XYZ0", [K.PACKING_X8, K.PACKING_X8, K.PACKING_X128, 0]) == 0 and mk("XYZ0", [K.PACKING_X8, K.PACKING_X8, K.PACKING_X192, 0]) == INVALID
    # colour rules
    f = C.c_uint64()
    assert nv.nvcvMakeColorImageFormat(C.byref(f), K.COLOR_MODEL_RAW, K.COLOR_SPEC_UNDEFINED, 0, 0, K.SWIZZLE_X000, K.PACKING_X8, 0, 0, 0, 0, None) == INVALID
    assert make_color(nv, K, "UNDEFINED", "BT601", "PL", "UNSIGNED", "X000", ["X8"])[0] == INVALID
    assert make_color(nv, K, "HSV", "BT601", "PL", "UNSIGNED", "XYZ0", ["X8_Y8_Z8"])[0] == INVALID
    assert make_color(nv, K, "HSV", "UNDEFINED", "PL", "UNSIGNED", "XYZ0", ["X8_Y8_Z8"]) == (0, K.IMAGE_FORMAT_HSV8)
    assert nv.nvcvMakeColorImageFormat(None, K.COLOR_MODEL_RGB, K.COLOR_SPEC_UNDEFINED, 0, 0, K.SWIZZLE_X000, K.PACKING_X8, 0, 0, 0, 0, None) == INVALID
    # extra channels
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZ0", ["X8", "X8", "X8"], ex=ExtraInfo(2, 8, 0, 0))[0] == INVALID_IMAGE_FORMAT
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZ0", ["X8_Y8_Z8"], ex=ExtraInfo(8, 8, 0, 0))[0] == INVALID
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZ0", ["X8_Y8_Z8"], ex=ExtraInfo(2, 256, 0, 0))[0] == INVALID
    assert make_color(nv, K, "RGB", "UNDEFINED", "PL", "UNSIGNED", "XYZ1", ["X8_Y8_Z8"], ex=ExtraInfo(0, 0, 0, 0)) == (0, K.IMAGE_FORMAT_RGB8)


def test_packed_422_formats(nv, K):
    # TestImageFormat.cpp:1597-1689
    assert make_ycbcr(nv, K, "BT601", "422", "PL", "UNSIGNED", "XYZ1", ["X8_Y8__X8_Z8"]) == (0, K.IMAGE_FORMAT_YUYV)
    assert make_ycbcr(nv, K, "BT601", "422", "PL", "UNSIGNED", "XYZ1", ["Y8_X8__Z8_X8"]) == (0, K.IMAGE_FORMAT_UYVY)
    assert make_ycbcr(nv, K, "BT601", "422", "PL", "UNSIGNED", "XZY1", ["Y8_X8__Z8_X8"]) == (0, K.IMAGE_FORMAT_VYUY)
    st, yvyu = make_ycbcr(nv, K, "BT601", "422", "PL", "UNSIGNED", "XZY1", ["X8_Y8__X8_Z8"])
    out = C.c_int()
    assert st == 0 and nv.nvcvImageFormatGetNumChannels(yvyu, C.byref(out)) == 0 and out.value == 3
    ex = ExtraInfo(3, 16, K.DATA_KIND_SIGNED, K.EXTRA_CHANNEL_D)
    st, with_extra = make_ycbcr(nv, K, "BT601", "422", "PL", "UNSIGNED", "XYZ1", ["X8_Y8__X8_Z8"], ex=ex)
    got = ExtraInfo()
    assert st == 0 and nv.nvcvImageFormatGetExtraChannelInfo(with_extra, C.byref(got)) == 0
    assert (got.numChannels, got.bitsPerPixel, got.datakind, got.channelType) == (3, 16, K.DATA_KIND_SIGNED, K.EXTRA_CHANNEL_D)
    for fmt, stride in ((K.IMAGE_FORMAT_YUYV, 2), (K.IMAGE_FORMAT_UYVY, 2), (K.IMAGE_FORMAT_RGB8, 3), (K.IMAGE_FORMAT_NV12, 1), (K.IMAGE_FORMAT_RGBAf32, 16)):
        assert nv.nvcvImageFormatGetPlanePixelStrideBytes(fmt, 0, C.byref(out)) == 0 and out.value == stride
    assert nv.nvcvImageFormatGetPlanePixelStrideBytes(K.IMAGE_FORMAT_NV12, 1, C.byref(out)) == 0 and out.value == 2


def test_names(nv, K):
    # TestImageFormat.cpp:1691-1936
    for n in ("NONE", "U8", "U8_BL", "S16_BL", "S32", "Y8_BL", "Y8_ER", "Y8_ER_BL", "Y16_BL", "Y16_ER", "Y16_ER_BL", "NV12_BL", "NV12_ER_BL",
              "NV24", "NV24_BL", "NV24_ER", "NV24_ER_BL", "2S16_BL", "UYVY_BL", "UYVY_ER_BL", "YUYV_BL", "YUYV_ER_BL", "RGB8", "CMYK8", "YCCK8",
              "RGB8_1U_U8", "RGBA8"):
        assert nv.nvcvImageFormatGetName(getattr(K, "IMAGE_FORMAT_" + n)) == b"NVCV_IMAGE_FORMAT_" + n.encode()
    name = lambda st_fmt: nv.nvcvImageFormatGetName(st_fmt[1]).decode() if st_fmt[0] == 0 else st_fmt[0]
    assert name(make_noncolor(nv, K, "BLOCK4_LINEAR", "FLOAT", "YZWX", ["X16", "X32_Y32", "X1"])) == \
        "NVCVImageFormat(UNDEFINED,BLOCK4_LINEAR,FLOAT,YZWX,ASSOCIATED,X16,X32_Y32,X1)"
    assert name(make_color(nv, K, "RGB", "BT2020", "BLOCK16_LINEAR", "FLOAT", "YZWX", ["X8", "X8_Y8", "X32"])) == \
        "NVCVImageFormat(RGB,BT2020,BLOCK16_LINEAR,FLOAT,YZWX,ASSOCIATED,X8,X8_Y8,X32)"
    assert name(make_color(nv, K, "RGB", "BT2020", "BLOCK16_LINEAR", "FLOAT", "XYZW", ["X8_Y8_Z8_W8"], ex=ExtraInfo(3, 16, K.DATA_KIND_SIGNED, K.EXTRA_CHANNEL_D))) == \
        "NVCVImageFormat(RGB,BT2020,BLOCK16_LINEAR,FLOAT,XYZW,ASSOCIATED,3,16,SIGNED,D,X8_Y8_Z8_W8)"
    assert name(make_raw(nv, K, "BAYER_CRCC", "BLOCK8_LINEAR", "FLOAT", "YZWX", ["X16", "X8_Y8", "X1"])) == \
        "NVCVImageFormat(RAW,BAYER_CRCC,BLOCK8_LINEAR,FLOAT,YZWX,ASSOCIATED,X16,X8_Y8,X1)"
    assert name(make_ycbcr(nv, K, "BT2020", "422R", "BLOCK16_LINEAR", "FLOAT", "YZWX", ["X8", "X8_Y8", "X32"])) == \
        "NVCVImageFormat(YCbCr,BT2020,4:2:2R,BLOCK16_LINEAR,FLOAT,YZWX,ASSOCIATED,X8,X8_Y8,X32)"
    spec, sw = C.c_int(), C.c_int()
    assert nv.nvcvMakeColorSpec(C.byref(spec), K.COLOR_SPACE_DCIP3, K.YCbCr_ENC_SMPTE240M, K.COLOR_XFER_BT2020, K.COLOR_RANGE_LIMITED,
                                K.CHROMA_LOC_EVEN, K.CHROMA_LOC_ODD) == 0
    assert nv.nvcvMakeSwizzle(C.byref(sw), K.CHANNEL_Z, K.CHANNEL_Y, K.CHANNEL_W, K.CHANNEL_1) == 0
    assert name(make_ycbcr(nv, K, spec.value, "411R", "BLOCK16_LINEAR", "FLOAT", sw.value, ["X8", "X16_Y16"])) == \
        ("NVCVImageFormat(YCbCr,NVCVColorSpec(SPACE_DCIP3,ENC_SMPTE240M,XFER_BT2020,RANGE_LIMITED,LOC_EVEN,LOC_ODD),4:1:1R,"
         "BLOCK16_LINEAR,FLOAT,ZYW1,ASSOCIATED,X8,X16_Y16)")
    assert name(make_ycbcr(nv, K, "SMPTE240M", "422", "BLOCK16_LINEAR", "FLOAT", "XZY1", ["X8_Y8__X8_Z8"])) == \
        "NVCVImageFormat(YCbCr,SMPTE240M,4:2:2,BLOCK16_LINEAR,FLOAT,XZY1,ASSOCIATED,X8_Y8__X8_Z8)"
    assert name(make_ycbcr(nv, K, "BT2020", "444", "BLOCK16_LINEAR", "FLOAT", "YZWX", ["X8", "X8_Y8", "X32"])) == \
        "NVCVImageFormat(YCbCr,BT2020,4:4:4,BLOCK16_LINEAR,FLOAT,YZWX,ASSOCIATED,X8,X8_Y8,X32)"
    assert name(make_ycbcr(nv, K, "BT2020", "444", "BLOCK16_LINEAR", "FLOAT", "YZWX", ["X2Y10Z10W10"])) == \
        "NVCVImageFormat(YCbCr,BT2020,4:4:4,BLOCK16_LINEAR,FLOAT,YZWX,ASSOCIATED,X2Y10Z10W10)"
    # TestDataLayout.cpp:674-760
    assert nv.nvcvPackingGetName(K.PACKING_X16) == b"NVCV_PACKING_X16"
    assert nv.nvcvPackingGetName(0x7FFFFFFF) == b"NVCVPacking(2147483647)"
    assert nv.nvcvByteOrderGetName(K.ORDER_LSB) == b"LSB" and nv.nvcvByteOrderGetName(-1) == b"NVCVByteOrder(-1)"
    assert nv.nvcvSwizzleGetName(K.SWIZZLE_XYZ1) == b"XYZ1"
    assert nv.nvcvChannelGetName(K.CHANNEL_Y) == b"Y" and nv.nvcvChannelGetName(255) == b"NVCVChannel(255)"
    assert nv.nvcvChannelGetName(7) == b"NVCVChannel(7)"
    for n in ("BLOCK1_LINEAR", "BLOCK2_LINEAR", "BLOCK32_LINEAR"):
        assert nv.nvcvMemLayoutGetName(getattr(K, "MEM_LAYOUT_" + n)) == b"NVCV_MEM_LAYOUT_" + n.encode()
    assert nv.nvcvMemLayoutGetName(-1) == b"NVCVMemLayout(-1)"
    assert nv.nvcvDataKindGetName(K.DATA_KIND_FLOAT) == b"NVCV_DATA_KIND_FLOAT"
    assert nv.nvcvDataKindGetName(-1) == b"NVCV_DATA_KIND_UNSPECIFIED" and nv.nvcvDataKindGetName(-128) == b"NVCVDataKind(-128)"


def fcc(s):
    return sum(ord(c) << (8 * i) for i, c in enumerate(s))


FROM_FOURCC = [("RGB3", "RGB8"), ("BGR3", "BGR8"), ("RGB4", "RGBA8"), ("BGR4", "BGRA8"), ("GRAY", "Y8"), ("Y8  ", "Y8"), ("Y16 ", "Y16"),
               ("UYVY", "UYVY"), ("YUY2", "YUYV"), ("YUYV", "YUYV"), ("YUNV", "YUYV"), ("NV12", "NV12")]


@pytest.mark.parametrize("code,name", FROM_FOURCC)
def test_fourcc_to_format(nv, K, code, name):
    # TestImageFormat.cpp:2472-2558
    fmt = getattr(K, "IMAGE_FORMAT_" + name)
    spec, f, gold = C.c_int(), C.c_uint64(), C.c_uint64(fmt)
    assert nv.nvcvImageFormatGetColorSpec(fmt, C.byref(spec)) == 0
    assert nv.nvcvMakeImageFormatFromFourCC(C.byref(f), fcc(code), spec.value, K.MEM_LAYOUT_PL) == 0 and f.value == fmt
    assert nv.nvcvMakeImageFormatFromFourCC(C.byref(f), fcc(code.lower()), spec.value, K.MEM_LAYOUT_PL) == 0 and f.value == fmt
    assert nv.nvcvImageFormatSetColorSpec(C.byref(gold), K.COLOR_SPEC_UNDEFINED) == 0
    assert nv.nvcvMakeImageFormatFromFourCC(C.byref(f), fcc(code), K.COLOR_SPEC_UNDEFINED, K.MEM_LAYOUT_PL) == 0 and f.value == gold.value
    gold = C.c_uint64(fmt)
    assert nv.nvcvImageFormatSetMemLayout(C.byref(gold), K.MEM_LAYOUT_BL) == 0
    assert nv.nvcvMakeImageFormatFromFourCC(C.byref(f), fcc(code), spec.value, K.MEM_LAYOUT_BL) == 0 and f.value == gold.value
    gold = C.c_uint64(fmt)
    assert nv.nvcvImageFormatSetColorSpec(C.byref(gold), K.COLOR_SPEC_BT2020) == 0
    assert nv.nvcvMakeImageFormatFromFourCC(C.byref(f), fcc(code), K.COLOR_SPEC_BT2020, K.MEM_LAYOUT_PL) == 0 and f.value == gold.value


def test_format_to_fourcc(nv, K):
    # TestImageFormat.cpp:2485-2595
    out = C.c_uint32()
    for name, code in (("RGB8", "RGB3"), ("BGR8", "BGR3"), ("RGBA8", "RGB4"), ("BGRA8", "BGR4"), ("Y8", "GRAY"), ("UYVY", "UYVY"),
                       ("YUYV", "YUY2"), ("NV12", "NV12"), ("NV12_ER_BL", "NV12")):
        assert nv.nvcvImageFormatToFourCC(getattr(K, "IMAGE_FORMAT_" + name), C.byref(out)) == 0 and out.value == fcc(code), name
    assert nv.nvcvImageFormatToFourCC(K.IMAGE_FORMAT_2F32, C.byref(out)) == INVALID
    assert nv.nvcvImageFormatToFourCC(K.IMAGE_FORMAT_RGB8, None) == INVALID
    f = C.c_uint64()
    assert nv.nvcvMakeImageFormatFromFourCC(C.byref(f), fcc("RODS"), K.COLOR_SPEC_BT601, K.MEM_LAYOUT_PL) == INVALID
    assert nv.nvcvMakeImageFormatFromFourCC(None, fcc("RGB3"), K.COLOR_SPEC_BT601, K.MEM_LAYOUT_PL) == INVALID


def test_same_data_layout_and_plane_size(nv, K):
    # TestImageFormat.cpp:2124-2218, :2339-2370
    b = C.c_int8(-1)
    same = [("RGB8", "BGR8"), ("RGBA8", "BGRA8"), ("NV12", "NV12_ER"), ("NV12", "NV21"), ("YUYV", "YUYV_ER"), ("U8", "Y8"), ("U8", "Y8_ER")]
    diff = [("RGB8", "RGBA8"), ("RGB8", "RGB8p"), ("NV12", "NV12_BL"), ("NV12", "NV24"), ("U8", "S8"), ("U8", "U16"), ("YUYV", "UYVY")]
    for a, c in same:
        assert nv.nvcvImageFormatHasSameDataLayout(getattr(K, "IMAGE_FORMAT_" + a), getattr(K, "IMAGE_FORMAT_" + c), C.byref(b)) == 0 and b.value == 1, (a, c)
    for a, c in diff:
        assert nv.nvcvImageFormatHasSameDataLayout(getattr(K, "IMAGE_FORMAT_" + a), getattr(K, "IMAGE_FORMAT_" + c), C.byref(b)) == 0 and b.value == 0, (a, c)
    w, h = C.c_int32(), C.c_int32()
    assert nv.nvcvImageFormatGetPlaneSize(K.IMAGE_FORMAT_NV12, 0, 1920, 1080, C.byref(w), C.byref(h)) == 0 and (w.value, h.value) == (1920, 1080)
    assert nv.nvcvImageFormatGetPlaneSize(K.IMAGE_FORMAT_NV12, 1, 1920, 1080, C.byref(w), C.byref(h)) == 0 and (w.value, h.value) == (960, 540)
    assert nv.nvcvImageFormatGetPlaneSize(K.IMAGE_FORMAT_NV12, 1, 1921, 1081, C.byref(w), None) == 0 and w.value == 961
    assert nv.nvcvImageFormatGetPlaneSize(K.IMAGE_FORMAT_NV24, 1, 1921, 1081, None, C.byref(h)) == 0 and h.value == 1081
    assert nv.nvcvImageFormatGetPlaneSize(K.IMAGE_FORMAT_NV12, 1, 1920, 1080, None, None) == INVALID


# ---- packings: TestDataLayout.cpp:202-420 (table), :426-533 (checks) -------------------------------------------
def P(name, bits, order, align, swz, fields):
    return (name, bits + [0] * (4 - len(bits)), order, align, swz, fields + [0] * (4 - len(fields)))


def lsb(*b):  # DEF_PACKn: one word, channels only
    return P("".join("XYZW"[i] + str(v) for i, v in enumerate(b)), list(b), "LSB", sum(b) // 8, "XYZW"[:len(b)].ljust(4, "0") if False else "0000", list(b))


def fix(*b):  # DEF_FIX_PACKn: one word per channel
    return P("_".join("XYZW"[i] + str(v) for i, v in enumerate(b)), list(b), "MSB", b[0] // 8, ("XYZW"[:len(b)]).ljust(4, "0"), list(b))


PACKINGS = [
    P("X8_Y8__X8_Z8", [8, 8, 8, 8], "MSB", 1, "XYXZ", [8, 8, 8, 8]), P("Y8_X8__Z8_X8", [8, 8, 8, 8], "MSB", 1, "YXZX", [8, 8, 8, 8]),
    P("X5Y5b1Z5", [5, 5, 5], "LSB", 2, "XYW0", [5, 5, 1, 5]), P("X32_Y24b8", [32, 24], "MSB", 4, "XY00", [32, 24, 8]),
    lsb(1), fix(1), lsb(2), fix(2), lsb(4), fix(4), lsb(8), fix(8), lsb(4, 4), lsb(3, 3, 2), lsb(16), fix(16), fix(8, 8),
    P("b4X4", [4], "LSB", 1, "Y000", [4, 4]), P("X4b4", [4], "MSB", 1, "X000", [4, 4]),
    P("b6X10", [10], "LSB", 2, "Y000", [6, 10]), P("X10b6", [10], "MSB", 2, "X000", [10, 6]),
    P("b2X14", [14], "LSB", 2, "Y000", [2, 14]), P("X14b2", [14], "MSB", 2, "X000", [14, 2]),
    P("X12b4", [12], "MSB", 2, "X000", [12, 4]), P("b4X12", [12], "LSB", 2, "Y000", [4, 12]),
    lsb(5, 5, 6), lsb(5, 6, 5), lsb(6, 5, 5), P("b4X4Y4Z4", [4, 4, 4], "LSB", 2, "YZW0", [4, 4, 4, 4]),
    P("X4Y4Z4W4", [4, 4, 4, 4], "LSB", 2, "XYZW", [4, 4, 4, 4]), P("b1X5Y5Z5", [5, 5, 5], "LSB", 2, "YZW0", [1, 5, 5, 5]),
    lsb(1, 5, 5, 5), lsb(5, 1, 5, 5), lsb(5, 5, 1, 5), lsb(5, 5, 5, 1), lsb(24), fix(24), fix(8, 8, 8), lsb(32), fix(32), fix(16, 16),
    P("X20b12", [20], "MSB", 4, "X000", [20, 12]), P("b12X20", [20], "LSB", 4, "Y000", [12, 20]),
    P("X24b8", [24], "MSB", 4, "X000", [24, 8]), P("b8X24", [24], "LSB", 4, "Y000", [8, 24]),
    lsb(10, 11, 11), lsb(11, 11, 10), lsb(2, 10, 10, 10), fix(8, 8, 8, 8), P("X10b6_Y10b6", [10, 10], "MSB", 2, "XZ00", [10, 6, 10, 6]),
    lsb(10, 10, 10, 2), P("X12b4_Y12b4", [12, 12], "MSB", 2, "XZ00", [12, 4, 12, 4]),
    P("b2X10Y10Z10", [10, 10, 10], "LSB", 4, "YZW0", [2, 10, 10, 10]), P("X10Y10Z10b2", [10, 10, 10], "MSB", 4, "XYZ0", [10, 10, 10, 2]),
    lsb(48), fix(48), fix(16, 16, 16), lsb(64), fix(64), fix(32, 32), fix(16, 16, 16, 16), lsb(96), fix(96), fix(32, 32, 32),
    lsb(128), fix(128), fix(64, 64), fix(32, 32, 32, 32), lsb(192), fix(192), fix(64, 64, 64), lsb(256), fix(256), fix(128, 128),
    fix(64, 64, 64, 64),
]


@pytest.mark.parametrize("name,bits,order,align,swz,fields", PACKINGS, ids=["%s-%s" % (p[0], p[2]) for p in PACKINGS])
def test_packing_from_and_to_parameters(nv, K, name, bits, order, align, swz, fields):
    packing = const(K, "PACKING_" + name)
    prm = PackingParams(const(K, "ORDER_" + order), align, const(K, "SWIZZLE_" + swz), (C.c_int32 * 4)(*fields))
    out = C.c_int(-1)
    assert nv.nvcvMakePacking(C.byref(out), C.byref(prm)) == 0 and out.value == packing
    nch = C.c_int()
    assert nv.nvcvSwizzleGetNumChannels(prm.swizzle, C.byref(nch)) == 0
    if nch.value == 1:  # one channel: either byte order names the same packing
        prm.byteOrder ^= 1
        assert nv.nvcvMakePacking(C.byref(out), C.byref(prm)) == 0 and out.value == packing
    got = PackingParams()
    assert nv.nvcvPackingGetParams(packing, C.byref(got)) == 0
    assert got.byteOrder == (K.ORDER_LSB if fields[1] == 0 else const(K, "ORDER_" + order))
    assert list(got.bits) == fields
    b = (C.c_int32 * 4)()
    assert nv.nvcvPackingGetBitsPerComponent(packing, b) == 0 and list(b) == bits
    n = C.c_int()
    assert nv.nvcvPackingGetNumComponents(packing, C.byref(n)) == 0 and n.value == sum(1 for v in bits if v)
    assert nv.nvcvPackingGetBitsPerPixel(packing, C.byref(n)) == 0
    assert n.value == (16 if "__" in name else sum(fields))


def test_packing_edge_cases(nv, K):
    # TestDataLayout.cpp:127-130, :680-720
    out = C.c_int(-1)
    zero = PackingParams(K.ORDER_LSB, 0, K.SWIZZLE_0000, (C.c_int32 * 4)(0, 0, 0, 0))
    assert nv.nvcvMakePacking(C.byref(out), C.byref(zero)) == 0 and out.value == 0
    for name, align in (("X24", 4), ("X4b4", 1), ("X10b6", 2), ("b4X12", 2), ("X8_Y8", 1), ("X5Y5Z6", 2), ("b4X4Y4Z4", 2), ("X1Y5Z5W5", 2),
                        ("X8_Y8__X8_Z8", 1), ("X8_Y8_Z8", 1), ("b2X10Y10Z10", 4), ("X12b4_Y12b4", 2), ("X32_Y24b8", 4)):
        assert nv.nvcvPackingGetAlignment(const(K, "PACKING_" + name), C.byref(out)) == 0 and out.value == align, name
    prm = PackingParams()
    assert nv.nvcvPackingGetParams(K.PACKING_X16, None) == INVALID
    assert nv.nvcvPackingGetParams(K.PACKING_X16, C.byref(prm)) == 0
    assert nv.nvcvMakePacking(C.byref(out), None) == INVALID and nv.nvcvMakePacking(None, C.byref(prm)) == INVALID
    none = PackingParams(K.ORDER_LSB, 0, K.SWIZZLE_0000, (C.c_int32 * 4)(7, 9, 0, 0))
    assert nv.nvcvMakePacking(C.byref(out), C.byref(none)) == INVALID
    # two channels in one word exist only in LSB order, in separate words only in MSB order
    assert nv.nvcvMakePacking(C.byref(out), C.byref(PackingParams(K.ORDER_MSB, 0, K.SWIZZLE_XY00, (C.c_int32 * 4)(4, 4, 0, 0)))) == INVALID
    assert nv.nvcvMakePacking(C.byref(out), C.byref(PackingParams(K.ORDER_LSB, 0, K.SWIZZLE_XY00, (C.c_int32 * 4)(8, 8, 0, 0)))) == INVALID
    # the alignment asked for does not take part in the choice
    for align in (0, 1, 8):
        assert nv.nvcvMakePacking(C.byref(out), C.byref(PackingParams(K.ORDER_MSB, align, K.SWIZZLE_XY00, (C.c_int32 * 4)(16, 16, 0, 0)))) == 0
        assert out.value == K.PACKING_X16_Y16


# ---- data types: tests/nvcv_types/system/TestDataType.cpp ---------------------------------------------------
def make_type(nv, K, kind, packing):
    t = C.c_uint64()
    assert nv.nvcvMakeDataType(C.byref(t), const(K, "DATA_KIND_" + kind), const(K, "PACKING_" + packing)) == 0
    return t.value


def dtype(nv, K, spec):
    """'U8' -> the named constant, ('FLOAT', 'X8_Y8_Z8') -> made from kind and packing."""
    return getattr(K, "DATA_TYPE_" + spec) if isinstance(spec, str) else make_type(nv, K, *spec)


DATA_TYPES = [  # TestDataType.cpp:55-74: type, kind, packing, channels, bits per pixel
    (("FLOAT", "X32_Y32_Z32_W32"), "FLOAT", "X32_Y32_Z32_W32", 4, 128), ("U8", "UNSIGNED", "X8", 1, 8), ("S8", "SIGNED", "X8", 1, 8),
    ("U16", "UNSIGNED", "X16", 1, 16), ("S16", "SIGNED", "X16", 1, 16), ("2U8", "UNSIGNED", "X8_Y8", 2, 16),
    ("3U8", "UNSIGNED", "X8_Y8_Z8", 3, 24), ("4U8", "UNSIGNED", "X8_Y8_Z8_W8", 4, 32), ("F32", "FLOAT", "X32", 1, 32),
    ("F64", "FLOAT", "X64", 1, 64), ("C64", "COMPLEX", "X64", 1, 64), ("4C64", "COMPLEX", "X64_Y64_Z64_W64", 4, 256),
    ("C128", "COMPLEX", "X128", 1, 128), ("2C128", "COMPLEX", "X128_Y128", 2, 256), (("UNSIGNED", "X10Y11Z11"), "UNSIGNED", "X10Y11Z11", 3, 32),
    (("UNSIGNED", "X5Y6Z5"), "UNSIGNED", "X5Y6Z5", 3, 16), (("UNSIGNED", "X10b6_Y10b6"), "UNSIGNED", "X10b6_Y10b6", 2, 32),
    ("2F32", "FLOAT", "X32_Y32", 2, 64)]


@pytest.mark.parametrize("spec,kind,packing,channels,bpp", DATA_TYPES, ids=[str(d[0]) for d in DATA_TYPES])
def test_data_type_properties(nv, K, spec, kind, packing, channels, bpp):
    t = dtype(nv, K, spec)
    out = C.c_int(-9)
    assert nv.nvcvDataTypeGetPacking(C.c_uint64(t), C.byref(out)) == 0 and out.value == const(K, "PACKING_" + packing)
    assert nv.nvcvDataTypeGetBitsPerPixel(C.c_uint64(t), C.byref(out)) == 0 and out.value == bpp
    assert nv.nvcvDataTypeGetDataKind(C.c_uint64(t), C.byref(out)) == 0 and out.value == const(K, "DATA_KIND_" + kind)
    assert nv.nvcvDataTypeGetNumChannels(C.c_uint64(t), C.byref(out)) == 0 and out.value == channels
    assert make_type(nv, K, kind, packing) == t
    bits, want = (C.c_int32 * 4)(), (C.c_int32 * 4)()
    assert nv.nvcvDataTypeGetBitsPerChannel(C.c_uint64(t), bits) == 0
    assert nv.nvcvPackingGetBitsPerComponent(const(K, "PACKING_" + packing), want) == 0 and list(bits) == list(want)


def test_data_types_equal_their_image_formats_and_names(nv, K):
    # TestDataType.cpp:145-224
    for n in ("U8", "S8", "U16", "S16", "F32", "2F32", "C64", "2C64", "C128", "2C128"):
        assert getattr(K, "IMAGE_FORMAT_" + n) == getattr(K, "DATA_TYPE_" + n)
    assert K.DATA_TYPE_NONE == 0
    nv.nvcvDataTypeGetName.restype = C.c_char_p
    nv.nvcvDataTypeGetName.argtypes = [C.c_uint64]
    names = ["NONE", "U8", "2S8", "3S8", "4S8", "2U16", "3U16", "4U16", "2S16", "3S16", "4S16", "U32", "2U32", "3U32", "4U32", "S32",
             "2S32", "3S32", "4S32", "F16", "2F16", "3F16", "4F16", "3F32", "U64", "2U64", "3U64", "4U64", "S64", "2S64", "3S64", "4S64",
             "2F64", "3F64", "4F64", "3C64"]
    for n in names:
        assert nv.nvcvDataTypeGetName(getattr(K, "DATA_TYPE_" + n)) == b"NVCV_DATA_TYPE_" + n.encode(), n
    assert nv.nvcvDataTypeGetName(make_type(nv, K, "FLOAT", "X8_Y8_Z8")) == b"NVCVDataType(FLOAT,X8_Y8_Z8)"
    out = C.c_int()
    assert nv.nvcvMakeDataType(None, K.DATA_KIND_FLOAT, K.PACKING_X8_Y8_Z8) == INVALID
    for f in ("nvcvDataTypeGetPacking", "nvcvDataTypeGetBitsPerPixel", "nvcvDataTypeGetBitsPerChannel", "nvcvDataTypeGetDataKind",
              "nvcvDataTypeGetNumChannels", "nvcvDataTypeGetStrideBytes", "nvcvDataTypeGetAlignment"):
        assert getattr(nv, f)(C.c_uint64(K.DATA_TYPE_U8), None) == INVALID, f
    assert nv.nvcvDataTypeGetChannelType(C.c_uint64(K.DATA_TYPE_U8), 0, None) == INVALID


CHANNEL_TYPES = [  # TestDataType.cpp:246-290: type, channel, type of that channel (None = INVALID_ARGUMENT)
    ("U8", 0, "U8"), ("U8", 4, "NONE"), (("FLOAT", "X32"), 0, ("FLOAT", "X32")), (("FLOAT", "X8_Y8_Z8"), 2, ("FLOAT", "X8")),
    ("2F32", 0, "F32"), ("2F32", 1, "F32"), ("2C64", 0, "C64"), ("2C64", 1, "C64"), ("2C128", 0, "C128"), ("2C128", 1, "C128"),
    (("SIGNED", "X64_Y64_Z64_W64"), 3, "S64"), (("UNSIGNED", "X4Y4"), 0, ("UNSIGNED", "X4")), (("UNSIGNED", "b4X4Y4Z4"), 2, ("UNSIGNED", "X4")),
    (("UNSIGNED", "X3Y3Z2"), 2, ("UNSIGNED", "X2")), (("UNSIGNED", "X1"), 0, ("UNSIGNED", "X1")), (("UNSIGNED", "X2"), 0, ("UNSIGNED", "X2")),
    ("3S16", 2, "S16"), (("SIGNED", "X24"), 0, ("SIGNED", "X24")), ("2F64", 1, "F64"), (("SIGNED", "X96"), 0, ("SIGNED", "X96")),
    (("SIGNED", "X128"), 0, ("SIGNED", "X128")), (("SIGNED", "X192"), 0, ("SIGNED", "X192")), (("SIGNED", "X256"), 0, ("SIGNED", "X256")),
    ("U8", 1, "NONE"), ("2F32", 2, "NONE"), (("UNSIGNED", "b4X4Y4Z4"), 3, "NONE"),
    ("U8", -1, None), (("UNSIGNED", "X5Y5b1Z5"), 0, None), (("UNSIGNED", "X3Y3Z2"), 1, None)]


@pytest.mark.parametrize("spec,channel,want", CHANNEL_TYPES, ids=["%s-%d" % (str(c[0]), c[1]) for c in CHANNEL_TYPES])
def test_channel_type_of_a_data_type(nv, K, spec, channel, want):
    out = C.c_uint64(99)
    st = nv.nvcvDataTypeGetChannelType(C.c_uint64(dtype(nv, K, spec)), channel, C.byref(out))
    if want is None:
        assert st == INVALID
    else:
        assert st == 0 and out.value == dtype(nv, K, want)


def test_data_type_stride_and_alignment(nv, K):
    # TestDataType.cpp:313-375
    out = C.c_int32()
    for spec, stride in (("U8", 1), ("U16", 2), ("3S8", 3), ("2U16", 4), (("SIGNED", "X256"), 32), ("2F32", 8), ("C64", 8), ("4C64", 32),
                         ("C128", 16), ("2C128", 32), (("FLOAT", "X8_Y8_Z8"), 3)):
        assert nv.nvcvDataTypeGetStrideBytes(C.c_uint64(dtype(nv, K, spec)), C.byref(out)) == 0 and out.value == stride, spec
    for spec, align in (("U8", 1), ("U16", 2), ("3S8", 1), ("2U16", 2), (("SIGNED", "X256"), 32), ("2F32", 4), ("C64", 8), ("2C64", 8),
                        ("C128", 16), ("2C128", 16), (("SIGNED", "X5Y1Z5W5"), 2), (("SIGNED", "X3Y3Z2"), 1), (("SIGNED", "X4b4"), 1),
                        (("SIGNED", "b4X4"), 1), (("SIGNED", "b4X12"), 2), (("SIGNED", "X10b6"), 2), (("SIGNED", "X4Y4Z4W4"), 2),
                        (("SIGNED", "X8_Y8__X8_Z8"), 1), (("SIGNED", "X32_Y24b8"), 4)):
        assert nv.nvcvDataTypeGetAlignment(C.c_uint64(dtype(nv, K, spec)), C.byref(out)) == 0 and out.value == align, spec
