"""Host-side logic of the NVCV core library (no GPU needed): status slot, formats, layouts,
requirements arithmetic, stride rules, wrap validation, reference counting, handle reuse.

Expectations follow the reference's behaviour (cited per test) -- shape->stride rules of
src/nvcv/src/priv/Tensor.cpp:172-185, validation of TensorWrapDataStrided.cpp:35-105, status
semantics of priv/Status.cpp:31-110 -- with this library's alignment constants (128-byte rows,
512-byte base)."""
import ctypes as C
import os

import numpy as np
import pytest


@pytest.fixture(scope="module")
def capi(cv):
    import cvcuda_amd._capi as capi
    return capi


def fake_tensor(cv, shape, strides, dtype, layout, ptr=0x10000):
    return cv.Tensor.wrap(ptr, shape, strides, dtype, layout)


# ------------------------------------------------------------------------------------------ status
def test_status_slot_semantics(cv, capi):
    nv = capi.nvcv
    nv.nvcvGetLastError()
    buf = C.create_string_buffer(256)
    assert nv.nvcvPeekAtLastErrorMessage(buf, 256) == 0 and buf.value == b"success"
    with pytest.raises(cv.Error) as e:
        cv.Tensor.requirements([2, 2], np.uint8, "NHWC")
    assert e.value.status == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvPeekAtLastError() == 2  # peek does not clear
    # a successful call leaves the last error in place
    cv.Tensor.requirements([2, 2, 2, 2], np.uint8, "NHWC")
    assert nv.nvcvPeekAtLastError() == 2
    assert nv.nvcvGetLastErrorMessage(buf, 256) == 2 and b"must be equal to layout" in buf.value
    assert nv.nvcvGetLastError() == 0  # get cleared it
    assert nv.nvcvStatusGetName(10) == b"NVCV_ERROR_OVERFLOW"
    # tiny buffers are NUL-terminated, never overrun
    small = C.create_string_buffer(b"xxxxxxxx", 8)
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_INTERNAL, b"%s-%d", b"abcdefghij", 42)
    assert nv.nvcvGetLastErrorMessage(small, 4) == 8 and small.value == b"abc"


def test_status_is_per_thread(cv, capi):
    import threading
    nv = capi.nvcv
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_NOT_READY, None)
    seen = []
    t = threading.Thread(target=lambda: seen.append(nv.nvcvPeekAtLastError()))
    t.start()
    t.join()
    assert seen == [0] and nv.nvcvGetLastError() == capi.NVCV_ERROR_NOT_READY


# ------------------------------------------------------------------------------------------ formats
def test_format_queries(cv, capi, K):
    nv = capi.nvcv

    def q(fn, *a):
        out = C.c_int32()
        assert getattr(nv, fn)(*a, C.byref(out)) == 0
        return out.value

    assert q("nvcvImageFormatGetNumPlanes", K.IMAGE_FORMAT_RGB8) == 1
    assert q("nvcvImageFormatGetNumChannels", K.IMAGE_FORMAT_RGB8) == 3
    assert q("nvcvImageFormatGetNumPlanes", K.IMAGE_FORMAT_RGBf32p) == 3
    assert q("nvcvImageFormatGetNumPlanes", K.IMAGE_FORMAT_RGBA8p) == 4
    assert q("nvcvImageFormatGetPlaneBitsPerPixel", K.IMAGE_FORMAT_RGBA8p, 3) == 8
    assert q("nvcvImageFormatGetNumPlanes", K.IMAGE_FORMAT_NV12) == 2
    assert q("nvcvImageFormatGetNumChannels", K.IMAGE_FORMAT_NV12) == 3
    assert q("nvcvImageFormatGetPlaneNumChannels", K.IMAGE_FORMAT_NV12, 1) == 2
    assert q("nvcvImageFormatGetPlanePixelStrideBytes", K.IMAGE_FORMAT_NV12, 1) == 2
    assert q("nvcvImageFormatGetPlanePixelStrideBytes", K.IMAGE_FORMAT_RGBAf32, 0) == 16
    assert q("nvcvImageFormatGetNumChannels", K.IMAGE_FORMAT_U8) == 1
    assert q("nvcvImageFormatGetNumChannels", K.IMAGE_FORMAT_NONE) == 0
    pw, ph = C.c_int32(), C.c_int32()
    assert nv.nvcvImageFormatGetPlaneSize(K.IMAGE_FORMAT_NV12, 1, 1921, 1081, C.byref(pw), C.byref(ph)) == 0
    assert (pw.value, ph.value) == (961, 541)  # ceil(w/2), ceil(h/2)
    dt = C.c_uint64()
    assert nv.nvcvImageFormatGetPlaneDataType(K.IMAGE_FORMAT_RGB8, 0, C.byref(dt)) == 0 and dt.value == K.DATA_TYPE_3U8
    assert nv.nvcvImageFormatGetPlaneDataType(K.IMAGE_FORMAT_NV12, 1, C.byref(dt)) == 0 and dt.value == K.DATA_TYPE_2U8
    assert nv.nvcvImageFormatGetPlaneDataType(K.IMAGE_FORMAT_RGBf32p, 2, C.byref(dt)) == 0 and dt.value == K.DATA_TYPE_F32
    v = C.c_int()
    assert nv.nvcvImageFormatGetColorModel(K.IMAGE_FORMAT_NV12, C.byref(v)) == 0 and v.value == K.COLOR_MODEL_YCbCr
    assert nv.nvcvImageFormatGetColorModel(K.IMAGE_FORMAT_BGR8, C.byref(v)) == 0 and v.value == K.COLOR_MODEL_RGB
    assert nv.nvcvImageFormatGetColorModel(K.IMAGE_FORMAT_HSV8, C.byref(v)) == 0 and v.value == K.COLOR_MODEL_HSV
    assert nv.nvcvImageFormatGetColorModel(K.IMAGE_FORMAT_F32, C.byref(v)) == 0 and v.value == K.COLOR_MODEL_UNDEFINED
    assert nv.nvcvImageFormatGetChromaSubsampling(K.IMAGE_FORMAT_NV12, C.byref(v)) == 0 and v.value == K.CSS_420
    assert nv.nvcvImageFormatGetSwizzle(K.IMAGE_FORMAT_BGRA8, C.byref(v)) == 0 and v.value == K.SWIZZLE_ZYXW
    assert nv.nvcvImageFormatGetColorSpec(K.IMAGE_FORMAT_NV12_ER, C.byref(v)) == 0 and v.value == K.COLOR_SPEC_BT601_ER
    assert nv.nvcvImageFormatGetName(K.IMAGE_FORMAT_RGB8) == b"NVCV_IMAGE_FORMAT_RGB8"
    assert nv.nvcvDataTypeGetName(K.DATA_TYPE_3F32) == b"NVCV_DATA_TYPE_3F32"
    # constructors reproduce the header constants
    f = C.c_uint64()
    assert nv.nvcvMakeColorImageFormat(C.byref(f), K.COLOR_MODEL_RGB, K.COLOR_SPEC_UNDEFINED, K.MEM_LAYOUT_PL,
                                       K.DATA_KIND_UNSIGNED, K.SWIZZLE_ZYX1, K.PACKING_X8_Y8_Z8, 0, 0, 0,
                                       K.ALPHA_ASSOCIATED, None) == 0
    assert f.value == K.IMAGE_FORMAT_BGR8
    assert nv.nvcvMakeYCbCrImageFormat(C.byref(f), K.COLOR_SPEC_BT601, K.CSS_420, K.MEM_LAYOUT_PL,
                                       K.DATA_KIND_UNSIGNED, K.SWIZZLE_XYZ0, K.PACKING_X8, K.PACKING_X8_Y8, 0, 0,
                                       K.ALPHA_ASSOCIATED, None) == 0
    assert f.value == K.IMAGE_FORMAT_NV12
    assert nv.nvcvMakeNonColorImageFormat(C.byref(f), K.MEM_LAYOUT_PL, K.DATA_KIND_FLOAT, K.SWIZZLE_X000,
                                          K.PACKING_X32, 0, 0, 0, K.ALPHA_ASSOCIATED, None) == 0
    assert f.value == K.IMAGE_FORMAT_F32
    assert nv.nvcvMakeDataType(C.byref(f), K.DATA_KIND_SIGNED, K.PACKING_X16_Y16_Z16_W16) == 0
    assert f.value == K.DATA_TYPE_4S16


def test_data_type_queries(cv, capi, K):
    nv = capi.nvcv
    v = C.c_int32()
    for dt, (bpp, nch, stride, align) in {K.DATA_TYPE_U8: (8, 1, 1, 1), K.DATA_TYPE_3U8: (24, 3, 3, 1),
                                         K.DATA_TYPE_4F32: (128, 4, 16, 4), K.DATA_TYPE_2S16: (32, 2, 4, 2),
                                         K.DATA_TYPE_F64: (64, 1, 8, 8)}.items():
        assert nv.nvcvDataTypeGetBitsPerPixel(dt, C.byref(v)) == 0 and v.value == bpp
        assert nv.nvcvDataTypeGetNumChannels(dt, C.byref(v)) == 0 and v.value == nch
        assert nv.nvcvDataTypeGetStrideBytes(dt, C.byref(v)) == 0 and v.value == stride
        assert nv.nvcvDataTypeGetAlignment(dt, C.byref(v)) == 0 and v.value == align
    ch = C.c_uint64()
    assert nv.nvcvDataTypeGetChannelType(K.DATA_TYPE_3F32, 2, C.byref(ch)) == 0 and ch.value == K.DATA_TYPE_F32
    assert nv.nvcvDataTypeGetChannelType(K.DATA_TYPE_3F32, 3, C.byref(ch)) == 0 and ch.value == K.DATA_TYPE_NONE
    assert nv.nvcvDataTypeGetChannelType(K.DATA_TYPE_3F32, -1, C.byref(ch)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    n = C.c_int32()
    assert nv.nvcvSwizzleGetNumChannels(K.SWIZZLE_XXX1, C.byref(n)) == 0 and n.value == 1
    assert nv.nvcvSwizzleGetNumChannels(K.SWIZZLE_ZYXW, C.byref(n)) == 0 and n.value == 4
    sw = C.c_int()
    assert nv.nvcvMakeSwizzle(C.byref(sw), K.CHANNEL_Z, K.CHANNEL_Y, K.CHANNEL_X, K.CHANNEL_1) == 0
    assert sw.value == K.SWIZZLE_ZYX1


# ------------------------------------------------------------------------------------------ layouts
def test_layout_builders_and_permute(cv, capi):
    nv = capi.nvcv
    L = capi.TensorLayout
    out = L()
    assert nv.nvcvTensorLayoutMake(b"NHWC", C.byref(out)) == 0 and str(out) == "NHWC" and out.rank == 4
    assert nv.nvcvTensorLayoutMake(None, C.byref(out)) == 0 and out.rank == 0
    assert nv.nvcvTensorLayoutMake(b"ABCDEFGHIJKLMNOP", C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    nhwc = L.make("NHWC")
    assert nv.nvcvTensorLayoutMakeFirst(nhwc, 2, C.byref(out)) == 0 and str(out) == "NH"
    assert nv.nvcvTensorLayoutMakeLast(nhwc, 2, C.byref(out)) == 0 and str(out) == "WC"
    assert nv.nvcvTensorLayoutMakeFirst(nhwc, -3, C.byref(out)) == 0 and str(out) == "HWC"
    assert nv.nvcvTensorLayoutMakeLast(nhwc, 9, C.byref(out)) == 0 and str(out) == "NHWC"
    assert nv.nvcvTensorLayoutMakeSubRange(nhwc, 1, -1, C.byref(out)) == 0 and str(out) == "HW"
    assert nv.nvcvTensorLayoutMakeSubRange(nhwc, 3, 1, C.byref(out)) == 0 and out.rank == 0
    src = (C.c_int64 * 4)(5, 7, 9, 3)
    dst = (C.c_int64 * 4)()
    assert nv.nvcvTensorShapePermute(nhwc, src, L.make("NCHW"), dst) == 0 and list(dst) == [5, 3, 7, 9]
    dst3 = (C.c_int64 * 3)()
    assert nv.nvcvTensorShapePermute(L.make("HW"), (C.c_int64 * 2)(4, 6), L.make("CHW"), dst3) == 0
    assert list(dst3) == [1, 4, 6]


# ------------------------------------------------------------------------------------------ requirements
def test_mem_requirements_arithmetic(cv, capi):
    nv = capi.nvcv
    req = capi.Requirements()
    assert nv.nvcvRequirementsInit(C.byref(req)) == 0
    m = req.cudaMem
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), 1000, 256) == 0
    assert m.numBlocks[8] == 4  # ceil(1000/256) blocks of 2^8
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), 1, 64) == 0 and m.numBlocks[6] == 1
    total = C.c_int64()
    assert nv.nvcvMemRequirementsCalcTotalSizeBytes(C.byref(m), C.byref(total)) == 0 and total.value == 4 * 256 + 64
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), -600, 256) == 0 and m.numBlocks[8] == 1
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), -6000, 256) == 0 and m.numBlocks[8] == 0
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), 10, 3) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), 10, 0) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), 10, 1 << 32) == capi.NVCV_ERROR_INVALID_ARGUMENT
    other = capi.Requirements()
    other.hostMem.numBlocks[4] = 3
    assert nv.nvcvRequirementsAdd(C.byref(req), C.byref(other)) == 0 and req.hostMem.numBlocks[4] == 3


def test_tensor_stride_rules(cv, K):
    def strides(shape, dt, layout, **kw):
        r = cv.Tensor.requirements(shape, dt, layout, **kw)
        return [r.strides[i] for i in range(len(shape))], r.alignBytes

    # ...WC layouts: W and C packed, the row (H stride) padded to 128 bytes
    assert strides([64, 1080, 1920, 3], np.uint8, "NHWC") == ([1080 * 5760, 5760, 3, 1], 512)
    assert strides([8, 224, 224, 3], np.uint8, "NHWC") == ([224 * 768, 768, 3, 1], 512)
    assert strides([224, 224, 3], np.uint8, "HWC") == ([768, 3, 1], 512)
    assert strides([16, 360, 640, 4], np.float32, "NHWC") == ([360 * 10240, 10240, 16, 4], 512)
    # other layouts: only the innermost dimension packed, the next one padded
    assert strides([64, 3, 224, 224], np.float32, "NCHW") == ([3 * 224 * 896, 224 * 896, 896, 4], 512)
    assert strides([2, 3, 5, 7], np.uint8, "NCHW") == ([3 * 5 * 128, 5 * 128, 128, 1], 512)
    assert strides([32, 1620, 1920, 1], np.uint8, "NHWC") == ([1620 * 1920, 1920, 1, 1], 512)
    assert strides([10], np.float32, "W") == ([4], 512)
    assert strides([3, 10], np.int16, "NW") == ([128, 2], 512)
    assert strides([5, 6], np.float32, "WC") == ([24, 4], 512)  # nothing outside the packed pair
    # caller-chosen alignments
    assert strides([2, 4, 5, 3], np.uint8, "NHWC", row_align=32, base_align=64) == ([128, 32, 3, 1], 64)
    assert strides([2, 4, 5, 3], np.uint8, "NHWC", row_align=1, base_align=1) == ([60, 15, 3, 1], 1)
    r = cv.Tensor.requirements([2, 4, 5, 3], np.uint8, "NHWC")
    assert r.mem.cudaMem.numBlocks[9] == 2  # 2 images x 4 rows x 128 B = 1024 B = 2 blocks of 512
    for bad in ({"row_align": 3}, {"base_align": 48}):
        with pytest.raises(cv.Error) as e:
            cv.Tensor.requirements([2, 4, 5, 3], np.uint8, "NHWC", **bad)
        assert e.value.status == 2
    with pytest.raises(cv.Error):
        cv.Tensor.requirements([], np.uint8, "")


def test_tensor_requirements_for_images(cv, capi, K):
    nv = capi.nvcv
    r = capi.TensorRequirements()
    assert nv.nvcvTensorCalcRequirementsForImages(4, 100, 50, K.IMAGE_FORMAT_RGB8, 0, 0, C.byref(r)) == 0
    assert str(r.layout) == "NHWC" and [r.shape[i] for i in range(4)] == [4, 50, 100, 3] and r.dtype == K.DATA_TYPE_U8
    assert [r.strides[i] for i in range(4)] == [50 * 384, 384, 3, 1]
    assert nv.nvcvTensorCalcRequirementsForImages(1, 100, 50, K.IMAGE_FORMAT_RGBf32p, 0, 0, C.byref(r)) == 0
    assert str(r.layout) == "NCHW" and [r.shape[i] for i in range(4)] == [1, 3, 50, 100] and r.dtype == K.DATA_TYPE_F32
    assert nv.nvcvTensorCalcRequirementsForImages(1, 100, 50, K.IMAGE_FORMAT_NV12, 0, 0, C.byref(r)) \
        == capi.NVCV_ERROR_NOT_IMPLEMENTED  # subsampled planes cannot form a tensor


def test_image_requirements(cv, capi, K):
    nv = capi.nvcv
    r = capi.ImageRequirements()
    assert nv.nvcvImageCalcRequirements(1921, 1081, K.IMAGE_FORMAT_NV12, 0, 0, C.byref(r)) == 0
    assert r.planeRowStride[0] == 1920 + 128 and r.planeRowStride[1] == 1920 + 128  # 961 px x 2 B -> 1922 -> 2048
    assert nv.nvcvImageCalcRequirements(100, 10, K.IMAGE_FORMAT_RGBA8, 0, 0, C.byref(r)) == 0
    assert r.planeRowStride[0] == 512 and r.alignBytes == 512 and r.mem.cudaMem.numBlocks[9] == 10
    assert nv.nvcvImageCalcRequirements(100, 10, K.IMAGE_FORMAT_RGB8, 256, 16, C.byref(r)) == 0
    assert r.planeRowStride[0] == 304 and r.alignBytes == 256
    assert nv.nvcvImageCalcRequirements(100, 10, K.IMAGE_FORMAT_RGB8, 0, 24, C.byref(r)) == 2


# ------------------------------------------------------------------------------------------ wrapping
def test_wrap_validation(cv, capi):
    ok = fake_tensor(cv, [2, 4, 5, 3], [128, 32, 3, 1], np.uint8, "NHWC")
    assert ok.shape == [2, 4, 5, 3] and ok.strides == [128, 32, 3, 1] and ok.layout == "NHWC"
    bad = [
        ([2, 4, 5, 3], [128, 32, 4, 1], np.uint8, "NHWC", 0x10000),   # W stride not packed
        ([2, 4, 5, 3], [128, 32, 3, 2], np.uint8, "NHWC", 0x10000),   # element stride wrong
        ([2, 4, 5, 3], [128, 14, 3, 1], np.uint8, "NHWC", 0x10000),   # rows overlap
        ([2, 4, 5, 3], [100, 32, 3, 1], np.uint8, "NHWC", 0x10000),   # samples overlap
        ([2, 0, 5, 3], [128, 32, 3, 1], np.uint8, "NHWC", 0x10000),   # empty dimension
        ([2, 4, 5, 3], [128, 32, 3, 1], np.uint8, "NHWC", 0),         # NULL buffer
        ([2, 4, 5], [128, 32, 3], np.uint8, "NHWC", 0x10000),         # rank != layout rank
        ([2, 3, 4, 5], [60, 20, 5, 2], np.uint8, "NCHW", 0x10000),    # innermost not packed
    ]
    for shape, strides, dt, layout, ptr in bad:
        with pytest.raises(cv.Error) as e:
            fake_tensor(cv, shape, strides, dt, layout, ptr)
        assert e.value.status == capi.NVCV_ERROR_INVALID_ARGUMENT, (shape, strides)
    # dimensions of extent 1 may carry any stride
    fake_tensor(cv, [1, 4, 5, 3], [7, 32, 3, 1], np.uint8, "NHWC")
    # NCHW: rows may be padded
    fake_tensor(cv, [2, 3, 4, 5], [3 * 4 * 8, 4 * 8, 8, 1], np.uint8, "NCHW")


def test_refcounts_cleanup_and_stale_handles(cv, capi):
    nv = capi.nvcv
    calls = []
    CB = capi.TensorCleanupFunc(lambda ctx, data: calls.append((ctx, data.contents.rank)))
    d = capi.TensorData()
    d.dtype = cv._as_dtype(np.uint8)
    d.layout = capi.TensorLayout.make("HW")
    d.rank = 2
    d.shape[0], d.shape[1] = 4, 8
    d.buffer.strides[0], d.buffer.strides[1] = 8, 1
    d.bufferType = 1
    d.buffer.basePtr = 0x4000
    h = C.c_void_p()
    assert nv.nvcvTensorWrapDataConstruct(C.byref(d), C.cast(CB, C.c_void_p), C.c_void_p(1234), C.byref(h)) == 0
    n = C.c_int()
    assert nv.nvcvTensorRefCount(h, C.byref(n)) == 0 and n.value == 1
    assert nv.nvcvTensorIncRef(h, C.byref(n)) == 0 and n.value == 2
    up = C.c_void_p()
    assert nv.nvcvTensorSetUserPointer(h, C.c_void_p(77)) == 0
    assert nv.nvcvTensorGetUserPointer(h, C.byref(up)) == 0 and up.value == 77
    assert nv.nvcvTensorDecRef(h, C.byref(n)) == 0 and n.value == 1 and calls == []
    assert nv.nvcvTensorDecRef(h, C.byref(n)) == 0 and n.value == 0 and calls == [(1234, 2)]
    # the handle is now stale: every use is rejected instead of touching freed state
    assert nv.nvcvTensorRefCount(h, C.byref(n)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvTensorDecRef(h, None) == capi.NVCV_ERROR_INVALID_ARGUMENT
    out = capi.TensorData()
    assert nv.nvcvTensorExportData(h, C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    # a new object reusing the slot gets a different handle value (generation tag)
    h2 = C.c_void_p()
    assert nv.nvcvTensorWrapDataConstruct(C.byref(d), None, None, C.byref(h2)) == 0
    assert h2.value != h.value and (h2.value & ~0xF) == (h.value & ~0xF)
    assert nv.nvcvTensorExportData(h, C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvTensorDecRef(h2, None) == 0
    # NULL and foreign pointers
    assert nv.nvcvTensorExportData(None, C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    junk = (C.c_char * 64)()
    assert nv.nvcvTensorExportData(C.cast(junk, C.c_void_p), C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    # a tensor handle is not an image handle
    t = fake_tensor(cv, [4, 4], [4, 1], np.uint8, "HW")
    w, hh = C.c_int32(), C.c_int32()
    assert nv.nvcvImageGetSize(t.handle, C.byref(w), C.byref(hh)) == capi.NVCV_ERROR_INVALID_ARGUMENT


def test_get_shape_and_reshape(cv, capi):
    nv = capi.nvcv
    t = fake_tensor(cv, [2, 4, 5, 3], [60, 15, 3, 1], np.uint8, "NHWC")
    rank = C.c_int32(6)
    shape = (C.c_int64 * 6)()
    assert nv.nvcvTensorGetShape(t.handle, C.byref(rank), shape) == 0
    assert rank.value == 4 and list(shape) == [1, 1, 2, 4, 5, 3]
    rank = C.c_int32(2)
    assert nv.nvcvTensorGetShape(t.handle, C.byref(rank), shape) == 0 and list(shape)[:2] == [5, 3]
    r = t.reshape([8, 15], "HW")
    assert r.shape == [8, 15] and r.strides == [15, 1] and t.refcount() == 2
    r2 = t.reshape([2, 1, 20, 3], "NHWC")
    assert r2.strides == [60, 60, 3, 1]
    with pytest.raises(cv.Error):
        t.reshape([7, 17], "HW")  # volume mismatch
    padded = fake_tensor(cv, [2, 4, 5, 3], [128, 32, 3, 1], np.uint8, "NHWC")
    v = padded.reshape([8, 5, 3], "HWC")  # N and H merge: 128 == 4*32
    assert v.strides == [32, 3, 1]
    with pytest.raises(cv.Error):
        padded.reshape([2, 60], "NW")  # rows are padded, cannot be flattened
    r.close()
    r2.close()
    assert t.refcount() == 1


def test_image_wrap_and_tensor_view(cv, capi, K):
    nv = capi.nvcv
    img = cv.Image.wrap(K.IMAGE_FORMAT_RGB8, [(0x20000, 50, 40, 256)])
    assert img.size == (50, 40) and img.format == K.IMAGE_FORMAT_RGB8
    ty = C.c_int()
    assert nv.nvcvImageGetType(img.handle, C.byref(ty)) == 0 and ty.value == 1
    h = C.c_void_p()
    assert nv.nvcvTensorWrapImageConstruct(img.handle, C.byref(h)) == 0
    t = cv.Tensor(h)
    assert t.shape == [1, 40, 50, 3] and t.strides == [256 * 40, 256, 3, 1] and t.layout == "NHWC"
    assert img.refcount() == 2
    t.close()
    assert img.refcount() == 1
    planar = cv.Image.wrap(K.IMAGE_FORMAT_RGBf32p, [(0x30000 + i * 0x4000, 20, 10, 128) for i in range(3)])
    assert nv.nvcvTensorWrapImageConstruct(planar.handle, C.byref(h)) == 0
    t = cv.Tensor(h)
    assert t.shape == [1, 3, 10, 20] and t.strides == [3 * 0x4000, 0x4000, 128, 4] and t.layout == "NCHW"
    nv12 = cv.Image.wrap(K.IMAGE_FORMAT_NV12, [(0x50000, 64, 32, 64), (0x58000, 32, 16, 64)])
    assert nv.nvcvTensorWrapImageConstruct(nv12.handle, C.byref(h)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    for bad in ([(0, 50, 40, 256)], [(0x1000, 0, 40, 256)]):
        with pytest.raises(cv.Error):
            cv.Image.wrap(K.IMAGE_FORMAT_RGB8, bad)


def test_custom_allocator(cv, capi):
    nv = capi.nvcv
    log = []
    libc = C.CDLL(None)
    libc.aligned_alloc.restype = C.c_void_p
    libc.aligned_alloc.argtypes = [C.c_size_t, C.c_size_t]
    libc.free.argtypes = [C.c_void_p]

    def alloc(ctx, size, align):
        log.append(("alloc", size, align))
        a = max(align, 8)
        return libc.aligned_alloc(a, (max(size, a) + a - 1) // a * a)  # C11: size is a multiple of the alignment

    def free(ctx, ptr, size, align):
        log.append(("free", size, align))
        libc.free(ptr)

    cleaned = []
    ra = capi.ResourceAllocator()
    ra.ctx = 5
    ra.resType = 0  # host memory
    ra.res.fnAlloc = capi.MemAllocFunc(alloc)
    ra.res.fnFree = capi.MemFreeFunc(free)
    ra.cleanup = capi.ResourceAllocatorCleanupFunc(lambda ctx, data: cleaned.append(ctx))
    h = C.c_void_p()
    assert nv.nvcvAllocatorConstructCustom(C.byref(ra), 1, C.byref(h)) == 0
    p = C.c_void_p()
    assert nv.nvcvAllocatorAllocHostMemory(h, C.byref(p), 128, 64) == 0 and p.value and p.value % 64 == 0
    assert nv.nvcvAllocatorFreeHostMemory(h, p, 128, 64) == 0
    assert log == [("alloc", 128, 64), ("free", 128, 64)]
    assert nv.nvcvAllocatorAllocHostMemory(h, C.byref(p), 100, 48) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvAllocatorAllocHostMemory(h, C.byref(p), -1, 64) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvAllocatorAllocHostMemory(h, C.byref(p), 100, 64) == capi.NVCV_ERROR_INVALID_ARGUMENT  # not whole units
    two = (capi.ResourceAllocator * 2)(ra, ra)
    h2 = C.c_void_p()
    assert nv.nvcvAllocatorConstructCustom(two, 2, C.byref(h2)) == capi.NVCV_ERROR_INVALID_ARGUMENT  # duplicate type
    assert nv.nvcvAllocatorDecRef(h, None) == 0 and cleaned == [5]
    # default allocator (NULL handle) serves host memory too
    assert nv.nvcvAllocatorAllocHostMemory(None, C.byref(p), 256, 128) == 0 and p.value % 128 == 0
    assert nv.nvcvAllocatorFreeHostMemory(None, p, 256, 128) == 0


def test_tensor_layout_cases_of_the_reference(cv, tmp_path):
    """tests/golden/tensor_layout_cases.c restates the cases of the reference's TestTensorLayout.cpp; it exercises the
    exported functions and the header-inline accessors from plain C."""
    import subprocess
    import cvcuda_amd._capi as capi_mod
    libdir = os.path.dirname(capi_mod.nvcv._name)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = tmp_path / "layout_cases"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-DCVCUDA_NO_HIP_HEADERS", "-I" + os.path.join(root, "include"),
                    os.path.join(root, "tests", "golden", "tensor_layout_cases.c"), "-L" + libdir, "-lnvcv_types",
                    # a sanitizer build of the library leaves its runtime's symbols to the preloaded runtime
                    "-Wl,--allow-shlib-undefined", "-Wl,-rpath," + libdir, "-o", str(exe)], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip() == "0 failures", r.stdout


def test_requirements_cases_of_the_reference(cv, capi):
    # tests/nvcv_types/system/TestRequirements.cpp:57-290
    nv = capi.nvcv
    n = len(capi.Requirements().cudaMem.numBlocks)
    ceil = lambda a, b: -(-a // b)
    # add_buffer / sub_buffer
    req = capi.Requirements()
    assert nv.nvcvRequirementsInit(C.byref(req)) == 0
    m = req.cudaMem
    a1, a2 = 256, 16384
    s1, s2 = 3 * a1 - 5, 6 * a2 - 17
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), s1, a1) == 0
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), s2, a2) == 0
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), a2 // 3, a2) == 0
    want = [0] * n
    want[8], want[14] = ceil(s1, a1), ceil(s2 + a2 // 3, a2)
    assert list(m.numBlocks) == want
    assert nv.nvcvRequirementsInit(C.byref(req)) == 0
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), s1, a1) == 0 and nv.nvcvMemRequirementsAddBuffer(C.byref(m), -511, a1) == 0
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), s2, a2) == 0 and nv.nvcvMemRequirementsAddBuffer(C.byref(m), -s2 * 5, a2) == 0
    want = [0] * n
    want[8] = ceil(s1 - 512, a1)
    assert list(m.numBlocks) == want
    # add and total size
    total, gold, sizes = capi.Requirements(), [[0] * n for _ in range(3)], [0, 0, 0]
    assert nv.nvcvRequirementsInit(C.byref(total)) == 0
    for factors in ((3, 5, 7), (17, 21, 37)):
        part = capi.Requirements()
        assert nv.nvcvRequirementsInit(C.byref(part)) == 0
        for i in range(n):
            align = 1 << i
            for k, mem in enumerate((part.cudaMem, part.hostMem, part.hostPinnedMem)):
                size = factors[k] * (i + 1) * align - (k + 1)
                assert nv.nvcvMemRequirementsAddBuffer(C.byref(mem), size, align) == 0
                gold[k][i] += ceil(size, align)
                sizes[k] += ceil(size, align) * align
        assert nv.nvcvRequirementsAdd(C.byref(total), C.byref(part)) == 0
        assert [list(total.cudaMem.numBlocks), list(total.hostMem.numBlocks), list(total.hostPinnedMem.numBlocks)] == gold
    out = C.c_int64()
    for k, mem in enumerate((total.cudaMem, total.hostMem, total.hostPinnedMem)):
        assert nv.nvcvMemRequirementsCalcTotalSizeBytes(C.byref(mem), C.byref(out)) == 0 and out.value == sizes[k]
    assert nv.nvcvRequirementsAdd(C.byref(total), C.byref(total)) == 0
    assert list(total.cudaMem.numBlocks) == [2 * v for v in gold[0]]
    # invalid arguments and overflow
    assert nv.nvcvRequirementsInit(None) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvRequirementsAdd(None, C.byref(req)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvRequirementsAdd(C.byref(req), None) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvMemRequirementsCalcTotalSizeBytes(None, C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvMemRequirementsCalcTotalSizeBytes(C.byref(m), None) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvMemRequirementsAddBuffer(None, 256, 256) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), 256, 3) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(m), 256, (1 << 32) + 1) == capi.NVCV_ERROR_INVALID_ARGUMENT
    big = capi.Requirements()
    assert nv.nvcvRequirementsInit(C.byref(big)) == 0
    big.cudaMem.numBlocks[0], big.cudaMem.numBlocks[1] = (1 << 63) - 1, 2
    assert nv.nvcvMemRequirementsCalcTotalSizeBytes(C.byref(big.cudaMem), C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    big.cudaMem.numBlocks[1] = (1 << 63) - 1
    assert nv.nvcvMemRequirementsCalcTotalSizeBytes(C.byref(big.cudaMem), C.byref(out)) == capi.NVCV_ERROR_INVALID_ARGUMENT
    big.cudaMem.numBlocks[1] = 0
    assert nv.nvcvMemRequirementsAddBuffer(C.byref(big.cudaMem), 2, 1) == capi.NVCV_ERROR_OVERFLOW


def test_status_cases_of_the_reference(cv, capi):
    # tests/nvcv_types/system/TestStatus.cpp:30-170
    nv = capi.nvcv
    nv.nvcvStatusGetName.restype = C.c_char_p
    names = ["NVCV_SUCCESS", "NVCV_ERROR_NOT_IMPLEMENTED", "NVCV_ERROR_INVALID_ARGUMENT", "NVCV_ERROR_INVALID_IMAGE_FORMAT",
             "NVCV_ERROR_INVALID_OPERATION", "NVCV_ERROR_DEVICE", "NVCV_ERROR_NOT_READY", "NVCV_ERROR_OUT_OF_MEMORY", "NVCV_ERROR_INTERNAL"]
    for code, name in enumerate(names):
        assert nv.nvcvStatusGetName(code) == name.encode()
    assert nv.nvcvStatusGetName(capi.NVCV_ERROR_OVERFLOW) == b"NVCV_ERROR_OVERFLOW"
    assert nv.nvcvStatusGetName(capi.NVCV_ERROR_OVERFLOW + 1) == b"NVCV_ERROR_UNDERFLOW"
    assert nv.nvcvStatusGetName(255) == b"Unknown error"
    msg = C.create_string_buffer(256)
    nv.nvcvGetLastError()
    assert nv.nvcvGetLastError() == 0 and nv.nvcvPeekAtLastError() == 0
    assert nv.nvcvGetLastErrorMessage(msg, 256) == 0 and msg.value == b"success"
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_DEVICE, b"%s", b"")
    assert nv.nvcvGetLastError() == capi.NVCV_ERROR_DEVICE and nv.nvcvGetLastError() == 0
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_DEVICE, b"%s", b"")
    assert nv.nvcvPeekAtLastError() == capi.NVCV_ERROR_DEVICE and nv.nvcvPeekAtLastError() == capi.NVCV_ERROR_DEVICE
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_INTERNAL, b"test message")
    assert nv.nvcvGetLastErrorMessage(msg, 256) == capi.NVCV_ERROR_INTERNAL and msg.value == b"test message"
    assert nv.nvcvGetLastErrorMessage(msg, 256) == 0 and msg.value == b"success"
    assert nv.nvcvPeekAtLastErrorMessage(msg, 256) == 0 and msg.value == b"success"
    reqs = capi.ImageRequirements()
    assert nv.nvcvImageCalcRequirements(640, 480, C.c_uint64(cv.K.IMAGE_FORMAT_U8), 0, 0, None) == capi.NVCV_ERROR_INVALID_ARGUMENT
    assert nv.nvcvImageCalcRequirements(640, 480, C.c_uint64(cv.K.IMAGE_FORMAT_U8), 0, 0, C.byref(reqs)) == 0
    assert nv.nvcvGetLastError() == capi.NVCV_ERROR_INVALID_ARGUMENT  # the success in between did not reset it
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_DEVICE, b"test message")
    for _ in range(2):
        msg.value = b""
        assert nv.nvcvPeekAtLastErrorMessage(msg, 256) == capi.NVCV_ERROR_DEVICE and msg.value == b"test message"
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_DEVICE, b"test message %d %c %s", 123, ord("r"), b"lima")
    assert nv.nvcvGetLastErrorMessage(msg, 256) == capi.NVCV_ERROR_DEVICE and msg.value == b"test message 123 r lima"
    nv.nvcvSetThreadStatus(capi.NVCV_ERROR_DEVICE, None)
    assert nv.nvcvGetLastErrorMessage(msg, 256) == capi.NVCV_ERROR_DEVICE and msg.value == b""


WRAP_CASES = [  # tests/nvcv_types/system/TestTensor.cpp:448-470: shape, layout, strides, dtype, accepted?
    ([2], "C", [4], np.float32, True), ([1], "W", [1], np.uint8, True), ([10, 5], "HW", [5, 1], np.uint8, True),
    ([1, 10, 5], "NHW", [1, 5, 1], np.uint8, True), ([3, 1, 5], "NHW", [20, 1, 4], np.float32, True),
    ([3, 1, 1], "NHW", [20, 1, 1], np.float32, True), ([10, 5, 3], "HWC", [60, 12, 4], np.float32, True),
    ([2], "C", [3], np.float32, False), ([2], "C", [5], np.float32, False), ([10, 5], "HW", [1, 10], np.uint8, False),
    ([10, 5, 3], "HWC", [4, 40, 200], np.float32, False), ([1, 10, 5], "NHW", [1, 19, 4], np.float32, False),
    ([3, 1, 5], "NHW", [19, 1, 4], np.float32, False)]


@pytest.mark.parametrize("shape,layout,strides,dt,ok", WRAP_CASES, ids=[str(c[:3]) for c in WRAP_CASES])
def test_wrap_parameter_cases_of_the_reference(cv, capi, shape, layout, strides, dt, ok):
    if not ok:
        with pytest.raises(cv.Error) as e:
            fake_tensor(cv, shape, strides, dt, layout, 0xDEADBEEF)
        assert e.value.status == capi.NVCV_ERROR_INVALID_ARGUMENT
        return
    t = fake_tensor(cv, shape, strides, dt, layout, 0xDEADBEEF)
    assert t.shape == shape and t.layout == layout and t.strides == strides


def build_c_cases(name, tmp_path, extra=()):
    """Compiles tests/golden/<name>.c with gcc against the public headers and the core library."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.environ.get("CVCUDA_AMD_LIBDIR", os.path.join(root, "cv-cuda_amd", "lib"))
    exe = str(tmp_path / name)
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-D_POSIX_C_SOURCE=200112L", "-DCVCUDA_NO_HIP_HEADERS",
                    "-I" + os.path.join(root, "include"), os.path.join(root, "tests", "golden", name + ".c"), "-o", exe,
                    "-L" + libdir, "-lnvcv_types", "-Wl,-rpath," + libdir, "-Wl,--allow-shlib-undefined"]
                   + list(extra), check=True)
    return exe


def test_argument_checks_of_the_reference_from_plain_c(cv, tmp_path):
    import subprocess
    r = subprocess.run([build_c_cases("core_negative_cases", tmp_path)], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.strip().endswith("0 failed"), r.stdout + r.stderr


def test_handles_created_shared_and_destroyed_by_many_threads(cv, tmp_path):
    """tests/golden/handle_pool_stress.c: 8 threads create, share by reference count and destroy tensors, images and
    allocator-backed tensors; every cleanup runs once, nothing stays alive, destroyed handles are refused."""
    import subprocess
    r = subprocess.run([build_c_cases("handle_pool_stress", tmp_path, ["-pthread"]), "8", "5000"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().endswith(" 0 failed"), r.stdout + r.stderr


@pytest.mark.gpu
def test_argument_checks_of_the_reference_from_plain_c_with_image_batches(cv, gpu, tmp_path):
    import subprocess
    r = subprocess.run([build_c_cases("core_negative_cases", tmp_path), "device"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0 and r.stdout.strip().endswith("0 failed"), r.stdout + r.stderr



@pytest.mark.parametrize("shape_arg,layout_arg,expected", [
    ((1, 10, 10, 3), "XHWC", (320, 32, 3, 1)), ((10, 10, 3, 1), "HWCX", (32, 3, 1, 1)), ((10, 1, 10, 3), "HXWC", (32, 32, 3, 1)),
    ((10, 2, 5, 3), "HABC", (32, 15, 3, 1)), ((2, 5, 10, 3), "ABWC", (160, 32, 3, 1)),
])
def test_reshape_of_padded_rows_gives_the_reference_strides(cv, shape_arg, layout_arg, expected):
    """tests/nvcv_types/python/test_tensor.py:372-395 on a tensor with the 32-byte row pitch of the reference's device:
    a unit dimension takes the stride of the group it is split from (src/nvcv/src/priv/TensorData.cpp:248-276)."""
    t = cv.Tensor.wrap(0x10000, [10, 10, 3], [32, 3, 1], np.uint8, "HWC")
    assert tuple(t.reshape(list(shape_arg), layout_arg).strides) == expected
    with pytest.raises(cv.Error):
        t.reshape([300], "A")  # padded rows cannot become one dense dimension
