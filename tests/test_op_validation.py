"""Argument validation of every operator Submit, on the CPU: tensors wrap a fake device address, every
case is rejected on the host before any launch. Status codes follow the reference's negative tests
(tests/cvcuda/system/TestOpResizeCropConvertReformat.cpp:574-603, TestOpResize.cpp:317-325,
TestOpCvtColor.cpp, TestOpNormalize.cpp, TestOpReformat.cpp:186-194, TestOpWarpAffine.cpp) and its
operator handle rules (src/cvcuda/priv/IOperator.hpp:59-72)."""
import ctypes as C

import numpy as np
import pytest

INVALID_ARGUMENT, NOT_COMPATIBLE, OVERFLOW = 2, 9, 10
FAKE = 0x7F0000000000
NEAREST, LINEAR, CUBIC, AREA, LANCZOS = 0, 1, 2, 3, 4


def fake(cv, shape, dtype, layout):
    """Tensor over a made-up address with packed strides."""
    es = np.dtype(dtype).itemsize
    strides, acc = [], es
    for s in reversed(shape):
        strides.insert(0, acc)
        acc *= s
    return cv.Tensor.wrap(FAKE, shape, strides, dtype, layout)


def expect(cv, status, fn, *args, **kw):
    with pytest.raises(cv.Error) as e:
        fn(*args, **kw)
    assert e.value.status == status, str(e.value)
    st, msg = cv.last_error()
    assert st == status and msg  # message recorded for the thread, then cleared
    assert cv.last_error()[0] == 0


def test_fused_negative_table(cv, K):
    op = cv.ResizeCropConvertReformat()
    u8, f32 = np.uint8, np.float32

    def run(interp=LINEAR, nin=2, nout=2, cin=3, cout=3, tin=u8, tout=u8, crop=(4, 4), pos=(0, 0), rs=(16, 16),
            lin="NHWC", lout="NHWC"):
        shp_in = [nin, 20, 24, cin] if lin == "NHWC" else [nin, cin, 20, 24]
        shp_out = [nout, crop[1], crop[0], cout] if lout == "NHWC" else [nout, cout, crop[1], crop[0]]
        op(0, fake(cv, shp_in, tin, lin), fake(cv, shp_out, tout, lout), rs, interp, pos)

    for interp in (CUBIC, AREA, LANCZOS):
        expect(cv, INVALID_ARGUMENT, run, interp=interp)
    expect(cv, INVALID_ARGUMENT, run, nin=1, nout=2)
    expect(cv, INVALID_ARGUMENT, run, nin=2, nout=1)
    expect(cv, NOT_COMPATIBLE, run, cout=4)
    expect(cv, NOT_COMPATIBLE, run, cin=4, cout=4)
    expect(cv, NOT_COMPATIBLE, run, tin=f32)
    expect(cv, NOT_COMPATIBLE, run, tout=np.float16)
    expect(cv, INVALID_ARGUMENT, run, pos=(-1, 0))
    expect(cv, INVALID_ARGUMENT, run, pos=(0, -1))
    expect(cv, INVALID_ARGUMENT, run, crop=(32, 4))
    expect(cv, INVALID_ARGUMENT, run, crop=(4, 32))
    expect(cv, NOT_COMPATIBLE, run, lin="NCHW")
    expect(cv, INVALID_ARGUMENT, run, rs=(0, 0))
    expect(cv, INVALID_ARGUMENT, run, rs=(1, 16))
    # input larger than 2 GiB - 1
    big_in = cv.Tensor.wrap(FAKE, [1, 30000, 30000, 3], [2700000000, 90000, 3, 1], u8, "NHWC")
    expect(cv, OVERFLOW, op, 0, big_in, fake(cv, [1, 4, 4, 3], u8, "NHWC"), (16, 16), LINEAR, (0, 0))
    # extension entry: NULL parameter block, unknown flag
    st = cv._cv.cvcudaxResizeCropConvertReformatNormalizeSubmit(
        op.handle, 0, fake(cv, [1, 20, 24, 3], u8, "NHWC").handle, fake(cv, [1, 4, 4, 3], f32, "NHWC").handle,
        cv.capi.Size2D(16, 16), LINEAR, cv.capi.Int2(0, 0), 0, 1.0, 0.0, False, None)
    assert st == INVALID_ARGUMENT and cv.last_error()[0] == INVALID_ARGUMENT


def test_operator_handle_rules(cv):
    a, b = fake(cv, [1, 8, 8, 3], np.uint8, "NHWC"), fake(cv, [1, 4, 4, 3], np.uint8, "NHWC")
    # NULL handle -> INVALID_ARGUMENT; handle of another operator type -> NOT_COMPATIBLE
    assert cv._cv.cvcudaResizeSubmit(None, 0, a.handle, b.handle, LINEAR) == INVALID_ARGUMENT
    cv.last_error()
    other = cv.Reformat()
    assert cv._cv.cvcudaResizeSubmit(other.handle, 0, a.handle, b.handle, LINEAR) == NOT_COMPATIBLE
    cv.last_error()
    assert cv._cv.cvcudaResizeCreate(None) == INVALID_ARGUMENT
    cv.last_error()
    # NULL tensors
    op = cv.Resize()
    assert cv._cv.cvcudaResizeSubmit(op.handle, 0, None, b.handle, LINEAR) == INVALID_ARGUMENT
    cv.last_error()
    h = C.c_void_p()
    assert cv._cv.cvcudaWarpAffineCreate(C.byref(h), -1) == INVALID_ARGUMENT
    cv.last_error()


def test_resize_negative(cv):
    op = cv.Resize()
    a = fake(cv, [2, 8, 8, 3], np.uint8, "NHWC")
    expect(cv, INVALID_ARGUMENT, op, 0, a, fake(cv, [2, 4, 4, 3], np.float32, "NHWC"), LINEAR)   # dtype differs
    expect(cv, INVALID_ARGUMENT, op, 0, a, fake(cv, [2, 4, 4, 4], np.uint8, "NHWC"), LINEAR)     # channels differ
    expect(cv, INVALID_ARGUMENT, op, 0, a, fake(cv, [3, 4, 4, 3], np.uint8, "NHWC"), LINEAR)     # batch differs
    expect(cv, INVALID_ARGUMENT, op, 0, a, fake(cv, [2, 3, 4, 4], np.uint8, "NCHW"), LINEAR)     # layout
    expect(cv, INVALID_ARGUMENT, op, 0, a, fake(cv, [2, 4, 4, 3], np.uint8, "NHWC"), LANCZOS)    # interpolation
    expect(cv, INVALID_ARGUMENT, op, 0, fake(cv, [2, 8, 8, 3], np.float64, "NHWC"),
           fake(cv, [2, 4, 4, 3], np.float64, "NHWC"), LINEAR)                                   # unsupported type


def test_cvtcolor_negative(cv, K):
    op = cv.CvtColor()
    rgb = fake(cv, [2, 8, 8, 3], np.uint8, "NHWC")
    expect(cv, INVALID_ARGUMENT, op, 0, rgb, fake(cv, [2, 8, 8, 3], np.uint8, "NHWC"), K.COLOR_BGR2BGRA)  # needs 4 ch out
    expect(cv, INVALID_ARGUMENT, op, 0, rgb, fake(cv, [2, 8, 9, 3], np.uint8, "NHWC"), K.COLOR_BGR2RGB)   # size differs
    expect(cv, INVALID_ARGUMENT, op, 0, rgb, fake(cv, [1, 8, 8, 3], np.uint8, "NHWC"), K.COLOR_BGR2RGB)   # batch differs
    nv12 = fake(cv, [2, 12, 8, 1], np.uint8, "NHWC")
    expect(cv, INVALID_ARGUMENT, op, 0, nv12, fake(cv, [2, 8, 8, 2], np.uint8, "NHWC"), K.COLOR_YUV2RGB_NV12)
    expect(cv, INVALID_ARGUMENT, op, 0, nv12, fake(cv, [2, 7, 8, 3], np.uint8, "NHWC"), K.COLOR_YUV2RGB_NV12)
    expect(cv, INVALID_ARGUMENT, op, 0, fake(cv, [2, 12, 8, 1], np.float32, "NHWC"),
           fake(cv, [2, 8, 8, 3], np.float32, "NHWC"), K.COLOR_YUV2RGB_NV12)                            # u8 only
    expect(cv, INVALID_ARGUMENT, op, 0, fake(cv, [2, 9, 6, 1], np.uint8, "NHWC"),
           fake(cv, [2, 6, 6, 3], np.uint8, "NHWC"), K.COLOR_YUV2RGB_NV12 + 1000)                        # unknown code


def test_normalize_reformat_warp_negative(cv, K):
    u8, f32 = np.uint8, np.float32
    norm = cv.Normalize()
    a, one = fake(cv, [2, 8, 8, 3], u8, "NHWC"), fake(cv, [1, 1, 1, 1], f32, "NHWC")
    out = fake(cv, [2, 8, 8, 3], u8, "NHWC")
    expect(cv, INVALID_ARGUMENT, norm, 0, a, one, one, fake(cv, [2, 8, 8, 3], f32, "NHWC"))
    expect(cv, INVALID_ARGUMENT, norm, 0, a, fake(cv, [1, 1, 1, 2], f32, "NHWC"), one, out)
    expect(cv, INVALID_ARGUMENT, norm, 0, a, one, fake(cv, [1, 1, 1, 1], u8, "NHWC"), out)
    expect(cv, INVALID_ARGUMENT, norm, 0, fake(cv, [2, 8, 8, 5], u8, "NHWC"), one, one, fake(cv, [2, 8, 8, 5], u8, "NHWC"))

    ref = cv.Reformat()
    expect(cv, INVALID_ARGUMENT, ref, 0, a, fake(cv, [2, 3, 8, 8], f32, "NCHW"))            # dtype
    expect(cv, INVALID_ARGUMENT, ref, 0, a, fake(cv, [2, 3, 8, 9], u8, "NCHW"))             # shape
    expect(cv, INVALID_ARGUMENT, ref, 0, a, fake(cv, [3, 8, 8], u8, "CHW"))                 # batched vs not

    warp = cv.WarpAffine(0)
    ident = [1, 0, 0, 0, 1, 0]
    expect(cv, INVALID_ARGUMENT, warp, 0, a, fake(cv, [2, 8, 8, 3], f32, "NHWC"), ident, LINEAR)
    expect(cv, INVALID_ARGUMENT, warp, 0, a, fake(cv, [3, 8, 8, 3], u8, "NHWC"), ident, LINEAR)
    expect(cv, INVALID_ARGUMENT, warp, 0, a, out, ident, AREA)
    expect(cv, INVALID_ARGUMENT, warp, 0, a, out, ident, LINEAR, 7)                         # border mode
    st = cv._cv.cvcudaWarpAffineSubmit(warp.handle, 0, a.handle, out.handle, None, LINEAR, 0, cv.capi.Float4(0, 0, 0, 0))
    assert st == INVALID_ARGUMENT
    cv.last_error()
    persp = cv.WarpPerspective(0)
    expect(cv, INVALID_ARGUMENT, persp, 0, a, fake(cv, [2, 8, 8, 4], u8, "NHWC"), [1, 0, 0, 0, 1, 0, 0, 0, 1], LINEAR)
