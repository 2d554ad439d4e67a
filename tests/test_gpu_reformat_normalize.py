"""GPU parity of cvcudaReformatSubmit (bit-exact, padding untouched: reference test
tests/cvcuda/system/TestOpReformat.cpp:52-71, 172-182) and cvcudaNormalize[VarShape]Submit (reference
rows tests/cvcuda/system/TestOpNormalize.cpp:86-101; exact for integer types, 1e-5 relative for f32)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def rand(orc, shape, dt, seed):
    if np.dtype(dt) == np.float32:
        return orc.fill_f32(shape, seed) * 200 - 50
    return orc.fill_u8(tuple(shape) + (np.dtype(dt).itemsize,), seed).view(dt).reshape(shape)


@pytest.mark.parametrize("dt", [np.uint8, np.int8, np.uint16, np.int16, np.int32, np.float32, np.float64])
@pytest.mark.parametrize("shape", [(2, 37, 53, 3), (1, 224, 224, 3), (3, 16, 20, 4), (2, 9, 11, 1), (1, 8, 9, 6),
                                   (1, 5, 531, 3), (2, 3, 300, 4)])
def test_reformat_nhwc_nchw_roundtrip(cv, orc, gpu, dt, shape):
    n, h, w, c = shape
    if dt == np.float64:
        a = (orc.fill_f32(shape, 3).astype(np.float64) - 0.5) * 1e6
    else:
        a = rand(orc, shape, dt, 3 + c)
    tin = cv.Tensor.from_numpy(a, "NHWC")
    tmid = cv.Tensor.alloc([n, c, h, w], dt, "NCHW")
    d = tmid.export()
    raw = cv._bytes_view(d.buffer.basePtr, d.buffer.strides[0] * n, tmid)
    raw.fill_(0xCD)
    op = cv.Reformat()
    op(None, tin, tmid)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tmid.numpy(), a.transpose(0, 3, 1, 2))
    # bytes between the end of a row and the next row start keep their previous content
    es, pitch = np.dtype(dt).itemsize, d.buffer.strides[2]
    if pitch > w * es:
        rows = raw.view(n * c * h, pitch)[:, w * es:].cpu().numpy()
        assert (rows == 0xCD).all()
    tback = cv.Tensor.alloc(list(shape), dt, "NHWC")
    op(None, tmid, tback)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tback.numpy(), a)


def test_reformat_hwc_chw_copy_and_errors(cv, orc, gpu):
    a = rand(orc, (30, 40, 3), np.float32, 9)
    t_hwc = cv.Tensor.from_numpy(a, "HWC")
    t_chw = cv.Tensor.alloc([3, 30, 40], np.float32, "CHW")
    op = cv.Reformat()
    op(None, t_hwc, t_chw)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(t_chw.numpy(), a.transpose(2, 0, 1))
    same = cv.Tensor.alloc([30, 40, 3], np.float32, "HWC", row_align=256)  # same layout, other pitch: copy
    op(None, t_hwc, same)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(same.numpy(), a)
    for bad in (cv.Tensor.alloc([1, 3, 30, 40], np.float32, "NCHW"),     # HWC -> NCHW mixes batch/no batch
                cv.Tensor.alloc([3, 30, 40], np.uint8, "CHW"),           # dtype
                cv.Tensor.alloc([3, 30, 41], np.float32, "CHW")):        # shape
        with pytest.raises(cv.Error) as e:
            op(None, t_hwc, bad)
        assert e.value.status == 2


def test_reformat_typical_pipeline_shape(cv, orc, gpu):
    a = rand(orc, (64, 224, 224, 3), np.float32, 12)
    tin = cv.Tensor.from_numpy(a, "NHWC")
    tout = cv.Tensor.alloc([64, 3, 224, 224], np.float32, "NCHW")
    cv.Reformat()(None, tin, tout)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tout.numpy(), a.transpose(0, 3, 1, 2))


NORM_ROWS = [  # width, height, images, scalarBase, scalarScale, stddev, globalScale, globalShift, epsilon
    (32, 33, 1, True, True, False, 0.0, 0.0, 0.0), (66, 55, 1, True, True, False, 1.0, 0.0, 0.0),
    (122, 212, 2, True, True, False, 1.234, 43.21, 0.0), (211, 102, 3, False, False, False, 1.1, 0.1, 0.0),
    (21, 12, 5, True, True, True, 1.2, 0.2, 0.0), (22, 12, 5, False, True, True, 1.3, 0.3, 0.0),
    (55, 23, 5, True, False, True, 1.2, 0.2, 0.0), (72, 88, 5, False, False, True, 1.2, 0.2, 0.0),
    (63, 32, 7, False, True, False, 1.3, 0.3, 0.0), (22, 13, 9, True, False, False, 1.4, 0.4, 0.0),
    (55, 33, 2, True, False, True, 2.1, 1.1, 1.23), (444, 222, 4, True, False, True, 2.2, 2.2, 12.3),
]


def compare_norm(res, ref):
    if res.dtype == np.float32:
        assert (np.abs(res - ref) <= 1e-5 * np.maximum(1.0, np.abs(ref))).all()
    else:
        np.testing.assert_array_equal(res, ref)


@pytest.mark.parametrize("row", NORM_ROWS, ids=lambda r: "%dx%dx%d-%s%s%s" % (r[0], r[1], r[2], "b" if r[3] else "B",
                                                                            "s" if r[4] else "S", "d" if r[5] else ""))
@pytest.mark.parametrize("dt,c", [(np.uint8, 4), (np.uint8, 3), (np.int16, 1), (np.float32, 3), (np.int32, 4),
                                  (np.uint16, 3), (np.int8, 1)])
def test_normalize_tensor_rows(cv, K, orc, gpu, row, dt, c):
    w, h, n, sb, ss, stddev, gs, sh, eps = row
    a = rand(orc, (n, h, w, c), dt, w + h)
    if dt == np.int32:
        a = a >> 8
    base = orc.fill_f32((1, 1, 1, 1 if sb else c), 5) * 100
    scale = orc.fill_f32((1, 1, 1, 1 if ss else c), 6) + 0.25
    tin = cv.Tensor.from_numpy(a, "NHWC")
    tout = cv.Tensor.alloc([n, h, w, c], dt, "NHWC")
    cv.Normalize()(None, tin, cv.Tensor.from_numpy(base, "NHWC"), cv.Tensor.from_numpy(scale, "NHWC"), tout, gs, sh,
                   eps, K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV if stddev else 0)
    torch.cuda.synchronize()
    compare_norm(tout.numpy(), orc.normalize(a, base, scale, gs, sh, eps, stddev))


def test_normalize_full_broadcast_matrix_and_identity(cv, K, orc, gpu):
    a = rand(orc, (3, 20, 30, 3), np.float32, 1)
    for bshape in [(3, 20, 30, 3), (1, 20, 1, 3), (3, 1, 30, 1), (1, 1, 1, 1), (3, 1, 1, 3)]:
        base = orc.fill_f32(bshape, 2) * 10
        scale = orc.fill_f32(bshape[::1], 3) + 0.5
        tout = cv.Tensor.alloc([3, 20, 30, 3], np.float32, "NHWC")
        cv.Normalize()(None, cv.Tensor.from_numpy(a, "NHWC"), cv.Tensor.from_numpy(base, "NHWC"),
                       cv.Tensor.from_numpy(scale, "NHWC"), tout, 0.7, -0.3)
        torch.cuda.synchronize()
        compare_norm(tout.numpy(), orc.normalize(a, base, scale, 0.7, -0.3))
    u = rand(orc, (2, 16, 16, 4), np.uint8, 4)
    tout = cv.Tensor.alloc([2, 16, 16, 4], np.uint8, "NHWC")
    one = np.ones((1, 1, 1, 1), np.float32)
    cv.Normalize()(None, cv.Tensor.from_numpy(u, "NHWC"), cv.Tensor.from_numpy(0 * one, "NHWC"),
                   cv.Tensor.from_numpy(one, "NHWC"), tout, 1.0, 0.0)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tout.numpy(), u)
    # imagenet-style use: (x/255 - mean)/std through STDDEV mode on f32
    x = orc.fill_f32((4, 224, 224, 3), 8)
    mean = np.array([0.485, 0.456, 0.406], np.float32).reshape(1, 1, 1, 3)
    std = np.array([0.229, 0.224, 0.225], np.float32).reshape(1, 1, 1, 3)
    tout = cv.Tensor.alloc([4, 224, 224, 3], np.float32, "NHWC")
    cv.Normalize()(None, cv.Tensor.from_numpy(x, "NHWC"), cv.Tensor.from_numpy(mean, "NHWC"),
                   cv.Tensor.from_numpy(std, "NHWC"), tout, 1.0, 0.0, 0.0, K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV)
    torch.cuda.synchronize()
    assert np.abs(tout.numpy() - (x - mean) / std).max() < 1e-5


def test_normalize_varshape(cv, K, orc, gpu):
    rng = np.random.default_rng(4)
    for in_dt, fmt_in, out_dt, fmt_out in [(np.uint8, K.IMAGE_FORMAT_RGB8, np.float32, K.IMAGE_FORMAT_RGBf32),
                                           (np.uint8, K.IMAGE_FORMAT_RGBA8, np.uint8, K.IMAGE_FORMAT_RGBA8),
                                           (np.float32, K.IMAGE_FORMAT_F32, np.uint8, K.IMAGE_FORMAT_U8)]:
        c = {K.IMAGE_FORMAT_RGB8: 3, K.IMAGE_FORMAT_RGBA8: 4, K.IMAGE_FORMAT_F32: 1}[fmt_in]
        n = 6
        bi, bo, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
        for i in range(n):
            w, h = int(rng.integers(5, 300)), int(rng.integers(5, 200))
            a = rand(orc, (h, w, c), in_dt, 30 + i)
            hosts.append(a)
            bi.push_back(cv.Image.from_numpy(a, fmt_in))
            o = cv.Image.alloc((w, h), fmt_out)
            outs.append(o)
            bo.push_back(o)
        for vec in (False, True):
            base = orc.fill_f32((1, 1, 1, c if vec else 1), 1) * 50
            scale = orc.fill_f32((1, 1, 1, c if vec else 1), 2) + 0.5
            for stddev in (False, True):
                cv.Normalize()(None, bi, cv.Tensor.from_numpy(base, "NHWC"), cv.Tensor.from_numpy(scale, "NHWC"), bo,
                               0.9, 3.0, 0.01, K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV if stddev else 0)
                torch.cuda.synchronize()
                for a, o in zip(hosts, outs):
                    res = o.plane_view(0, out_dt, c).cpu().numpy()
                    # oracle computes in the input type; convert through float for a different output type
                    ref_f = orc.normalize(a[None].astype(np.float32), base, scale, 0.9, 3.0, 0.01, stddev)[0]
                    ref = ref_f if out_dt == np.float32 else np.clip(np.rint(ref_f), 0, 255).astype(np.uint8)
                    compare_norm(res, ref)


def test_normalize_negative(cv, K, gpu):
    op = cv.Normalize()
    a = cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC")
    one = cv.Tensor.alloc([1, 1, 1, 1], np.float32, "NHWC")
    bad = [
        (a, one, one, cv.Tensor.alloc([2, 8, 8, 3], np.float32, "NHWC")),                    # dtype differs
        (a, cv.Tensor.alloc([1, 1, 1, 2], np.float32, "NHWC"), one, cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC")),
        (a, one, cv.Tensor.alloc([1, 4, 1, 1], np.float32, "NHWC"), cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC")),
        (a, cv.Tensor.alloc([1, 1, 1, 1], np.uint8, "NHWC"), one, cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC")),
        (a, one, one, cv.Tensor.alloc([2, 3, 8, 8], np.uint8, "NCHW")),
    ]
    for tin, b, s, tout in bad:
        with pytest.raises(cv.Error) as e:
            op(None, tin, b, s, tout)
        assert e.value.status == 2
