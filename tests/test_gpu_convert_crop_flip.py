"""GPU parity of cvcudaConvertToSubmit, cvcudaCustomCropSubmit, cvcudaCenterCropSubmit and
cvcudaFlip[VarShape]Submit. Crops and flips are bit-exact against numpy slicing (the reference's
goldens are the same index maps: tests/cvcuda/system/TestOpCustomCrop.cpp:37-61, TestOpCenterCrop.cpp,
tests/cvcuda/system/FlipUtils.cpp); ConvertTo is bit-exact against the device-arithmetic restatement
and, for integer results, within 1 of the float64 golden (TestOpConvertTo.cpp:132)."""
import itertools

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TYPES = [np.uint8, np.int8, np.uint16, np.int16, np.int32, np.float32, np.float64]


def rand(orc, shape, dt, seed):
    dt = np.dtype(dt)
    if dt.kind == "f":
        return ((orc.fill_f32(shape, seed) - 0.3) * 400).astype(dt)
    a = orc.fill_u8(tuple(shape) + (dt.itemsize,), seed).view(dt).reshape(shape)
    return a >> 12 if dt == np.int32 else a


@pytest.mark.parametrize("tin,tout", list(itertools.product(TYPES, TYPES)))
def test_convert_to_all_type_pairs(cv, orc, gpu, tin, tout):
    op = cv.ConvertTo()
    for shape, alpha, beta in [((2, 13, 37, 3), 1.0, 0.0), ((1, 5, 5, 4), 2.1, 2.0), ((3, 9, 130, 1), -0.731, 40.25),
                               ((1, 1, 1, 2), 2.1, -1.0)]:
        a = rand(orc, shape, tin, 3)
        t_out = cv.Tensor.alloc(list(shape), tout, "NHWC")
        op(None, cv.Tensor.from_numpy(a, "NHWC"), t_out, alpha, beta)
        torch.cuda.synchronize()
        res = t_out.numpy()
        np.testing.assert_array_equal(res, orc.convert_to(a, tout, alpha, beta, 1))
        gold = orc.convert_to(a, tout, alpha, beta, 0)
        if np.dtype(tout).kind != "f":
            assert np.abs(res.astype(np.int64) - gold.astype(np.int64)).max() <= 1
        else:
            assert np.allclose(res, gold, rtol=1e-5, atol=1e-4)


def test_float_to_u8_rounding_and_saturation_cases(cv, orc, gpu):
    # every half-way case around the u8 range, their float neighbours, the range ends, non-finite values:
    # round half to even, saturate, NaN -> 0 (cuda_tools/detail/SaturateCastImpl.hpp:41-50)
    ties = np.arange(-4, 261, dtype=np.float32) + np.float32(0.5)
    vals = np.concatenate([ties, np.nextafter(ties, np.float32(-1e9)), np.nextafter(ties, np.float32(1e9)),
                           np.arange(-4, 261, dtype=np.float32),
                           np.array([np.nan, np.inf, -np.inf, 1e9, -1e9, 3e38, -3e38, 1e-40, -1e-40, 0.0, -0.0,
                                     254.5, 255.5, 255.49998, 256.0], np.float32)])
    vals = np.resize(vals, (1, 1, -(-vals.size // 4), 4)).astype(np.float32)  # padded by repeating the start
    out = cv.Tensor.alloc(list(vals.shape), np.uint8, "NHWC")
    cv.ConvertTo()(None, cv.Tensor.from_numpy(vals, "NHWC"), out, 1.0, 0.0)
    torch.cuda.synchronize()
    with np.errstate(invalid="ignore"):
        exp = np.clip(np.rint(np.nan_to_num(vals, nan=0.0, posinf=1e9, neginf=-1e9)), 0, 255).astype(np.uint8)
    np.testing.assert_array_equal(out.numpy(), exp)


def test_convert_to_reference_rows_and_pipeline_shape(cv, orc, gpu):
    # constant 0x10 images of the reference's table; expected value by its formula
    op = cv.ConvertTo()
    for (w, h, alpha, beta, n), (tin, tout, c) in itertools.product(
            [(5, 5, 1.0, 1.0, 1), (5, 5, 2.1, 2.0, 5), (1, 1, 2.1, -1.0, 1)],
            [(np.uint8, np.uint8, 4), (np.uint8, np.float32, 4), (np.float32, np.uint8, 4), (np.float32, np.float32, 4),
             (np.uint8, np.uint16, 1), (np.uint16, np.float32, 2), (np.uint8, np.float32, 3)]):
        a = np.full((n, h, w, c), 16, tin)
        t_out = cv.Tensor.alloc([n, h, w, c], tout, "NHWC")
        op(None, cv.Tensor.from_numpy(a, "NHWC"), t_out, alpha, beta)
        torch.cuda.synchronize()
        exp = alpha * 16 + beta
        exp = np.float32(exp) if tout == np.float32 else np.clip(np.rint(exp), 0, np.iinfo(tout).max)
        assert np.allclose(t_out.numpy(), exp, rtol=1e-6)
    # u8 -> f32 /255 at the fused operator's output shape
    a = rand(orc, (64, 224, 224, 3), np.uint8, 9)
    t_out = cv.Tensor.alloc([64, 224, 224, 3], np.float32, "NHWC")
    op(None, cv.Tensor.from_numpy(a, "NHWC"), t_out, 1 / 255.0, 0.0)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(t_out.numpy(), a.astype(np.float32) * np.float32(1 / 255.0))


@pytest.mark.parametrize("dt,c", [(np.uint8, 1), (np.uint8, 3), (np.uint8, 4), (np.uint16, 3), (np.int16, 2),
                                  (np.float32, 1), (np.float32, 4), (np.float64, 3), (np.int32, 3)])
def test_custom_and_center_crop(cv, orc, gpu, dt, c):
    n, h, w = 3, 61, 97
    a = rand(orc, (n, h, w, c), dt, 21)
    tin = cv.Tensor.from_numpy(a, "NHWC")
    crop, center = cv.CustomCrop(), cv.CenterCrop()
    for x, y, cw, ch in [(0, 0, w, h), (5, 7, 33, 21), (96, 60, 1, 1), (1, 0, 96, 61), (13, 2, 70, 5)]:
        for oh, ow in [(ch, cw), (ch + 3, cw + 5)]:
            out = cv.Tensor.alloc([n, oh, ow, c], dt, "NHWC")
            raw = out.torch_view()
            raw.fill_(7)
            crop(None, tin, out, (x, y, cw, ch))
            torch.cuda.synchronize()
            res = out.numpy()
            np.testing.assert_array_equal(res[:, :ch, :cw], a[:, y:y + ch, x:x + cw])
            assert (res[:, ch:] == 7).all() and (res[:, :, cw:] == 7).all()  # outside the region: untouched
    for cw, ch in [(w, h), (32, 32), (1, 1), (96, 60), (33, 20)]:
        out = cv.Tensor.alloc([n, ch, cw, c], dt, "NHWC")
        center(None, tin, out, (cw, ch))
        torch.cuda.synchronize()
        top, left = (h - ch) // 2, (w - cw) // 2
        np.testing.assert_array_equal(out.numpy(), a[:, top:top + ch, left:left + cw])


def test_crop_negative(cv, gpu):
    a = cv.Tensor.alloc([2, 24, 24, 3], np.uint8, "NHWC")
    out = cv.Tensor.alloc([2, 24, 24, 3], np.uint8, "NHWC")
    crop, center = cv.CustomCrop(), cv.CenterCrop()
    for rect in [(-1, 0, 4, 4), (0, -1, 4, 4), (21, 0, 4, 4), (0, 21, 4, 4), (0, 0, 25, 4), (0, 0, 4, 25)]:
        with pytest.raises(cv.Error) as e:
            crop(None, a, out, rect)
        assert e.value.status == 2
    for bad in [cv.Tensor.alloc([2, 24, 24, 3], np.uint16, "NHWC"), cv.Tensor.alloc([2, 3, 24, 24], np.uint8, "NCHW"),
                cv.Tensor.alloc([2, 2, 2, 3], np.uint8, "NHWC")]:
        with pytest.raises(cv.Error) as e:
            crop(None, a, bad, (0, 0, 4, 4))
        assert e.value.status == 2
        with pytest.raises(cv.Error) as e:
            center(None, a, bad, (4, 4))
        assert e.value.status == 2
    with pytest.raises(cv.Error) as e:
        center(None, a, out, (25, 4))
    assert e.value.status == 2


@pytest.mark.parametrize("dt,c", [(np.uint8, 1), (np.uint8, 3), (np.uint8, 4), (np.uint16, 3), (np.int32, 4),
                                  (np.float32, 1), (np.float32, 3)])
@pytest.mark.parametrize("code", [1, 0, -1, 5, -7])
def test_flip_tensor(cv, orc, gpu, dt, c, code):
    op = cv.Flip(0)
    for shape in [(2, 37, 53, c), (1, 1, 1, c), (3, 8, 300, c), (1, 200, 7, c)]:
        a = rand(orc, shape, dt, 31)
        out = cv.Tensor.alloc(list(shape), dt, "NHWC")
        op(None, cv.Tensor.from_numpy(a, "NHWC"), out, code)
        torch.cuda.synchronize()
        ref = a[:, :, ::-1] if code > 0 else a[:, ::-1] if code == 0 else a[:, ::-1, ::-1]
        np.testing.assert_array_equal(out.numpy(), ref)


def test_flip_varshape_and_negative(cv, K, orc, gpu):
    rng = np.random.default_rng(6)
    for fmt, dt, c in [(K.IMAGE_FORMAT_RGB8, np.uint8, 3), (K.IMAGE_FORMAT_RGBA8, np.uint8, 4),
                       (K.IMAGE_FORMAT_U8, np.uint8, 1), (K.IMAGE_FORMAT_RGBf32, np.float32, 3),
                       (K.IMAGE_FORMAT_F32, np.float32, 1)]:
        n = 7
        bi, bo, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
        for i in range(n):
            w, h = int(rng.integers(1, 300)), int(rng.integers(1, 120))
            a = rand(orc, (h, w, c), dt, 60 + i)
            hosts.append(a)
            bi.push_back(cv.Image.from_numpy(a, fmt))
            o = cv.Image.alloc((w, h), fmt)
            outs.append(o)
            bo.push_back(o)
        codes = np.array([1, 0, -1, 2, -3, 1, 0], np.int32)
        cv.Flip(n)(None, bi, bo, cv.Tensor.from_numpy(codes, "N"))
        torch.cuda.synchronize()
        for a, o, code in zip(hosts, outs, codes):
            ref = {1: a[:, ::-1], 0: a[::-1], -1: a[::-1, ::-1]}.get(int(code), a)
            np.testing.assert_array_equal(o.plane_view(0, dt, c).cpu().numpy(), ref)
    op = cv.Flip(4)
    a = cv.Tensor.alloc([2, 24, 24, 3], np.uint8, "NHWC")
    for bad in [cv.Tensor.alloc([2, 24, 24, 3], np.float32, "NHWC"), cv.Tensor.alloc([2, 3, 24, 24], np.uint8, "NCHW"),
                cv.Tensor.alloc([2, 24, 25, 3], np.uint8, "NHWC")]:
        with pytest.raises(cv.Error) as e:
            op(None, a, bad, 0)
        assert e.value.status == 2
    f64 = cv.Tensor.alloc([2, 24, 24, 3], np.float64, "NHWC")
    with pytest.raises(cv.Error) as e:
        op(None, f64, cv.Tensor.alloc([2, 24, 24, 3], np.float64, "NHWC"), 0)
    assert e.value.status == 2
    with pytest.raises(cv.Error) as e:  # too few codes
        cv.Flip(n)(None, bi, bo, cv.Tensor.from_numpy(np.zeros(3, np.int32), "N"))
    assert e.value.status == 2
