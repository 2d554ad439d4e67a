"""Where this build's results deliberately differ from the reference's bytes, one test per difference that
states the chosen behaviour by name. Each is listed under "Differences a caller can observe" in the
integration notes."""
import importlib.util
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NEAREST, LINEAR, CUBIC = 0, 1, 2


@pytest.fixture(scope="module")
def col():
    spec = importlib.util.spec_from_file_location("color_oracle", os.path.join(ROOT, "oracle", "color_oracle.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


def reference_image_batch_i420_layout(y_u_v, h, w):
    """Planar 4:2:0 layout as the reference's IMAGE-BATCH encoder writes it
    (src/cvcuda/priv/legacy/cvt_color_var_shape.cu:614-626): chroma sample (sy/2, sx/2) goes to row h + sy/4 of
    its plane and to column sx/2, plus h/2 -- not w/2 -- for odd sy/2."""
    y, u, v = y_u_v
    out = np.zeros((h * 3 // 2, w), np.uint8)
    out[:h] = y
    for cy in range(h // 2):
        for cx in range(w // 2):
            col_ = cx + ((h // 2) if (cy & 1) else 0)
            if col_ < w:
                out[h + cy // 2, col_] = u[cy, cx]
                out[h + h // 4 + cy // 2, col_] = v[cy, cx]
    return out


def test_image_batch_rgb_to_i420_puts_odd_chroma_rows_at_half_the_width_not_half_the_height(cv, K, orc, col, gpu):
    # The tensor encoder, both decoders (cvt_color.cu:559, 594; cvt_color_var_shape.cu:684) and this build place
    # the chroma of odd row pairs at column W/2 + x/2. The reference's image-batch encoder uses H/2 + x/2
    # (cvt_color_var_shape.cu:622), which its own decoder would not read back for W != H. This build writes the
    # layout the decoders read, for image batches too; on a non-square image the bytes therefore differ from
    # the reference's, on a square one they are the same.
    for (w, h) in ((24, 8), (8, 24), (16, 16)):
        rgb = orc.fill_u8((h, w, 3), 5 * w + h)
        bi, bo = cv.ImageBatchVarShape(1), cv.ImageBatchVarShape(1)
        bi.push_back(cv.Image.from_numpy(rgb, K.IMAGE_FORMAT_RGB8))
        out = cv.Image.alloc((w, h * 3 // 2), K.IMAGE_FORMAT_U8)
        bo.push_back(out)
        cv.CvtColor()(None, bi, bo, K.COLOR_RGB2YUV_I420)
        torch.cuda.synchronize()
        got = out.plane_view(0, np.uint8, 1).cpu().numpy()[:, :, 0]
        chosen = col.yuv420_from_bgr(rgb[None], False, 0, True)[0, :, :, 0]
        np.testing.assert_array_equal(got, chosen)
        # the same bytes as the tensor operator gives for this image
        tout = cv.Tensor.alloc([1, h * 3 // 2, w, 1], np.uint8, "NHWC")
        cv.CvtColor()(None, cv.Tensor.from_numpy(rgb[None], "NHWC"), tout, K.COLOR_RGB2YUV_I420)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(tout.numpy()[0, :, :, 0], got)
        # and what the reference's image-batch encoder would have written
        y = chosen[:h]
        u = chosen[h:h + h // 4].reshape(h // 2, w // 2)
        v = chosen[h + h // 4:].reshape(h // 2, w // 2)
        theirs = reference_image_batch_i420_layout((y, u, v), h, w)
        if w == h:
            np.testing.assert_array_equal(got, theirs)
        else:
            assert (got != theirs).any()
        # round trip through this build's decoder returns to within the 4:2:0 quantisation of the input
        back = cv.Tensor.alloc([1, h, w, 3], np.uint8, "NHWC")
        cv.CvtColor()(None, cv.Tensor.from_numpy(got[None, :, :, None].copy(), "NHWC"), back, K.COLOR_YUV2RGB_I420)
        torch.cuda.synchronize()
        flat = np.full((h, w, 3), 100, np.uint8)  # a flat image survives subsampling exactly up to rounding
        bi2, bo2 = cv.ImageBatchVarShape(1), cv.ImageBatchVarShape(1)
        bi2.push_back(cv.Image.from_numpy(flat, K.IMAGE_FORMAT_RGB8))
        enc = cv.Image.alloc((w, h * 3 // 2), K.IMAGE_FORMAT_U8)
        bo2.push_back(enc)
        cv.CvtColor()(None, bi2, bo2, K.COLOR_RGB2YUV_I420)
        torch.cuda.synchronize()
        dec = cv.Tensor.alloc([1, h, w, 3], np.uint8, "NHWC")
        cv.CvtColor()(None, cv.Tensor.from_numpy(enc.plane_view(0, np.uint8, 1).cpu().numpy()[None].copy(), "NHWC"), dec,
                      K.COLOR_YUV2RGB_I420)
        torch.cuda.synchronize()
        assert np.abs(dec.numpy().astype(np.int16) - 100).max() <= 2


def test_signed_linear_resize_follows_the_device_expression_without_the_goldens_abs(cv, orc, gpu):
    # The reference's golden takes |.| of the bilinear sum (tests/cvcuda/system/ResizeUtils.cpp:241-247), its device
    # kernel does not (src/cvcuda/priv/OpResize.cu:225-228); they differ only for negative samples of signed
    # types, which the reference never tests. This build follows the device: a negative image stays negative.
    src = np.full((1, 12, 16, 1), -1000, np.int16)
    src[0, ::2] = -3000
    tout = cv.Tensor.alloc([1, 7, 9, 1], np.int16, "NHWC")
    cv.Resize()(None, cv.Tensor.from_numpy(src, "NHWC"), tout, LINEAR)
    torch.cuda.synchronize()
    res = tout.numpy()
    assert res.max() < 0
    np.testing.assert_array_equal(res, orc.resize(src, (7, 9), LINEAR, variant=1))  # device expression
    assert (orc.resize(src, (7, 9), LINEAR, variant=0) > 0).all()                   # the golden's abs


@pytest.mark.parametrize("interp", [LINEAR, CUBIC])
def test_sources_narrower_than_the_tap_window_read_clamped_taps(cv, orc, gpu, interp):
    # A LINEAR sample has 2 taps per axis, a CUBIC one 4. On sources with fewer pixels than that along an axis the
    # reference's golden and kernels index outside the image; this build clamps those taps to the image, so a
    # constant source gives a constant result of the same value.
    for (h, w) in ((1, 1), (1, 9), (9, 1), (3, 2)):
        src = np.full((2, h, w, 3), 77, np.uint8)
        tout = cv.Tensor.alloc([2, 5, 6, 3], np.uint8, "NHWC")
        cv.Resize()(None, cv.Tensor.from_numpy(src, "NHWC"), tout, interp)
        torch.cuda.synchronize()
        res = tout.numpy()
        assert np.abs(res.astype(np.int16) - 77).max() <= (0 if interp == LINEAR else 1), (h, w)
        np.testing.assert_array_equal(res, orc.resize_shipped(src, (5, 6), interp))


def test_crops_require_equal_batch_sizes_where_the_reference_reads_out_of_bounds(cv, gpu):
    # CustomCrop / CenterCrop with an output batch larger than the input: the reference launches over the
    # output's batch and reads input samples that do not exist; this build reports INVALID_ARGUMENT.
    tin = cv.Tensor.alloc([2, 16, 16, 3], np.uint8, "NHWC")
    tout = cv.Tensor.alloc([3, 8, 8, 3], np.uint8, "NHWC")
    with pytest.raises(cv.Error) as e:
        cv.CustomCrop()(None, tin, tout, (0, 0, 8, 8))
    assert e.value.status == 2
    with pytest.raises(cv.Error) as e:
        cv.CenterCrop()(None, tin, tout, (8, 8))
    assert e.value.status == 2
