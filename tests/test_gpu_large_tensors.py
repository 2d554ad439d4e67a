"""Tensors whose samples lie beyond the 2 GiB and 4 GiB marks. CvtColor is the one operator on the path that takes
them (the others refuse tensors that span more than INT32_MAX bytes, like the reference): every kernel form it
uses must address the last samples with 64-bit offsets. All samples but the last hold one image and the last
holds another: an offset that wrapped would convert the common image where the special one is expected."""
import importlib.util
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def col():
    spec = importlib.util.spec_from_file_location("color_oracle", os.path.join(ROOT, "oracle", "color_oracle.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


H, W = 540, 960


def run_big(cv, common, special, n, out_shape, code):
    """n samples of `common`, the last replaced by `special`; returns output samples 0, n - 2 and n - 1."""
    tin = cv.Tensor.alloc([n] + list(common.shape), np.uint8, "NHWC")
    tout = cv.Tensor.alloc([n] + list(out_shape), np.uint8, "NHWC")
    vin, vout = tin.torch_view(), tout.torch_view()
    assert vin.stride(0) * (n - 1) > 2 ** 32 or vout.stride(0) * (n - 1) > 2 ** 32
    vin[:] = torch.from_numpy(common).cuda()
    vin[n - 1] = torch.from_numpy(special).cuda()
    vout.fill_(0x5A)
    cv.CvtColor()(None, tin, tout, code)
    torch.cuda.synchronize()
    return [vout[i].cpu().numpy() for i in (0, n - 2, n - 1)]


def test_colour_conversions_address_samples_beyond_4_gib(cv, K, orc, col, gpu):
    bgr_a, bgr_b = orc.fill_u8((H, W, 3), 71), orc.fill_u8((H, W, 3), 72)
    n3 = 2 ** 32 // (H * W * 3) + 40  # samples of a 3-channel image that reach past 4 GiB
    # channel swizzle (run kernel)
    first, before, last = run_big(cv, bgr_a, bgr_b, n3, (H, W, 3), K.COLOR_BGR2RGB)
    np.testing.assert_array_equal(first, bgr_a[..., ::-1])
    np.testing.assert_array_equal(before, bgr_a[..., ::-1])
    np.testing.assert_array_equal(last, bgr_b[..., ::-1])
    # one pixel in, one pixel out (map kernel), output a third of the input
    first, before, last = run_big(cv, bgr_a, bgr_b, n3, (H, W, 1), K.COLOR_BGR2GRAY)
    np.testing.assert_array_equal(before, col.gray_from_bgr(bgr_a[None], True)[0])
    np.testing.assert_array_equal(last, col.gray_from_bgr(bgr_b[None], True)[0])
    # 4:2:0 encoder (item kernel): the input reaches past 4 GiB
    first, before, last = run_big(cv, bgr_a, bgr_b, n3, (H * 3 // 2, W, 1), K.COLOR_BGR2YUV_NV12)
    np.testing.assert_array_equal(before, col.yuv420_from_bgr(bgr_a[None], True, 0, False)[0])
    np.testing.assert_array_equal(last, col.yuv420_from_bgr(bgr_b[None], True, 0, False)[0])
    # 4:2:0 decoder: the output reaches past 4 GiB
    nv_a, nv_b = orc.fill_u8((H * 3 // 2, W, 1), 73), orc.fill_u8((H * 3 // 2, W, 1), 74)
    first, before, last = run_big(cv, nv_a, nv_b, n3, (H, W, 3), K.COLOR_YUV2BGR_NV12)
    np.testing.assert_array_equal(before, orc.yuv420_to_rgb(nv_a[None], 3, True, 0, True, variant=0)[0])
    np.testing.assert_array_equal(last, orc.yuv420_to_rgb(nv_b[None], 3, True, 0, True, variant=0)[0])
    # 4:2:2 decoder
    yuy_a, yuy_b = orc.fill_u8((H, 2 * W, 1), 75), orc.fill_u8((H, 2 * W, 1), 76)
    first, before, last = run_big(cv, yuy_a, yuy_b, n3, (H, W, 3), K.COLOR_YUV2BGR_YUY2)
    np.testing.assert_array_equal(before, col.bgr_from_yuv422(yuy_a[None], True, 0, 0, 3)[0])
    np.testing.assert_array_equal(last, col.bgr_from_yuv422(yuy_b[None], True, 0, 0, 3)[0])
