"""GPU parity of cvcudaCvtColor[VarShape]Submit: NV12/NV21/I420/YV12 -> RGB family (bit-exact against
the integer BT.601 restatement, <= 2 against the reference's double-precision golden, its own
tolerance: tests/cvcuda/system/TestOpCvtColor.cpp:626-649) and the bit-exact channel swizzles
(rows :449-470)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def nv12_input(orc, n, w, h, seed):
    y = orc.fill_u8((n, h, w), seed, 16, 235)
    uv = orc.fill_u8((n, h // 2, w), seed + 1, 16, 240)
    return np.concatenate([y, uv], axis=1)[..., None]


YUV_CODES = {  # code name: (dcn, bgr, uidx, semi-planar)
    "YUV2RGB_NV12": (3, False, 0, True), "YUV2BGR_NV12": (3, True, 0, True),
    "YUV2RGB_NV21": (3, False, 1, True), "YUV2BGR_NV21": (3, True, 1, True),
    "YUV2RGBA_NV12": (4, False, 0, True), "YUV2BGRA_NV12": (4, True, 0, True),
    "YUV2RGBA_NV21": (4, False, 1, True), "YUV2BGRA_NV21": (4, True, 1, True),
    "YUV2RGB_YV12": (3, False, 1, False), "YUV2BGR_YV12": (3, True, 1, False),
    "YUV2RGB_IYUV": (3, False, 0, False), "YUV2BGR_IYUV": (3, True, 0, False),
    "YUV2RGBA_YV12": (4, False, 1, False), "YUV2BGRA_IYUV": (4, True, 0, False),
}


@pytest.mark.parametrize("name", sorted(YUV_CODES))
@pytest.mark.parametrize("size", [(64, 48, 2), (130, 36, 3), (1920, 1080, 1), (6, 4, 1), (2, 4, 2)])
def test_yuv420_to_rgb(cv, K, orc, gpu, name, size):
    w, h, n = size
    dcn, bgr, uidx, semi = YUV_CODES[name]
    if not semi and h % 4:
        pytest.skip("planar 4:2:0 needs height % 4 == 0")
    src = nv12_input(orc, n, w, h, w * 3 + h)
    tin = cv.Tensor.from_numpy(src, "NHWC")
    tout = cv.Tensor.alloc([n, h, w, dcn], np.uint8, "NHWC")
    tout.torch_view().fill_(7)
    cv.CvtColor()(None, tin, tout, getattr(K, "COLOR_" + name))
    torch.cuda.synchronize()
    res = tout.numpy()
    ref = orc.yuv420_to_rgb(src, dcn, bgr, uidx, semi, variant=0)
    np.testing.assert_array_equal(res, ref)
    if semi:
        gold = orc.yuv420_to_rgb(src, dcn, bgr, uidx, semi, variant=1)
        assert np.abs(res.astype(np.int16) - gold.astype(np.int16)).max() <= 2


def test_config3_full_size(cv, K, orc, gpu):
    # BASELINE config 3: batch 32, 1080p NV12 -> RGB; Y in [16,235], UV in [16,240]
    src = nv12_input(orc, 32, 1920, 1080, 0xC0FFEE03)
    tin = cv.Tensor.from_numpy(src, "NHWC")
    tout = cv.Tensor.alloc([32, 1080, 1920, 3], np.uint8, "NHWC")
    cv.CvtColor()(None, tin, tout, K.COLOR_YUV2RGB_NV12)
    torch.cuda.synchronize()
    res = tout.numpy()
    np.testing.assert_array_equal(res, orc.yuv420_to_rgb(src, threads=8))


def test_yuv_exhaustive_triples_on_device(cv, K, orc, gpu):
    # all 2^24 (Y,U,V) combinations through the kernel
    W = H = 4096
    by, bx = np.meshgrid(np.arange(H // 2), np.arange(W // 2), indexing="ij")
    blk = by * (W // 2) + bx
    Y = np.zeros((H, W), np.uint8)
    yb = (blk // 65536) * 4
    Y[0::2, 0::2], Y[0::2, 1::2], Y[1::2, 0::2], Y[1::2, 1::2] = yb, yb + 1, yb + 2, yb + 3
    uv = np.zeros((H // 2, W), np.uint8)
    uv[:, 0::2], uv[:, 1::2] = blk % 256, (blk // 256) % 256
    src = np.concatenate([Y, uv])[None, :, :, None]
    tout = cv.Tensor.alloc([1, H, W, 3], np.uint8, "NHWC")
    cv.CvtColor()(None, cv.Tensor.from_numpy(src, "NHWC"), tout, K.COLOR_YUV2RGB_NV12)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tout.numpy(), orc.yuv420_to_rgb(src, threads=8))


SWIZZLES = {"BGR2BGRA": (3, 4, False), "BGRA2BGR": (4, 3, False), "BGR2RGBA": (3, 4, True), "RGBA2BGR": (4, 3, True),
            "BGR2RGB": (3, 3, True), "BGRA2RGBA": (4, 4, True)}
ALPHA = {np.uint8: 255, np.int8: -1, np.uint16: 65535, np.int16: -1, np.int32: 2147483647, np.float32: 1.0,
         np.float64: 1.0}


@pytest.mark.parametrize("name", sorted(SWIZZLES))
@pytest.mark.parametrize("dt", [np.uint8, np.uint16, np.int32, np.float32, np.float64])
def test_swizzles(cv, K, orc, gpu, name, dt):
    sch, dch, swap = SWIZZLES[name]
    n, h, w = 2, 37, 129
    raw = orc.fill_u8((n, h, w, sch, np.dtype(dt).itemsize), 77 + sch)
    src = raw.view(dt).reshape(n, h, w, sch)
    if np.issubdtype(dt, np.floating):
        src = np.nan_to_num(src, nan=0.5, posinf=1.0, neginf=-1.0)
    tin = cv.Tensor.from_numpy(src, "NHWC")
    tout = cv.Tensor.alloc([n, h, w, dch], dt, "NHWC")
    cv.CvtColor()(None, tin, tout, getattr(K, "COLOR_" + name))
    torch.cuda.synchronize()
    want = np.zeros((n, h, w, dch), dt)
    want[..., :3] = src[..., 2::-1] if swap else src[..., :3]
    if dch == 4:
        want[..., 3] = src[..., 3] if sch == 4 else ALPHA[dt]
    np.testing.assert_array_equal(tout.numpy(), want)


def test_varshape_nv12_and_swizzle(cv, K, orc, gpu):
    rng = np.random.default_rng(2)
    n = 5
    bin_, bout, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
    for i in range(n):
        w, h = 2 * int(rng.integers(5, 200)), 2 * int(rng.integers(3, 100))
        a = nv12_input(orc, 1, w, h, 50 + i)[0]
        hosts.append(a)
        bin_.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_U8))
        o = cv.Image.alloc((w, h), K.IMAGE_FORMAT_BGR8)
        outs.append(o)
        bout.push_back(o)
    cv.CvtColor()(None, bin_, bout, K.COLOR_YUV2BGR_NV12)
    torch.cuda.synchronize()
    for a, o in zip(hosts, outs):
        np.testing.assert_array_equal(o.plane_view(0, np.uint8, 3).cpu().numpy()[None],
                                      orc.yuv420_to_rgb(a[None], 3, True, 0, True))
    # swizzle on the results: BGR -> RGBA
    bout2, outs2 = cv.ImageBatchVarShape(n), []
    for o in outs:
        o2 = cv.Image.alloc(o.size, K.IMAGE_FORMAT_RGBA8)
        outs2.append(o2)
        bout2.push_back(o2)
    cv.CvtColor()(None, bout, bout2, K.COLOR_BGR2RGBA)
    torch.cuda.synchronize()
    for o, o2 in zip(outs, outs2):
        a = o.plane_view(0, np.uint8, 3).cpu().numpy()
        b = o2.plane_view(0, np.uint8, 4).cpu().numpy()
        np.testing.assert_array_equal(b[..., :3], a[..., ::-1])
        assert (b[..., 3] == 255).all()


def test_negative_cases(cv, K, gpu):
    op = cv.CvtColor()
    nv = cv.Tensor.alloc([1, 12, 8, 1], np.uint8, "NHWC")
    bad = [
        (nv, cv.Tensor.alloc([1, 8, 8, 2], np.uint8, "NHWC"), K.COLOR_YUV2RGB_NV12),    # 2 output channels
        (nv, cv.Tensor.alloc([1, 6, 8, 3], np.uint8, "NHWC"), K.COLOR_YUV2RGB_NV12),    # wrong height
        (nv, cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC"), K.COLOR_YUV2RGB_NV12),    # batch mismatch
        (cv.Tensor.alloc([1, 10, 8, 1], np.uint8, "NHWC"), cv.Tensor.alloc([1, 6, 8, 3], np.uint8, "NHWC"),
         K.COLOR_YUV2RGB_NV12),                                                           # H % 3 != 0
        (cv.Tensor.alloc([1, 9, 8, 1], np.uint8, "NHWC"), cv.Tensor.alloc([1, 6, 8, 3], np.uint8, "NHWC"),
         K.COLOR_YUV2RGB_YV12),                                                           # planar needs H % 4 == 0
        (cv.Tensor.alloc([1, 8, 8, 3], np.uint8, "NHWC"), cv.Tensor.alloc([1, 8, 8, 3], np.uint8, "NHWC"),
         K.COLOR_BGR2BGRA),                                                               # needs 4 output channels
        (cv.Tensor.alloc([1, 8, 8, 3], np.uint8, "NHWC"), cv.Tensor.alloc([1, 8, 8, 3], np.float32, "NHWC"),
         K.COLOR_BGR2RGB),                                                                # dtype mismatch
        (cv.Tensor.alloc([1, 8, 8, 3], np.uint8, "NHWC"), cv.Tensor.alloc([1, 3, 8, 8], np.uint8, "NCHW"),
         K.COLOR_BGR2RGB),                                                                # layout
        (cv.Tensor.alloc([1, 8, 8, 3], np.uint8, "NHWC"), cv.Tensor.alloc([1, 8, 8, 3], np.uint8, "NHWC"),
         K.COLOR_BGR2Lab),                                                                # code not provided (by the reference either)
    ]
    for tin, tout, code in bad:
        with pytest.raises(cv.Error) as e:
            op(None, tin, tout, code)
        assert e.value.status == 2
