"""GPU parity of the per-pixel colour families of cvcudaCvtColor[VarShape]Submit against
oracle/color_oracle.py: integer results bit-exact, float32 results within 1e-4 (HSV hue 2e-3, the
reference's own bounds tests/cvcuda/system/TestOpCvtColor.cpp:538-700). Shapes follow its table."""
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


def image(orc, shape, dt, seed):
    if dt == np.float32:
        return orc.fill_f32(shape, seed)
    a = orc.fill_u8(tuple(shape) + (np.dtype(dt).itemsize,), seed).view(dt).reshape(shape)
    return a


def run(cv, a, out_shape, out_dt, code):
    tout = cv.Tensor.alloc(list(out_shape), out_dt, "NHWC")
    cv.CvtColor()(None, cv.Tensor.from_numpy(a, "NHWC"), tout, code)
    torch.cuda.synchronize()
    return tout.numpy()


def check(res, ref, tol=0.0):
    assert res.shape == ref.shape
    if ref.dtype.kind == "f":
        assert np.abs(res - ref).max() <= tol, np.abs(res - ref).max()
    else:
        np.testing.assert_array_equal(res, ref)


@pytest.mark.parametrize("dt", [np.uint8, np.uint16, np.float32])
def test_gray_and_yuv444(cv, K, orc, col, gpu, dt):
    for (w, h, n) in [(21, 22, 3), (201, 102, 2), (64, 21, 3), (513, 40, 1)]:
        a = image(orc, (n, h, w, 3), dt, w + n)
        check(run(cv, a, (n, h, w, 1), dt, K.COLOR_BGR2GRAY), col.gray_from_bgr(a, True), 1e-6)
        check(run(cv, a, (n, h, w, 1), dt, K.COLOR_RGB2GRAY), col.gray_from_bgr(a, False), 1e-6)
        g = a[..., :1].copy()
        check(run(cv, g, (n, h, w, 3), dt, K.COLOR_GRAY2BGR), col.bgr_from_gray(g), 0)
        check(run(cv, a, (n, h, w, 3), dt, K.COLOR_BGR2YUV), col.yuv_from_bgr(a, True), 1e-6)
        check(run(cv, a, (n, h, w, 3), dt, K.COLOR_RGB2YUV), col.yuv_from_bgr(a, False), 1e-6)
        check(run(cv, a, (n, h, w, 3), dt, K.COLOR_YUV2BGR), col.bgr_from_yuv(a, True), 1e-5)
        check(run(cv, a, (n, h, w, 3), dt, K.COLOR_YUV2RGB), col.bgr_from_yuv(a, False), 1e-5)


def test_gray2bgr_other_types_and_negative(cv, K, orc, col, gpu):
    for dt in (np.int8, np.int16, np.int32, np.float64):
        g = image(orc, (2, 9, 33, 1), np.uint8, 3).astype(dt)
        check(run(cv, g, (2, 9, 33, 3), dt, K.COLOR_GRAY2BGR), col.bgr_from_gray(g), 0)
    a = cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC")
    op = cv.CvtColor()
    bad = [(cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC"), K.COLOR_BGR2GRAY),      # 3 channels out
           (cv.Tensor.alloc([2, 8, 8, 1], np.uint16, "NHWC"), K.COLOR_BGR2GRAY),     # type differs
           (cv.Tensor.alloc([2, 8, 9, 1], np.uint8, "NHWC"), K.COLOR_RGB2GRAY),      # size differs
           (cv.Tensor.alloc([2, 8, 8, 4], np.uint8, "NHWC"), K.COLOR_BGR2YUV),
           (cv.Tensor.alloc([2, 8, 8, 1], np.uint8, "NHWC"), K.COLOR_BGR2HSV),
           (cv.Tensor.alloc([2, 12, 8, 3], np.uint8, "NHWC"), K.COLOR_BGR2YUV_NV12),  # must be 1 channel
           (cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC"), 9),                      # GRAY2BGRA: not implemented
           (cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC"), 109)]                    # VYUY: not implemented
    for out, code in bad:
        with pytest.raises(cv.Error) as e:
            op(None, a, out, code)
        assert e.value.status == 2
    s8 = cv.Tensor.alloc([2, 8, 8, 3], np.int8, "NHWC")
    with pytest.raises(cv.Error) as e:
        op(None, s8, cv.Tensor.alloc([2, 8, 8, 1], np.int8, "NHWC"), K.COLOR_BGR2GRAY)
    assert e.value.status == 2


@pytest.mark.parametrize("full", [False, True])
def test_hsv(cv, K, orc, col, gpu, full):
    for (w, h, n) in [(55, 257, 2), (366, 14, 3), (112, 157, 1)]:
        a = image(orc, (n, h, w, 3), np.uint8, w)
        a[0, 0, :16] = np.array([[0, 0, 0], [255, 255, 255], [255, 0, 0], [0, 255, 0], [0, 0, 255], [7, 7, 7], [1, 0, 0],
                                 [0, 1, 0], [254, 255, 255], [255, 254, 255], [128, 128, 127], [10, 200, 10],
                                 [200, 10, 200], [3, 2, 1], [1, 2, 3], [90, 90, 91]], np.uint8)
        c_bgr = K.COLOR_BGR2HSV_FULL if full else K.COLOR_BGR2HSV
        c_rgb = K.COLOR_RGB2HSV_FULL if full else K.COLOR_RGB2HSV
        hsv = run(cv, a, (n, h, w, 3), np.uint8, c_bgr)
        check(hsv, col.hsv_from_bgr(a, True, full))
        check(run(cv, a, (n, h, w, 3), np.uint8, c_rgb), col.hsv_from_bgr(a, False, full))
        d_bgr = K.COLOR_HSV2BGR_FULL if full else K.COLOR_HSV2BGR
        d_rgb = K.COLOR_HSV2RGB_FULL if full else K.COLOR_HSV2RGB
        # hue values a real image holds (< 180 for the half range) and arbitrary bytes as well
        for src in (hsv, a):
            res = run(cv, src, (n, h, w, 3), np.uint8, d_bgr)
            ref = col.bgr_from_hsv(src, True, full)
            assert np.abs(res.astype(int) - ref.astype(int)).max() <= 1  # float path: products may round apart
            assert (res != ref).mean() < 1e-3
            res4 = run(cv, src, (n, h, w, 4), np.uint8, d_rgb)
            assert (res4[..., 3] == 255).all()
            np.testing.assert_array_equal(res4[..., :3], res[..., ::-1])
    if not full:
        f = image(orc, (2, 33, 125, 3), np.float32, 9)
        f[0, 0, :4] = np.array([[0, 0, 0], [1, 1, 1], [0.5, 0.5, 0.5], [0.25, 0.75, 0.25]], np.float32)
        res = run(cv, f, (2, 33, 125, 3), np.float32, K.COLOR_BGR2HSV)
        ref = col.hsv_from_bgr(f, True)
        assert np.abs(res[..., 1:] - ref[..., 1:]).max() <= 1e-5
        dh = np.abs(res[..., 0] - ref[..., 0])
        assert np.minimum(dh, 360 - dh).max() <= 2e-3
        hs = ref.copy()
        back = run(cv, hs, (2, 33, 125, 3), np.float32, K.COLOR_HSV2BGR)
        check(back, col.bgr_from_hsv(hs, True), 1e-5)
        back4 = run(cv, hs, (2, 33, 125, 4), np.float32, K.COLOR_HSV2RGB)
        assert (back4[..., 3] == 1.0).all()
        check(back4[..., :3], col.bgr_from_hsv(hs, False), 1e-5)


ENCODE = [  # code name, bgr order, uidx, planar, channels
    ("COLOR_RGB2YUV_NV12", False, 0, False, 3), ("COLOR_BGR2YUV_NV12", True, 0, False, 3),
    ("COLOR_RGB2YUV_NV21", False, 1, False, 3), ("COLOR_BGR2YUV_NV21", True, 1, False, 3),
    ("COLOR_RGBA2YUV_NV12", False, 0, False, 4), ("COLOR_BGRA2YUV_NV12", True, 0, False, 4),
    ("COLOR_RGBA2YUV_NV21", False, 1, False, 4), ("COLOR_BGRA2YUV_NV21", True, 1, False, 4),
    ("COLOR_RGB2YUV_I420", False, 0, True, 3), ("COLOR_BGR2YUV_I420", True, 0, True, 3),
    ("COLOR_RGBA2YUV_I420", False, 0, True, 4), ("COLOR_BGRA2YUV_I420", True, 0, True, 4),
    ("COLOR_RGB2YUV_YV12", False, 1, True, 3), ("COLOR_BGR2YUV_YV12", True, 1, True, 3),
    ("COLOR_RGBA2YUV_YV12", False, 1, True, 4), ("COLOR_BGRA2YUV_YV12", True, 1, True, 4),
]


@pytest.mark.parametrize("name,bgr,uidx,planar,c", ENCODE, ids=[e[0] for e in ENCODE])
def test_rgb_to_yuv420(cv, K, orc, col, gpu, name, bgr, uidx, planar, c):
    for (w, h, n) in [(120, 20, 2), (100, 40, 3), (2, 4, 1), (1920, 1080 if not planar else 1080, 1)]:
        a = image(orc, (n, h, w, c), np.uint8, w + c)
        res = run(cv, a, (n, h * 3 // 2, w, 1), np.uint8, getattr(K, name))
        check(res, col.yuv420_from_bgr(a, bgr, uidx, planar))
    # and back through the decoder of this build: within the reference's round-trip bound on smooth data
    g = np.repeat(np.repeat(image(orc, (1, 10, 16, c), np.uint8, 5), 4, axis=1), 4, axis=2)
    yuv = run(cv, g, (1, 60, 64, 1), np.uint8, getattr(K, name))
    dec = {(False, 0, False): "COLOR_YUV2RGB_NV12", (True, 0, False): "COLOR_YUV2BGR_NV12",
           (False, 1, False): "COLOR_YUV2RGB_NV21", (True, 1, False): "COLOR_YUV2BGR_NV21",
           (False, 0, True): "COLOR_YUV2RGB_I420", (True, 0, True): "COLOR_YUV2BGR_I420",
           (False, 1, True): "COLOR_YUV2RGB_YV12", (True, 1, True): "COLOR_YUV2BGR_YV12"}[(bgr, uidx, planar)]
    back = run(cv, yuv, (1, 40, 64, 3), np.uint8, getattr(K, dec))
    assert np.abs(back.astype(int) - g[..., :3].astype(int)).max() <= 3


def test_rgb_to_yuv420_negative(cv, K, gpu):
    op = cv.CvtColor()
    for shape_in, shape_out, code in [([2, 9, 8, 3], [2, 13, 8, 1], K.COLOR_RGB2YUV_NV12),     # odd height
                                      ([2, 8, 9, 3], [2, 12, 9, 1], K.COLOR_RGB2YUV_NV12),     # odd width
                                      ([2, 6, 8, 3], [2, 9, 8, 1], K.COLOR_RGB2YUV_I420),      # planar: H % 4
                                      ([2, 8, 8, 3], [2, 8, 8, 1], K.COLOR_RGB2YUV_NV12),      # output height
                                      ([2, 8, 8, 1], [2, 12, 8, 1], K.COLOR_RGB2YUV_NV12)]:    # input channels
        with pytest.raises(cv.Error) as e:
            op(None, cv.Tensor.alloc(shape_in, np.uint8, "NHWC"), cv.Tensor.alloc(shape_out, np.uint8, "NHWC"), code)
        assert e.value.status == 2


DECODE422 = [  # code name, bgr, yidx, uidx, dcn
    ("COLOR_YUV2RGB_UYVY", False, 1, 0, 3), ("COLOR_YUV2BGR_UYVY", True, 1, 0, 3),
    ("COLOR_YUV2RGBA_UYVY", False, 1, 0, 4), ("COLOR_YUV2BGRA_UYVY", True, 1, 0, 4),
    ("COLOR_YUV2RGB_YUY2", False, 0, 0, 3), ("COLOR_YUV2BGR_YUY2", True, 0, 0, 3),
    ("COLOR_YUV2RGB_YVYU", False, 0, 2, 3), ("COLOR_YUV2BGR_YVYU", True, 0, 2, 3),
    ("COLOR_YUV2RGBA_YUY2", False, 0, 0, 4), ("COLOR_YUV2BGRA_YUY2", True, 0, 0, 4),
    ("COLOR_YUV2RGBA_YVYU", False, 0, 2, 4), ("COLOR_YUV2BGRA_YVYU", True, 0, 2, 4),
]


@pytest.mark.parametrize("name,bgr,yidx,uidx,dcn", DECODE422, ids=[e[0] for e in DECODE422])
def test_yuv422_to_rgb(cv, K, orc, col, gpu, name, bgr, yidx, uidx, dcn):
    for (w, h, n) in [(120, 20, 2), (100, 40, 3), (2, 1, 1), (1920, 270, 1)]:
        a = image(orc, (n, h, 2 * w, 1), np.uint8, w + dcn)
        check(run(cv, a, (n, h, w, dcn), np.uint8, getattr(K, name)), col.bgr_from_yuv422(a, bgr, yidx, uidx, dcn))


def test_yuv_to_gray(cv, K, orc, col, gpu):
    a = image(orc, (3, 40, 200, 1), np.uint8, 2)  # 100 pixels per row
    check(run(cv, a, (3, 40, 100, 1), np.uint8, K.COLOR_YUV2GRAY_UYVY), col.gray_from_yuv422(a, 1))
    check(run(cv, a, (3, 40, 100, 1), np.uint8, K.COLOR_YUV2GRAY_YUY2), col.gray_from_yuv422(a, 0))
    nv = image(orc, (2, 180, 80, 1), np.uint8, 3)
    check(run(cv, nv, (2, 120, 80, 1), np.uint8, K.COLOR_YUV2GRAY_420), nv[:, :120])
    op = cv.CvtColor()
    with pytest.raises(cv.Error) as e:
        op(None, cv.Tensor.from_numpy(a, "NHWC"), cv.Tensor.alloc([3, 40, 100, 3], np.uint8, "NHWC"), K.COLOR_YUV2GRAY_UYVY)
    assert e.value.status == 2
    with pytest.raises(cv.Error) as e:
        op(None, cv.Tensor.alloc([1, 8, 6, 1], np.uint8, "NHWC"), cv.Tensor.alloc([1, 8, 3, 3], np.uint8, "NHWC"),
           K.COLOR_YUV2RGB_UYVY)  # width not a multiple of 4
    assert e.value.status == 2


def test_varshape_per_pixel_families(cv, K, orc, col, gpu):
    rng = np.random.default_rng(8)
    cases = [(K.COLOR_BGR2GRAY, K.IMAGE_FORMAT_RGB8, K.IMAGE_FORMAT_U8, np.uint8, 3, 1, lambda a: col.gray_from_bgr(a[None])[0]),
             (K.COLOR_GRAY2BGR, K.IMAGE_FORMAT_U8, K.IMAGE_FORMAT_RGB8, np.uint8, 1, 3, lambda a: col.bgr_from_gray(a[None])[0]),
             (K.COLOR_RGB2YUV, K.IMAGE_FORMAT_RGB8, K.IMAGE_FORMAT_RGB8, np.uint8, 3, 3, lambda a: col.yuv_from_bgr(a[None], False)[0]),
             (K.COLOR_YUV2BGR, K.IMAGE_FORMAT_RGBf32, K.IMAGE_FORMAT_RGBf32, np.float32, 3, 3, lambda a: col.bgr_from_yuv(a[None], True)[0]),
             (K.COLOR_BGR2HSV, K.IMAGE_FORMAT_RGB8, K.IMAGE_FORMAT_RGB8, np.uint8, 3, 3, lambda a: col.hsv_from_bgr(a[None], True)[0]),
             (K.COLOR_HSV2RGB_FULL, K.IMAGE_FORMAT_RGB8, K.IMAGE_FORMAT_RGBA8, np.uint8, 3, 4,
              lambda a: col.bgr_from_hsv(a[None], False, True, 4)[0])]
    for code, fin, fout, dt, cin, cout, ref in cases:
        n = 5
        bi, bo, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
        for i in range(n):
            w, h = int(rng.integers(1, 260)), int(rng.integers(1, 90))
            a = image(orc, (h, w, cin), dt, 70 + i)
            hosts.append(a)
            bi.push_back(cv.Image.from_numpy(a, fin))
            o = cv.Image.alloc((w, h), fout)
            outs.append(o)
            bo.push_back(o)
        cv.CvtColor()(None, bi, bo, code)
        torch.cuda.synchronize()
        for a, o in zip(hosts, outs):
            res = o.plane_view(0, dt, cout).cpu().numpy()
            r = ref(a)
            if code == K.COLOR_HSV2RGB_FULL:
                assert np.abs(res.astype(int) - r.astype(int)).max() <= 1
            else:
                check(res, r, 1e-5)


def test_varshape_subsampled_families(cv, K, orc, col, gpu):
    # image batches through the 4:2:0 encoders, the 4:2:2 decoders and the luma extractions (the
    # reference: legacy/cvt_color_var_shape.cu:1416-1640): single-plane u8 images, every image its own size
    rng = np.random.default_rng(21)
    n = 7
    sizes = [(2 * int(rng.integers(1, 150)), 4 * int(rng.integers(1, 30))) for _ in range(n)]
    sizes[0], sizes[1] = (2, 4), (516, 8)

    def batch_from(arrays, fmt):
        b = cv.ImageBatchVarShape(len(arrays))
        for a in arrays:
            b.push_back(cv.Image.from_numpy(a, fmt))
        return b

    def batch_alloc(dims, fmt):
        b, outs = cv.ImageBatchVarShape(len(dims)), []
        for wh in dims:
            outs.append(cv.Image.alloc(wh, fmt))
            b.push_back(outs[-1])
        return b, outs

    def results(outs, c):
        torch.cuda.synchronize()
        return [o.plane_view(0, np.uint8, c).cpu().numpy() for o in outs]

    for c, fmt in ((3, K.IMAGE_FORMAT_RGB8), (4, K.IMAGE_FORMAT_RGBA8)):
        rgb = [image(orc, (h, w, c), np.uint8, 31 * i + c) for i, (w, h) in enumerate(sizes)]
        bi = batch_from(rgb, fmt)
        for name, bgr, uidx, planar in [("COLOR_RGB2YUV_NV12", False, 0, False), ("COLOR_BGR2YUV_NV21", True, 1, False),
                                        ("COLOR_BGR2YUV_I420", True, 0, True), ("COLOR_RGB2YUV_YV12", False, 1, True)]:
            name = name.replace("RGB2", "RGBA2").replace("BGR2", "BGRA2") if c == 4 else name
            bo, outs = batch_alloc([(w, h * 3 // 2) for w, h in sizes], K.IMAGE_FORMAT_U8)
            cv.CvtColor()(None, bi, bo, getattr(K, name))
            for a, r in zip(rgb, results(outs, 1)):
                check(r[None], col.yuv420_from_bgr(a[None], bgr, uidx, planar))
    packed = [image(orc, (h, 2 * w, 1), np.uint8, 17 * i) for i, (w, h) in enumerate(sizes)]
    bi = batch_from(packed, K.IMAGE_FORMAT_U8)
    for name, bgr, yidx, uidx, dcn in [("COLOR_YUV2BGR_YUY2", True, 0, 0, 3), ("COLOR_YUV2RGBA_UYVY", False, 1, 0, 4),
                                       ("COLOR_YUV2RGB_YVYU", False, 0, 2, 3)]:
        bo, outs = batch_alloc(sizes, K.IMAGE_FORMAT_RGB8 if dcn == 3 else K.IMAGE_FORMAT_RGBA8)
        cv.CvtColor()(None, bi, bo, getattr(K, name))
        for a, r in zip(packed, results(outs, dcn)):
            check(r[None], col.bgr_from_yuv422(a[None], bgr, yidx, uidx, dcn))
    bo, outs = batch_alloc(sizes, K.IMAGE_FORMAT_U8)
    cv.CvtColor()(None, bi, bo, K.COLOR_YUV2GRAY_YUY2)
    for a, r in zip(packed, results(outs, 1)):
        check(r[None], col.gray_from_yuv422(a[None], 0))
    planes = [image(orc, (h * 3 // 2, w, 1), np.uint8, 13 * i) for i, (w, h) in enumerate(sizes)]
    bo, outs = batch_alloc(sizes, K.IMAGE_FORMAT_U8)
    cv.CvtColor()(None, batch_from(planes, K.IMAGE_FORMAT_U8), bo, K.COLOR_YUV2GRAY_420)
    for a, r, (w, h) in zip(planes, results(outs, 1), sizes):
        check(r, a[:h])
    # one image of the batch with the wrong output height
    bi = batch_from([image(orc, (8, 8, 3), np.uint8, 1), image(orc, (8, 16, 3), np.uint8, 2)], K.IMAGE_FORMAT_RGB8)
    bo, _ = batch_alloc([(8, 12), (16, 8)], K.IMAGE_FORMAT_U8)
    with pytest.raises(cv.Error) as e:
        cv.CvtColor()(None, bi, bo, K.COLOR_RGB2YUV_NV12)
    assert e.value.status == 2


def test_every_width_residue_of_the_grouped_kernels(cv, K, orc, col, gpu):
    # the byte-pixel kernels move 8 or 16 pixels per lane and finish a row's ragged end item by item: every
    # even width from 2 to 40 (all residues modulo 16, rows shorter than one group included) plus widths
    # around a whole wave's 512 pixels, through each of those kernels
    widths = list(range(2, 42, 2)) + [510, 512, 514, 516, 520, 526]
    for w in widths:
        h, n = 4, 2
        nv = np.concatenate([orc.fill_u8((n, h, w), w, 16, 235), orc.fill_u8((n, h // 2, w), w + 1, 16, 240)], axis=1)[..., None]
        for name, dcn, bgr, uidx, semi in [("COLOR_YUV2RGB_NV12", 3, False, 0, True), ("COLOR_YUV2BGRA_NV21", 4, True, 1, True),
                                           ("COLOR_YUV2RGB_IYUV", 3, False, 0, False), ("COLOR_YUV2BGRA_YV12", 4, True, 1, False)]:
            check(run(cv, nv, (n, h, w, dcn), np.uint8, getattr(K, name)), orc.yuv420_to_rgb(nv, dcn, bgr, uidx, semi, variant=0))
        check(run(cv, nv, (n, h, w, 1), np.uint8, K.COLOR_YUV2GRAY_420), nv[:, :h])
        a = image(orc, (n, h, w, 3), np.uint8, 3 * w)
        a4 = image(orc, (n, h, w, 4), np.uint8, 5 * w)
        check(run(cv, a, (n, h * 3 // 2, w, 1), np.uint8, K.COLOR_RGB2YUV_NV12), col.yuv420_from_bgr(a, False, 0, False))
        check(run(cv, a4, (n, h * 3 // 2, w, 1), np.uint8, K.COLOR_BGRA2YUV_NV21), col.yuv420_from_bgr(a4, True, 1, False))
        check(run(cv, a, (n, h * 3 // 2, w, 1), np.uint8, K.COLOR_BGR2YUV_I420), col.yuv420_from_bgr(a, True, 0, True))
        check(run(cv, a4, (n, h * 3 // 2, w, 1), np.uint8, K.COLOR_RGBA2YUV_YV12), col.yuv420_from_bgr(a4, False, 1, True))
        check(run(cv, a, (n, h, w, 1), np.uint8, K.COLOR_BGR2GRAY), col.gray_from_bgr(a, True))
        check(run(cv, a, (n, h, w, 3), np.uint8, K.COLOR_RGB2HSV), col.hsv_from_bgr(a, False, False))
        check(run(cv, a, (n, h, w, 3), np.uint8, K.COLOR_BGR2YUV), col.yuv_from_bgr(a, True))
        y2 = image(orc, (n, h, 2 * w, 1), np.uint8, 7 * w)
        check(run(cv, y2, (n, h, w, 3), np.uint8, K.COLOR_YUV2BGR_YUY2), col.bgr_from_yuv422(y2, True, 0, 0, 3))
        check(run(cv, y2, (n, h, w, 4), np.uint8, K.COLOR_YUV2RGBA_UYVY), col.bgr_from_yuv422(y2, False, 1, 0, 4))
        check(run(cv, y2, (n, h, w, 1), np.uint8, K.COLOR_YUV2GRAY_UYVY), col.gray_from_yuv422(y2, 1))
    for w in (1, 3, 5, 7, 9, 15, 17, 511, 513):  # odd widths: the one-in, one-out maps only
        a = image(orc, (2, 3, w, 3), np.uint8, 11 * w)
        check(run(cv, a, (2, 3, w, 1), np.uint8, K.COLOR_RGB2GRAY), col.gray_from_bgr(a, False))
        check(run(cv, a, (2, 3, w, 3), np.uint8, K.COLOR_BGR2HSV_FULL), col.hsv_from_bgr(a, True, True))
        g = a[..., :1].copy()
        check(run(cv, g, (2, 3, w, 3), np.uint8, K.COLOR_GRAY2BGR), col.bgr_from_gray(g))
