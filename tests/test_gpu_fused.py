"""GPU parity of cvcudaResizeCropConvertReformat[VarShape]Submit against the CPU oracle.

Rows follow the reference's own table (tests/cvcuda/system/TestOpResizeCropConvertReformat.cpp:232-329:
sizes, resize targets, crops, interpolation, scale/offset, srcCast, layouts) with its deterministic
input recipe (x+y+c)&255 (:198-221), plus seeded random inputs and the benchmark configuration.
Tolerances: nearest bit-exact; u8 output <= 1 LSB; f32 output |d| <= 1e-5*max(1,|ref|).
"""
import itertools

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NEAREST, LINEAR = 0, 1


def ramp(n, h, w):
    y, x, c = np.meshgrid(np.arange(h), np.arange(w), np.arange(3), indexing="ij")
    img = ((x + y + c) & 255).astype(np.uint8)
    return np.stack([np.roll(img, i, axis=1) for i in range(n)])


def run_tensor(cv, src, out_hw, resize_dim, crop, interp, out_dtype, planar, manip, scale, offset, src_cast,
               batch_dim=True):
    n = src.shape[0]
    tin = cv.Tensor.from_numpy(src if batch_dim else src[0], "NHWC" if batch_dim else "HWC")
    h, w = out_hw
    if planar:
        shape, layout = ([n, 3, h, w], "NCHW") if batch_dim else ([3, h, w], "CHW")
    else:
        shape, layout = ([n, h, w, 3], "NHWC") if batch_dim else ([h, w, 3], "HWC")
    tout = cv.Tensor.alloc(shape, out_dtype, layout)
    tout.torch_view().zero_()
    op = cv.ResizeCropConvertReformat()
    op(None, tin, tout, resize_dim, interp, crop, manip, scale, offset, src_cast)
    torch.cuda.synchronize()
    res = tout.numpy()
    return res if batch_dim else res[None]


def compare(res, ref, interp, out_dtype):
    assert res.shape == ref.shape
    if out_dtype == np.uint8:
        d = np.abs(res.astype(np.int32) - ref.astype(np.int32))
        assert d.max() <= (0 if interp == NEAREST else 1), "max diff %d" % d.max()
    else:
        if interp == NEAREST:
            np.testing.assert_array_equal(res, ref)
        else:
            tol = 1e-5 * np.maximum(1.0, np.abs(ref))
            bad = np.abs(res - ref) > tol
            assert not bad.any(), "max err %g at %d elements" % (np.abs(res - ref).max(), bad.sum())


# srcW, srcH, newW, newH, cropX, cropY, outW, outH, N, interp, out dtype, planar, manip, scale, offset, srcCast
ROWS = [
    (8, 8, 8, 8, 0, 0, 8, 8, 1, NEAREST, np.uint8, False, 0, 1.0, 0.0, True),
    (8, 8, 8, 8, 0, 0, 8, 8, 1, LINEAR, np.uint8, False, 0, 1.0, 0.0, True),
    (8, 8, 16, 16, 0, 0, 16, 16, 2, LINEAR, np.uint8, False, 0, 1.0, 0.0, True),
    (42, 48, 23, 24, 0, 0, 23, 24, 2, NEAREST, np.uint8, False, 0, 1.0, 0.0, True),
    (42, 40, 21, 20, 0, 0, 21, 20, 2, LINEAR, np.uint8, True, 1, 1.0, 0.0, True),
    (17, 151, 23, 191, 1, 2, 21, 185, 3, LINEAR, np.float32, True, 0, 1.0, 0.0, False),
    (353, 450, 256, 326, 16, 51, 224, 224, 3, LINEAR, np.float32, True, 1, 1 / 127.5, -1.0, False),
    (353, 450, 256, 326, 16, 51, 224, 224, 2, LINEAR, np.float32, False, 0, 1 / 255.0, 0.0, True),
    (353, 450, 256, 326, 16, 51, 224, 224, 2, NEAREST, np.float32, True, 1, 1 / 127.5, -1.0, False),
    (1080, 1920, 400, 711, 88, 243, 224, 224, 2, LINEAR, np.uint8, True, 0, 1.0, 0.0, True),
    (1920, 1080, 455, 256, 115, 16, 224, 224, 2, LINEAR, np.float32, True, 0, 1 / (255 * 0.226), -0.449 / 0.226, False),
    (1920, 1080, 455, 256, 115, 16, 224, 224, 2, NEAREST, np.uint8, False, 1, 1.0, 0.0, False),
    (640, 480, 1280, 960, 100, 50, 1000, 800, 1, LINEAR, np.float32, True, 0, 2.0, -3.0, False),
    (31, 29, 97, 93, 0, 0, 97, 93, 1, NEAREST, np.float32, False, 0, 0.5, 0.25, False),
    (1, 1, 2, 2, 0, 0, 2, 2, 2, LINEAR, np.float32, True, 0, 1.0, 0.0, False),   # images smaller than one 8-byte load
    (2, 1, 5, 3, 1, 0, 3, 3, 1, LINEAR, np.uint8, False, 1, 1.0, 0.0, True),
    (3, 1, 7, 2, 0, 0, 7, 2, 1, LINEAR, np.float32, False, 0, 1.0, 0.0, False),  # exactly 9 bytes: shifted tail load
    # interleaved 8-bit outputs whose last wave holds one column (width = 1 mod 64): its 3 bytes are a row's tail
    (130, 40, 65, 20, 0, 0, 65, 20, 2, LINEAR, np.uint8, False, 0, 1.0, 0.0, True),
    (130, 40, 140, 30, 11, 3, 129, 20, 1, NEAREST, np.uint8, False, 1, 1.0, 0.0, False),
    (6, 61, 12, 150, 8, 59, 1, 67, 1, NEAREST, np.uint8, False, 0, 2.0, -100.0, False),
    (6, 61, 12, 150, 8, 59, 1, 67, 2, LINEAR, np.uint8, False, 1, 0.5, 3.0, False),
]


@pytest.mark.parametrize("row", ROWS, ids=lambda r: "%dx%d-%dx%d-%s-%s%s" % (
    r[0], r[1], r[6], r[7], "nn" if r[9] == 0 else "lin", np.dtype(r[10]).name, "p" if r[11] else "i"))
@pytest.mark.parametrize("data", ["ramp", "random"])
def test_tensor_rows(cv, orc, gpu, row, data):
    sw, sh, nw, nh, cx, cy, ow, oh, n, interp, odt, planar, manip, scale, offset, cast = row
    src = ramp(n, sh, sw) if data == "ramp" else orc.fill_u8((n, sh, sw, 3), 0xC0FFEE00 + sw * 7 + sh)
    ref = orc.fused_rccr(src, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast, order=0)
    res = run_tensor(cv, src, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast)
    compare(res, ref, interp, odt)
    # the device-order restatement must agree with the golden-order one within the same bar
    ref1 = orc.fused_rccr(src, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast, order=1)
    compare(ref1, ref, interp, odt)


# The reference's own table, all 63 rows (tests/cvcuda/system/TestOpResizeCropConvertReformat.cpp:232-329):
# source (w, h, n), resize (w, h), interpolation, destination (w, h), crop (x, y), scale, offset, source format,
# destination format, srcCast. The formats give the channel manipulation (order differs -> REVERSE), the layout
# (a trailing p -> planar) and the output type.
REFERENCE_ROWS = [
    (8, 8, 1, 8, 8, LINEAR, 6, 6, 1, 1, 1, 0, "RGB8", "BGRf32p", False),
    (8, 8, 1, 16, 16, LINEAR, 12, 12, 2, 2, 1, 0, "RGB8", "BGRf32p", False),
    (42, 48, 1, 23, 24, LINEAR, 15, 13, 0, 0, 1, 0, "RGB8", "BGRf32p", False),
    (42, 40, 3, 21, 20, LINEAR, 17, 13, 1, 1, 1, 0, "RGB8", "BGRf32p", False),
    (21, 21, 5, 42, 42, LINEAR, 32, 32, 10, 10, 1, 0, "RGB8", "BGRf32p", False),
    (113, 12, 7, 12, 36, LINEAR, 7, 13, 3, 11, 1, 0, "RGB8", "BGRf32p", False),
    (17, 151, 7, 48, 16, LINEAR, 32, 16, 4, 0, 1, 0, "RGB8", "BGRf32p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "BGRf32p", False),
    (1080, 1920, 13, 800, 600, LINEAR, 640, 480, 101, 64, 1, 0, "RGB8", "BGRf32p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "BGRf32p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "BGR8p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "BGR8p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "RGBf32p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "RGBf32p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "RGB8p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "RGB8p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "BGR8", "RGBf32p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "BGR8", "RGBf32p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "BGR8", "RGB8p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "BGR8", "RGB8p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "BGR8", "BGRf32p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "BGR8", "BGRf32p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "BGR8", "BGR8p", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "BGR8", "BGR8p", False),
    (8, 8, 1, 8, 8, LINEAR, 6, 6, 1, 1, 1, 0, "RGB8", "BGRf32", False),
    (8, 8, 1, 16, 16, LINEAR, 12, 12, 2, 2, 1, 0, "RGB8", "BGRf32", False),
    (113, 12, 7, 12, 36, LINEAR, 7, 13, 3, 11, 1, 0, "RGB8", "BGRf32", False),
    (17, 151, 7, 48, 16, LINEAR, 32, 16, 4, 0, 1, 0, "RGB8", "BGRf32", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "BGRf32", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "BGRf32", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "BGR8", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "BGR8", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "RGBf32", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "RGBf32", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "RGB8", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "RGB8", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "RGBf32", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "RGBf32", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "RGB8", "RGB8", False),
    (1280, 960, 3, 300, 225, LINEAR, 250, 200, 15, 16, 1, 0, "RGB8", "RGB8", False),
    (8, 8, 1, 8, 8, NEAREST, 6, 6, 1, 1, 1, 0, "RGB8", "BGRf32p", False),
    (8, 8, 5, 16, 16, NEAREST, 12, 12, 2, 2, 1, 0, "RGB8", "BGRf32p", False),
    (42, 48, 1, 23, 24, NEAREST, 15, 13, 0, 0, 1, 0, "RGB8", "BGRf32p", False),
    (313, 212, 4, 412, 336, NEAREST, 412, 336, 0, 0, 1, 0, "RGB8", "BGRf32p", False),
    (1080, 1920, 13, 800, 600, NEAREST, 640, 480, 101, 64, 1, 0, "RGB8", "BGRf32p", False),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 1, 0, "RGB8", "BGRf32p", False),
    (313, 212, 4, 412, 336, NEAREST, 412, 336, 0, 0, 1, 0, "RGB8", "BGR8p", False),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 1, 0, "RGB8", "BGR8p", False),
    (313, 212, 4, 412, 336, NEAREST, 412, 336, 0, 0, 1, 0, "BGR8", "RGBf32p", False),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 1, 0, "BGR8", "RGBf32p", False),
    (313, 212, 4, 412, 336, NEAREST, 412, 336, 0, 0, 1, 0, "BGR8", "RGB8p", False),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 1, 0, "BGR8", "RGB8p", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1/127.5, -1, "BGR8", "RGBf32p", False),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 2, -255, "BGR8", "RGBf32p", False),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, -1, 255, "BGR8", "RGB8", False),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 0.5, 0, "BGR8", "RGB8p", False),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 2, 0, "BGR8", "RGB8p", False),
    (353, 450, 3, 256, 256, LINEAR, 224, 224, 16, 16, 1, 0, "BGR8", "RGBf32p", True),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1/127.5, -1, "BGR8", "RGBf32p", True),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 2, -255, "BGR8", "RGBf32p", True),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, -1, 255, "BGR8", "RGB8", True),
    (313, 212, 4, 412, 336, LINEAR, 412, 336, 0, 0, 1, 0, "BGR8", "RGB8p", True),
    (1280, 960, 3, 300, 225, NEAREST, 250, 200, 15, 16, 1, 0, "BGR8", "RGB8p", True),
]


@pytest.mark.parametrize("index", range(len(REFERENCE_ROWS)))
def test_reference_table_rows(cv, orc, gpu, index):
    sw, sh, n, nw, nh, interp, ow, oh, cx, cy, scale, offset, sfmt, dfmt, cast = REFERENCE_ROWS[index]
    odt = np.float32 if "f32" in dfmt else np.uint8
    planar, manip = dfmt.endswith("p"), int(sfmt[:3] != dfmt[:3])
    src = ramp(n, sh, sw)  # the reference test's input recipe
    ref = orc.fused_rccr(src, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast, order=0)
    res = run_tensor(cv, src, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast)
    if cast and interp == LINEAR and odt == np.float32:
        # srcCast rounds the bilinear value to 8 bits before scale and offset: where that value is a tie within
        # float32 rounding, the golden's order of summation and the kernel's round to neighbouring integers, one
        # unit of `scale` apart (the reference's own tolerance is 1 in output units, its line 437). The kernel's
        # order (oracle order 1) is reproduced to the float bar, the golden's to one unit on a handful of pixels.
        compare(res, orc.fused_rccr(src, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast,
                                    order=1), interp, odt)
        d = np.abs(res - ref)
        assert d.max() <= abs(scale) * (1 + 1e-5) and (d > 1e-5 * np.maximum(1.0, np.abs(ref))).mean() < 1e-4
    else:
        compare(res, ref, interp, odt)


def test_single_image_layouts(cv, orc, gpu):
    src = orc.fill_u8((1, 37, 53, 3), 11)
    for planar in (True, False):
        ref = orc.fused_rccr(src, (20, 30), (40, 24), (3, 2), LINEAR, np.float32, planar, 0, 0.25, 1.0, False)
        res = run_tensor(cv, src, (20, 30), (40, 24), (3, 2), LINEAR, np.float32, planar, 0, 0.25, 1.0, False,
                         batch_dim=False)
        compare(res, ref, LINEAR, np.float32)


def test_identity_and_constant_closed_forms(cv, gpu):
    # resize to the source size with no crop is an exact cast; a constant image maps to scale*k+offset
    rng = np.random.default_rng(5)
    src = rng.integers(0, 256, (2, 19, 23, 3), dtype=np.uint8)
    res = run_tensor(cv, src, (19, 23), (23, 19), (0, 0), LINEAR, np.float32, False, 0, 1.0, 0.0, False)
    np.testing.assert_array_equal(res, src.astype(np.float32))
    const = np.full((1, 64, 48, 3), 77, np.uint8)
    res = run_tensor(cv, const, (20, 20), (30, 33), (5, 6), LINEAR, np.float32, True, 0, 0.5, 3.0, False)
    assert np.abs(res - (0.5 * 77 + 3.0)).max() <= 0.5 * 4 * 77 * np.finfo(np.float32).eps


def test_pitched_unaligned_source_view(cv, orc, gpu):
    # source tensor that is a window into a larger buffer: odd base address, pitch not a multiple of 4,
    # last row ends exactly at the end of the allocation (exercises the tail path of the 8-byte loads)
    H, W = 45, 71
    pitch = W * 3 + 5
    host = orc.fill_u8((2 * H * pitch + 1,), 99)
    buf = torch.from_numpy(host).cuda()
    base = 1
    nbytes = (2 * H - 1) * pitch + W * 3
    assert base + nbytes <= buf.numel()
    view = buf[base:base + nbytes]
    tin = cv.Tensor.wrap(view.data_ptr(), [2, H, W, 3], [H * pitch, pitch, 3, 1], np.uint8, "NHWC", keep=buf)
    dense = np.zeros((2, H, W, 3), np.uint8)
    for n in range(2):
        for y in range(H):
            o = base + n * H * pitch + y * pitch
            dense[n, y] = host[o:o + W * 3].reshape(W, 3)
    tout = cv.Tensor.alloc([2, 3, 30, 40], np.float32, "NCHW")
    op = cv.ResizeCropConvertReformat()
    op(None, tin, tout, (50, 33), LINEAR, (4, 2), 0, 1.0, 0.0, False)
    torch.cuda.synchronize()
    ref = orc.fused_rccr(dense, (30, 40), (50, 33), (4, 2), LINEAR, np.float32, True)
    compare(tout.numpy(), ref, LINEAR, np.float32)


def test_varshape(cv, K, orc, gpu):
    rng = np.random.default_rng(3)
    sizes = [(int(rng.integers(60, 140)), int(rng.integers(50, 120))) for _ in range(5)]
    # (65 columns: an interleaved 8-bit row whose second wave holds the last column alone)
    for (interp, odt, planar), ow in itertools.product(((LINEAR, np.float32, True), (NEAREST, np.uint8, False),
                                                        (LINEAR, np.uint8, True), (LINEAR, np.uint8, False)), (40, 65)):
        batch = cv.ImageBatchVarShape(8)
        hosts = []
        for i, (w, h) in enumerate(sizes):
            a = orc.fill_u8((h, w, 3), 1000 + i)
            hosts.append(a)
            batch.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_RGB8))
        shape, layout = ([5, 3, 32, ow], "NCHW") if planar else ([5, 32, ow, 3], "NHWC")
        tout = cv.Tensor.alloc(shape, odt, layout)
        op = cv.ResizeCropConvertReformat()
        op(None, batch, tout, (ow + 8, 40), interp, (4, 3), 1, 0.5, 1.0, False)
        torch.cuda.synchronize()
        res = tout.numpy()
        for i, a in enumerate(hosts):
            ref = orc.fused_rccr(a[None], (32, ow), (ow + 8, 40), (4, 3), interp, odt, planar, 1, 0.5, 1.0, False)
            compare(res[i:i + 1], ref, interp, odt)


# seeded random cases: sizes from 1 pixel to 1080p-sized, resize factors 0.1 to 3, any crop of the resized image
# (1-pixel-wide outputs included), both interpolations, output types and layouts, channel order, scale / offset, the
# cast before scaling; as tensors, as views with odd leads and pitches whose last row ends the allocation, and as
# image batches. Exact against the device-order restatement; against the golden order within one unit of |scale|
# where the cast's rounding can tie, 1 LSB for 8-bit outputs and 1e-3 * max(1, |scale|) otherwise (a float32 sum in
# another order, scaled, before an offset that may cancel it).
@pytest.mark.parametrize("seed", [21, 22])
def test_random_cases(cv, K, orc, gpu, seed):
    rng = np.random.default_rng(seed)
    op = cv.ResizeCropConvertReformat()
    for it in range(120):
        if rng.random() < 0.25:
            sw, sh = int(rng.integers(500, 2000)), int(rng.integers(300, 1200))
        else:
            sw, sh = int(rng.integers(1, 300)), int(rng.integers(1, 200))
        f = float(np.exp(rng.uniform(np.log(0.1), np.log(3))))
        nw = max(2, min(1500, int(sw * f * rng.uniform(0.8, 1.25))))
        nh = max(2, min(1000, int(sh * f * rng.uniform(0.8, 1.25))))
        ow, oh = int(rng.integers(1, nw + 1)), int(rng.integers(1, nh + 1))
        cx, cy = int(rng.integers(0, nw - ow + 1)), int(rng.integers(0, nh - oh + 1))
        n = int(rng.integers(1, 5))
        interp, odt = int(rng.integers(0, 2)), [np.uint8, np.float32][int(rng.integers(0, 2))]
        planar, manip, cast = bool(rng.integers(0, 2)), int(rng.integers(0, 2)), bool(rng.integers(0, 2))
        scale, offset = [(1.0, 0.0), (1 / 127.5, -1.0), (0.5, 3.25), (-1.0, 255.0), (2.0, -100.0)][int(rng.integers(0, 5))]
        kind = str(rng.choice(["tensor", "view", "varshape"]))
        case = "seed %d case %d: %s %dx%d -> %dx%d crop (%d,%d) %dx%d n %d interp %d %s planar %d manip %d scale %g cast %d" % (
            seed, it, kind, sw, sh, nw, nh, cx, cy, ow, oh, n, interp, np.dtype(odt).name, planar, manip, scale, cast)
        tout = cv.Tensor.alloc([n, 3, oh, ow] if planar else [n, oh, ow, 3], odt, "NCHW" if planar else "NHWC")
        args = ((nw, nh), interp, (cx, cy), manip, scale, offset, cast)

        def exact(res, a):
            dev = orc.fused_rccr(a, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast, order=1)
            gold = orc.fused_rccr(a, (oh, ow), (nw, nh), (cx, cy), interp, odt, planar, manip, scale, offset, cast, order=0)
            np.testing.assert_array_equal(res, dev, err_msg=case)
            bar = 0.0 if interp == NEAREST else max(1.0, abs(scale)) * (1.0 if cast or odt == np.uint8 else 1e-3)
            assert np.abs(res.astype(np.float64) - gold.astype(np.float64)).max() <= bar, case

        if kind == "varshape":
            batch, hosts = cv.ImageBatchVarShape(n), []
            for i in range(n):
                w, h = max(1, sw + int(rng.integers(-20, 20))), max(1, sh + int(rng.integers(-20, 20)))
                hosts.append(orc.fill_u8((h, w, 3), 1000 * it + i + seed))
                batch.push_back(cv.Image.from_numpy(hosts[-1], K.IMAGE_FORMAT_RGB8))
            op(None, batch, tout, *args)
            torch.cuda.synchronize()
            res = tout.numpy()
            for i, a in enumerate(hosts):
                exact(res[i:i + 1], a[None])
            continue
        src = orc.fill_u8((n, sh, sw, 3), 31 * it + seed)
        if kind == "view":
            pad, lead = int(rng.integers(0, 9)), int(rng.integers(0, 5))
            pitch = sw * 3 + pad
            buf = torch.zeros((lead + (n * sh - 1) * pitch + sw * 3,), dtype=torch.uint8, device="cuda")
            torch.as_strided(buf[lead:], (n, sh, sw, 3), (pitch * sh, pitch, 3, 1)).copy_(torch.from_numpy(src).cuda())
            tin = cv.Tensor.wrap(buf.data_ptr() + lead, [n, sh, sw, 3], [pitch * sh, pitch, 3, 1], np.uint8, "NHWC", keep=buf)
        else:
            tin = cv.Tensor.from_numpy(src, "NHWC")
        op(None, tin, tout, *args)
        torch.cuda.synchronize()
        exact(tout.numpy(), src)


def test_benchmark_config_full_size(cv, orc, gpu):
    # BASELINE config 2 at full size: batch 64 of 1080p, every image different (one random image rolled by
    # 7 * n columns and n rows, so an image index that aliases would show), the oracle on all 64.
    N = 64
    one = orc.fill_u8((1080, 1920, 3), 0xC0FFEE02)
    src = np.stack([np.roll(one, (n, 7 * n), axis=(0, 1)) for n in range(N)])
    res = run_tensor(cv, src, (224, 224), (455, 256), (115, 16), LINEAR, np.float32, True, 0,
                     1 / (255 * 0.226), -0.449 / 0.226, False)
    ref = orc.fused_rccr(src, (224, 224), (455, 256), (115, 16), LINEAR, np.float32, True, 0,
                         1 / (255 * 0.226), -0.449 / 0.226, False, threads=8)
    compare(res, ref, LINEAR, np.float32)
    assert not (res[1] == res[0]).all()


# ---- extension: fused + per-channel normalisation in one kernel -------------------------------------
IMAGENET_MEAN, IMAGENET_STD = (0.485, 0.456, 0.406), (0.229, 0.224, 0.225)


@pytest.mark.parametrize("interp", [0, 1])
@pytest.mark.parametrize("manip", [0, 1])
def test_normalize_extension_equals_three_operator_chain(cv, K, orc, gpu, interp, manip):
    # the reference-faithful way: fused (scale 1/255, f32 NHWC) -> Normalize(STDDEV) -> Reformat(NCHW);
    # the extension must give the same bits in one pass
    src = orc.fill_u8((3, 135, 240, 3), 77)
    tin = cv.Tensor.from_numpy(src, "NHWC")
    fused, norm, reformat = cv.ResizeCropConvertReformat(), cv.Normalize(), cv.Reformat()
    t1 = cv.Tensor.alloc([3, 56, 56, 3], np.float32, "NHWC")
    t2 = cv.Tensor.alloc([3, 56, 56, 3], np.float32, "NHWC")
    t3 = cv.Tensor.alloc([3, 3, 56, 56], np.float32, "NCHW")
    fused(None, tin, t1, (114, 64), interp, (29, 4), manip, 1 / 255.0, 0.0, False)
    mean = np.asarray(IMAGENET_MEAN, np.float32).reshape(1, 1, 1, 3)
    std = np.asarray(IMAGENET_STD, np.float32).reshape(1, 1, 1, 3)
    norm(None, t1, cv.Tensor.from_numpy(mean, "NHWC"), cv.Tensor.from_numpy(std, "NHWC"), t2, 1.0, 0.0, 0.0,
         K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV)
    reformat(None, t2, t3)
    one = cv.Tensor.alloc([3, 3, 56, 56], np.float32, "NCHW")
    fused.normalized(None, tin, one, (114, 64), interp, (29, 4), IMAGENET_MEAN, IMAGENET_STD, manip, 1 / 255.0, 0.0,
                     False, 1.0, 0.0, 0.0, K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(one.numpy(), t3.numpy())
    # and against the oracle: golden fused composed with the Normalize formula
    x = orc.fused_rccr(src, (56, 56), (114, 64), (29, 4), interp, np.float32, False, manip, 1 / 255.0, 0.0, False)
    ref = orc.normalize(x, mean, std, 1.0, 0.0, 0.0, True).transpose(0, 3, 1, 2)
    assert (np.abs(one.numpy() - ref) <= 1e-5 * np.maximum(1.0, np.abs(ref))).all()


def test_normalize_extension_varshape_plain_scale_and_errors(cv, K, orc, gpu):
    rng = np.random.default_rng(3)
    n = 4
    batch, hosts = cv.ImageBatchVarShape(n), []
    for i in range(n):
        a = orc.fill_u8((int(rng.integers(60, 200)), int(rng.integers(80, 300)), 3), 500 + i)
        hosts.append(a)
        batch.push_back(cv.Image.from_numpy(a, K.IMAGE_FORMAT_RGB8))
    out = cv.Tensor.alloc([n, 3, 32, 48], np.float32, "NCHW")
    op = cv.ResizeCropConvertReformat()
    base, nscale = (10.0, 20.0, 30.0), (0.5, 0.25, 2.0)
    op.normalized(None, batch, out, (64, 40), 1, (8, 4), base, nscale, 0, 1.0, 0.0, False, 0.9, 0.1)
    torch.cuda.synchronize()
    got = out.numpy()
    for i, a in enumerate(hosts):
        x = orc.fused_rccr(a[None], (32, 48), (64, 40), (8, 4), 1, np.float32, False, 0, 1.0, 0.0, False)
        ref = orc.normalize(x, np.asarray(base, np.float32).reshape(1, 1, 1, 3),
                            np.asarray(nscale, np.float32).reshape(1, 1, 1, 3), 0.9, 0.1)[0].transpose(2, 0, 1)
        assert (np.abs(got[i] - ref) <= 1e-5 * np.maximum(1.0, np.abs(ref))).all()
    with pytest.raises(cv.Error) as e:
        op.normalized(None, batch, out, (64, 40), 1, (8, 4), base, nscale, flags=4)
    assert e.value.status == 2
    st = cv._cv.cvcudaxResizeCropConvertReformatNormalizeVarShapeSubmit(
        op.handle, cv.stream_ptr(None), batch.handle, out.handle, cv.capi.Size2D(64, 40), 1, cv.capi.Int2(8, 4), 0, 1.0,
        0.0, False, None)
    assert st == 2


def test_zero_copy_interop_torch_dlpack_cuda_array_interface(cv, orc, gpu):
    # the pipeline edge: a PyTorch-ROCm tensor in, an NCHW f32 torch tensor out, no copies on either side
    src = orc.fill_u8((2, 135, 240, 3), 31)
    t_in = torch.from_numpy(src).cuda()
    t_out = torch.empty((2, 3, 56, 56), dtype=torch.float32, device="cuda")
    op = cv.ResizeCropConvertReformat()
    ref = orc.fused_rccr(src, (56, 56), (114, 64), (29, 4), 1, np.float32, True, 0, 1 / 255.0, 0.0, False)
    for wrap_in, wrap_out in [(cv.Tensor.from_torch(t_in, "NHWC"), cv.Tensor.from_torch(t_out, "NCHW")),
                              (cv.Tensor.from_dlpack(torch.utils.dlpack.to_dlpack(t_in), "NHWC"),
                               cv.Tensor.from_dlpack(t_out, "NCHW")),
                              (cv.Tensor.from_cuda_array_interface(t_in, "NHWC"),
                               cv.Tensor.from_cuda_array_interface(t_out, "NCHW"))]:
        t_out.zero_()
        op(None, wrap_in, wrap_out, (114, 64), 1, (29, 4), 0, 1 / 255.0, 0.0, False)
        torch.cuda.synchronize()
        got = t_out.cpu().numpy()
        assert (np.abs(got - ref) <= 1e-5 * np.maximum(1.0, np.abs(ref))).all()
        assert wrap_out.export().buffer.basePtr == t_out.data_ptr()
    # and outwards: a library-allocated (pitched) tensor seen by torch through both protocols
    own = cv.Tensor.alloc([2, 56, 56, 3], np.float32, "NHWC")
    op(None, cv.Tensor.from_torch(t_in, "NHWC"), own, (114, 64), 1, (29, 4), 0, 1 / 255.0, 0.0, False)
    torch.cuda.synchronize()
    via_dlpack = torch.utils.dlpack.from_dlpack(own.to_dlpack())
    via_cai = torch.as_tensor(own, device="cuda")
    for view in (via_dlpack, via_cai):
        assert view.data_ptr() == own.export().buffer.basePtr
        assert np.abs(view.cpu().numpy().transpose(0, 3, 1, 2) - ref).max() <= 1e-5 * np.abs(ref).max()
