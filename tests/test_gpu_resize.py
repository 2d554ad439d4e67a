"""GPU parity of cvcudaResize[VarShape]Submit against the CPU oracle.

Rows are the reference's own table (tests/cvcuda/system/TestOpResize.cpp:49-91)
with seeded random inputs, plus the two benchmark configurations at full size.
Bars: NEAREST bit-exact vs the golden; LINEAR/CUBIC on integer types <= 1 LSB vs the golden (the
reference's own tolerance) and bit-exact vs the restatement of the shipped arithmetic (the float32 device
formula; for 8-bit LINEAR the 15-bit fixed-point blend, oracle variant 4); f32 cubic within 1e-4 of it.
"""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
NEAREST, LINEAR, CUBIC = 0, 1, 2


def make_input(orc, shape, dtype, seed):
    if np.dtype(dtype) == np.float32:
        return orc.fill_f32(shape, seed)
    raw = orc.fill_u8(tuple(shape) + (np.dtype(dtype).itemsize,), seed)
    return raw.view(dtype).reshape(shape)


def check(res, src, out_hw, interp, orc, varshape=False):
    golden = orc.resize(src, out_hw, interp, variant=0)
    device = orc.resize_shipped(src, out_hw, interp, varshape)
    if interp == NEAREST:
        np.testing.assert_array_equal(res, golden)
    elif res.dtype == np.float32:
        assert np.abs(res - device).max() <= 1e-4
    else:
        # The reference golden takes |.| of the bilinear sum as well (ResizeUtils.cpp:241-247) although
        # its device kernel does not (OpResize.cu:225-228); they only differ for negative signed
        # inputs, which the reference never tests. Follow the device there.
        if not (interp == LINEAR and np.issubdtype(res.dtype, np.signedinteger)):
            # 1 LSB is the reference's bound, which it only exercises on uint8. The device computes
            # source coordinates in float32, the golden in double: for 16-bit samples the coordinate
            # rounding (width * 2^-24 pixels) times the sample range exceeds 1 LSB on wide sources.
            lsb = 1 if res.dtype.itemsize == 1 else 1 + int(np.ceil(max(src.shape[1:3]) * 2.0 ** -24 * 65536 * 2))
            assert np.abs(res.astype(np.int64) - golden.astype(np.int64)).max() <= lsb
        # no FMA contraction on either side (integers for 8-bit LINEAR): the restatement is reproduced exactly
        np.testing.assert_array_equal(res, device)


TABLE = [
    (42, 48, 23, 24, NEAREST, 1, np.uint8, 4), (113, 12, 12, 36, NEAREST, 1, np.uint8, 4),
    (421, 148, 223, 124, NEAREST, 2, np.uint8, 4), (313, 212, 412, 336, NEAREST, 3, np.uint8, 4),
    (42, 40, 21, 20, LINEAR, 1, np.uint8, 4), (21, 21, 42, 42, LINEAR, 1, np.uint8, 4),
    (420, 420, 210, 210, LINEAR, 4, np.uint8, 4), (210, 210, 420, 420, LINEAR, 5, np.uint8, 4),
    (42, 40, 21, 20, CUBIC, 1, np.uint8, 4), (21, 21, 42, 42, CUBIC, 6, np.uint8, 4),
    (420, 420, 420, 420, CUBIC, 2, np.uint8, 4), (420, 420, 40, 42, CUBIC, 1, np.uint8, 4),
    (1920, 1080, 640, 320, CUBIC, 2, np.uint8, 4), (1080, 1920, 720, 1280, LINEAR, 1, np.uint8, 4),
    (720, 1280, 480, 854, CUBIC, 1, np.uint8, 4), (2160, 3840, 1080, 1920, LINEAR, 1, np.uint8, 4),
    (1080, 1920, 360, 640, CUBIC, 1, np.uint8, 4),
] + [(42, 48, 23, 24, interp, 1, dt, c) for dt in (np.uint8, np.uint16, np.int16, np.float32) for c in (1, 3, 4)
     for interp in (NEAREST, LINEAR, CUBIC)]


@pytest.mark.parametrize("row", TABLE, ids=lambda r: "%dx%d-%dx%d-i%d-n%d-%s%d" % (r[:6] + (np.dtype(r[6]).name, r[7])))
def test_tensor_table(cv, orc, gpu, row):
    sw, sh, dw, dh, interp, n, dt, c = row
    src = make_input(orc, (n, sh, sw, c), dt, 0xC0FFEE01 + sw + 31 * sh + c)
    tin = cv.Tensor.from_numpy(src, "NHWC")
    tout = cv.Tensor.alloc([n, dh, dw, c], dt, "NHWC")
    cv.Resize()(None, tin, tout, interp)
    torch.cuda.synchronize()
    check(tout.numpy(), src, (dh, dw), interp, orc)


# bicubic reductions by 2x or more take the tap-major kernel (pixels of whole dwords only): ragged
# tiles, sources narrower than the 4-tap window, every staged pixel size
STAGED = [(sw, sh, dw, dh, CUBIC, n, dt, c)
          for (sw, sh, dw, dh, n) in [(131, 37, 65, 9, 2), (640, 50, 67, 13, 1), (3, 9, 1, 2, 1), (7, 5, 3, 6, 3),
                                      (1000, 20, 130, 10, 1)]
          for dt, c in [(np.uint8, 4), (np.uint16, 4), (np.int16, 4), (np.float32, 1), (np.float32, 3),
                        (np.float32, 4)]]


@pytest.mark.parametrize("row", STAGED, ids=lambda r: "%dx%d-%dx%d-i%d-n%d-%s%d" % (r[:6] + (np.dtype(r[6]).name, r[7])))
def test_tensor_cubic_reduction(cv, orc, gpu, row):
    test_tensor_table(cv, orc, gpu, row)


# 8-bit bicubic at vertical scales of 1/2 to 2 runs as strips of 16 rows per wave once the launch has 2048 strips: the
# benchmark's shape, ragged widths and heights, scale 2 exactly (every window advances by 2), 1.25, an enlargement
# beyond 2 vertically (every strip takes the row-by-row path), horizontal enlargement with vertical reduction
STRIPS = [(sw, sh, dw, dh, CUBIC, n, np.uint8, c)
          for c in (3, 4, 1)  # (one channel stays with wave patches at these sizes too)
          for (sw, sh, dw, dh, n) in [(1920, 1080, 1280, 720, 3), (1917, 1083, 1283, 719, 3), (1024, 1408, 512, 704, 8),
                                      (1600, 900, 1280, 720, 3), (640, 360, 1000, 1100, 2), (300, 1080, 700, 720, 6),
                                      # enlargements: by 1.5, by 2 exactly (the limit of the enlarging strips), by 1.2 with
                                      # ragged sizes, and equal heights (every window advances by 1)
                                      (1280, 720, 1920, 1080, 2), (640, 360, 1280, 720, 3), (1003, 601, 1201, 721, 3),
                                      (1920, 720, 1280, 720, 3)]]


@pytest.mark.parametrize("row", STRIPS, ids=lambda r: "%dx%d-%dx%d-i%d-n%d-%s%d" % (r[:6] + (np.dtype(r[6]).name, r[7])))
def test_tensor_cubic_u8_strips(cv, orc, gpu, row):
    test_tensor_table(cv, orc, gpu, row)


# 8-bit nearest neighbour enlarging by 1.5 or more horizontally (and not reducing vertically) runs as strips once the
# launch has 2048 of them: 1.5, 2 and 3 times, ragged sizes, mixed scales (2.5 across, 1 down: every source row once),
# and a vertical reduction with the same widths (wave patches)
NN_STRIPS = [(sw, sh, dw, dh, NEAREST, n, np.uint8, c)
             for c in (3, 1, 4)
             for (sw, sh, dw, dh, n) in [(1280, 720, 1920, 1080, 2), (640, 360, 1280, 720, 6), (427, 241, 1283, 725, 6),
                                         (512, 720, 1280, 720, 6), (512, 720, 1280, 700, 6), (9, 2000, 30, 2100, 8)]]


@pytest.mark.parametrize("row", NN_STRIPS, ids=lambda r: "%dx%d-%dx%d-i%d-n%d-%s%d" % (r[:6] + (np.dtype(r[6]).name, r[7])))
def test_tensor_nearest_u8_strips(cv, orc, gpu, row):
    test_tensor_table(cv, orc, gpu, row)


# the strip kernels on views that start at an odd byte and have an odd row pitch (their window loads take the aligned
# dwords around a pixel: nothing may be assumed of where a row starts), output bytes outside the rows untouched
@pytest.mark.parametrize("c", [3, 1, 4])
@pytest.mark.parametrize("shape", [(1531, 700, 1021, 467, LINEAR), (701, 500, 1283, 915, LINEAR), (1531, 700, 1021, 467, CUBIC),
                                   (701, 500, 1283, 915, CUBIC), (701, 500, 1283, 915, NEAREST)],
                         ids=lambda sh: "%dx%d-%dx%d-i%d" % sh)
def test_strips_on_odd_bases_and_pitches(cv, orc, gpu, shape, c):
    sw, sh, dw, dh, interp = shape
    n = 6
    src = make_input(orc, (n, sh, sw, c), np.uint8, 0xBEEF + sw + c)

    def view(w, h, fill):
        pitch, plane = w * c + 3, (w * c + 3) * h + 7
        buf = torch.full((n * plane + 64,), fill, dtype=torch.uint8, device="cuda")
        t = cv.Tensor.wrap(buf.data_ptr() + 1, [n, h, w, c], [plane, pitch, c, 1], np.uint8, "NHWC", keep=buf)
        return buf, t, torch.as_strided(buf[1:], (n, h, w, c), (plane, pitch, c, 1)), (plane, pitch)

    big_in, tin, in_view, _ = view(sw, sh, 0)
    in_view.copy_(torch.from_numpy(src).cuda())
    big_out, tout, out_view, (plane, pitch) = view(dw, dh, 0xCD)
    cv.Resize()(None, tin, tout, interp)
    torch.cuda.synchronize()
    check(out_view.cpu().numpy(), src, (dh, dw), interp, orc)
    mask = torch.ones_like(big_out, dtype=torch.bool)
    torch.as_strided(mask[1:], (n, dh, dw * c), (plane, pitch, 1)).fill_(False)
    assert bool((big_out[mask] == 0xCD).all())


# 8-bit bilinear at horizontal scales up to 2 takes the kernel in which a lane owns two columns: both
# directions, the scale limit itself, ragged widths (1 - 3 columns left over), odd heights, tiny outputs
PAIRS = [(sw, sh, dw, dh, LINEAR, n, np.uint8, c)
         for c in (3, 1, 4)
         for (sw, sh, dw, dh, n) in [(131, 37, 66, 19, 2), (100, 40, 50, 20, 1), (64, 48, 97, 71, 2), (640, 360, 431, 243, 1),
                                     (33, 9, 130, 30, 1), (5, 4, 7, 3, 3), (4, 4, 2, 2, 1), (257, 33, 129, 17, 1),
                                     (1280, 720, 1920, 1080, 1), (1920, 1080, 1280, 720, 1),
                                     # enlargements by 1.5 or more: four columns per lane; ragged widths, odd heights,
                                     # the limit itself (3 * src == 2 * dst), one wave's worth and less
                                     (100, 40, 151, 61, 2), (257, 33, 771, 99, 1), (40, 30, 61, 46, 1), (4, 4, 7, 9, 2),
                                     (640, 360, 1921, 1079, 1), (86, 20, 129, 30, 1), (171, 7, 257, 11, 1),
                                     (6, 5, 9, 8, 1), (341, 50, 1023, 75, 1)]]


@pytest.mark.parametrize("row", PAIRS, ids=lambda r: "%dx%d-%dx%d-i%d-n%d-%s%d" % (r[:6] + (np.dtype(r[6]).name, r[7])))
def test_tensor_linear_u8_pair_columns(cv, orc, gpu, row):
    test_tensor_table(cv, orc, gpu, row)


def test_output_padding_is_untouched_and_hwc_layout(cv, orc, gpu):
    src = make_input(orc, (1, 33, 47, 3), np.uint8, 5)
    tin = cv.Tensor.from_numpy(src[0], "HWC")
    tout = cv.Tensor.alloc([20, 30, 3], np.uint8, "HWC")
    d = tout.export()
    pitch = d.buffer.strides[0]
    assert pitch > 30 * 3
    raw = cv._bytes_view(d.buffer.basePtr, pitch * 20, tout)
    raw.fill_(0xAB)
    cv.Resize()(None, tin, tout, LINEAR)
    torch.cuda.synchronize()
    check(tout.numpy()[None], src, (20, 30), LINEAR, orc)
    pad = raw.view(20, pitch)[:, 30 * 3:].cpu().numpy()
    assert (pad == 0xAB).all()


def test_config1_full_size_and_knife_edge_columns(cv, orc, gpu):
    # BASELINE config 1: batch 8, u8 NHWC 3ch 1920x1080 -> 224x224; nearest bit-exact, linear <= 1 LSB.
    src = orc.fill_u8((8, 1080, 1920, 3), 0xC0FFEE01)
    tin = cv.Tensor.from_numpy(src, "NHWC")
    for interp in (NEAREST, LINEAR):
        tout = cv.Tensor.alloc([8, 224, 224, 3], np.uint8, "NHWC")
        cv.Resize()(None, tin, tout, interp)
        torch.cuda.synchronize()
        check(tout.numpy(), src, (224, 224), interp, orc)
    # a ramp image (value = column index) exposes any deviation of the nearest index on the 32
    # columns dx = 3 (mod 7) where (dx+.5)*1920/224 is an exact integer
    ramp = np.tile(np.arange(1920, dtype=np.uint16).reshape(1, 1, 1920, 1), (1, 4, 1, 1))
    tout = cv.Tensor.alloc([1, 4, 224, 1], np.uint16, "NHWC")
    cv.Resize()(None, cv.Tensor.from_numpy(ramp, "NHWC"), tout, NEAREST)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(tout.numpy(), orc.resize(ramp, (4, 224), NEAREST))


def test_config5_bicubic_f32_full_size(cv, orc, gpu):
    # BASELINE config 5: batch 16 f32 NHWC 4ch 3840x2160 -> 640x360, values in [0,1), 1e-4 abs. Every image
    # is different (one random image rolled by 5 * n columns and 3 * n rows) and all 16 go through the oracle.
    N = 16
    one = orc.fill_f32((2160, 3840, 4), 0xC0FFEE05)
    tin = cv.Tensor.alloc([N, 2160, 3840, 4], np.float32, "NHWC")
    view = tin.torch_view()
    refs = []
    for n in range(N):
        img = np.roll(one, (3 * n, 5 * n), axis=(0, 1))
        view[n].copy_(torch.from_numpy(img))
        refs.append(orc.resize(img[None], (360, 640), CUBIC, variant=1, threads=8)[0])
    tout = cv.Tensor.alloc([N, 360, 640, 4], np.float32, "NHWC")
    cv.Resize()(None, tin, tout, CUBIC)
    torch.cuda.synchronize()
    res = tout.numpy()
    for n in range(N):
        assert np.abs(res[n] - refs[n]).max() <= 1e-4, n
    assert not (res[1] == res[0]).all()


def _format_for(cv, K, dt, c):
    import cvcuda_amd._capi as capi
    kind = {np.uint8: K.DATA_KIND_UNSIGNED, np.uint16: K.DATA_KIND_UNSIGNED, np.int16: K.DATA_KIND_SIGNED,
            np.float32: K.DATA_KIND_FLOAT}[dt]
    bits = np.dtype(dt).itemsize * 8
    pack = getattr(K, "PACKING_" + "_".join("%s%d" % (n, bits) for n in "XYZW"[:c]))
    swz = [K.SWIZZLE_X000, None, K.SWIZZLE_XYZ1, K.SWIZZLE_XYZW][c - 1]
    f = C.c_uint64()
    cv.check(capi.nvcv.nvcvMakeNonColorImageFormat(C.byref(f), K.MEM_LAYOUT_PL, kind, swz, pack, 0, 0, 0,
                                                   K.ALPHA_ASSOCIATED, None))
    return f.value


@pytest.mark.parametrize("interp", [NEAREST, LINEAR, CUBIC])
@pytest.mark.parametrize("dt,c", [(np.uint8, 3), (np.uint8, 4), (np.uint8, 1), (np.uint16, 3), (np.int16, 4),
                                  (np.float32, 1), (np.float32, 4)])
def test_varshape(cv, K, orc, gpu, interp, dt, c):
    rng = np.random.default_rng(17)
    fmt = _format_for(cv, K, dt, c)
    n = 7
    bin_, bout, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
    for i in range(n):
        sw, sh = int(rng.integers(20, 300)), int(rng.integers(20, 200))
        dw, dh = int(rng.integers(10, 350)), int(rng.integers(10, 250))
        a = make_input(orc, (sh, sw, c), dt, 100 + i)
        hosts.append(a)
        bin_.push_back(cv.Image.from_numpy(a, fmt))
        o = cv.Image.alloc((dw, dh), fmt)
        outs.append(o)
        bout.push_back(o)
    cv.Resize()(None, bin_, bout, interp)
    torch.cuda.synchronize()
    for a, o in zip(hosts, outs):
        w, h = o.size
        res = o.plane_view(0, dt, c).cpu().numpy()[None]
        check(res, a[None], (h, w), interp, orc, varshape=True)


# large image batches of 8-bit bilinear resizes run in the tensor kernels' strips: mostly enlarged by 1.5 or more (wide
# tiles, with a reduced and a strongly reduced image among them), mostly reduced or slightly enlarged (narrow tiles)
@pytest.mark.parametrize("c", [3, 1, 4])
@pytest.mark.parametrize("mix", ["enlarging", "reducing"])
def test_varshape_linear_u8_strips(cv, K, orc, gpu, mix, c):
    rng = np.random.default_rng(23 + c)
    fmt = _format_for(cv, K, np.uint8, c)
    n = 16  # (2048 tiles and more of 256 x 32, respectively 128 x 16)
    bin_, bout, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
    for i in range(n):
        if mix == "enlarging":
            sw, sh = int(rng.integers(700, 900)), int(rng.integers(500, 650))
            f = [1.5, 1.9, 2.0, 3.1][i % 4] if i < n - 2 else [0.7, 0.3][i - (n - 2)]
        else:
            sw, sh = int(rng.integers(900, 1300)), int(rng.integers(500, 800))
            f = [1 / 1.5, 0.5, 0.9, 1.2, 1 / 1.51][i % 5] if i < n - 2 else [0.31, 1.6][i - (n - 2)]
        dw, dh = max(1, int(sw * f) + int(rng.integers(0, 3))), max(1, int(sh * f) + int(rng.integers(0, 3)))
        a = make_input(orc, (sh, sw, c), np.uint8, 500 + i)
        hosts.append(a)
        bin_.push_back(cv.Image.from_numpy(a, fmt))
        o = cv.Image.alloc((dw, dh), fmt)
        outs.append(o)
        bout.push_back(o)
    cv.Resize()(None, bin_, bout, LINEAR)
    torch.cuda.synchronize()
    for a, o in zip(hosts, outs):
        w, h = o.size
        res = o.plane_view(0, np.uint8, c).cpu().numpy()[None]
        check(res, a[None], (h, w), LINEAR, orc, varshape=True)


# large image batches of 8-bit nearest-neighbour enlargements of 1 and 3 channels run in the tensor kernel's strips
# (256 x 32 tiles, 2048 and more), images of other scales among them as patches
@pytest.mark.parametrize("c", [3, 1])
def test_varshape_nearest_u8_strips(cv, K, orc, gpu, c):
    rng = np.random.default_rng(61 + c)
    fmt = _format_for(cv, K, np.uint8, c)
    n = 16
    bin_, bout, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
    for i in range(n):
        sw, sh = int(rng.integers(700, 900)), int(rng.integers(500, 650))
        f = [1.5, 1.9, 2.0, 3.1][i % 4] if i < n - 2 else [0.7, 1.2][i - (n - 2)]
        dw, dh = max(1, int(sw * f) + int(rng.integers(0, 3))), max(1, int(sh * f) + int(rng.integers(0, 3)))
        a = make_input(orc, (sh, sw, c), np.uint8, 900 + i)
        hosts.append(a)
        bin_.push_back(cv.Image.from_numpy(a, fmt))
        o = cv.Image.alloc((dw, dh), fmt)
        outs.append(o)
        bout.push_back(o)
    cv.Resize()(None, bin_, bout, NEAREST)
    torch.cuda.synchronize()
    for a, o in zip(hosts, outs):
        w, h = o.size
        res = o.plane_view(0, np.uint8, c).cpu().numpy()[None]
        check(res, a[None], (h, w), NEAREST, orc, varshape=True)


# large image batches of 8-bit bicubic resizes of 3 and 4 channels run in the tensor kernels' strips (64 x 64 tiles,
# 2048 and more): reductions up to 2, enlargements up to 2, and a few images outside both among them
@pytest.mark.parametrize("c", [3, 4])
def test_varshape_cubic_u8_strips(cv, K, orc, gpu, c):
    rng = np.random.default_rng(41 + c)
    fmt = _format_for(cv, K, np.uint8, c)
    n = 16
    bin_, bout, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
    for i in range(n):
        sw, sh = int(rng.integers(600, 900)), int(rng.integers(400, 650))
        f = [1 / 1.5, 1.5, 2.0, 0.5, 1.0, 1.25][i % 6] if i < n - 2 else [0.3, 2.6][i - (n - 2)]
        dw, dh = max(1, int(sw * f) + int(rng.integers(0, 3))), max(1, int(sh * f) + int(rng.integers(0, 3)))
        a = make_input(orc, (sh, sw, c), np.uint8, 700 + i)
        hosts.append(a)
        bin_.push_back(cv.Image.from_numpy(a, fmt))
        o = cv.Image.alloc((dw, dh), fmt)
        outs.append(o)
        bout.push_back(o)
    cv.Resize()(None, bin_, bout, CUBIC)
    torch.cuda.synchronize()
    for a, o in zip(hosts, outs):
        w, h = o.size
        res = o.plane_view(0, np.uint8, c).cpu().numpy()[None]
        check(res, a[None], (h, w), CUBIC, orc, varshape=True)


AREA = 3
AREA_ROWS = [(44, 40, 22, 20, 2, np.uint8, 4), (30, 30, 20, 20, 2, np.uint8, 4), (30, 30, 60, 60, 4, np.uint8, 4),
             (1440, 2560, 1080, 1920, 1, np.uint8, 4), (720, 1280, 360, 640, 1, np.uint8, 4),
             (1440, 2560, 720, 1280, 1, np.uint8, 4), (1920, 1080, 224, 224, 2, np.uint8, 3),
             (97, 61, 13, 9, 2, np.uint16, 1), (97, 61, 13, 9, 2, np.int16, 3), (97, 61, 40, 33, 2, np.float32, 4),
             # u8x3 at horizontal scales up to 2 (one 12-byte load per source row): 1.5, fractional, exactly 2 and 1,
             # an enlargement, a mixed pair of scales, sources barely wider than the load
             (1920, 1080, 1280, 720, 1, np.uint8, 3), (97, 61, 61, 40, 2, np.uint8, 3), (64, 48, 32, 24, 2, np.uint8, 3),
             (33, 21, 33, 21, 1, np.uint8, 3), (50, 40, 75, 60, 2, np.uint8, 3), (40, 90, 31, 20, 2, np.uint8, 3),
             (4, 4, 3, 3, 1, np.uint8, 3), (5, 9, 3, 2, 2, np.uint8, 3), (640, 3, 427, 2, 1, np.uint8, 3),
             # the same form for 1- and 4-byte pixels
             (97, 61, 61, 40, 2, np.uint8, 1), (64, 48, 32, 24, 2, np.uint8, 1), (50, 40, 75, 60, 2, np.uint8, 1),
             (5, 9, 3, 2, 2, np.uint8, 1), (97, 61, 61, 40, 2, np.uint8, 4), (50, 40, 75, 60, 2, np.uint8, 4),
             (5, 9, 3, 2, 2, np.uint8, 4), (1920, 1080, 1280, 720, 1, np.uint8, 4)]


@pytest.mark.parametrize("row", AREA_ROWS, ids=lambda r: "%dx%d-%dx%d-n%d-%s%d" % (r[:5] + (np.dtype(r[5]).name, r[6])))
def test_area_tensor(cv, orc, gpu, row):
    # box-filter resize, tensors (reference rows TestOpResize.cpp:67-78 plus other types and the
    # 1080p -> 224 case): <= 1 LSB against the float64 golden, and against the restatement of the shipped
    # arithmetic (8-bit pixels at reductions of up to 3: the fixed-point form; otherwise the reference's device
    # order in float32) exactly for integers, within float rounding of the long sums for float32
    sw, sh, dw, dh, n, dt, c = row
    src = make_input(orc, (n, sh, sw, c), dt, 0xA0EA + sw + dh)
    tout = cv.Tensor.alloc([n, dh, dw, c], dt, "NHWC")
    cv.Resize()(None, cv.Tensor.from_numpy(src, "NHWC"), tout, AREA)
    torch.cuda.synchronize()
    res = tout.numpy()
    golden = orc.resize(src, (dh, dw), AREA, variant=0, threads=8)
    device = orc.resize_shipped(src, (dh, dw), AREA, threads=8)
    if dt == np.float32:
        assert np.abs(res - device).max() <= 1e-5 and np.abs(res - golden).max() <= 1e-4
    else:
        np.testing.assert_array_equal(res, device)
        # the golden's box filter and the device expression part ways on fractional enlargements (there the device
        # weights do not sum to 1); the reference's own rows hold reductions and the exact 2x enlargement
        if (sw >= dw and sh >= dh) or (dw == 2 * sw and dh == 2 * sh):
            assert np.abs(res.astype(np.int64) - golden.astype(np.int64)).max() <= 1


def test_area_sources_one_and_two_pixels_wide(cv, orc, gpu):
    # u8x3 rows shorter than the 4- and 8-byte tap loads: 1 x 1, 1 x H, 2 x 1 and W x 1 sources, every
    # interpolation (the tap loads of the last row must not be moved in front of the row)
    for (sw, sh) in ((1, 1), (1, 7), (2, 1), (2, 5), (9, 1)):
        src = make_input(orc, (2, sh, sw, 3), np.uint8, 31 * sw + sh)
        for interp in (NEAREST, LINEAR, CUBIC, AREA):
            for (dw, dh) in ((1, 1), (3, 2), (5, 9)):
                tout = cv.Tensor.alloc([2, dh, dw, 3], np.uint8, "NHWC")
                cv.Resize()(None, cv.Tensor.from_numpy(src, "NHWC"), tout, interp)
                torch.cuda.synchronize()
                device = orc.resize_shipped(src, (dh, dw), interp)
                np.testing.assert_array_equal(tout.numpy(), device, err_msg=str((sw, sh, dw, dh, interp)))


@pytest.mark.parametrize("dt,c", [(np.uint8, 4), (np.uint8, 3), (np.uint8, 1), (np.uint16, 1), (np.int16, 3), (np.float32, 4)])
def test_area_varshape(cv, K, orc, gpu, dt, c):
    # image batches run the reference's separate AREA kernel (reductions: same sums, corners last;
    # enlargements: a bilinear variant). Sizes: the reference's rows (TestOpResize.cpp:67-69) plus
    # fractional factors in both directions and mixed reduce/enlarge.
    fmt = _format_for(cv, K, dt, c)
    sizes = [(44, 40, 22, 20), (30, 30, 20, 20), (30, 30, 60, 60), (97, 61, 13, 9), (50, 70, 75, 90), (64, 48, 32, 96),
             (33, 21, 33, 21), (120, 90, 47, 31)]
    n = len(sizes)
    bin_, bout, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
    for i, (sw, sh, dw, dh) in enumerate(sizes):
        a = make_input(orc, (sh, sw, c), dt, 0xA0EA + i)
        hosts.append(a)
        bin_.push_back(cv.Image.from_numpy(a, fmt))
        o = cv.Image.alloc((dw, dh), fmt)
        outs.append(o)
        bout.push_back(o)
    cv.Resize()(None, bin_, bout, AREA)
    torch.cuda.synchronize()
    for a, o, (sw, sh, dw, dh) in zip(hosts, outs, sizes):
        res = o.plane_view(0, dt, c).cpu().numpy()[None]
        golden = orc.resize(a[None], (dh, dw), AREA, variant=3)
        device = orc.resize_shipped(a[None], (dh, dw), AREA, varshape=True)
        if dt == np.float32:
            assert np.abs(res - device).max() <= 1e-5 and np.abs(res - golden).max() <= 1e-4
        else:
            np.testing.assert_array_equal(res, device)
            # float32 source coordinates against the golden's double: a pixel whose box edge lands on an
            # integer can take a different tap, so the 1-LSB bar is required of all but a few pixels
            # (the reference's own rows have none)
            bad = np.abs(res.astype(np.int64) - golden.astype(np.int64)) > 1
            assert bad.mean() <= (0.0 if (sw, sh, dw, dh) in sizes[:3] else 0.02), (sw, sh, dw, dh, bad.mean())


# seeded random cases: 8-bit pixels of 1, 3 and 4 channels, every interpolation, scales of 0.42 to 2.4 per axis (now
# and then equal, or exactly 1/2, 2/3, 1, 1.5, 2), small and 1080p-sized images, batches below and above the sizes
# at which the strip kernels take over, as packed tensors, as views with odd leads and pitches (bytes outside the
# rows must stay untouched) and as image batches of mixed sizes
@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_scales_and_pitches(cv, K, orc, gpu, seed):
    rng = np.random.default_rng(seed)
    for it in range(36):
        c = int(rng.choice([3, 3, 4, 1]))
        interp = int(rng.choice([NEAREST, LINEAR, LINEAR, CUBIC, CUBIC, AREA]))
        kind = str(rng.choice(["tensor", "view", "varshape"]))
        fx, fy = (float(np.exp(rng.uniform(np.log(0.42), np.log(2.4)))) for _ in range(2))
        if rng.random() < 0.2:
            fy = fx
        if rng.random() < 0.1:
            fx = float(rng.choice([0.5, 1.0, 1.5, 2.0, 2 / 3]))
        if rng.random() < 0.4:
            sw, sh = int(rng.integers(600, 2300)), int(rng.integers(400, 1300))
        else:
            sw, sh = int(rng.integers(4, 700)), int(rng.integers(4, 500))
        dw, dh = max(1, int(round(sw * fx))), max(1, int(round(sh * fy)))
        n = int(np.clip(rng.choice([1, 2, 2048 * 64 * 16 // (dw * dh) + 1, 2048 * 256 * 8 // (dw * dh) + 1]), 1, 16))
        n = min(n, max(1, int(60e6 / ((sw * sh + dw * dh) * c))))
        case = "seed %d case %d: %s u8x%d interp %d %dx%d -> %dx%d n %d" % (seed, it, kind, c, interp, sw, sh, dw, dh, n)

        def compare(res, src, out_hw, varshape):
            if interp == AREA:  # (the golden's box filter parts ways with the device expression on enlargements)
                np.testing.assert_array_equal(res, orc.resize_shipped(src, out_hw, AREA, varshape), err_msg=case)
            else:
                check(res, src, out_hw, interp, orc, varshape)

        try:
            if kind == "varshape":
                fmt = _format_for(cv, K, np.uint8, c)
                bin_, bout, hosts, outs = cv.ImageBatchVarShape(n), cv.ImageBatchVarShape(n), [], []
                for i in range(n):
                    w, h = max(8, sw + int(rng.integers(-30, 30))), max(8, sh + int(rng.integers(-30, 30)))
                    gx, gy = (fx, fy) if rng.random() < 0.8 else (float(rng.uniform(0.3, 3)), float(rng.uniform(0.3, 3)))
                    hosts.append(make_input(orc, (h, w, c), np.uint8, 1000 * it + i + seed))
                    bin_.push_back(cv.Image.from_numpy(hosts[-1], fmt))
                    outs.append(cv.Image.alloc((max(1, int(w * gx)), max(1, int(h * gy))), fmt))
                    bout.push_back(outs[-1])
                cv.Resize()(None, bin_, bout, interp)
                torch.cuda.synchronize()
                for a, o in zip(hosts, outs):
                    w, h = o.size
                    compare(o.plane_view(0, np.uint8, c).cpu().numpy()[None], a[None], (h, w), True)
                continue
            src = make_input(orc, (n, sh, sw, c), np.uint8, 77 * it + seed)
            if kind == "tensor":
                tout = cv.Tensor.alloc([n, dh, dw, c], np.uint8, "NHWC")
                cv.Resize()(None, cv.Tensor.from_numpy(src, "NHWC"), tout, interp)
                torch.cuda.synchronize()
                compare(tout.numpy(), src, (dh, dw), False)
                continue

            def view(w, h, fill):
                pad, lead = int(rng.integers(0, 9)), int(rng.integers(0, 5))
                pitch = w * c + pad
                plane = pitch * h + int(rng.integers(0, 9))
                buf = torch.full((n * plane + 64,), fill, dtype=torch.uint8, device="cuda")
                t = cv.Tensor.wrap(buf.data_ptr() + lead, [n, h, w, c], [plane, pitch, c, 1], np.uint8, "NHWC", keep=buf)
                return buf, t, lead, plane, pitch

            _, tin, lead, plane, pitch = view(sw, sh, 0)
            torch.as_strided(_[lead:], (n, sh, sw, c), (plane, pitch, c, 1)).copy_(torch.from_numpy(src).cuda())
            big_out, tout, lead, plane, pitch = view(dw, dh, 0xCD)
            cv.Resize()(None, tin, tout, interp)
            torch.cuda.synchronize()
            compare(torch.as_strided(big_out[lead:], (n, dh, dw, c), (plane, pitch, c, 1)).cpu().numpy(), src, (dh, dw), False)
            mask = torch.ones_like(big_out, dtype=torch.bool)
            torch.as_strided(mask[lead:], (n, dh, dw * c), (plane, pitch, 1)).fill_(False)
            assert bool((big_out[mask] == 0xCD).all()), "bytes outside the rows written"
        except AssertionError as e:
            raise AssertionError(case + ": " + str(e)) from e


def test_negative_cases(cv, gpu):
    a = cv.Tensor.alloc([2, 8, 8, 3], np.uint8, "NHWC")
    op = cv.Resize()
    cases = [
        (cv.Tensor.alloc([2, 4, 4, 3], np.float32, "NHWC"), LINEAR),   # dtype differs
        (cv.Tensor.alloc([3, 4, 4, 3], np.uint8, "NHWC"), LINEAR),     # batch differs
        (cv.Tensor.alloc([2, 4, 4, 4], np.uint8, "NHWC"), LINEAR),     # channels differ
        (cv.Tensor.alloc([2, 3, 4, 4], np.uint8, "NCHW"), LINEAR),     # layout differs
        (cv.Tensor.alloc([2, 4, 4, 3], np.uint8, "NHWC"), 4),          # LANCZOS unsupported
    ]
    for out, interp in cases:
        with pytest.raises(cv.Error) as e:
            op(None, a, out, interp)
        assert e.value.status == 2
    with pytest.raises(cv.Error) as e:
        cv.ResizeCropConvertReformat()(None, a, a, LINEAR) if False else cv.check(
            __import__("cvcuda_amd")._capi.cvcuda.cvcudaResizeSubmit(cv.ResizeCropConvertReformat().handle, None,
                                                                     a.handle, a.handle, LINEAR))
    assert e.value.status == 9  # handle of another operator -> NOT_COMPATIBLE
