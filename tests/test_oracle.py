"""Pins the CPU oracle (oracle/cv_oracle.cpp) WITHOUT running the reference: closed forms, textbook
values, brute force and independent library routines (torch interpolate, numpy pad), chosen so that a
dropped term, a wrong sign/index or a swapped operand fails at least one check.

Known answers taken from the reference's texts are cited where used.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

NEAREST, LINEAR, CUBIC, AREA = 0, 1, 2, 3


# ------------------------------------------------------------------------------------------ saturate
def test_saturate_cast_known_answers(orc):
    # round-half-to-even then clamp (reference: cuda_tools/detail/SaturateCastImpl.hpp:41-50, 125;
    # known-answer style of tests/nvcv_types/cudatools_system/TestSaturateCast.cpp)
    ka = [(0.5, 0), (1.5, 2), (2.5, 2), (3.5, 4), (-0.5, 0), (-1.0, 0), (254.5, 254), (255.5, 255), (300.0, 255),
          (1e9, 255), (-1e9, 0), (127.49, 127), (float("nan"), 0)]
    for v, want in ka:
        assert orc.saturate_f32(v, np.uint8) == want, v
    for v, want in [(32767.5, 32767), (-32768.5, -32768), (-40000.0, -32768), (1.5, 2), (-1.5, -2), (-2.5, -2)]:
        assert orc.saturate_f32(v, np.int16) == want, v
    for v, want in [(65535.5, 65535), (70000.0, 65535), (-1.0, 0), (1234.5, 1234)]:
        assert orc.saturate_f32(v, np.uint16) == want, v
    xs = np.linspace(-3, 258, 4177).astype(np.float32)
    want = np.clip(np.rint(xs), 0, 255).astype(np.int64)  # np.rint is half-to-even
    got = np.array([orc.saturate_f32(float(x), np.uint8) for x in xs])
    np.testing.assert_array_equal(got, want)


# ------------------------------------------------------------------------------------------ borders
def test_border_index_maps_against_numpy_pad(orc):
    modes = {1: "edge", 2: "symmetric", 3: "wrap", 4: "reflect"}  # replicate, reflect, wrap, reflect101
    for s in range(1, 9):
        for mode, npmode in modes.items():
            if npmode == "reflect" and s == 1:
                assert all(orc.border_index(mode, c, 1) == 0 for c in range(-5, 6))
                continue
            pad = 24
            padded = np.pad(np.arange(s), pad, mode=npmode)
            for c in range(-20, 21):
                assert orc.border_index(mode, c, s) == padded[c + pad], (mode, s, c)
    # the device's closed form for REFLECT (BorderWrap.hpp:100-108) equals the golden's branchy form
    for s in range(1, 9):
        for c in range(-40, 41):
            assert orc.border_index_reflect_device(c, s) == orc.border_index(2, c, s)


# ------------------------------------------------------------------------------------------ fused op
def test_fused_identity_constant_and_crop_consistency(orc):
    rng = np.random.default_rng(1)
    src = rng.integers(0, 256, (2, 13, 17, 3), dtype=np.uint8)
    for order in (0, 1):
        out = orc.fused_rccr(src, (13, 17), (17, 13), (0, 0), LINEAR, np.float32, False, order=order)
        np.testing.assert_array_equal(out, src.astype(np.float32))  # same size, no crop: exact cast
    const = np.full((1, 40, 50, 3), 200, np.uint8)
    out = orc.fused_rccr(const, (9, 11), (23, 19), (3, 4), LINEAR, np.float32, True, scale=0.25, offset=-7.0)
    # a constant image stays constant up to a few float32 roundings of the lerp
    assert np.abs(out - (0.25 * 200 - 7.0)).max() <= 0.25 * 4 * 200 * np.finfo(np.float32).eps
    # cropping the uncropped result == asking for the crop (same per-pixel coordinates)
    full = orc.fused_rccr(src, (11, 9), (9, 11), (0, 0), LINEAR, np.float32, False)
    part = orc.fused_rccr(src, (5, 4), (9, 11), (3, 2), LINEAR, np.float32, False)
    np.testing.assert_array_equal(part, full[:, 2:7, 3:7])
    # channel reversal and planar layout are pure index permutations
    a = orc.fused_rccr(src, (7, 8), (12, 9), (1, 1), LINEAR, np.float32, False, manip=0)
    b = orc.fused_rccr(src, (7, 8), (12, 9), (1, 1), LINEAR, np.float32, True, manip=1)
    np.testing.assert_array_equal(b, a[..., ::-1].transpose(0, 3, 1, 2))


def test_fused_bilinear_matches_torch_interpolate(orc):
    # half-pixel-centre bilinear without antialias is exactly torch's align_corners=False mode
    # (edge handling by tap clamping is equivalent); differences are float rounding only.
    rng = np.random.default_rng(2)
    for (h, w, nh, nw) in [(40, 56, 17, 23), (23, 31, 50, 64), (1080 // 8, 1920 // 8, 32, 57)]:
        src = rng.integers(0, 256, (2, h, w, 3), dtype=np.uint8)
        ref = F.interpolate(torch.from_numpy(src).permute(0, 3, 1, 2).double(), size=(nh, nw), mode="bilinear",
                            align_corners=False, antialias=False).numpy()
        for order in (0, 1):
            out = orc.fused_rccr(src, (nh, nw), (nw, nh), (0, 0), LINEAR, np.float32, True, order=order)
            assert np.abs(out - ref).max() < 1e-2  # float32 coordinate rounding (|coord|*eps) times a slope of up to 255
        # the two summation orders agree far inside the parity bar
        o0 = orc.fused_rccr(src, (nh, nw), (nw, nh), (0, 0), LINEAR, np.float32, True, order=0)
        o1 = orc.fused_rccr(src, (nh, nw), (nw, nh), (0, 0), LINEAR, np.float32, True, order=1)
        assert np.abs(o0 - o1).max() <= 4 * 255 * np.finfo(np.float32).eps


def test_fused_nearest_matches_torch_nearest_exact_and_srccast(orc):
    rng = np.random.default_rng(3)
    src = rng.integers(0, 256, (1, 33, 47, 3), dtype=np.uint8)
    # sizes with no coordinate landing within float rounding of an integer
    out = orc.fused_rccr(src, (13, 19), (19, 13), (0, 0), NEAREST, np.uint8, False)
    ref = F.interpolate(torch.from_numpy(src).permute(0, 3, 1, 2).float(), size=(13, 19), mode="nearest-exact")
    np.testing.assert_array_equal(out, ref.permute(0, 2, 3, 1).numpy().astype(np.uint8))
    # srcCast rounds the interpolated value to u8 (half-to-even) before scaling
    lin = orc.fused_rccr(src, (13, 19), (19, 13), (0, 0), LINEAR, np.float32, False, scale=1.0, src_cast=False)
    cast = orc.fused_rccr(src, (13, 19), (19, 13), (0, 0), LINEAR, np.float32, False, scale=1.0, src_cast=True)
    np.testing.assert_array_equal(cast, np.clip(np.rint(lin), 0, 255))
    u8 = orc.fused_rccr(src, (13, 19), (19, 13), (0, 0), LINEAR, np.uint8, False, scale=2.0, offset=-100.0)
    np.testing.assert_array_equal(u8, np.clip(np.rint(np.float32(2.0) * lin + np.float32(-100.0)), 0, 255))


# ------------------------------------------------------------------------------------------ resize
def test_resize_nearest_knife_edge_columns(orc):
    # 1920 -> 224: (dx+.5)*60/7 is an exact integer for dx = 3 (mod 7). The golden's float32 expression
    # floor(scaleW*(dx+0.5f)) and the reference device's pack expression floor((dx0+.5f)*s + k*s)
    # disagree on exactly these 13 columns (documented analysis of tests/cvcuda/system/ResizeUtils.cpp:195-215
    # vs src/cvcuda/priv/OpResize.cu:79-83,152-162); the oracle must follow the golden.
    w_src, w_dst = 1920, 224
    src = np.arange(w_src, dtype=np.uint16).reshape(1, 1, w_src, 1).repeat(2, axis=1)
    out = orc.resize(src, (2, w_dst), NEAREST)[0, 0, :, 0].astype(np.int64)
    s = np.float32(w_src) / np.float32(w_dst)
    dx = np.arange(w_dst)
    golden = np.minimum(np.floor(s * (dx.astype(np.float32) + np.float32(0.5))), w_src - 1).astype(np.int64)
    np.testing.assert_array_equal(out, golden)
    dx0 = (dx // 4) * 4
    k = (dx % 4).astype(np.float32)
    pack = np.floor((dx0.astype(np.float32) + np.float32(0.5)) * s + k * s).astype(np.int64)
    assert list(np.nonzero(pack != golden)[0]) == [59, 73, 101, 115, 122, 143, 150, 171, 178, 185, 199, 206, 213]
    # away from the knife edges the result is the exact rational floor
    exact = ((2 * dx + 1) * w_src) // (2 * w_dst)
    safe = (dx % 7) != 3
    np.testing.assert_array_equal(out[safe], exact[safe])


def test_resize_identity_and_constant(orc):
    rng = np.random.default_rng(4)
    for dt in (np.uint8, np.uint16, np.int16, np.float32):
        a = (rng.random((2, 9, 11, 4)) * 200).astype(dt)
        for interp in (NEAREST, LINEAR):
            for variant in (0, 1, 2):
                if dt == np.float32 and variant == 0 and interp == LINEAR:
                    continue  # the golden rounds floats to integers (known quirk of the reference's golden)
                np.testing.assert_array_equal(orc.resize(a, (9, 11), interp, variant), a)
        c = np.full((1, 20, 30, 3), 37, dt)
        for interp in (NEAREST, LINEAR, CUBIC):
            for variant in (0, 1, 2):
                out = orc.resize(c, (7, 13), interp, variant)
                assert np.abs(out.astype(np.float64) - 37).max() <= (1e-4 if dt == np.float32 else 0)


def test_resize_linear_and_cubic_match_torch(orc):
    rng = np.random.default_rng(5)
    a = rng.random((1, 64, 80, 4)).astype(np.float32)
    t = torch.from_numpy(a).permute(0, 3, 1, 2).double()
    for (h, w) in [(16, 20), (31, 37), (100, 90)]:
        ref = F.interpolate(t, size=(h, w), mode="bilinear", align_corners=False).permute(0, 2, 3, 1).numpy()
        for variant in (1, 2):
            assert np.abs(orc.resize(a, (h, w), LINEAR, variant) - ref).max() < 1e-4
        # cubic: torch uses the same Keys kernel (A = -0.75); borders differ, compare the interior only
        ref = F.interpolate(t, size=(h, w), mode="bicubic", align_corners=False).permute(0, 2, 3, 1).numpy()
        sy, sx = 64 / h, 80 / w
        m_y, m_x = int(np.ceil(3 / sy)) + 1, int(np.ceil(3 / sx)) + 1
        for variant in (1, 2):
            out = orc.resize(a, (h, w), CUBIC, variant)
            inner = (slice(None), slice(m_y, h - m_y), slice(m_x, w - m_x))
            # |.| of the device formula only matters for negative overshoot; inputs are in [0,1)
            assert np.abs(out[inner] - np.abs(ref[inner])).max() < 1e-4
    # u8: golden (double, rint) vs device (float32) within 1 LSB, the reference's own tolerance
    b = rng.integers(0, 256, (1, 50, 70, 3), dtype=np.uint8)
    for interp in (LINEAR, CUBIC):
        g = orc.resize(b, (21, 33), interp, 0).astype(np.int32)
        for variant in (1, 2):
            d = orc.resize(b, (21, 33), interp, variant).astype(np.int32)
            assert np.abs(g - d).max() <= 1


def test_resize_cubic_edge_quirk(orc):
    # the x weight is forced to zero-offset when the centre column is within the border band, the y
    # weight is not (src/cvcuda/priv/OpResize.cu:357-366): with a horizontal ramp the first output
    # columns reproduce source column 1 exactly (taps (0,1,0,0) on clamped centre 1).
    w = 40
    img = np.tile(np.arange(w, dtype=np.float32), (12, 1)).reshape(1, 12, w, 1)
    out = orc.resize(img, (12, 20), CUBIC, 1)[0, :, :, 0]
    assert np.all(out[:, 0] == 1.0)



def _box_filter_float64(src, dh, dw):
    """Area resize straight from its definition, in float64: output pixel (i, j) is the mean of the source over the
    rectangle [j * sw / dw, (j + 1) * sw / dw) x [i * sh / dh, (i + 1) * sh / dh), pixels as unit squares."""
    n, sh, sw, c = src.shape

    def overlaps(s, d):
        edges = np.arange(d + 1, dtype=np.float64) * (s / d)
        lo, hi = edges[:-1, None], edges[1:, None]
        x = np.arange(s, dtype=np.float64)[None, :]
        w = np.clip(np.minimum(x + 1, hi) - np.maximum(x, lo), 0, None)
        return w / w.sum(axis=1, keepdims=True)

    return np.einsum("iy,nyxc,jx->nijc", overlaps(sh, dh), src.astype(np.float64), overlaps(sw, dw))


def test_resize_area_fixed_point_variant(orc):
    # Variants 5 and 6 (the product library's 8-bit box filter at reductions of up to 3) against the definition of
    # the box filter in float64: never more than 1 apart, equal wherever the exact value is further than 0.03 from a
    # rounding boundary (the horizontal weights are rounded to 2^-15: 4 * 255 * 2^-16 < 0.02), and equal to the
    # exact mean for the 2x reduction (weights 2^-1, nothing rounded before the end) and for equal sizes (a copy).
    # A dropped or misplaced partial pixel, a wrong normalisation at the image's far edge or a weight table shifted
    # by one fails the first two.
    rng = np.random.default_rng(55)
    for (sw, sh, dw, dh, c) in [(97, 61, 61, 40, 3), (90, 70, 31, 24, 4), (97, 61, 61, 40, 1), (50, 40, 17, 14, 3),
                                (120, 90, 47, 31, 3), (48, 27, 20, 13, 3), (64, 36, 43, 24, 3), (11, 4, 4, 2, 3)]:
        src = rng.integers(0, 256, (2, sh, sw, c), dtype=np.uint8)
        exact = _box_filter_float64(src, dh, dw)
        for variant in (5, 6):
            got = orc.resize(src, (dh, dw), AREA, variant=variant)
            assert np.abs(got - exact).max() <= 0.5 + 0.03, (sw, sh, dw, dh, c, variant)
            clear = np.abs(exact - np.floor(exact) - 0.5) > 0.03
            np.testing.assert_array_equal(got[clear], np.rint(exact)[clear].astype(np.uint8))
    src = rng.integers(0, 256, (1, 40, 64, 3), dtype=np.uint8)
    blocks = src.astype(np.float64).reshape(1, 20, 2, 32, 2, 3)
    np.testing.assert_array_equal(orc.resize(src, (20, 32), AREA, variant=5), np.rint(blocks.mean(axis=(2, 4))).astype(np.uint8))
    np.testing.assert_array_equal(orc.resize(src, (40, 64), AREA, variant=5), src)
    const = np.full((1, 33, 70, 3), 201, np.uint8)
    assert np.unique(orc.resize(const, (14, 37), AREA, variant=5)).tolist() == [201]
    # outside the form's scales (an enlargement, a reduction beyond 3, a source of under 32 bytes per row) the
    # variants are the device formulas
    for (sw, sh, dw, dh) in [(30, 30, 60, 60), (97, 61, 13, 9), (9, 40, 5, 20)]:
        src = rng.integers(0, 256, (1, sh, sw, 3), dtype=np.uint8)
        np.testing.assert_array_equal(orc.resize(src, (dh, dw), AREA, variant=5), orc.resize(src, (dh, dw), AREA, variant=1))
        np.testing.assert_array_equal(orc.resize(src, (dh, dw), AREA, variant=6), orc.resize(src, (dh, dw), AREA, variant=2))



def test_resize_cubic_fixed_point_variant(orc):
    # Variant 7 (the product library's 8-bit bicubic resize) against the float64 golden: never more than 1 apart,
    # under 1 % of the outputs differ (the horizontal weights are rounded to 2^-14 and add up to exactly 1); constant
    # images stay constant, equal sizes copy the interior (fractions 0: weights 0, 1, 0, 0), and the hand-computed pixels of
    # test_resize_cubic_hand_weights_interior_and_border_row hold for it as for the float32 variants. Other element
    # types take the float32 device formula.
    rng = np.random.default_rng(77)
    for (sw, sh, dw, dh, c) in [(97, 61, 61, 40, 3), (64, 48, 100, 77, 3), (50, 40, 17, 14, 4), (30, 20, 45, 33, 1), (5, 4, 9, 7, 3)]:
        src = rng.integers(0, 256, (2, sh, sw, c), dtype=np.uint8)
        got = orc.resize(src, (dh, dw), CUBIC, variant=7).astype(np.int32)
        gold = orc.resize(src, (dh, dw), CUBIC, variant=0).astype(np.int32)
        assert np.abs(got - gold).max() <= 1 and (got != gold).mean() < 0.01, (sw, sh, dw, dh, c)
    src = rng.integers(0, 256, (1, 23, 31, 3), dtype=np.uint8)
    # (the reference's border band, 1 pixel in front and 3 behind, moves the centre: equal sizes copy the interior)
    np.testing.assert_array_equal(orc.resize(src, (23, 31), CUBIC, variant=7)[:, 1:-3, 1:-3], src[:, 1:-3, 1:-3])
    const = np.full((1, 19, 27, 3), 143, np.uint8)
    assert np.unique(orc.resize(const, (31, 11), CUBIC, variant=7)).tolist() == [143]
    f = rng.random((1, 12, 14, 2)).astype(np.float32)
    np.testing.assert_array_equal(orc.resize(f, (7, 9), CUBIC, variant=7), orc.resize(f, (7, 9), CUBIC, variant=1))
    # 6 x 6 -> 4 x 4: the weights of fractions 0.75 and 0.25 are multiples of 2^-8, exact in 14 bits, so every pixel is
    # the hand-computed sum rounded once (interior, the row band that keeps its fraction, the column band that drops it)
    w75 = np.array([-0.03515625, 0.26171875, 0.87890625, -0.10546875])
    w25 = w75[::-1]
    img = rng.integers(0, 256, (1, 6, 6, 1), dtype=np.uint8)
    a = img[0, :, :, 0].astype(np.float64)
    out = orc.resize(img, (4, 4), CUBIC, variant=7)[0, :, :, 0].astype(np.float64)
    for got, want in [(out[1, 1], w75 @ a[0:4, 0:4] @ w75), (out[0, 1], w25 @ a[0:4, 0:4] @ w75), (out[1, 0], w75 @ a[0:4, 1]),
                      (out[0, 0], w25 @ a[0:4, 1]), (out[3, 1], w75 @ a[2:6, 0:4] @ w75), (out[1, 3], w75 @ a[0:4, 3])]:
        assert abs(got - min(abs(want), 255.0)) <= 0.5 + 1e-3, (got, want)


def test_resize_cubic_hand_weights_interior_and_border_row(orc):
    # 6 x 6 -> 4 x 4 (scale 1.5): output index 1 maps to source 1.75 (centre 1, fraction 0.75, interior), output
    # index 0 to 0.25 (centre 0, fraction 0.25, in the border band). Keys kernel with A = -0.75, written out by hand:
    #   W(x) = 1.25|x|^3 - 2.25|x|^2 + 1 (|x| <= 1),  -0.75|x|^3 + 3.75|x|^2 - 6|x| + 3 (1 < |x| < 2)
    #   fraction 0.75: taps at distances 1.75, 0.75, 0.25, 1.25
    w75 = np.array([-0.03515625, 0.26171875, 0.87890625, -0.10546875])
    w25 = w75[::-1]  # fraction 0.25: distances 1.25, 0.25, 0.75, 1.75
    assert w75.sum() == 1.0
    rng = np.random.default_rng(21)
    img = (rng.random((1, 6, 6, 1)) * 4 + 1).astype(np.float32)
    a = img[0, :, :, 0].astype(np.float64)
    for variant in (1, 2):
        out = orc.resize(img, (4, 4), CUBIC, variant)[0, :, :, 0]
        # interior in both axes: centre (1, 1), taps rows 0..3 x columns 0..3
        assert abs(out[1, 1] - w75 @ a[0:4, 0:4] @ w75) < 1e-5
        # border band along y only (output row 0): the centre is clamped to row 1 but the fraction 0.25 is KEPT
        # (src/cvcuda/priv/OpResize.cu:357-366 zeroes the horizontal fraction only), taps rows 0..3
        assert abs(out[0, 1] - w25 @ a[0:4, 0:4] @ w75) < 1e-5
        # border band along x only (output column 0): centre clamped to column 1 AND fraction forced to 0 -> column 1
        assert abs(out[1, 0] - w75 @ a[0:4, 1]) < 1e-5
        # both: column 1 with the vertical weights of fraction 0.25
        assert abs(out[0, 0] - w25 @ a[0:4, 1]) < 1e-5
        # the far side: output index 3 maps to 4.75 (centre 4 >= 6 - 3: band), centre clamped to 3, taps 2..5
        assert abs(out[3, 1] - w75 @ a[2:6, 0:4] @ w75) < 1e-5   # vertical fraction kept
        assert abs(out[1, 3] - w75 @ a[0:4, 3]) < 1e-5           # horizontal fraction zeroed: column 3


# ------------------------------------------------------------------------------------------ NV12
def _all_triples_nv12():
    W = H = 4096
    by, bx = np.meshgrid(np.arange(H // 2), np.arange(W // 2), indexing="ij")
    blk = by * (W // 2) + bx
    U = (blk % 256).astype(np.uint8)
    V = ((blk // 256) % 256).astype(np.uint8)
    yb = (blk // 65536) * 4
    Y = np.zeros((H, W), np.uint8)
    Y[0::2, 0::2] = yb
    Y[0::2, 1::2] = yb + 1
    Y[1::2, 0::2] = yb + 2
    Y[1::2, 1::2] = yb + 3
    uv = np.zeros((H // 2, W), np.uint8)
    uv[:, 0::2] = U
    uv[:, 1::2] = V
    return np.concatenate([Y, uv])[None], Y, np.repeat(np.repeat(U, 2, 0), 2, 1), np.repeat(np.repeat(V, 2, 0), 2, 1)


def test_nv12_textbook_colours_and_exhaustive_cross_check(orc):
    # BT.601 limited-range primaries (textbook YCbCr values of pure colours)
    for (y, u, v), rgb in {(16, 128, 128): (0, 0, 0), (235, 128, 128): (255, 255, 255), (81, 90, 240): (255, 0, 0),
                           (145, 54, 34): (0, 255, 0), (41, 240, 110): (0, 0, 255)}.items():
        got = orc.yuv_to_rgb_int(y, u, v)
        assert max(abs(int(g) - w) for g, w in zip(got, rgb)) <= 1, ((y, u, v), got)
    # every (Y,U,V) in 256^3: the integer device formula stays within 2 of the reference's
    # double-precision golden (its own test tolerance, tests/cvcuda/system/TestOpCvtColor.cpp:626-646)
    nv12, Y, U, V = _all_triples_nv12()
    seen = np.zeros(1 << 24, bool)
    seen[(Y.astype(np.int64) << 16 | U.astype(np.int64) << 8 | V).ravel()] = True
    assert seen.all()
    a = orc.yuv420_to_rgb(nv12, variant=0, threads=8).astype(np.int16)
    b = orc.yuv420_to_rgb(nv12, variant=1, threads=8).astype(np.int16)
    assert np.abs(a - b).max() <= 2
    # channel order / alpha / NV21 are index permutations of the same values
    small = nv12[:, :, :64][:, list(range(32)) + list(range(4096, 4096 + 16))]
    rgb = orc.yuv420_to_rgb(small)
    np.testing.assert_array_equal(orc.yuv420_to_rgb(small, bgr=True), rgb[..., ::-1])
    rgba = orc.yuv420_to_rgb(small, dcn=4)
    np.testing.assert_array_equal(rgba[..., :3], rgb)
    assert (rgba[..., 3] == 255).all()
    swapped = small.copy()
    swapped[:, 32:, 0::2], swapped[:, 32:, 1::2] = small[:, 32:, 1::2], small[:, 32:, 0::2]
    np.testing.assert_array_equal(orc.yuv420_to_rgb(swapped, uidx=1), rgb)


def test_i420_equals_nv12_after_deinterleave(orc):
    rng = np.random.default_rng(6)
    H, W = 8, 12
    Y = rng.integers(0, 256, (H, W), dtype=np.uint8)
    U = rng.integers(0, 256, (H // 2, W // 2), dtype=np.uint8)
    V = rng.integers(0, 256, (H // 2, W // 2), dtype=np.uint8)
    uv = np.zeros((H // 2, W), np.uint8)
    uv[:, 0::2], uv[:, 1::2] = U, V
    nv12 = np.concatenate([Y, uv])[None]
    i420 = np.concatenate([Y, U.reshape(H // 4, W), V.reshape(H // 4, W)])[None]
    np.testing.assert_array_equal(orc.yuv420_to_rgb(i420, semi_planar=False), orc.yuv420_to_rgb(nv12))


# ------------------------------------------------------------------------------------------ normalize
def test_normalize_identity_broadcast_and_stddev(orc):
    rng = np.random.default_rng(7)
    for dt in (np.uint8, np.int16, np.float32):
        a = (rng.random((3, 5, 7, 3)) * 100).astype(dt)
        one = np.ones((1, 1, 1, 1), np.float32)
        np.testing.assert_array_equal(orc.normalize(a, 0 * one, one), a)
    a = rng.random((2, 4, 6, 3)).astype(np.float32)
    base = rng.random((1, 1, 1, 3)).astype(np.float32)
    scale = (rng.random((2, 4, 1, 1)) + 0.5).astype(np.float32)
    out = orc.normalize(a, base, scale, 1.5, 0.25)
    want = (a - base) * scale * np.float32(1.5) + np.float32(0.25)  # float32, left to right
    np.testing.assert_array_equal(out, want.astype(np.float32))
    out = orc.normalize(a, base, scale, 2.0, 1.0, epsilon=0.5, stddev=True)
    mul = np.float32(1.0) / np.sqrt(scale * scale + np.float32(0.5))
    np.testing.assert_array_equal(out, ((a - base) * mul * np.float32(2.0) + np.float32(1.0)).astype(np.float32))
    # u8 saturates and rounds half to even
    b = np.array([[[[10, 250, 3]]]], np.uint8)
    out = orc.normalize(b, np.zeros((1, 1, 1, 1), np.float32), np.full((1, 1, 1, 1), 1.5, np.float32), 1.0, 0.0)
    np.testing.assert_array_equal(out, np.array([[[[15, 255, 4]]]], np.uint8))  # 4.5 -> 4


# ------------------------------------------------------------------------------------------ warp
def test_invert_affine(orc):
    m = np.array([1.2, 0.3, 5.0, -0.4, 0.9, -7.0], np.float32)
    inv = orc.invert_affine(m).astype(np.float64)
    A = np.vstack([m.reshape(2, 3).astype(np.float64), [0, 0, 1]])
    B = np.vstack([inv.reshape(2, 3), [0, 0, 1]])
    assert np.abs(A @ B - np.eye(3)).max() < 1e-5
    np.testing.assert_array_equal(orc.invert_affine([1, 2, 3, 2, 4, 5]), np.zeros(6, np.float32))  # singular


def test_warp_identity_translation_borders_rotation(orc):
    rng = np.random.default_rng(8)
    src = rng.integers(0, 256, (1, 7, 9, 3), dtype=np.uint8)
    ident = [1, 0, 0, 0, 1, 0]
    for interp in (NEAREST, LINEAR, CUBIC):
        for variant in (0, 1):
            np.testing.assert_array_equal(orc.warp(src, (7, 9), ident, interp, variant=variant), src)
    # integer translation: dst(x,y) = src(x+3, y-2); outside -> border policy == numpy pad
    pads = {0: ("constant", {"constant_values": 0}), 1: ("edge", {}), 2: ("symmetric", {}), 3: ("wrap", {}),
            4: ("reflect", {})}
    for border, (mode, kw) in pads.items():
        padded = np.pad(src[0], ((12, 12), (12, 12), (0, 0)), mode=mode, **kw)
        want = padded[12 - 2:12 - 2 + 7, 12 + 3:12 + 3 + 9]
        for interp in (NEAREST, LINEAR):
            for variant in (0, 1):
                got = orc.warp(src, (7, 9), [1, 0, 3, 0, 1, -2], interp, border=border, variant=variant)[0]
                np.testing.assert_array_equal(got, want)
    # constant border takes the per-channel value
    got = orc.warp(src, (7, 9), [1, 0, 100, 0, 1, 0], NEAREST, border=0, border_value=(7, 8, 9, 0))[0]
    assert (got == np.array([7, 8, 9], np.uint8)).all()
    # 90-degree rotation with an integer matrix is an exact index permutation
    sq = rng.integers(0, 256, (1, 6, 6, 1), dtype=np.uint8)
    got = orc.warp(sq, (6, 6), [0, 1, 0, -1, 0, 5], LINEAR)[0, :, :, 0]  # src = (y, 5 - x)
    np.testing.assert_array_equal(got, np.rot90(sq[0, :, :, 0], 1).T[::-1].T if False else
                                  np.array([[sq[0, 5 - x, y, 0] for x in range(6)] for y in range(6)]))
    # half-pixel shift in x: bilinear is the mean of horizontal neighbours
    f = rng.random((1, 5, 8, 1)).astype(np.float32)
    got = orc.warp(f, (5, 7), [1, 0, 0.5, 0, 1, 0], LINEAR, variant=1)[0, :, :, 0]
    np.testing.assert_allclose(got, 0.5 * (f[0, :, :-1, 0] + f[0, :, 1:, 0]), rtol=0, atol=1e-6)


def _bilinear_float64(src, out_hw, m, border_value=0.0):
    """Bilinear sample of src[H,W,C] at the float32 coordinates of the warp, everything after the coordinates
    in float64 with exact weights; taps outside the image take border_value. Returns the unrounded sums."""
    h, w = out_hw
    m = np.asarray(m, np.float32)
    xs, ys = np.meshgrid(np.arange(w, dtype=np.float32), np.arange(h, dtype=np.float32))
    sx = (m[0] * xs + m[1] * ys + m[2]).astype(np.float64)  # float32 products and sums, as the operator forms them
    sy = (m[3] * xs + m[4] * ys + m[5]).astype(np.float64)
    x1, y1 = np.floor(sx).astype(np.int64), np.floor(sy).astype(np.int64)
    fx, fy = sx - x1, sy - y1
    H, W, C = src.shape
    pad = np.full((H + 2, W + 2, C), float(border_value))
    pad[1:-1, 1:-1] = src

    def tap(x, y):
        return pad[np.clip(y + 1, 0, H + 1), np.clip(x + 1, 0, W + 1)]

    return (tap(x1, y1) * ((1 - fx) * (1 - fy))[..., None] + tap(x1 + 1, y1) * (fx * (1 - fy))[..., None]
            + tap(x1, y1 + 1) * ((1 - fx) * fy)[..., None] + tap(x1 + 1, y1 + 1) * (fx * fy)[..., None])


def test_resize_linear_fixed_point_variant(orc):
    # variant 4 (8-bit bilinear resize: weights cut to 2^-15, four integer weights that add up to 2^15, one
    # rounding) against torch's bilinear interpolation in float64 (same half-pixel map and edge clamp): the unrounded
    # sums differ by < 0.032 + the float32 coordinate error, so the results agree wherever the exact value is clear of
    # a tie and never differ by more than 1; against the golden (variant 0): at most 1 apart, rarely different
    rng = np.random.default_rng(14)
    src = rng.integers(0, 256, (2, 37, 53, 3), dtype=np.uint8)
    for out_hw in ((23, 31), (61, 90), (37, 53), (5, 200)):
        got = orc.resize(src, out_hw, LINEAR, variant=4).astype(np.int64)
        x = torch.from_numpy(src).permute(0, 3, 1, 2).double()
        exact = F.interpolate(x, size=out_hw, mode="bilinear", align_corners=False, antialias=False)
        exact = exact.permute(0, 2, 3, 1).numpy()
        assert np.abs(got - exact).max() <= 0.5 + 0.04
        clear = np.abs(exact - np.floor(exact) - 0.5) > 0.05
        np.testing.assert_array_equal(got[clear], np.rint(exact[clear]).astype(np.int64))
        gold = orc.resize(src, out_hw, LINEAR, variant=0).astype(np.int64)
        assert np.abs(got - gold).max() <= 1 and (got != gold).mean() < 0.03
    # same size: identity; 2x reduction: the mean of each 2 x 2 block, ties to even; a constant stays constant
    np.testing.assert_array_equal(orc.resize(src, (37, 53), LINEAR, variant=4), src)
    even = src[:, :36, :52].astype(np.int64)
    blocks = even.reshape(2, 18, 2, 26, 2, 3).sum(axis=(2, 4))
    np.testing.assert_array_equal(orc.resize(src[:, :36, :52], (18, 26), LINEAR, variant=4), np.rint(blocks / 4.0))
    assert (orc.resize(np.full((1, 9, 11, 1), 131, np.uint8), (20, 7), LINEAR, variant=4) == 131).all()
    # other element types keep the float32 sum of variant 1
    u16 = rng.integers(0, 60000, (1, 20, 30, 1)).astype(np.uint16)
    np.testing.assert_array_equal(orc.resize(u16, (11, 47), LINEAR, variant=4), orc.resize(u16, (11, 47), LINEAR, variant=1))


def test_warp_linear_fixed_point_variant(orc):
    # variant 2 (8-bit pixels: 15-bit fractions, four integer weights that add up to 2^15, one rounding) against
    # an exact float64 bilinear sum at the same float32 coordinates: its unrounded sum may be off by at most
    # 4 * 255 * 2^-15 < 0.032, so it must give round(exact) wherever exact is further than that from a tie and
    # never be more than 1 away; and against the golden (variant 0): at most 1 apart, rarely different
    rng = np.random.default_rng(12)
    src = rng.integers(0, 256, (1, 61, 83, 3), dtype=np.uint8)
    t = np.deg2rad(21.0)
    fwd = [1.1 * np.cos(t), -1.1 * np.sin(t), 7.3, 1.1 * np.sin(t), 1.1 * np.cos(t), -11.9]
    m = orc.invert_affine(fwd)
    got = orc.warp(src, (70, 90), m, LINEAR, border=0, border_value=(5, 5, 5, 0), variant=2)[0].astype(np.int64)
    exact = _bilinear_float64(src[0].astype(np.float64), (70, 90), m, 5.0)
    assert np.abs(got - exact).max() <= 0.5 + 0.032
    clear = np.abs(exact - np.floor(exact) - 0.5) > 0.04
    np.testing.assert_array_equal(got[clear], np.rint(exact[clear]).astype(np.int64))
    assert clear.mean() > 0.9
    gold = orc.warp(src, (70, 90), m, LINEAR, border=0, border_value=(5, 5, 5, 0), variant=0)[0].astype(np.int64)
    assert np.abs(got - gold).max() <= 1 and (got != gold).mean() < 0.02
    # dyadic weights (quarter-step maps, as in the reference's table): nothing is rounded before the final
    # rounding, ties go to even as in the golden -> bit-equal, all borders
    for border in range(5):
        for mm in ([1, 0, 0.25, 0, 1, 0.75], [0.5, 0, 0.5, 0.25, 1, -2.5], [1, 0.75, -3, 0.5, 1, 1]):
            a = orc.warp(src, (50, 70), mm, LINEAR, border=border, border_value=(1, 2, 3, 4), variant=2)
            b = orc.warp(src, (50, 70), mm, LINEAR, border=border, border_value=(1, 2, 3, 4), variant=0)
            np.testing.assert_array_equal(a, b)
    # ties: a half-pixel shift of a two-column image whose neighbours differ by an odd number rounds to even
    pair = np.array([[[[2], [5], [4], [7]]]], np.uint8)  # means 3.5, 4.5, 5.5 -> 4, 4, 6
    got = orc.warp(pair, (1, 3), [1, 0, 0.5, 0, 1, 0], LINEAR, border=1, variant=2)[0, 0, :, 0]
    np.testing.assert_array_equal(got, [4, 4, 6])
    # other element types keep the float32 sum of variant 0
    s16 = rng.integers(-3000, 3000, (1, 20, 30, 1)).astype(np.int16)
    np.testing.assert_array_equal(orc.warp(s16, (20, 30), m, LINEAR, variant=2), orc.warp(s16, (20, 30), m, LINEAR, variant=0))


def test_warp_cubic_fixed_point_variant(orc):
    # variant 2 for CUBIC on 8-bit pixels: horizontal Catmull-Rom weights rounded to 2^-14 (sum exactly 1), exact
    # integer row sums, float32 vertical sum. Against a float64 evaluation of the same 16-tap sum with the exact
    # Catmull-Rom polynomials: the unrounded values differ by < 0.06, so the results agree wherever the exact value
    # is that far from a tie, and never differ by more than 1
    rng = np.random.default_rng(13)
    src = rng.integers(0, 256, (1, 40, 52, 3), dtype=np.uint8)
    t = np.deg2rad(-14.0)
    m = orc.invert_affine([0.93 * np.cos(t), -0.93 * np.sin(t), 3.7, 0.93 * np.sin(t), 0.93 * np.cos(t), 1.2])
    got = orc.warp(src, (44, 56), m, CUBIC, border=1, variant=2)[0].astype(np.int64)
    m32 = np.asarray(m, np.float32)
    xs, ys = np.meshgrid(np.arange(56, dtype=np.float32), np.arange(44, dtype=np.float32))
    sx = (m32[0] * xs + m32[1] * ys + m32[2]).astype(np.float64)
    sy = (m32[3] * xs + m32[4] * ys + m32[5]).astype(np.float64)

    def catmull_rom(d):  # weights of taps -1, 0, 1, 2 at fraction d (A = -0.5)
        return np.stack([((-0.5 * d + 1.0) * d - 0.5) * d, (1.5 * d - 2.5) * d * d + 1.0,
                         ((-1.5 * d + 2.0) * d + 0.5) * d, (0.5 * d - 0.5) * d * d])

    ix, iy = np.floor(sx).astype(np.int64), np.floor(sy).astype(np.int64)
    wx, wy = catmull_rom(sx - ix), catmull_rom(sy - iy)
    img = src[0].astype(np.float64)
    exact = np.zeros((44, 56, 3))
    for j in range(4):
        for i in range(4):
            tap = img[np.clip(iy + j - 1, 0, 39), np.clip(ix + i - 1, 0, 51)]  # replicate border
            exact += tap * (wx[i] * wy[j])[..., None]
    want = np.clip(np.rint(exact), 0, 255).astype(np.int64)
    assert np.abs(got - np.clip(exact, 0, 255)).max() <= 0.5 + 0.06
    clear = np.abs(exact - np.floor(exact) - 0.5) > 0.07
    np.testing.assert_array_equal(got[clear], want[clear])
    assert clear.mean() > 0.8
    dev = orc.warp(src, (44, 56), m, CUBIC, border=1, variant=1)[0].astype(np.int64)
    assert np.abs(got - dev).max() <= 1 and (got != dev).mean() < 0.05
    # whole-pixel translation: weights (0, 1, 0, 0) on both axes -> a shifted copy; a constant image stays constant
    sh = orc.warp(src, (40, 52), [1, 0, 2, 0, 1, -3], CUBIC, border=3, variant=2)[0]
    np.testing.assert_array_equal(sh, np.roll(src[0], (3, -2), axis=(0, 1)))
    const = np.full((1, 20, 20, 1), 201, np.uint8)
    assert (orc.warp(const, (20, 20), m, CUBIC, border=1, variant=2) == 201).all()


def test_warp_cubic_reproduces_quadratics(orc):
    # Catmull-Rom (A = -0.5) interpolation reproduces polynomials up to degree 2: a CUBIC warp of a quadratic image by a
    # fractional translation equals the quadratic at the shifted coordinates, both for the golden (variant 0, which
    # normalises by the weight sum) and the device formula (variant 1). With any other A (the resize's -0.75, say) the
    # second-order term is off by (A + 0.5) * f'' * t(1 - t) per axis: ~1e-3 here.
    h, w = 24, 28
    ys, xs = np.meshgrid(np.arange(h, dtype=np.float64), np.arange(w, dtype=np.float64), indexing="ij")

    def quad(x, y):
        return 0.011 * x * x - 0.007 * x * y + 0.013 * y * y + 0.05 * x - 0.03 * y + 2.0

    img = quad(xs, ys).astype(np.float32).reshape(1, h, w, 1)
    tx, ty = 0.3125, 0.6875
    for variant in (0, 1):
        out = orc.warp(img, (h, w), [1, 0, tx, 0, 1, ty], CUBIC, border=1, variant=variant)[0, :, :, 0]
        want = quad(xs + tx, ys + ty)
        inner = (slice(2, h - 3), slice(2, w - 3))
        assert np.abs(out[inner] - want[inner]).max() < 2e-5, variant


def test_warp_cubic_golden_vs_device_and_perspective(orc):
    rng = np.random.default_rng(9)
    src = rng.integers(0, 256, (2, 20, 24, 3), dtype=np.uint8)
    m = orc.invert_affine([0.9, 0.2, 1.5, -0.15, 1.1, -2.0])
    g = orc.warp(src, (20, 24), m, CUBIC, border=1, variant=0).astype(np.int32)
    d = orc.warp(src, (20, 24), m, CUBIC, border=1, variant=1).astype(np.int32)
    assert np.abs(g - d).max() <= 1  # Catmull-Rom taps; golden normalises by the weight sum (== 1)
    # a perspective matrix with last row (0,0,1) is the affine map
    a = orc.warp(src, (20, 24), m, LINEAR, border=4, variant=1)
    p = orc.warp(src, (20, 24), list(m) + [0, 0, 1], LINEAR, border=4, perspective=True, variant=1)
    np.testing.assert_array_equal(a, p)


def _homography(src_pts, dst_pts):
    """3x3 matrix H (float64, H[2,2] = 1) with H @ (x, y, 1) ~ (u, v, 1) for the four pairs (x, y) -> (u, v):
    the textbook direct linear solve."""
    A, b = [], []
    for (x, y), (u, v) in zip(src_pts, dst_pts):
        A.append([x, y, 1, 0, 0, 0, -u * x, -u * y])
        b.append(u)
        A.append([0, 0, 0, x, y, 1, -v * x, -v * y])
        b.append(v)
    h = np.linalg.solve(np.asarray(A, np.float64), np.asarray(b, np.float64))
    return np.append(h, 1.0).reshape(3, 3)


def test_warp_true_homography_against_float64_coordinates(orc):
    # Pins the projective branch (reference: src/cvcuda/priv/legacy/CvCudaLegacy.h:157-183) with a matrix whose
    # last row is not (0, 0, 1) and has m6 != m7: a dropped "coeff *" on one axis, m6 and m7 swapped or a
    # transposed matrix all fail here. The matrix maps destination pixels to source positions (what the
    # oracle takes); it is built from four corner correspondences in float64.
    W, H, w, h = 40, 32, 36, 28
    dst_corners = [(0, 0), (w - 1, 0), (w - 1, h - 1), (0, h - 1)]
    src_points = [(2, 3), (37, 1), (33, 29), (5, 24)]
    M = _homography(dst_corners, src_points)
    assert abs(M[2, 0]) > 1e-4 and abs(M[2, 1]) > 1e-4 and abs(M[2, 0] - M[2, 1]) > 1e-4
    xs, ys = np.meshgrid(np.arange(w, dtype=np.float64), np.arange(h, dtype=np.float64))
    den = M[2, 0] * xs + M[2, 1] * ys + M[2, 2]
    u = (M[0, 0] * xs + M[0, 1] * ys + M[0, 2]) / den
    v = (M[1, 0] * xs + M[1, 1] * ys + M[1, 2]) / den
    # NEAREST on an image that holds its own pixel index: the output names the pixel that was read
    index = (np.arange(H)[:, None] * W + np.arange(W)[None, :]).astype(np.float32)[None, :, :, None]
    iu, iv = np.floor(u + 0.5), np.floor(v + 0.5)
    inside = (iu >= 0) & (iu < W) & (iv >= 0) & (iv < H)
    # away from the half-integer coordinates, where float32 and float64 may round to different pixels
    safe = inside & (np.abs(u + 0.5 - np.round(u + 0.5)) > 1e-3) & (np.abs(v + 0.5 - np.round(v + 0.5)) > 1e-3)
    assert safe.mean() > 0.9
    for variant in (0, 1):
        got = orc.warp(index, (h, w), M.reshape(9), NEAREST, border=0, border_value=(-1, 0, 0, 0), perspective=True,
                       variant=variant)[0, :, :, 0]
        np.testing.assert_array_equal(got[safe], (iv * W + iu)[safe].astype(np.float32))
        # the four corners land on the stated source points
        for (x, y), (px, py) in zip(dst_corners, src_points):
            assert got[y, x] == py * W + px
    # LINEAR reproduces an image that is linear in (x, y) at the float64 coordinates
    ramp = (0.25 * np.arange(W)[None, :] + 1.5 * np.arange(H)[:, None] + 3.0).astype(np.float32)[None, :, :, None]
    well_inside = (u >= 0) & (u <= W - 1) & (v >= 0) & (v <= H - 1)
    assert well_inside.mean() > 0.9
    for variant in (0, 1):
        got = orc.warp(ramp, (h, w), M.reshape(9), LINEAR, border=1, perspective=True, variant=variant)[0, :, :, 0]
        np.testing.assert_allclose(got[well_inside], (0.25 * u + 1.5 * v + 3.0)[well_inside], rtol=0, atol=2e-3)


# ------------------------------------------------------------------------------------------ generator
def test_seeded_generators(orc):
    a = orc.fill_u8((1000,), 42)
    b = orc.fill_u8((1000,), 42)
    np.testing.assert_array_equal(a, b)
    assert a.min() < 5 and a.max() > 250
    c = orc.fill_u8((4096,), 7, 16, 235)
    assert c.min() == 16 and c.max() == 235
    f = orc.fill_f32((4096,), 3)
    assert 0.0 <= f.min() and f.max() < 1.0 and abs(f.mean() - 0.5) < 0.03
    # splitmix64 reference value: first output for seed 0 is 0xE220A8397B1DCDAF (published test vector)
    first8 = orc.fill_u8((8,), 0)
    assert int.from_bytes(bytes(first8), "little") == 0xE220A8397B1DCDAF


def test_convert_to_known_answers_and_numpy_cross_check(orc):
    # rows of the reference's own test (tests/cvcuda/system/TestOpConvertTo.cpp:119-240): value 0x10
    v = np.full((7,), 16, np.uint8)
    for variant in (0, 1):
        assert (orc.convert_to(v, np.uint8, 1.0, 1.0, variant) == 17).all()
        assert (orc.convert_to(v, np.uint8, 2.1, 2.0, variant) == 36).all()
        assert (orc.convert_to(v, np.uint8, 2.1, -1.0, variant) == 33).all()
        assert (orc.convert_to(v, np.uint16, 2.1, 2.0, variant) == 36).all()
    assert (orc.convert_to(v, np.float32, 2.1, 2.0, 1) == np.float32(2.1) * np.float32(16) + np.float32(2)).all()
    assert (orc.convert_to(v.astype(np.float32), np.float64, 2.1, 2.0, 1) == 2.1 * 16 + 2.0).all()
    # identity, saturation at both ends, ties to even, NaN
    x = np.arange(-300, 300, dtype=np.int16)
    np.testing.assert_array_equal(orc.convert_to(x, np.int16), x)
    np.testing.assert_array_equal(orc.convert_to(x, np.uint8), np.clip(x, 0, 255))
    np.testing.assert_array_equal(orc.convert_to(x, np.int8), np.clip(x, -128, 127))
    np.testing.assert_array_equal(orc.convert_to(np.array([1, 3, 5, 7], np.uint8), np.uint8, 0.5, 0.0), [0, 2, 2, 4])
    assert orc.convert_to(np.array([np.nan, 1e20, -1e20], np.float32), np.int32).tolist() == [0, 2**31 - 1, -2**31]
    # every integer target against numpy arithmetic in float32
    f = (orc.fill_f32((4096,), 5) - 0.5) * 1e5
    for dt in (np.uint8, np.int8, np.uint16, np.int16, np.int32):
        info = np.iinfo(dt)
        ref = np.clip(np.rint(np.float32(0.37) * f + np.float32(-11.5)), info.min, info.max).astype(dt)
        np.testing.assert_array_equal(orc.convert_to(f, dt, 0.37, -11.5), ref)


def test_crop_flip_normalize_closed_forms(orc):
    a = orc.fill_u8((20, 30, 3), 8)
    # identity parameters = numpy crop (+ flips), zeros beyond the rectangle
    for code, pick in [(7, lambda w: w), (1, lambda w: w[:, ::-1]), (0, lambda w: w[::-1]), (-1, lambda w: w[::-1, ::-1])]:
        r = orc.crop_flip_normalize(a, (16, 24), np.uint8, (4, 2, 20, 12), code, 0, 0.0, [0], [1])
        np.testing.assert_array_equal(r[:12, :20], pick(a[2:14, 4:24]))
        assert (r[12:] == 0).all() and (r[:, 20:] == 0).all()
    # rectangle leaving the image: numpy.pad supplies the border
    pads = {0: dict(mode="constant", constant_values=9), 1: dict(mode="edge"), 2: dict(mode="symmetric"),
            3: dict(mode="wrap"), 4: dict(mode="reflect")}
    for border, kw in pads.items():
        padded = np.pad(a, ((5, 5), (5, 5), (0, 0)), **kw)
        r = orc.crop_flip_normalize(a, (26, 36), np.uint8, (-3, -4, 36, 26), 2, border, 9.0, [0], [1])
        np.testing.assert_array_equal(r, padded[1:27, 2:38])
    # normalisation arithmetic against numpy float32, scalar and per-channel, stddev mode
    base, scale = np.array([10.5, 20.25, 3.0], np.float32), np.array([0.5, 0.25, 2.0], np.float32)
    x = a[2:14, 4:24].astype(np.float32)
    r = orc.crop_flip_normalize(a, (12, 20), np.float32, (4, 2, 20, 12), 2, 0, 0.0, base, scale, 1.5, -2.0)
    np.testing.assert_array_equal(r, (x - base) * scale * np.float32(1.5) + np.float32(-2.0))
    r = orc.crop_flip_normalize(a, (12, 20), np.float32, (4, 2, 20, 12), 2, 0, 0.0, base, scale, 1.0, 0.0, 0.01, True)
    mul = np.float32(1) / np.sqrt(scale * scale + np.float32(0.01))
    np.testing.assert_array_equal(r, (x - base) * mul * np.float32(1.0) + np.float32(0.0))
    r8 = orc.crop_flip_normalize(a, (12, 20), np.int8, (4, 2, 20, 12), 2, 0, 0.0, [128], [1])
    np.testing.assert_array_equal(r8, np.clip(a[2:14, 4:24].astype(np.int32) - 128, -128, 127))


def test_resize_area_closed_forms(orc):
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, (1, 24, 36, 3), dtype=np.uint8)
    # integer factors: the plain block mean
    for fy, fx in ((2, 2), (3, 4), (1, 6)):
        ref = a.reshape(1, 24 // fy, fy, 36 // fx, fx, 3).astype(np.float64).mean(axis=(2, 4))
        for variant in (0, 1, 2, 3):  # 2 / 3: the image-batch kernel and its golden
            r = orc.resize(a, (24 // fy, 36 // fx), 3, variant=variant)
            assert np.abs(r - ref).max() <= 0.5 + 1e-4
    # same size: identity; constant image: constant (weights sum to the covered area)
    for variant in (0, 1, 2, 3):
        np.testing.assert_array_equal(orc.resize(a, (24, 36), 3, variant=variant), a)
        k = np.full((1, 31, 47, 1), 200, np.uint8)
        r = orc.resize(k, (13, 10), 3, variant=variant)
        assert np.abs(r.astype(int) - 200).max() <= 1
    # fractional factor: exact area-weighted mean computed by brute force on a 60x finer grid
    f = rng.random((1, 7, 9, 1)).astype(np.float32)
    fine = np.repeat(np.repeat(f, 60, axis=1), 60, axis=2)  # 420 x 540
    ref = fine.reshape(1, 5, 84, 6, 90, 1).mean(axis=(2, 4))  # 7 -> 5 rows, 9 -> 6 columns
    for variant in (0, 1, 2, 3):
        r = orc.resize(f, (5, 6), 3, variant=variant)
        assert np.abs(r - ref).max() < 1e-5
    # image batches, enlargement by an integer factor: every fraction is 0, so the result is pixel
    # replication -- except that the last source row and column are never reached (the reference steps
    # back to the one before and takes that with weight 1)
    for variant in (2, 3):
        for k in (2, 3):
            r = orc.resize(a, (24 * k, 36 * k), 3, variant=variant)
            iy, ix = np.minimum(np.arange(24 * k) // k, 22), np.minimum(np.arange(36 * k) // k, 34)
            np.testing.assert_array_equal(r, a[:, iy][:, :, ix])
    # enlargement by 1.5: output pixel 1 lies half-way between source pixels 0 and 1
    ramp = np.tile(np.arange(0, 80, 10, dtype=np.float32).reshape(1, 1, 8, 1), (1, 4, 1, 1))
    for variant in (2, 3):
        r = orc.resize(ramp, (6, 12), 3, variant=variant)
        assert abs(float(r[0, 0, 1, 0]) - 5.0) < 1e-4 and float(r[0, 0, 0, 0]) == 0.0


def test_committed_golden_vectors_are_reproduced(orc):
    # tests/golden/vectors.npz was written by tests/golden/make_vectors.py from the golden forms; the
    # oracle of today must still produce every array bit for bit
    import importlib.util
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("make_vectors", os.path.join(here, "golden", "make_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    stored = np.load(os.path.join(here, "golden", "vectors.npz"))
    fresh = mod.cases()
    assert sorted(stored.files) == sorted(fresh)
    for name, arr in fresh.items():
        assert stored[name].dtype == arr.dtype and stored[name].shape == arr.shape, name
        np.testing.assert_array_equal(stored[name], arr, err_msg=name)
