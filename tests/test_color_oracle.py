"""Pins oracle/color_oracle.py (numpy restatement of the reference's per-pixel colour arithmetic) without
the reference: textbook colours, float64 definitions of the colour spaces, symmetries, round trips."""
import colorsys
import importlib.util
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def col():
    spec = importlib.util.spec_from_file_location("color_oracle", os.path.join(ROOT, "oracle", "color_oracle.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


def cube(step=5):
    v = np.arange(0, 256, step, dtype=np.uint8)
    v[-1] = 255
    b, g, r = np.meshgrid(v, v, v, indexing="ij")
    return np.stack([b, g, r], axis=-1).reshape(1, -1, len(v), 3)


def test_gray(col):
    a = cube()
    g = col.gray_from_bgr(a)
    # grays stay, weights are the BT.601 luma weights within 1 LSB of the float64 definition
    eq = np.repeat(np.arange(256, dtype=np.uint8).reshape(1, 1, 256, 1), 3, axis=-1)
    np.testing.assert_array_equal(col.gray_from_bgr(eq)[..., 0], eq[..., 0])
    ref = 0.114 * a[..., 0] + 0.587 * a[..., 1] + 0.299 * a[..., 2]
    assert np.abs(g[..., 0] - ref).max() <= 0.51
    np.testing.assert_array_equal(col.gray_from_bgr(a[..., ::-1], bgr=False), g)
    a16 = (a.astype(np.uint16) * 257)
    # 15-bit coefficients: the quantisation error grows with the range (the reference's own bound for u16 is 2)
    assert np.abs(col.gray_from_bgr(a16)[..., 0] - ref * 257).max() <= 2.0
    af = a.astype(np.float32) / 255
    assert np.abs(col.gray_from_bgr(af)[..., 0] - ref / 255).max() < 1e-6
    np.testing.assert_array_equal(col.bgr_from_gray(g), np.repeat(g, 3, axis=-1))


def test_yuv444(col):
    a = cube()
    yuv = col.yuv_from_bgr(a)
    b, g, r = (a[..., i].astype(np.float64) for i in range(3))
    y = 0.299 * r + 0.587 * g + 0.114 * b
    ref = np.stack([y, (b - y) * 0.492 + 128, (r - y) * 0.877 + 128], axis=-1)
    assert np.abs(yuv - np.clip(ref, 0, 255)).max() <= 1.0
    # white/black/gray have neutral chroma
    for v in (0, 128, 255):
        np.testing.assert_array_equal(col.yuv_from_bgr(np.full((1, 1, 1, 3), v, np.uint8))[0, 0, 0], [v, 128, 128])
    back = col.bgr_from_yuv(yuv)
    sat = (yuv == 0) | (yuv == 255)  # chroma clipped on the way in: not invertible
    ok = ~sat.any(axis=-1)
    assert np.abs(back.astype(int) - a.astype(int))[ok].max() <= 2
    np.testing.assert_array_equal(col.yuv_from_bgr(a[..., ::-1], bgr=False), yuv)
    np.testing.assert_array_equal(col.bgr_from_yuv(yuv, bgr=False), back[..., ::-1])
    af = a.astype(np.float32) / 255
    yf = col.yuv_from_bgr(af)
    assert np.abs(yf[..., 0] - y / 255).max() < 1e-6
    assert np.abs(col.bgr_from_yuv(yf) - af).max() < 2e-3  # the rounded 3-digit constants are not exact inverses
    a16 = a.astype(np.uint16) * 257
    y16 = col.yuv_from_bgr(a16)
    assert np.abs(y16[..., 0] - y * 257).max() <= 3
    ok16 = ~((y16 == 0) | (y16 == 65535)).any(axis=-1)
    assert np.abs(col.bgr_from_yuv(y16).astype(int) - a16.astype(int))[ok16].max() <= 300  # ~0.4 % like the u8 case


def test_hsv(col):
    a = cube(15)
    for full in (False, True):
        hsv = col.hsv_from_bgr(a, full=full)
        hr = 256 if full else 180
        ref = np.array([colorsys.rgb_to_hsv(p[2] / 255, p[1] / 255, p[0] / 255) for p in a.reshape(-1, 3)])
        got = hsv.reshape(-1, 3).astype(np.float64)
        dh = np.abs(got[:, 0] - ref[:, 0] * hr)
        dh = np.minimum(dh, hr - dh)  # hue wraps
        assert dh.max() <= 1.0 and np.abs(got[:, 1] - ref[:, 1] * 255).max() <= 1.0
        np.testing.assert_array_equal(got[:, 2], a.reshape(-1, 3).max(axis=1))
        back = col.bgr_from_hsv(hsv, full=full)
        assert np.abs(back.astype(int) - a.astype(int)).max() <= (4 if full else 6)  # hue quantisation
        np.testing.assert_array_equal(col.hsv_from_bgr(a[..., ::-1], bgr=False, full=full), hsv)
        rgba = col.bgr_from_hsv(hsv, bgr=False, full=full, dcn=4)
        np.testing.assert_array_equal(rgba[..., :3], back[..., ::-1])
        assert (rgba[..., 3] == 255).all()
    # textbook primaries (half-range hue: degrees / 2)
    prim = np.array([[[[0, 0, 255], [0, 255, 0], [255, 0, 0], [255, 255, 255], [0, 0, 0]]]], np.uint8)  # BGR
    np.testing.assert_array_equal(col.hsv_from_bgr(prim)[0, 0],
                                  [[0, 255, 255], [60, 255, 255], [120, 255, 255], [0, 0, 255], [0, 0, 0]])
    af = a.astype(np.float32) / 255
    hf = col.hsv_from_bgr(af)
    ref = np.array([colorsys.rgb_to_hsv(p[2], p[1], p[0]) for p in af.reshape(-1, 3).astype(np.float64)])
    got = hf.reshape(-1, 3)
    dh = np.abs(got[:, 0] - ref[:, 0] * 360)
    assert np.minimum(dh, 360 - dh).max() < 1e-2 and np.abs(got[:, 1] - ref[:, 1]).max() < 1e-5
    assert np.abs(col.bgr_from_hsv(hf) - af).max() < 1e-4


def test_yuv420_encode_layout_and_values(col):
    rng = np.random.default_rng(1)
    a = rng.integers(0, 256, (2, 8, 12, 3), dtype=np.uint8)
    b, g, r = (a[..., i].astype(np.float64) for i in range(3))
    y = 16 + (65.481 * r + 128.553 * g + 24.966 * b) / 255
    u = 128 + (-37.797 * r - 74.203 * g + 112.0 * b) / 255
    v = 128 + (112.0 * r - 93.786 * g - 18.214 * b) / 255
    nv12 = col.yuv420_from_bgr(a, bgr=True, uidx=0, planar=False)[..., 0]
    assert nv12.shape == (2, 12, 12)
    assert np.abs(nv12[:, :8] - y).max() <= 1.0
    assert np.abs(nv12[:, 8:, 0::2] - u[:, ::2, ::2]).max() <= 1.0 and np.abs(nv12[:, 8:, 1::2] - v[:, ::2, ::2]).max() <= 1.0
    nv21 = col.yuv420_from_bgr(a, bgr=True, uidx=1, planar=False)[..., 0]
    np.testing.assert_array_equal(nv21[:, 8:, 0::2], nv12[:, 8:, 1::2])
    np.testing.assert_array_equal(nv21[:, 8:, 1::2], nv12[:, 8:, 0::2])
    i420 = col.yuv420_from_bgr(a, bgr=True, uidx=0, planar=True)[..., 0]
    np.testing.assert_array_equal(i420[:, :8], nv12[:, :8])
    # chroma row k of the (H/2 x W/2) plane sits in storage row k // 2, half k % 2
    for k in range(4):
        np.testing.assert_array_equal(i420[:, 8 + k // 2, (k % 2) * 6:(k % 2) * 6 + 6], nv12[:, 8 + k, 0::2])
        np.testing.assert_array_equal(i420[:, 10 + k // 2, (k % 2) * 6:(k % 2) * 6 + 6], nv12[:, 8 + k, 1::2])
    yv12 = col.yuv420_from_bgr(a, bgr=True, uidx=1, planar=True)[..., 0]
    np.testing.assert_array_equal(yv12[:, 8:10], i420[:, 10:12])
    np.testing.assert_array_equal(col.yuv420_from_bgr(a[..., ::-1], bgr=False)[..., 0], nv12)
    # limited range end points
    for val, yy in ((0, 16), (255, 235)):
        e = col.yuv420_from_bgr(np.full((1, 2, 2, 3), val, np.uint8))[0, :, :, 0]
        assert (e[:2] == yy).all() and (e[2] == 128).all()


def test_yuv422_decode(col):
    rng = np.random.default_rng(2)
    a = rng.integers(0, 256, (2, 5, 16, 1), dtype=np.uint8)  # 8 pixels per row
    q = a.reshape(2, 5, 4, 4).astype(np.float64)

    def ref(y, u, v):
        c = np.maximum(y - 16, 0) * 1.164383
        return np.stack([c + 2.017232 * (u - 128), c - 0.391762 * (u - 128) - 0.812968 * (v - 128),
                         c + 1.596027 * (v - 128)], axis=-1)

    yuyv = col.bgr_from_yuv422(a, bgr=True, yidx=0, uidx=0)
    assert yuyv.shape == (2, 5, 8, 3)
    exp = np.stack([ref(q[..., 0], q[..., 1], q[..., 3]), ref(q[..., 2], q[..., 1], q[..., 3])], axis=3).reshape(2, 5, 8, 3)
    assert np.abs(yuyv - np.clip(exp, 0, 255)).max() <= 1.0
    uyvy = col.bgr_from_yuv422(a, bgr=True, yidx=1, uidx=0)
    exp = np.stack([ref(q[..., 1], q[..., 0], q[..., 2]), ref(q[..., 3], q[..., 0], q[..., 2])], axis=3).reshape(2, 5, 8, 3)
    assert np.abs(uyvy - np.clip(exp, 0, 255)).max() <= 1.0
    yvyu = col.bgr_from_yuv422(a, bgr=True, yidx=0, uidx=2)
    exp = np.stack([ref(q[..., 0], q[..., 3], q[..., 1]), ref(q[..., 2], q[..., 3], q[..., 1])], axis=3).reshape(2, 5, 8, 3)
    assert np.abs(yvyu - np.clip(exp, 0, 255)).max() <= 1.0
    rgba = col.bgr_from_yuv422(a, bgr=False, yidx=0, uidx=0, dcn=4)
    np.testing.assert_array_equal(rgba[..., :3], yuyv[..., ::-1])
    assert (rgba[..., 3] == 255).all()
    np.testing.assert_array_equal(col.gray_from_yuv422(a, 0)[..., 0], a[..., 0][:, :, 0::2])
    np.testing.assert_array_equal(col.gray_from_yuv422(a, 1)[..., 0], a[..., 0][:, :, 1::2])
