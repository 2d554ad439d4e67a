"""CPU oracle (numpy) of the per-pixel colour conversions. TEST INFRASTRUCTURE ONLY: nothing in the
product imports this file.

Each function restates the reference's device arithmetic of src/cvcuda/priv/legacy/cvt_color.cu
(integer fixed point evaluated in int64, floating point in float32 one operation at a time, so no
fused multiply-add): gray :34-43, 250-274; YUV 4:4:4 :45-62, 276-346; HSV :368-413, 436-503;
RGB -> YUV 4:2:0 :70-78, 567-615; YUV 4:2:2 :618-638, 676-759.

Parity pinning (tests/test_color_oracle.py): textbook colours (primaries, white, black, grays),
channel-order symmetry, float64 formulas of the colour spaces within 1 LSB, encode/decode round
trips, and the layout of the subsampled formats checked element by element. No function here is
"parity unpinned".
"""
import numpy as np

F = np.float32
FLT_EPSILON = F(1.1920929e-07)


def _split(a, bgr):
    """(b, g, r) planes of a [...,>=3] array in BGR or RGB order."""
    return (a[..., 0], a[..., 1], a[..., 2]) if bgr else (a[..., 2], a[..., 1], a[..., 0])


def _merge(b, g, r, bgr, dtype, alpha=None):
    ch = [b, g, r] if bgr else [r, g, b]
    if alpha is not None:
        ch.append(np.full(b.shape, alpha, dtype))
    return np.stack(ch, axis=-1).astype(dtype)


def _descale(x, n):
    return (x + (1 << (n - 1))) >> n


def _sat(v, dtype):
    info = np.iinfo(dtype)
    return np.clip(v, info.min, info.max).astype(dtype)


def _sat_f(v, dtype):
    """float32 -> integer type: round half to even, saturate."""
    info = np.iinfo(dtype)
    return np.clip(np.rint(v), info.min, info.max).astype(dtype)


def gray_from_bgr(a, bgr=True):
    b, g, r = _split(a, bgr)
    if a.dtype.kind == "f":
        return (b * F(0.114) + g * F(0.587) + r * F(0.299)).astype(np.float32)[..., None]
    b, g, r = (c.astype(np.int64) for c in (b, g, r))
    return _descale(b * 3735 + g * 19235 + r * 9798, 15).astype(a.dtype)[..., None]


def bgr_from_gray(a):
    return np.repeat(a.reshape(a.shape[:3] + (1,)), 3, axis=-1)


def yuv_from_bgr(a, bgr=True):
    b, g, r = _split(a, bgr)
    if a.dtype.kind == "f":
        y = r * F(0.299) + g * F(0.587) + b * F(0.114)
        cr = (r - y) * F(0.877) + F(0.5)
        cb = (b - y) * F(0.492) + F(0.5)
        return np.stack([y, cb, cr], axis=-1).astype(np.float32)
    delta = (int(np.iinfo(a.dtype).max) // 2 + 1) << 14
    b, g, r = (c.astype(np.int64) for c in (b, g, r))
    y = _descale(r * 4899 + g * 9617 + b * 1868, 14)
    cr = _descale((r - y) * 14369 + delta, 14)
    cb = _descale((b - y) * 8061 + delta, 14)
    return np.stack([_sat(y, a.dtype), _sat(cb, a.dtype), _sat(cr, a.dtype)], axis=-1)


def bgr_from_yuv(a, bgr=True):
    y, cb, cr = a[..., 0], a[..., 1], a[..., 2]
    if a.dtype.kind == "f":
        b = y + (cb - F(0.5)) * F(2.032)
        g = y + (cb - F(0.5)) * F(-0.395) + (cr - F(0.5)) * F(-0.581)
        r = y + (cr - F(0.5)) * F(1.140)
        return _merge(b, g, r, bgr, np.float32)
    delta = int(np.iinfo(a.dtype).max) // 2 + 1
    y, cb, cr = (c.astype(np.int64) for c in (y, cb, cr))
    b = y + _descale((cb - delta) * 33292, 14)
    g = y + _descale((cb - delta) * -6472 + (cr - delta) * -9519, 14)
    r = y + _descale((cr - delta) * 18678, 14)
    return _merge(_sat(b, a.dtype), _sat(g, a.dtype), _sat(r, a.dtype), bgr, a.dtype)


def hsv_from_bgr(a, bgr=True, full=False):
    b, g, r = _split(a, bgr)
    if a.dtype.kind == "f":
        vmin = np.minimum(r, np.minimum(g, b))
        v = np.maximum(r, np.maximum(g, b))
        diff = v - vmin
        s = diff / (np.abs(v) + FLT_EPSILON)
        d = F(60.0) / (diff + FLT_EPSILON)
        h = np.where(v == r, (g - b) * d, np.where(v == g, (b - r) * d + F(120.0), (r - g) * d + F(240.0)))
        h = np.where(h < 0, h + F(360.0), h)
        return np.stack([h, s, v], axis=-1).astype(np.float32)
    hrange = 256 if full else 180
    b, g, r = (c.astype(np.int64) for c in (b, g, r))
    vmin = np.minimum(b, np.minimum(g, r))
    v = np.maximum(b, np.maximum(g, r))
    diff = v - vmin
    with np.errstate(divide="ignore", invalid="ignore"):
        hdiv = np.where(diff == 0, 0, np.rint(F(hrange << 12) / (F(6.0) * diff.astype(np.float32)))).astype(np.int64)
        sdiv = np.where(v == 0, 0, np.rint(F(255 << 12) / v.astype(np.float32))).astype(np.int64)
    s = (diff * sdiv + (1 << 11)) >> 12
    h = np.where(v == r, g - b, np.where(v == g, b - r + 2 * diff, r - g + 4 * diff))
    h = (h * hdiv + (1 << 11)) >> 12
    h = np.where(h < 0, h + hrange, h)
    return np.stack([_sat(h, a.dtype), s.astype(a.dtype), v.astype(a.dtype)], axis=-1)


def _hsv_to_bgr_float(h, s, v):
    h = h + F(6.0) * (h < 0)
    idx = h.astype(np.int32)  # truncation; h >= 0 here
    f = h - idx.astype(np.float32)
    sector = idx % 6
    one = F(1.0)
    tab = [v, v * (one - s), v * (one - s * f), v * (one - s * (one - f))]
    lut_b, lut_g, lut_r = 0x00200311, 0x00112003, 0x00031120

    def pick(lut):
        sel = (lut >> (sector << 2)) & 0xF
        return np.choose(sel, tab)

    gray = s == 0
    return (np.where(gray, v, pick(lut_b)), np.where(gray, v, pick(lut_g)), np.where(gray, v, pick(lut_r)))


def bgr_from_hsv(a, bgr=True, full=False, dcn=3):
    if a.dtype.kind == "f":
        b, g, r = _hsv_to_bgr_float(a[..., 0] * F(6.0 / 360.0), a[..., 1], a[..., 2])
        return _merge(b, g, r, bgr, np.float32, F(1.0) if dcn == 4 else None)
    scale_h = F(6.0) / F(256.0) if full else F(6.0) / F(180.0)
    sv = F(1.0) / F(255.0)
    b, g, r = _hsv_to_bgr_float(a[..., 0].astype(np.float32) * scale_h, a[..., 1].astype(np.float32) * sv,
                                a[..., 2].astype(np.float32) * sv)
    b, g, r = (_sat_f(c * F(255.0), a.dtype) for c in (b, g, r))
    return _merge(b, g, r, bgr, a.dtype, 255 if dcn == 4 else None)


def _bgr_to_yuv420_pixel(b, g, r):
    b, g, r = (c.astype(np.int64) for c in (b, g, r))
    half = 1 << 19
    yy = 269484 * r + 528482 * g + 102760 * b + half + (16 << 20)
    uu = -155188 * r + -305135 * g + 460324 * b + half + (128 << 20)
    vv = 460324 * r + -385875 * g + -74448 * b + half + (128 << 20)
    return _sat(yy >> 20, np.uint8), _sat(uu >> 20, np.uint8), _sat(vv >> 20, np.uint8)


def yuv420_from_bgr(a, bgr=True, uidx=0, planar=False):
    """a: [N,H,W,3|4] u8 -> [N,H*3/2,W,1]; chroma of each 2x2 block comes from its top-left pixel."""
    n, h, w = a.shape[:3]
    b, g, r = _split(a, bgr)
    y, u, v = _bgr_to_yuv420_pixel(b, g, r)
    out = np.zeros((n, h * 3 // 2, w), np.uint8)
    out[:, :h] = y
    us, vs = u[:, ::2, ::2], v[:, ::2, ::2]  # [N, H/2, W/2]
    first, second = (us, vs) if uidx == 0 else (vs, us)
    if not planar:
        out[:, h:, 0::2] = first
        out[:, h:, 1::2] = second
    else:
        # each chroma plane: H/2 rows of W/2 values stored as H/4 rows of W values
        out[:, h:h + h // 4] = first.reshape(n, h // 4, w)
        out[:, h + h // 4:] = second.reshape(n, h // 4, w)
    return out[..., None]


def _yuv42x_to_bgr(y, u, v):
    y, u, v = (c.astype(np.int64) for c in (y, u, v))
    yy = np.maximum(0, y - 16) * 1220542
    uu, vv = u - 128, v - 128
    r = _sat(_descale(yy + 1673527 * vv, 20), np.uint8)
    g = _sat(_descale(yy + -852492 * vv + -409993 * uu, 20), np.uint8)
    b = _sat(_descale(yy + 2116026 * uu, 20), np.uint8)
    return b, g, r


def bgr_from_yuv422(a, bgr=True, yidx=0, uidx=0, dcn=3):
    """a: [N,H,2W,1] u8 groups of 4 bytes per 2 pixels -> [N,H,W,dcn]."""
    q = a.reshape(a.shape[0], a.shape[1], -1, 4)
    y0, y1 = q[..., yidx], q[..., yidx + 2]
    u, v = q[..., (yidx ^ 1) + uidx], q[..., (yidx ^ 1) + (uidx ^ 2)]
    px = []
    for y in (y0, y1):
        b, g, r = _yuv42x_to_bgr(y, u, v)
        px.append(_merge(b, g, r, bgr, np.uint8, 255 if dcn == 4 else None))
    out = np.stack(px, axis=3)  # [N,H,W/2,2,dcn]
    return out.reshape(a.shape[0], a.shape[1], -1, dcn)


def gray_from_yuv422(a, yidx=0):
    q = a.reshape(a.shape[0], a.shape[1], -1, 4)
    return np.stack([q[..., yidx], q[..., yidx + 2]], axis=-1).reshape(a.shape[0], a.shape[1], -1, 1)
