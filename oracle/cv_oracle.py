"""ctypes front-end of the CPU oracle (liboracle.so, built from cv_oracle.cpp by `make -C oracle`).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg, never by the product package. All functions take and return dense numpy arrays.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "cv_oracle.cpp")):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True, capture_output=True)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
    return _lib


DTYPE_CODE = {np.dtype(np.uint8): 0, np.dtype(np.int8): 1, np.dtype(np.uint16): 2, np.dtype(np.int16): 3,
              np.dtype(np.int32): 4, np.dtype(np.float32): 5, np.dtype(np.float64): 6, np.dtype(np.uint32): 8}


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _i64(v):
    return C.c_int64(int(v))


def fused_rccr(src, out_hw, resize_dim, crop_pos, interp, out_dtype=np.float32, planar=True, manip=0, scale=1.0,
               offset=0.0, src_cast=False, order=0, threads=1):
    """src: [N,H,W,3] u8. Returns [N,3,h,w] (planar) or [N,h,w,3]."""
    src = np.ascontiguousarray(src, dtype=np.uint8)
    N, H, W, Cc = src.shape
    assert Cc == 3
    h, w = out_hw
    dt = np.dtype(out_dtype)
    assert dt in (np.dtype(np.float32), np.dtype(np.uint8))
    if planar:
        dst = np.zeros((N, 3, h, w), dt)
        sn, sx, sy, sc = 3 * h * w, 1, w, h * w
    else:
        dst = np.zeros((N, h, w, 3), dt)
        sn, sx, sy, sc = 3 * h * w, 3, 3 * w, 1
    rc = lib().orc_fused_rccr(_p(src), _i64(W * 3), _i64(H * W * 3), N, W, H, _p(dst), int(dt == np.float32),
                              _i64(sn), _i64(sx), _i64(sy), _i64(sc), w, h, int(resize_dim[0]), int(resize_dim[1]),
                              int(crop_pos[0]), int(crop_pos[1]), int(interp), int(manip), C.c_float(scale),
                              C.c_float(offset), int(bool(src_cast)), int(order), int(threads))
    assert rc == 0
    return dst


def resize(src, out_hw, interp, variant=0, threads=1):
    """src: [N,H,W,C]; returns [N,h,w,C] of the same dtype."""
    src = np.ascontiguousarray(src)
    N, H, W, Cc = src.shape
    h, w = out_hw
    dst = np.zeros((N, h, w, Cc), src.dtype)
    rc = lib().orc_resize(_p(src), _i64(W * Cc), _i64(H * W * Cc), N, W, H, _p(dst), _i64(w * Cc), _i64(h * w * Cc),
                          w, h, Cc, DTYPE_CODE[src.dtype], int(interp), int(variant), int(threads))
    assert rc == 0
    return dst


def resize_shipped(src, out_hw, interp, varshape=False, threads=1):
    """The restatement of what the product library's Resize computes for this element type and interpolation:
    8-bit bilinear and bicubic are the fixed-point blends (variants 4 and 7) for tensors and image batches alike; the
    8-bit box filter
    is the fixed-point form at reductions of up to 3 and the device formula elsewhere (variants 5 and, for image
    batches, 6); everything else is the reference's device formula (variant 1; variant 2, its image-batch
    association, with varshape)."""
    if int(interp) == 1 and np.dtype(src.dtype) == np.uint8:
        variant = 4
    elif int(interp) == 2 and np.dtype(src.dtype) == np.uint8:
        variant = 7
    elif int(interp) == 3 and np.dtype(src.dtype) == np.uint8:
        variant = 6 if varshape else 5
    else:
        variant = 2 if varshape else 1
    return resize(src, out_hw, interp, variant=variant, threads=threads)


def yuv420_to_rgb(src, dcn=3, bgr=False, uidx=0, semi_planar=True, variant=0, threads=1):
    """src: [N, H*3/2, W] u8 (or with a trailing 1); returns [N,H,W,dcn] u8."""
    src = np.ascontiguousarray(src, dtype=np.uint8).reshape(src.shape[0], src.shape[1], src.shape[2])
    N, H32, W = src.shape
    H = H32 * 2 // 3
    dst = np.zeros((N, H, W, dcn), np.uint8)
    rc = lib().orc_yuv420_to_rgb(_p(src), _i64(W), _i64(H32 * W), N, W, H, _p(dst), _i64(W * dcn),
                                 _i64(H * W * dcn), dcn, 0 if bgr else 2, int(uidx), int(bool(semi_planar)),
                                 int(variant), int(threads))
    assert rc == 0
    return dst


def yuv_to_rgb_int(y, u, v):
    out = (C.c_uint8 * 3)()
    lib().orc_yuv_to_rgb_int(int(y), int(u), int(v), out)
    return out[0], out[1], out[2]


def normalize(src, base, scale, global_scale=1.0, shift=0.0, epsilon=0.0, stddev=False, threads=1):
    """src: [N,H,W,C]; base/scale: float32 [n,h,w,c] with each extent 1 or matching."""
    src = np.ascontiguousarray(src)
    base = np.ascontiguousarray(base, dtype=np.float32)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    N, H, W, Cc = src.shape
    bN, bH, bW, bC = base.shape
    sN, sH, sW, sC = scale.shape
    dst = np.zeros_like(src)
    rc = lib().orc_normalize(_p(src), _i64(W * Cc), _i64(H * W * Cc), _p(dst), _i64(W * Cc), _i64(H * W * Cc), N, W,
                             H, Cc, DTYPE_CODE[src.dtype], _p(base), _i64(bW * bC), _i64(bH * bW * bC), bN, bW, bH,
                             bC, _p(scale), _i64(sW * sC), _i64(sH * sW * sC), sN, sW, sH, sC,
                             C.c_float(global_scale), C.c_float(shift), C.c_float(epsilon), int(bool(stddev)),
                             int(threads))
    assert rc == 0
    return dst


def convert_to(src, out_dtype, alpha=1.0, beta=0.0, variant=1):
    """Element-wise saturate_cast<out_dtype>(alpha*src+beta); variant 1 = device arithmetic, 0 = float64 golden."""
    src = np.ascontiguousarray(src)
    dst = np.zeros(src.shape, out_dtype)
    lib().orc_convert_to.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int64, C.c_double, C.c_double,
                                     C.c_int]
    rc = lib().orc_convert_to(_p(src), DTYPE_CODE[src.dtype], _p(dst), DTYPE_CODE[dst.dtype], src.size, alpha, beta,
                              int(variant))
    assert rc == 0
    return dst


def crop_flip_normalize(src, out_hw, out_dtype, crop, flip, border, border_value, base, scale, global_scale=1.0,
                        shift=0.0, epsilon=0.0, stddev=False):
    """One image src [H,W,C] -> [h,w,C]; crop = (x, y, width, height); base/scale: C floats."""
    src = np.ascontiguousarray(src)
    H, W, Cc = src.shape
    h, w = out_hw
    dst = np.zeros((h, w, Cc), out_dtype)
    cr = np.asarray(crop, np.int32)
    b = np.ascontiguousarray(np.broadcast_to(np.asarray(base, np.float32).reshape(-1), (Cc,)))
    sc = np.ascontiguousarray(np.broadcast_to(np.asarray(scale, np.float32).reshape(-1), (Cc,)))
    rc = lib().orc_crop_flip_normalize(_p(src), W, H, Cc, DTYPE_CODE[src.dtype], _p(dst), w, h, DTYPE_CODE[dst.dtype],
                                       _p(cr), int(flip), int(border), C.c_float(border_value), _p(b), _p(sc),
                                       C.c_float(global_scale), C.c_float(shift), C.c_float(epsilon),
                                       int(bool(stddev)))
    assert rc == 0
    return dst


def invert_affine(m):
    m = np.ascontiguousarray(m, dtype=np.float32).reshape(6)
    out = np.zeros(6, np.float32)
    lib().orc_invert_affine(_p(m), _p(out))
    return out


def warp(src, out_hw, xform, interp, border=0, border_value=(0, 0, 0, 0), perspective=False, variant=0,
         threads=1):
    """src: [N,H,W,C]; xform: [N,6] (or [N,9]) dst->src matrices (already inverted); returns [N,h,w,C]."""
    src = np.ascontiguousarray(src)
    N, H, W, Cc = src.shape
    h, w = out_hw
    mlen = 9 if perspective else 6
    xf = np.ascontiguousarray(np.broadcast_to(np.asarray(xform, np.float32).reshape(-1, mlen), (N, mlen)))
    bv = np.asarray(border_value, np.float32).reshape(4)
    dst = np.zeros((N, h, w, Cc), src.dtype)
    rc = lib().orc_warp(_p(src), _i64(W * Cc), _i64(H * W * Cc), N, W, H, _p(dst), _i64(w * Cc), _i64(h * w * Cc), w,
                        h, Cc, DTYPE_CODE[src.dtype], _p(xf), int(bool(perspective)), int(interp), int(border),
                        _p(bv), int(variant), int(threads))
    assert rc == 0
    return dst


def saturate_f32(v, np_dtype):
    lib().orc_saturate_f32.restype = C.c_int
    return lib().orc_saturate_f32(C.c_float(v), DTYPE_CODE[np.dtype(np_dtype)])


def border_index(mode, c, s):
    return lib().orc_border_index(int(mode), int(c), int(s))


def border_index_reflect_device(c, s):
    return lib().orc_border_index_reflect_device(int(c), int(s))


def fill_u8(shape, seed, lo=0, hi=255):
    a = np.empty(shape, np.uint8)
    lib().orc_fill_u8(_p(a), _i64(a.size), C.c_uint64(seed), int(lo), int(hi))
    return a


def fill_f32(shape, seed):
    a = np.empty(shape, np.float32)
    lib().orc_fill_f32(_p(a), _i64(a.size), C.c_uint64(seed))
    return a
