"""Writes tests/golden/vectors.npz: expected outputs of every operator of the path on small inputs
built from the reference tests' own recipe, value(x, y, c) = (x + y + c) & 255
(tests/cvcuda/system/TestOpResizeCropConvertReformat.cpp:198-221), computed by the CPU oracle's golden
forms. The fixture pins the oracle against drift (tests/test_oracle.py re-derives every array and
requires equality) and gives the GPU parity tests vectors that do not depend on the oracle of the
day. Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import cv_oracle as orc  # noqa: E402

NEAREST, LINEAR, CUBIC, AREA = 0, 1, 2, 3


def recipe(n, h, w, c, dtype=np.uint8, step=1):
    """(x + y + c [+ image index]) & 255, optionally scaled into the dtype's range."""
    i, y, x, ch = np.meshgrid(np.arange(n), np.arange(h), np.arange(w), np.arange(c), indexing="ij")
    v = ((x * step + y * 3 + ch * 7 + i * 11) & 255).astype(np.float64)
    if np.dtype(dtype) == np.float32:
        return (v / 255.0).astype(np.float32)
    if np.dtype(dtype).itemsize == 2:
        return (v * 257 - (32768 if np.dtype(dtype).kind == "i" else 0)).astype(dtype)
    return v.astype(dtype)


def cases():
    """name -> (function producing the expected array, description of the call)."""
    out = {}
    src = recipe(2, 54, 96, 3, step=5)
    for interp, nm in ((NEAREST, "nearest"), (LINEAR, "linear")):
        out["fused_%s_f32_nchw" % nm] = orc.fused_rccr(src, (24, 24), (46, 26), (11, 1), interp, np.float32, True, 0,
                                                       1.0 / (255 * 0.226), -0.449 / 0.226, False)
        out["fused_%s_u8_nhwc_reversed" % nm] = orc.fused_rccr(src, (24, 24), (46, 26), (11, 1), interp, np.uint8, False,
                                                               1, 1.0, 0.0, False)
    for dt, c in ((np.uint8, 3), (np.uint8, 4), (np.uint16, 1), (np.int16, 3), (np.float32, 4)):
        a = recipe(1, 27, 48, c, dt, step=5)
        for interp, nm in ((NEAREST, "nearest"), (LINEAR, "linear"), (CUBIC, "cubic"), (AREA, "area")):
            for hw, tag in (((13, 20), "down"), ((40, 70), "up")):
                # the reference's golden rounds every result to an integer (it is only used on 8-bit images):
                # float images take the float32 restatement of the device formula instead
                variant = 1 if dt == np.float32 and interp != NEAREST else 0
                out["resize_%s_%s%d_%s" % (nm, np.dtype(dt).name, c, tag)] = orc.resize(a, hw, interp, variant=variant)
                if interp == LINEAR and dt == np.uint8:
                    # the shipped 8-bit bilinear blend (15-bit fixed point), to be reproduced bit for bit
                    out["resize_linear_fixed_uint8%d_%s" % (c, tag)] = orc.resize(a, hw, interp, variant=4)
                if interp == CUBIC and dt == np.uint8:
                    # the shipped 8-bit bicubic blend (14-bit horizontal weights, integer row sums), bit for bit
                    out["resize_cubic_fixed_uint8%d_%s" % (c, tag)] = orc.resize(a, hw, interp, variant=7)
                if interp == AREA and dt == np.uint8 and tag == "down":
                    # the shipped 8-bit box filter at reductions of up to 3 (fixed-point rows), bit for bit
                    out["resize_area_fixed_uint8%d_down" % c] = orc.resize(a, hw, interp, variant=5)
    y = recipe(2, 12, 16, 1, step=9)[..., 0] // 2 + 60
    uv = recipe(2, 6, 16, 1, step=13)[..., 0] // 2 + 60
    nv = np.concatenate([y, uv], axis=1)
    for dcn in (3, 4):
        for bgr in (False, True):
            for uidx in (0, 1):
                out["yuv420sp_to_%s%d_u%d" % ("bgr" if bgr else "rgb", dcn, uidx)] = orc.yuv420_to_rgb(nv, dcn, bgr, uidx,
                                                                                                     True, variant=0)
    a = recipe(2, 9, 14, 3, step=7)
    base = np.array([[[[10.0, 20.0, 30.0]]]], np.float32)
    scale = np.array([[[[0.5, 0.25, 2.0]]]], np.float32)
    out["normalize_u8"] = orc.normalize(a, base, scale, 1.5, 3.0, 0.0, False)
    out["normalize_u8_stddev"] = orc.normalize(a, base, scale, 40.0, 100.0, 0.5, True)
    out["normalize_f32_stddev"] = orc.normalize(recipe(2, 9, 14, 3, np.float32, 7), base / 255, scale, 1.0, 0.0, 0.1, True)
    a = recipe(2, 30, 44, 3, step=5)
    for interp, nm in ((NEAREST, "nearest"), (LINEAR, "linear"), (CUBIC, "cubic")):
        for border in range(5):
            m = orc.invert_affine([0.9, -0.3, 6.0, 0.25, 1.1, -4.0])
            out["warp_affine_%s_border%d" % (nm, border)] = orc.warp(a, (30, 44), m, interp, border, (7, 8, 9, 0), False,
                                                                    variant=0)
    for border in range(5):
        # the shipped 8-bit bilinear blend (15-bit fixed point), which the kernels must reproduce bit for bit
        out["warp_affine_linear_fixed_border%d" % border] = orc.warp(a, (30, 44), m, LINEAR, border, (7, 8, 9, 0), False,
                                                                    variant=2)
    # the call of tests/golden/abi_gpu_calls.c: RGBA8, a border colour of four different values
    out["abi_warp_affine_rgba8_linear"] = orc.warp(recipe(1, 30, 44, 4, step=5), (30, 44), m, LINEAR, 0, (7, 80, 159, 250),
                                                   False, variant=2)
    out["convert_u8_to_f32"] = orc.convert_to(recipe(1, 5, 7, 3), np.float32, 1 / 255.0, 0.0, 0)
    out["convert_f32_to_u8"] = orc.convert_to(recipe(1, 5, 7, 3, np.float32) * 300 - 20, np.uint8, 1.0, 0.5, 0)
    img = recipe(1, 20, 28, 3, step=5)[0]
    for flip in (-1, 0, 1, 2):
        out["crop_flip_normalize_f32_flip%d" % flip] = orc.crop_flip_normalize(
            img, (16, 24), np.float32, (-2, 3, 22, 15), flip, 2, 0.0, [1.0, 2.0, 3.0], [0.5, 0.25, 0.125], 1.0, 0.0, 0.0,
            False)
    return out


if __name__ == "__main__":
    arrays = cases()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **arrays)
    print("%d arrays, %d bytes -> %s" % (len(arrays), os.path.getsize(path), path))
