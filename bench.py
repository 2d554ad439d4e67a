#!/usr/bin/env python3
"""Benchmark of the image pre-processing hot path on one MI355X.

Default workload (the headline one): a step = one cvcudaResizeCropConvertReformatSubmit over a batch
of 64 1080p u8 RGB images (bilinear resize to 455x256, centre crop 224x224, scale/offset, f32 NCHW
output). With no `--workload` the other BASELINE configurations (plain resize nearest and bilinear, NV12->RGB,
var-shape affine warp, 4K cubic resize) are timed after it, each the same way on a smaller budget, and reported
under the extra key `configs` (one entry per configuration, the headline first); `--workload` times one
workload only. Each is one Submit per step.

Inputs are generated on the host from a fixed seed and uploaded before the timed region. To keep
the reads coming from HBM rather than from the 256 MB on-die cache, consecutive steps cycle through
`--rotate` distinct input/output buffer sets (default: at least 3 and enough for 1.5 GB of algorithmic
bytes, so that even a kernel that reads only a fifth of its bytes cycles through twice the cache's
size in reads; with fewer sets the streaming kernels time up to 25 % shorter because part of the input is
still in that cache; 1 = same buffers every step).

Prints ONE JSON line: throughput (images/s), the HBM roofline fraction of the kernel (algorithmic
bytes / mean kernel time / 8 TB/s) and the CPU oracle's throughput on a bounded sample of the same
workload.
"""
import argparse
import json
import math
import os
import sys
import time

HBM_PEAK_GBS = 8000.0
SEED_BASE = 0xC0FFEE00
NEAREST, LINEAR, CUBIC, AREA = 0, 1, 2, 3

# HBM bytes one launch of a workload's kernel moves, from hardware counters (rocprofv3 --pmc
# FETCH_SIZE and --pmc WRITE_SIZE in separate runs, each scaled by what the same counter reads for a
# plain device copy of known size appended to the same run by --copy-probe). It is a property of the
# kernel and the workload, not of a run, so it is recorded here rather than re-measured; read and
# write parts are in the summary files named below. The counters sit between the L2s and the fabric:
# a batch that fits the memory-side cache (warp-affine-varshape) has part of those reads served there.
MEASURED_TRAFFIC_BYTES = {"fused": 122963893, "resize-cubic-4k": 1474458644, "resize-nearest": 12249763,
                          "resize-linear": 23286608, "nv12-to-rgb": 298659855, "warp-affine-varshape": 298562951}
# The rocprofv3 counter summary each figure above is the "total" line of (a CPU test compares them).
TRAFFIC_PROFILES = {"fused": "FusedBilinear_batch64_1080p_to_224",
                    "resize-cubic-4k": "ResizeCubicStagedKernel_f32x4_batch16_4k_to_640x360",
                    "resize-nearest": "ResizePatchTensorKernel_u8x3_NEAREST_batch8_1080p_to_224",
                    "resize-linear": "ResizePatchTensorKernel_u8x3_LINEAR_batch8_1080p_to_224",
                    "nv12-to-rgb": "Yuv420ToRgbTensor_NV12_batch32_1080p",
                    "warp-affine-varshape": "WarpVarShape_u8x3_LINEAR_batch32_varshape"}


def span_bytes(n_out, crop, src, new, interp, pixel_bytes):
    """Distinct source indices referenced along one axis and the byte span first..last (times
    pixel_bytes), from the operators' own float32 index maps."""
    import numpy as np
    f32 = np.float32
    s = f32(src) / f32(new)
    d = np.arange(n_out, dtype=np.float32) + f32(crop)
    if interp == NEAREST:
        idx = np.minimum(np.floor((d + f32(0.5)) * s).astype(np.int64), src - 1)
    elif interp == LINEAR:
        i0 = np.floor((d + f32(0.5)) * s - f32(0.5)).astype(np.int64)
        idx = np.concatenate([np.clip(i0, 0, src - 1), np.clip(i0 + 1, 0, src - 1)])
    else:
        i0 = np.clip(np.floor((d + f32(0.5)) * s - f32(0.5)).astype(np.int64), 1, src - 3)
        idx = np.concatenate([i0 - 1, i0, i0 + 1, i0 + 2])
    return len(np.unique(idx)), (int(idx.max()) - int(idx.min()) + 1) * pixel_bytes


def polygon_clip_area(poly, w, h):
    """Area of a convex polygon clipped to [0,w]x[0,h] (Sutherland-Hodgman + shoelace)."""
    def clip(pts, inside, inter):
        out = []
        for i in range(len(pts)):
            a, b = pts[i - 1], pts[i]
            ia, ib = inside(a), inside(b)
            if ia != ib:
                out.append(inter(a, b))
            if ib:
                out.append(b)
        return out

    def ix(x0):
        return lambda a, b: (x0, a[1] + (b[1] - a[1]) * (x0 - a[0]) / (b[0] - a[0]))

    def iy(y0):
        return lambda a, b: (a[0] + (b[0] - a[0]) * (y0 - a[1]) / (b[1] - a[1]), y0)

    pts = list(poly)
    for inside, inter in ((lambda p: p[0] >= 0, ix(0.0)), (lambda p: p[0] <= w, ix(float(w))),
                          (lambda p: p[1] >= 0, iy(0.0)), (lambda p: p[1] <= h, iy(float(h)))):
        if not pts:
            return 0.0
        pts = clip(pts, inside, inter)
    area = 0.0
    for i in range(len(pts)):
        area += pts[i - 1][0] * pts[i][1] - pts[i][0] * pts[i - 1][1]
    return abs(area) / 2


# ------------------------------------------------------------------------------------------------
# Workloads. Each class offers: key, kernel, workload (text), dtype, images (per step), alg_bytes
# (per step), make_set() -> buffer set, submit(stream, set), check(set) (oracle spot check of what
# the GPU produced), cpu(threads) -> images the oracle processed.
class Fused:
    """Configuration 2 in four forms (`form`):
    fused            one cvcudaResizeCropConvertReformatSubmit, normalisation as one scale/offset pair
    fused-normalize  one cvcudaxResizeCropConvertReformatNormalizeSubmit (extension): per-channel mean/std
    fused-chain      what the reference needs for per-channel mean/std: fused (x 1/255, f32 NHWC) ->
                     Normalize (scale is stddev) -> Reformat (NCHW), three Submits per step
    fused-copy-bound not an operator: a kernel with the fused kernel's grid, tap loads and stores but no
                     arithmetic (libcvamd_bench.so), i.e. what the memory system allows this access pattern
    """
    config_id = 2
    N, SRC_H, SRC_W = 64, 1080, 1920
    NEW_W, NEW_H, CROP_X, CROP_Y, OUT_H, OUT_W = 455, 256, 115, 16, 224, 224
    SCALE, OFFSET = 1.0 / (255.0 * 0.226), -0.449 / 0.226
    MEAN, STD = (0.485, 0.456, 0.406), (0.229, 0.224, 0.225)
    dtype = "f32"
    KERNELS = {"fused": "FusedBilinear<float,false,false,false,true>",
               "fused-normalize": "FusedBilinear<float,false,false,true,true>",
               "fused-chain": "FusedBilinear<float,false,false,false,false> + NormRunsTensor<float,float,3> + "
                              "ReformatKernel<unsigned int,3,true,false>",
               "fused-copy-bound": "FusedCopyBound"}
    TEXT = {"fused": "scale/offset", "fused-normalize": "per-channel mean/std in the same kernel (extension entry point)",
            "fused-chain": "per-channel mean/std as the three-operator chain fused -> Normalize -> Reformat",
            "fused-copy-bound": "copy-bound twin of the fused kernel (same grid, loads and stores, no arithmetic)"}

    def __init__(self, cv, orc, np, torch, form="fused"):
        self.cv, self.orc, self.np, self.torch, self.form = cv, orc, np, torch, form
        self.key, self.kernel = form, self.KERNELS[form]
        if form == "fused" and self.N == 64:  # the mover has the bytes of the configuration's own batch
            self.mover = "stream-mix-4-2"
        self.workload = ("fused ResizeCropConvertReformat: batch %d u8 NHWC 1920x1080 -> bilinear 455x256 -> " % self.N +
                         "crop 224x224 @(115,16) -> f32 NCHW, " + self.TEXT[form])
        self.images = self.N
        rows, _ = span_bytes(self.OUT_H, self.CROP_Y, self.SRC_H, self.NEW_H, LINEAR, 1)
        _, span = span_bytes(self.OUT_W, self.CROP_X, self.SRC_W, self.NEW_W, LINEAR, 3)
        self.alg_bytes = (rows * span + 3 * self.OUT_H * self.OUT_W * 4) * self.N
        cols, _ = span_bytes(self.OUT_W, self.CROP_X, self.SRC_W, self.NEW_W, LINEAR, 3)
        out_bytes = 3 * self.OUT_H * self.OUT_W * 4
        self.other_bytes = {"whole_tensors": (self.SRC_H * self.SRC_W * 3 + out_bytes) * self.N,
                            "referenced_pixels_only": (rows * cols * 3 + out_bytes) * self.N}
        self.host = orc.fill_u8((self.N, self.SRC_H, self.SRC_W, 3), SEED_BASE + self.config_id)
        self.dev = torch.from_numpy(self.host).cuda()
        self.op = cv.ResizeCropConvertReformat()
        if form == "fused-chain":
            self.norm, self.reformat = cv.Normalize(), cv.Reformat()
            self.tmean = cv.Tensor.from_numpy(np.asarray(self.MEAN, np.float32).reshape(1, 1, 1, 3), "NHWC")
            self.tstd = cv.Tensor.from_numpy(np.asarray(self.STD, np.float32).reshape(1, 1, 1, 3), "NHWC")
        if form == "fused-copy-bound":
            import ctypes as C
            lib = C.CDLL(os.path.join(os.path.dirname(os.path.abspath(cv.__file__)), "lib", "libcvamd_bench.so"))
            self.copy_fn = lib.cvamdBenchFusedCopyBound
            self.copy_fn.restype = C.c_int
            self.copy_fn.argtypes = [C.c_void_p, C.c_void_p, C.c_int64] + [C.c_int32] * 3 + [C.c_void_p] + [C.c_int32] * 7

    def make_set(self):
        cv, np = self.cv, self.np
        tin = cv.Tensor.alloc([self.N, self.SRC_H, self.SRC_W, 3], np.uint8, "NHWC")
        tin.torch_view().copy_(self.dev)
        out = cv.Tensor.alloc([self.N, 3, self.OUT_H, self.OUT_W], np.float32, "NCHW")
        if self.form == "fused-chain":
            return (tin, out, cv.Tensor.alloc([self.N, self.OUT_H, self.OUT_W, 3], np.float32, "NHWC"),
                    cv.Tensor.alloc([self.N, self.OUT_H, self.OUT_W, 3], np.float32, "NHWC"))
        return tin, out

    def submit(self, stream, s):
        geom = ((self.NEW_W, self.NEW_H), LINEAR, (self.CROP_X, self.CROP_Y))
        if self.form == "fused":
            self.op(stream, s[0], s[1], *geom, 0, self.SCALE, self.OFFSET, False)
        elif self.form == "fused-normalize":
            self.op.normalized(stream, s[0], s[1], *geom, self.MEAN, self.STD, 0, 1 / 255.0, 0.0, False, 1.0, 0.0, 0.0,
                               self.cv.K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV)
        elif self.form == "fused-chain":
            self.op(stream, s[0], s[2], *geom, 0, 1 / 255.0, 0.0, False)
            self.norm(stream, s[2], self.tmean, self.tstd, s[3], 1.0, 0.0, 0.0, self.cv.K.CVCUDA_NORMALIZE_SCALE_IS_STDDEV)
            self.reformat(stream, s[3], s[1])
        else:
            tv = s[0].torch_view()
            rc = self.copy_fn(self.cv.stream_ptr(stream), tv.data_ptr(), tv.stride(0), tv.stride(1), self.SRC_W,
                              self.SRC_H, s[1].torch_view().data_ptr(), self.N, self.OUT_W, self.OUT_H, self.NEW_W,
                              self.NEW_H, self.CROP_X, self.CROP_Y)
            assert rc == 0, "cvamdBenchFusedCopyBound failed: hipError %d" % rc

    def _oracle(self, src, threads=1):
        np, orc = self.np, self.orc
        size, geom = (self.OUT_H, self.OUT_W), ((self.NEW_W, self.NEW_H), (self.CROP_X, self.CROP_Y), LINEAR)
        if self.form in ("fused", "fused-copy-bound"):
            return orc.fused_rccr(src, size, *geom, np.float32, True, 0, self.SCALE, self.OFFSET, False, threads=threads)
        x = orc.fused_rccr(src, size, *geom, np.float32, False, 0, 1 / 255.0, 0.0, False, threads=threads)
        mean = np.asarray(self.MEAN, np.float32).reshape(1, 1, 1, 3)
        std = np.asarray(self.STD, np.float32).reshape(1, 1, 1, 3)
        return np.ascontiguousarray(orc.normalize(x, mean, std, 1.0, 0.0, 0.0, True, threads=threads).transpose(0, 3, 1, 2))

    def check(self, s):
        np = self.np
        got = s[1].torch_view()[:2].cpu().numpy()
        if self.form == "fused-copy-bound":
            # plane 0 holds the 3 bytes of the upper row's first tap: the same place the operator reads
            f32 = np.float32
            dx, dy = np.arange(self.OUT_W, dtype=f32), np.arange(self.OUT_H, dtype=f32)
            sx = np.maximum(np.floor((dx + f32(self.CROP_X) + f32(0.5)) * (f32(self.SRC_W) / f32(self.NEW_W)) - f32(0.5)), 0)
            sy = np.maximum(np.floor((dy + f32(self.CROP_Y) + f32(0.5)) * (f32(self.SRC_H) / f32(self.NEW_H)) - f32(0.5)), 0)
            px = self.host[:2][:, sy.astype(int)][:, :, sx.astype(int)].astype(np.uint32)
            want = px[..., 0] | (px[..., 1] << 8) | (px[..., 2] << 16)
            assert (got[:, 0].view(np.uint32) == want).all(), "copy-bound kernel read other pixels than the operator"
            return
        ref = self._oracle(self.host[:2])
        assert (np.abs(got - ref) <= 1e-5 * np.maximum(1.0, np.abs(ref))).all(), "bench output differs from oracle"

    def cpu(self, threads):
        n = min(8, self.N)
        self._oracle(self.host[:n], threads)
        return n


class ResizeC1:
    config_id = 1
    N, SRC_H, SRC_W, OUT_H, OUT_W = 8, 1080, 1920, 224, 224
    dtype = "f32"

    def __init__(self, cv, orc, np, torch, interp):
        self.cv, self.orc, self.np, self.torch, self.interp = cv, orc, np, torch, interp
        name = "NEAREST" if interp == NEAREST else "LINEAR"
        self.key = "resize-" + name.lower()
        self.kernel = "ResizePatchTensorKernel<uint8_t,3,%s>" % name
        self.dtype = "f32" if interp == NEAREST else "i32"  # index map in float32; bilinear blend in fixed point
        self.workload = "Resize %s: batch %d u8 NHWC 1920x1080 -> 224x224" % (name, self.N)
        self.images = self.N
        rows, _ = span_bytes(self.OUT_H, 0, self.SRC_H, self.OUT_H, interp, 1)
        _, span = span_bytes(self.OUT_W, 0, self.SRC_W, self.OUT_W, interp, 3)
        self.alg_bytes = (rows * span + self.OUT_H * self.OUT_W * 3) * self.N
        cols, _ = span_bytes(self.OUT_W, 0, self.SRC_W, self.OUT_W, interp, 3)
        self.other_bytes = {"whole_tensors": (self.SRC_H * self.SRC_W + self.OUT_H * self.OUT_W) * 3 * self.N,
                            "referenced_pixels_only": (rows * cols + self.OUT_H * self.OUT_W) * 3 * self.N}
        self.host = orc.fill_u8((self.N, self.SRC_H, self.SRC_W, 3), SEED_BASE + self.config_id)
        self.dev = torch.from_numpy(self.host).cuda()
        self.op = cv.Resize()

    def make_set(self):
        tin = self.cv.Tensor.alloc([self.N, self.SRC_H, self.SRC_W, 3], self.np.uint8, "NHWC")
        tin.torch_view().copy_(self.dev)
        return tin, self.cv.Tensor.alloc([self.N, self.OUT_H, self.OUT_W, 3], self.np.uint8, "NHWC")

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], self.interp)

    def check(self, s):
        ref = self.orc.resize(self.host[:2], (self.OUT_H, self.OUT_W), self.interp, variant=0)
        got = s[1].torch_view()[:2].cpu().numpy()
        tol = 0 if self.interp == NEAREST else 1
        assert self.np.abs(got.astype(self.np.int16) - ref.astype(self.np.int16)).max() <= tol

    def cpu(self, threads):
        self.orc.resize(self.host, (self.OUT_H, self.OUT_W), self.interp, variant=0, threads=threads)
        return self.N


class CubicC5:
    key, config_id, mover = "resize-cubic-4k", 5, "stream-mix-24-1"
    N, SRC_H, SRC_W, OUT_H, OUT_W = 16, 2160, 3840, 360, 640
    kernel = "ResizeCubicStagedKernel<float,4>"
    dtype = "f32"
    workload = "Resize CUBIC: batch 16 f32 NHWC 3840x2160x4 -> 640x360x4"

    def __init__(self, cv, orc, np, torch):
        self.cv, self.orc, self.np, self.torch = cv, orc, np, torch
        self.images = self.N
        rows, _ = span_bytes(self.OUT_H, 0, self.SRC_H, self.OUT_H, CUBIC, 1)
        _, span = span_bytes(self.OUT_W, 0, self.SRC_W, self.OUT_W, CUBIC, 16)
        self.alg_bytes = (rows * span + self.OUT_H * self.OUT_W * 16) * self.N
        cols, _ = span_bytes(self.OUT_W, 0, self.SRC_W, self.OUT_W, CUBIC, 16)
        self.other_bytes = {"whole_tensors": (self.SRC_H * self.SRC_W + self.OUT_H * self.OUT_W) * 16 * self.N,
                            "referenced_pixels_only": (rows * cols + self.OUT_H * self.OUT_W) * 16 * self.N}
        self.host = orc.fill_f32((self.N, self.SRC_H, self.SRC_W, 4), SEED_BASE + self.config_id)
        self.dev = torch.from_numpy(self.host).cuda()
        self.op = cv.Resize()

    def make_set(self):
        tin = self.cv.Tensor.alloc([self.N, self.SRC_H, self.SRC_W, 4], self.np.float32, "NHWC")
        tin.torch_view().copy_(self.dev)
        return tin, self.cv.Tensor.alloc([self.N, self.OUT_H, self.OUT_W, 4], self.np.float32, "NHWC")

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], CUBIC)

    def check(self, s):
        ref = self.orc.resize(self.host[:1], (self.OUT_H, self.OUT_W), CUBIC, variant=1)
        got = s[1].torch_view()[:1].cpu().numpy()
        assert self.np.abs(got - ref).max() <= 1e-4

    def cpu(self, threads):
        self.orc.resize(self.host[:4], (self.OUT_H, self.OUT_W), CUBIC, variant=1, threads=threads)
        return 4


class Nv12C3:
    key, config_id, mover = "nv12-to-rgb", 3, "stream-mix-1-2"
    N, H, W = 32, 1080, 1920
    kernel = "Yuv420ToRgbTensor<3,true>"
    dtype = "int32"
    workload = "CvtColor YUV2RGB_NV12: batch 32 u8 [1620,1920,1] -> [1080,1920,3]"

    def __init__(self, cv, orc, np, torch):
        self.cv, self.orc, self.np, self.torch = cv, orc, np, torch
        self.images = self.N
        self.alg_bytes = self.N * (self.H * 3 // 2 * self.W + self.H * self.W * 3)
        self.other_bytes = {"whole_tensors": self.alg_bytes, "referenced_pixels_only": self.alg_bytes}  # a streaming map
        y = orc.fill_u8((self.N, self.H, self.W, 1), SEED_BASE + self.config_id, 16, 235)
        uv = orc.fill_u8((self.N, self.H // 2, self.W, 1), SEED_BASE + self.config_id + 100, 16, 240)
        self.host = np.concatenate([y, uv], axis=1)
        self.dev = torch.from_numpy(self.host).cuda()
        self.op = cv.CvtColor()

    def make_set(self):
        tin = self.cv.Tensor.alloc([self.N, self.H * 3 // 2, self.W, 1], self.np.uint8, "NHWC")
        tin.torch_view().copy_(self.dev)
        return tin, self.cv.Tensor.alloc([self.N, self.H, self.W, 3], self.np.uint8, "NHWC")

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], 90)

    def check(self, s):
        ref = self.orc.yuv420_to_rgb(self.host[:1, :, :, 0], 3, False, 0, True, variant=0)
        got = s[1].torch_view()[:1].cpu().numpy()
        assert (got == ref).all()

    def cpu(self, threads):
        self.orc.yuv420_to_rgb(self.host[:16, :, :, 0], 3, False, 0, True, variant=0, threads=threads)
        return 16


class WarpC4:
    key, config_id = "warp-affine-varshape", 4
    N = 32
    kernel = "WarpVarShape<uint8_t,3,LINEAR>"
    dtype = "i32"  # coordinates in float32, the 8-bit blend in 15-bit fixed point
    workload = ("WarpAffine var-shape LINEAR: 32 u8 RGB images, W in [640,1920], H in [480,1080], rotation +-30 deg "
                "x scale 0.8-1.2 about the centre, constant border 0")

    def __init__(self, cv, orc, np, torch):
        self.cv, self.orc, self.np, self.torch = cv, orc, np, torch
        self.images = self.N
        rng = np.random.default_rng(SEED_BASE + self.config_id)
        self.sizes, mats, alg = [], [], 0
        for _ in range(self.N):
            w, h = int(rng.integers(640, 1921)), int(rng.integers(480, 1081))
            t, s = math.radians(float(rng.uniform(-30, 30))), float(rng.uniform(0.8, 1.2))
            c, sn, cx, cy = s * math.cos(t), s * math.sin(t), (w - 1) / 2.0, (h - 1) / 2.0
            m = [c, -sn, cx - c * cx + sn * cy, sn, c, cy - sn * cx - c * cy]
            self.sizes.append((w, h))
            mats.append(m)
            inv = orc.invert_affine(m).astype(np.float64)
            corners = [(inv[0] * x + inv[1] * y + inv[2], inv[3] * x + inv[4] * y + inv[5])
                       for x, y in ((0, 0), (w, 0), (w, h), (0, h))]
            alg += min(w * h * 3, int(3 * polygon_clip_area(corners, w, h))) + w * h * 3
        self.alg_bytes = alg
        self.other_bytes = {"whole_tensors": sum(2 * w * h * 3 for w, h in self.sizes)}
        self.mats = np.asarray(mats, np.float32)
        self.hosts = [orc.fill_u8((h, w, 3), SEED_BASE + self.config_id + 1000 + i)
                      for i, (w, h) in enumerate(self.sizes)]
        self.op = cv.WarpAffine(self.N)
        self.K = cv.K

    def make_set(self):
        cv = self.cv
        bi, bo, outs = cv.ImageBatchVarShape(self.N), cv.ImageBatchVarShape(self.N), []
        for a, (w, h) in zip(self.hosts, self.sizes):
            bi.push_back(cv.Image.from_numpy(a, self.K.IMAGE_FORMAT_RGB8))
            o = cv.Image.alloc((w, h), self.K.IMAGE_FORMAT_RGB8)
            outs.append(o)
            bo.push_back(o)
        return bi, bo, cv.Tensor.from_numpy(self.mats, "NW"), outs

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], s[2], LINEAR, 0, (0, 0, 0, 0))

    def check(self, s):
        np = self.np
        a = self.hosts[0]
        ref = self.orc.warp(a[None], a.shape[:2], self.orc.invert_affine(self.mats[0]), LINEAR, 0, variant=0)[0]
        got = s[3][0].plane_view(0, np.uint8, 3).cpu().numpy()
        assert np.abs(got.astype(np.int16) - ref.astype(np.int16)).max() <= 1

    def cpu(self, threads):
        # images differ in size: the oracle threads over the rows of one image at a time
        for i in range(8):
            a = self.hosts[i]
            self.orc.warp(a[None], a.shape[:2], self.orc.invert_affine(self.mats[i]), LINEAR, 0, variant=0,
                          threads=threads)
        return 8


class FusedVarShape:
    """Configuration 2's geometry on an image batch: 64 separately allocated u8 RGB images of mixed sizes, each resized
    to 455x256 (its own scale factors), cropped and written to one f32 NCHW tensor."""
    key, config_id = "fused-varshape", 2
    N = 64
    NEW_W, NEW_H, CROP_X, CROP_Y, OUT_H, OUT_W = Fused.NEW_W, Fused.NEW_H, Fused.CROP_X, Fused.CROP_Y, Fused.OUT_H, Fused.OUT_W
    SCALE, OFFSET = Fused.SCALE, Fused.OFFSET
    kernel = "FusedBilinear<float,true,false,false,true>"
    dtype = "f32"
    workload = ("fused ResizeCropConvertReformat, image batch: 64 u8 RGB images, W in [1280,1920], H in [720,1080] -> "
                "bilinear 455x256 -> crop 224x224 @(115,16) -> f32 NCHW tensor, scale/offset")

    def __init__(self, cv, orc, np, torch):
        self.cv, self.orc, self.np, self.torch = cv, orc, np, torch
        self.images = self.N
        rng = np.random.default_rng(SEED_BASE + 20)
        self.sizes = [(int(rng.integers(1280, 1921)), int(rng.integers(720, 1081))) for _ in range(self.N)]
        self.alg_bytes = 0
        for w, h in self.sizes:
            rows, _ = span_bytes(self.OUT_H, self.CROP_Y, h, self.NEW_H, LINEAR, 1)
            _, span = span_bytes(self.OUT_W, self.CROP_X, w, self.NEW_W, LINEAR, 3)
            self.alg_bytes += rows * span + 3 * self.OUT_H * self.OUT_W * 4
        self.hosts = [orc.fill_u8((h, w, 3), SEED_BASE + 2000 + i) for i, (w, h) in enumerate(self.sizes)]
        self.op = cv.ResizeCropConvertReformat()

    def make_set(self):
        cv = self.cv
        batch = cv.ImageBatchVarShape(self.N)
        for a in self.hosts:
            batch.push_back(cv.Image.from_numpy(a, cv.K.IMAGE_FORMAT_RGB8))
        return batch, cv.Tensor.alloc([self.N, 3, self.OUT_H, self.OUT_W], self.np.float32, "NCHW")

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], (self.NEW_W, self.NEW_H), LINEAR, (self.CROP_X, self.CROP_Y), 0, self.SCALE,
                self.OFFSET, False)

    def _oracle(self, a, threads=1):
        return self.orc.fused_rccr(a[None], (self.OUT_H, self.OUT_W), (self.NEW_W, self.NEW_H), (self.CROP_X, self.CROP_Y),
                                   LINEAR, self.np.float32, True, 0, self.SCALE, self.OFFSET, False, threads=threads)[0]

    def check(self, s):
        np = self.np
        got = s[1].torch_view()[:2].cpu().numpy()
        for i in range(2):
            ref = self._oracle(self.hosts[i])
            assert (np.abs(got[i] - ref) <= 1e-5 * np.maximum(1.0, np.abs(ref))).all(), "bench output differs from oracle"

    def cpu(self, threads):
        for a in self.hosts[:8]:
            self._oracle(a, threads)
        return 8


class ResizeVarShape:
    """Configuration 1's reduction on an image batch: 32 u8 RGB images of mixed sizes, each to its own 224x224 image."""
    key, config_id = "resize-linear-varshape", 1
    N, OUT = 32, 224
    kernel = "ResizePatchVarShapeKernel<uint8_t,3,LINEAR>"
    dtype = "i32"  # coordinates in float32, the 8-bit blend in 15-bit fixed point
    workload = "Resize LINEAR, image batch: 32 u8 RGB images, W in [1280,1920], H in [720,1080] -> 224x224 each"

    def __init__(self, cv, orc, np, torch):
        self.cv, self.orc, self.np, self.torch = cv, orc, np, torch
        self.images = self.N
        rng = np.random.default_rng(SEED_BASE + 21)
        self.sizes = [(int(rng.integers(1280, 1921)), int(rng.integers(720, 1081))) for _ in range(self.N)]
        self.alg_bytes = 0
        for w, h in self.sizes:
            rows, _ = span_bytes(self.OUT, 0, h, self.OUT, LINEAR, 1)
            _, span = span_bytes(self.OUT, 0, w, self.OUT, LINEAR, 3)
            self.alg_bytes += rows * span + self.OUT * self.OUT * 3
        self.hosts = [orc.fill_u8((h, w, 3), SEED_BASE + 3000 + i) for i, (w, h) in enumerate(self.sizes)]
        self.op = cv.Resize()

    def make_set(self):
        cv = self.cv
        bi, bo, outs = cv.ImageBatchVarShape(self.N), cv.ImageBatchVarShape(self.N), []
        for a in self.hosts:
            bi.push_back(cv.Image.from_numpy(a, cv.K.IMAGE_FORMAT_RGB8))
            o = cv.Image.alloc((self.OUT, self.OUT), cv.K.IMAGE_FORMAT_RGB8)
            outs.append(o)
            bo.push_back(o)
        return bi, bo, outs

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], LINEAR)

    def check(self, s):
        np = self.np
        for i in range(2):
            ref = self.orc.resize(self.hosts[i][None], (self.OUT, self.OUT), LINEAR, variant=0)[0]
            got = s[2][i].plane_view(0, np.uint8, 3).cpu().numpy()
            assert np.abs(got.astype(np.int16) - ref.astype(np.int16)).max() <= 1

    def cpu(self, threads):
        for a in self.hosts[:8]:
            self.orc.resize(a[None], (self.OUT, self.OUT), LINEAR, variant=0, threads=threads)
        return 8


class CropFlipNormalize:
    """CropFlipNormalizeReformat as the classification pipelines use it: a 224x224 crop of each image of a batch,
    mirrored or not, (x - mean) / std per channel, written as f32 NCHW."""
    key, config_id = "crop-flip-normalize-224", 0
    N, OUT = 64, 224
    kernel = "CfnrRunsKernel<uint8_t,float,3>"
    dtype = "f32"
    workload = ("CropFlipNormalizeReformat: 64 u8 RGB images, W in [256,512], H in [256,384] -> crop 224x224 at a random "
                "place, random flip code, per-channel (x - base) * scale -> f32 NCHW tensor")

    def __init__(self, cv, orc, np, torch):
        self.cv, self.orc, self.np, self.torch = cv, orc, np, torch
        self.images = self.N
        rng = np.random.default_rng(SEED_BASE + 22)
        self.sizes = [(int(rng.integers(256, 513)), int(rng.integers(256, 385))) for _ in range(self.N)]
        self.hosts = [orc.fill_u8((h, w, 3), SEED_BASE + 4000 + i) for i, (w, h) in enumerate(self.sizes)]
        self.crops = np.zeros((self.N, 1, 1, 4), np.int32)
        for i, (w, h) in enumerate(self.sizes):
            self.crops[i, 0, 0] = (rng.integers(0, w - self.OUT + 1), rng.integers(0, h - self.OUT + 1), self.OUT, self.OUT)
        self.flips = rng.integers(-1, 3, self.N).astype(np.int32)
        self.base = (np.asarray(Fused.MEAN, np.float32) * 255).reshape(1, 1, 1, 3)
        self.scale = (1 / (np.asarray(Fused.STD, np.float32) * 255)).astype(np.float32).reshape(1, 1, 1, 3)
        self.alg_bytes = self.N * self.OUT * self.OUT * 3 * (1 + 4)
        self.op = cv.CropFlipNormalizeReformat()

    def make_set(self):
        cv = self.cv
        batch = cv.ImageBatchVarShape(self.N)
        for a in self.hosts:
            batch.push_back(cv.Image.from_numpy(a, cv.K.IMAGE_FORMAT_RGB8))
        return (batch, cv.Tensor.alloc([self.N, 3, self.OUT, self.OUT], self.np.float32, "NCHW"),
                cv.Tensor.from_numpy(self.crops, "NHWC"), cv.Tensor.from_numpy(self.flips, "N"),
                cv.Tensor.from_numpy(self.base, "NHWC"), cv.Tensor.from_numpy(self.scale, "NHWC"))

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], s[2], 0, 0.0, s[3], s[4], s[5])

    def _oracle(self, i):
        return self.orc.crop_flip_normalize(self.hosts[i], (self.OUT, self.OUT), self.np.float32, self.crops[i, 0, 0],
                                            self.flips[i], 0, 0.0, self.base.reshape(-1), self.scale.reshape(-1), 1.0,
                                            0.0, 0.0, False)

    def check(self, s):
        np = self.np
        got = s[1].torch_view()[:2].cpu().numpy().transpose(0, 2, 3, 1)
        for i in range(2):
            ref = self._oracle(i)
            assert np.abs(got[i] - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max()), "bench output differs from oracle"

    def cpu_cores(self, threads):
        return 1

    def cpu(self, threads):
        for i in range(self.N):
            self._oracle(i)
        return self.N


class WarpTensor:
    """WarpAffine on a tensor: 32 u8 RGB images of 1280x780 rotated by 17 degrees about the centre at scale 1.05
    (forward map), constant border 0. Algorithmic bytes: the part of the source the destination's inverse image
    covers, plus the output."""
    config_id = 0
    N, H, W = 32, 780, 1280
    dtype = "f32"

    def __init__(self, cv, orc, np, torch, interp):
        self.cv, self.orc, self.np, self.torch, self.interp = cv, orc, np, torch, interp
        name = {NEAREST: "NEAREST", LINEAR: "LINEAR", CUBIC: "CUBIC"}[interp]
        self.key = "warp-affine-tensor-" + name.lower()
        self.kernel = "WarpTensor<uint8_t,3,%s>" % name
        self.dtype = "f32" if interp == NEAREST else "i32"  # coordinates in float32; 8-bit blends in fixed point
        self.workload = "WarpAffine %s: batch 32 u8 NHWC 1280x780x3, rotation 17 deg x scale 1.05, constant border 0" % name
        self.images = self.N
        w, h = self.W, self.H
        t, sc = math.radians(float(os.environ.get("CVAMD_BENCH_WARP_DEGREES", "17"))), 1.05
        c, sn, cx, cy = sc * math.cos(t), sc * math.sin(t), (w - 1) / 2.0, (h - 1) / 2.0
        self.m = [c, -sn, cx - c * cx + sn * cy, sn, c, cy - sn * cx - c * cy]
        inv = orc.invert_affine(self.m).astype(np.float64)
        corners = [(inv[0] * x + inv[1] * y + inv[2], inv[3] * x + inv[4] * y + inv[5])
                   for x, y in ((0, 0), (w, 0), (w, h), (0, h))]
        self.alg_bytes = self.N * (min(w * h * 3, int(3 * polygon_clip_area(corners, w, h))) + w * h * 3)
        self.host = orc.fill_u8((1, h, w, 3), SEED_BASE + 55)
        self.dev = torch.from_numpy(self.host).cuda()
        self.op = cv.WarpAffine(0)

    def make_set(self):
        tin = self.cv.Tensor.alloc([self.N, self.H, self.W, 3], self.np.uint8, "NHWC")
        tin.torch_view().copy_(self.dev.expand(self.N, -1, -1, -1))
        return tin, self.cv.Tensor.alloc([self.N, self.H, self.W, 3], self.np.uint8, "NHWC")

    def submit(self, stream, s):
        self.op(stream, s[0], s[1], self.m, self.interp, 0, (0, 0, 0, 0))

    def _oracle(self, src, threads=1):
        return self.orc.warp(src, (self.H, self.W), self.orc.invert_affine(self.m), self.interp, 0, (0, 0, 0, 0),
                             variant=0, threads=threads)

    def check(self, s):
        np = self.np
        got = s[1].torch_view()[:1].cpu().numpy()
        ref = self._oracle(self.host)
        assert np.abs(got.astype(np.int16) - ref.astype(np.int16)).max() <= (0 if self.interp == NEAREST else 1)

    def cpu(self, threads):
        self._oracle(self.host, threads)
        return 1


class EmptyLaunch:
    """Not an operator: one launch of a kernel that does nothing (libcvamd_bench.so), i.e. what a dependent
    launch costs in the same timed region as the operators. No bytes, so no roofline fraction."""
    key, config_id, kernel, dtype = "empty-launch", 0, "EmptyKernel", "none"
    workload = "one empty kernel launch per step (64 threads)"
    images, alg_bytes = 0, 0

    def __init__(self, cv, orc, np, torch):
        import ctypes as C
        lib = C.CDLL(os.path.join(os.path.dirname(os.path.abspath(cv.__file__)), "lib", "libcvamd_bench.so"))
        self.fn, self.cv = lib.cvamdBenchEmptyLaunch, cv
        self.fn.restype, self.fn.argtypes = C.c_int, [C.c_void_p]

    def make_set(self):
        return ()

    def submit(self, stream, s):
        assert self.fn(self.cv.stream_ptr(stream)) == 0

    def check(self, s):
        pass

    def cpu(self, threads):
        return 0


class StreamMix:
    """Not an operator: a kernel that only moves bytes (libcvamd_bench.so), dense 16-byte loads and streaming
    stores in the read : write ratio of one of the configurations and with its byte counts, i.e. what the memory
    system gives that mix. stream-mix-1-2 has the bytes of nv12-to-rgb, stream-mix-24-1 those of resize-cubic-4k,
    stream-mix-4-2 reads the 81.1 MB of the fused configuration's row spans (and writes half as much, 5 % more than
    the fused output; 4 loads and 2 stores per lane was the fastest of 2:1, 4:2 and 8:4), stream-mix-1-1 is a plain
    copy of the same size as the first."""
    config_id, dtype = 0, "none"
    SPECS = {"stream-mix-1-1": (1, 1, 149299200 // 16), "stream-mix-1-2": (1, 2, 99532800 // 16),
             "stream-mix-4-2": (4, 2, 64 * 1267392 // 64), "stream-mix-24-1": (24, 1, 58982400 // 16)}
    images = 0

    def __init__(self, cv, orc, np, torch, key):
        import ctypes as C
        self.key, self.cv, self.torch = key, cv, torch
        self.reads, self.writes, self.lanes = self.SPECS[key]
        self.kernel = "StreamMix<%d,%d>" % (self.reads, self.writes)
        self.workload = "plain byte mover: %d x 16 bytes read, %d x 16 written per lane, %d lanes" % (
            self.reads, self.writes, self.lanes)
        self.alg_bytes = 16 * self.lanes * (self.reads + self.writes)
        self.other_bytes = {"whole_tensors": self.alg_bytes, "referenced_pixels_only": self.alg_bytes}
        lib = C.CDLL(os.path.join(os.path.dirname(os.path.abspath(cv.__file__)), "lib", "libcvamd_bench.so"))
        self.fn = lib.cvamdBenchStreamMix
        self.fn.restype = C.c_int
        self.fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32]

    def make_set(self):
        src = self.torch.randint(0, 255, (16 * self.lanes * self.reads,), dtype=self.torch.uint8, device="cuda")
        return src, self.torch.empty(16 * self.lanes * self.writes, dtype=self.torch.uint8, device="cuda")

    def submit(self, stream, s):
        assert self.fn(self.cv.stream_ptr(stream), s[0].data_ptr(), s[1].data_ptr(), self.lanes, self.reads, self.writes) == 0

    def check(self, s):
        # chunk 0 of the output is the XOR of every input chunk of the lane
        n = min(self.lanes, 4096)
        src = s[0].view(self.reads, self.lanes, 16)[:, :n].cpu().numpy()
        want = src[0].copy()
        for k in range(1, self.reads):
            want ^= src[k]
        got = s[1].view(self.writes, self.lanes, 16)[0, :n].cpu().numpy()
        assert (got == want).all()

    def cpu(self, threads):
        return 0


class Streaming:
    """Operators either side of the five configurations, each on a 1080p batch: algorithmic bytes are
    the input plus the output, the check is the oracle (or the numpy index map) on the first image."""
    config_id = 0
    H, W = 1080, 1920
    SPECS = {
        # key: (operator, batch, in dtype/channels, out dtype/channels/layout, kernel, arithmetic type, text)
        "cvtcolor-bgr2rgb": ("CvtColor", 32, ("uint8", 3), ("uint8", 3, "NHWC"), "SwizzleTensor<uint8_t,3,3>", "u8",
                             "CvtColor BGR2RGB"),
        "cvtcolor-bgr2gray": ("CvtColor", 32, ("uint8", 3), ("uint8", 1, "NHWC"), "MapTensor<GrayFromBgr<uint8_t,3>>",
                              "int32", "CvtColor BGR2GRAY"),
        "normalize-u8": ("Normalize", 32, ("uint8", 3), ("uint8", 3, "NHWC"), "NormRunsTensor<uint8_t,uint8_t,3>",
                         "f32", "Normalize (per-channel base/scale)"),
        "normalize-f32": ("Normalize", 16, ("float32", 3), ("float32", 3, "NHWC"), "NormRunsTensor<float,float,3>",
                          "f32", "Normalize (per-channel base/scale)"),
        "reformat-nhwc-nchw": ("Reformat", 32, ("uint8", 3), ("uint8", 3, "NCHW"),
                               "ReformatRunsKernel<uint8_t,3,true,false>", "u8", "Reformat NHWC -> NCHW"),
        "convertto-u8-f32": ("ConvertTo", 32, ("uint8", 3), ("float32", 3, "NHWC"), "ConvertKernel<uint8_t,float>",
                             "f32", "ConvertTo x 1/255"),
        "flip-horizontal": ("Flip", 32, ("uint8", 3), ("uint8", 3, "NHWC"), "PixelMapTensor<uint8_t,3>", "u8",
                            "Flip (columns mirrored)"),
        "resize-linear-720p": ("Resize", 32, ("uint8", 3), ("uint8", 3, "NHWC", 720, 1280),
                               "ResizeLinearPairsU8Kernel<3>", "i32", "Resize LINEAR 1920x1080 -> 1280x720"),
        "resize-linear-upscale": ("Resize", 32, ("uint8", 3, 720, 1280), ("uint8", 3, "NHWC", 1080, 1920),
                                  "ResizeLinearQuadsU8Kernel<3>", "i32", "Resize LINEAR 1280x720 -> 1920x1080"),
        "resize-cubic-720p": ("Resize", 32, ("uint8", 3), ("uint8", 3, "NHWC", 720, 1280),
                              "ResizeCubicStripU8Kernel<3,4>", "i32", "Resize CUBIC 1920x1080 -> 1280x720"),
        "resize-cubic-upscale": ("Resize", 32, ("uint8", 3, 720, 1280), ("uint8", 3, "NHWC", 1080, 1920),
                                 "ResizeCubicStripU8Kernel<3,8>", "i32", "Resize CUBIC 1280x720 -> 1920x1080"),
        "resize-nearest-upscale": ("Resize", 32, ("uint8", 3, 720, 1280), ("uint8", 3, "NHWC", 1080, 1920),
                                   "ResizeNearestQuadsU8Kernel<3>", "f32", "Resize NEAREST 1280x720 -> 1920x1080"),
        "resize-area-720p": ("Resize", 32, ("uint8", 3), ("uint8", 3, "NHWC", 720, 1280),
                             "ResizeAreaFixedTensorKernel<3>", "i32", "Resize AREA 1920x1080 -> 1280x720"),
        "cvtcolor-bgr2hsv": ("CvtColor", 32, ("uint8", 3), ("uint8", 3, "NHWC"), "MapTensor<HsvFromBgr<uint8_t,false>>", "f32",
                             "CvtColor BGR2HSV"),
        "cvtcolor-bgr2nv12": ("CvtColor", 32, ("uint8", 3), ("uint8", 1, "NHWC", 1620, 1920),
                              "PixelTensor<Yuv420FromBgr<3,true>>", "int32", "CvtColor BGR2YUV_NV12"),
        "cvtcolor-yuy2-bgr": ("CvtColor", 32, ("uint8", 1, 1080, 3840), ("uint8", 3, "NHWC", 1080, 1920), "PixelTensor<BgrFromYuv422<3>>", "int32",
                              "CvtColor YUV2BGR_YUY2"),
    }
    # what differs from the operator's default call above: colour code by name, interpolation
    CODES = {"cvtcolor-bgr2rgb": "COLOR_BGR2RGB", "cvtcolor-bgr2gray": "COLOR_BGR2GRAY", "cvtcolor-bgr2hsv": "COLOR_BGR2HSV",
             "cvtcolor-bgr2nv12": "COLOR_BGR2YUV_NV12", "cvtcolor-yuy2-bgr": "COLOR_YUV2BGR_YUY2"}
    INTERP = {"resize-area-720p": AREA, "resize-cubic-720p": CUBIC, "resize-cubic-upscale": CUBIC,
              "resize-nearest-upscale": NEAREST}

    def __init__(self, cv, orc, np, torch, key):
        self.cv, self.orc, self.np, self.torch, self.key = cv, orc, np, torch, key
        opname, self.N, src, dst, self.kernel, self.dtype, text = self.SPECS[key]
        self.images = self.N
        self.sdt, self.sc = np.dtype(src[0]), src[1]
        self.sh, self.sw = (src[2], src[3]) if len(src) > 2 else (self.H, self.W)
        self.ddt, self.dc, self.dlayout = np.dtype(dst[0]), dst[1], dst[2]
        self.dh, self.dw = (dst[3], dst[4]) if len(dst) > 3 else (self.sh, self.sw)
        self.workload = "%s: batch %d %s NHWC %dx%dx%d -> %s %s %dx%dx%d" % (
            text, self.N, self.sdt.name, self.sw, self.sh, self.sc, self.ddt.name, self.dlayout, self.dw, self.dh, self.dc)
        self.alg_bytes = self.N * (self.sh * self.sw * self.sc * self.sdt.itemsize
                                   + self.dh * self.dw * self.dc * self.ddt.itemsize)
        one = orc.fill_u8((1, self.sh, self.sw, self.sc), SEED_BASE + 77)
        self.host1 = one if self.sdt == np.uint8 else (one.astype(np.float32) / 255.0)
        self.dev1 = torch.from_numpy(self.host1).cuda()
        self.op = getattr(cv, opname)()
        self.opname = opname
        if opname == "Normalize":
            self.base = np.array([[[[104.0, 117.0, 123.0]]]], np.float32) / (1.0 if self.sdt == np.uint8 else 255.0)
            self.scale = np.array([[[[0.9, 1.1, 1.3]]]], np.float32)
            self.tbase, self.tscale = cv.Tensor.from_numpy(self.base, "NHWC"), cv.Tensor.from_numpy(self.scale, "NHWC")

    def make_set(self):
        tin = self.cv.Tensor.alloc([self.N, self.sh, self.sw, self.sc], self.sdt, "NHWC")
        tin.torch_view().copy_(self.dev1.expand(self.N, -1, -1, -1))
        shape = [self.N, self.dc, self.dh, self.dw] if self.dlayout == "NCHW" else [self.N, self.dh, self.dw, self.dc]
        return tin, self.cv.Tensor.alloc(shape, self.ddt, self.dlayout)

    def submit(self, stream, s):
        K = self.cv.K
        if self.opname == "CvtColor":
            self.op(stream, s[0], s[1], getattr(K, self.CODES[self.key]))
        elif self.opname == "Normalize":
            self.op(stream, s[0], self.tbase, self.tscale, s[1], 1.0, 0.0, 0.0, 0)
        elif self.opname == "Reformat":
            self.op(stream, s[0], s[1])
        elif self.opname == "ConvertTo":
            self.op(stream, s[0], s[1], 1.0 / 255.0, 0.0)
        elif self.opname == "Flip":
            self.op(stream, s[0], s[1], 1)
        else:
            self.op(stream, s[0], s[1], self.INTERP.get(self.key, LINEAR))

    def _color_oracle(self):
        if not hasattr(self, "_col"):
            import importlib.util
            spec = importlib.util.spec_from_file_location(
                "color_oracle", os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle", "color_oracle.py"))
            self._col = importlib.util.module_from_spec(spec)
            spec.loader.exec_module(self._col)
        return self._col

    def _reference(self, a, threads=1):
        np, orc = self.np, self.orc
        if self.key == "cvtcolor-bgr2hsv":
            return self._color_oracle().hsv_from_bgr(a, True, False)
        if self.key == "cvtcolor-bgr2nv12":
            return self._color_oracle().yuv420_from_bgr(a, True, 0, False)
        if self.key == "cvtcolor-yuy2-bgr":
            return self._color_oracle().bgr_from_yuv422(a, True, 0, 0, 3)
        if self.opname == "CvtColor":
            if self.dc == 3:
                return np.ascontiguousarray(a[..., ::-1])
            b, g, r = (a[..., i].astype(np.int64) for i in range(3))
            return ((b * 3735 + g * 19235 + r * 9798 + (1 << 14)) >> 15).astype(np.uint8)[..., None]
        if self.opname == "Normalize":
            return orc.normalize(a, self.base, self.scale, 1.0, 0.0, 0.0, False, threads=threads)
        if self.opname == "Reformat":
            return np.ascontiguousarray(a.transpose(0, 3, 1, 2))
        if self.opname == "ConvertTo":
            return orc.convert_to(a, np.float32, 1.0 / 255.0, 0.0, 1)
        if self.opname == "Flip":
            return np.ascontiguousarray(a[:, :, ::-1])
        return orc.resize_shipped(a, (self.dh, self.dw), self.INTERP.get(self.key, LINEAR), threads=threads)

    def check(self, s):
        got = s[1].torch_view()[:1].cpu().numpy()
        ref = self._reference(self.host1)
        if self.ddt == self.np.float32:
            assert (self.np.abs(got - ref) <= 1e-5 * self.np.maximum(1.0, self.np.abs(ref))).all()
        elif self.key == "cvtcolor-bgr2hsv":  # float path: products may round apart by one step on a few pixels
            assert self.np.abs(got.astype(self.np.int16) - ref.astype(self.np.int16)).max() <= 1
            assert (got != ref).mean() < 1e-3
        else:
            assert (got == ref).all(), "bench output differs from the oracle"

    def cpu_cores(self, threads):
        # the numpy index maps and the element-wise conversion run on one thread
        return threads if self.opname in ("Normalize", "Resize") else 1

    def cpu(self, threads):
        self._reference(self.np.repeat(self.host1, 4, axis=0), threads)
        return 4


WORKLOADS = {
    "empty-launch": EmptyLaunch,
    "fused": Fused,
    "fused-normalize": lambda *a: Fused(*a, "fused-normalize"),
    "fused-chain": lambda *a: Fused(*a, "fused-chain"),
    "fused-copy-bound": lambda *a: Fused(*a, "fused-copy-bound"),
    "resize-nearest": lambda *a: ResizeC1(*a, NEAREST),
    "resize-linear": lambda *a: ResizeC1(*a, LINEAR),
    "nv12-to-rgb": Nv12C3,
    "warp-affine-varshape": WarpC4,
    "fused-varshape": FusedVarShape,
    "resize-linear-varshape": ResizeVarShape,
    "crop-flip-normalize-224": CropFlipNormalize,
    "warp-affine-tensor-nearest": lambda *a: WarpTensor(*a, NEAREST),
    "warp-affine-tensor-linear": lambda *a: WarpTensor(*a, LINEAR),
    "warp-affine-tensor-cubic": lambda *a: WarpTensor(*a, CUBIC),
    "resize-cubic-4k": CubicC5,
}
WORKLOADS.update({k: (lambda *a, k=k: Streaming(*a, k)) for k in Streaming.SPECS})
WORKLOADS.update({k: (lambda *a, k=k: StreamMix(*a, k)) for k in StreamMix.SPECS})


# What each workload's dominant kernel is bound by, from its hardware counters (profiles/*_sq_counters.txt):
# "hbm" unless named here. "valu-issue": the vector-ALU instructions of the launch take most of its time at one
# wave-instruction per CU and cycle; "vmem-issue": the texture addresser is busy for most of the launch (gathers and
# loads that are not dword aligned cost cache accesses, not bytes); "launch-latency": the launch floor plus one ramp
# of memory latency is more than half of the time (batch 8).
BOUNDS = {"warp-affine-varshape": "valu-issue", "warp-affine-tensor-linear": "valu-issue",
          "warp-affine-tensor-cubic": "valu-issue", "warp-affine-tensor-nearest": "vmem-issue",
          "resize-area-720p": "valu-issue", "resize-cubic-720p": "valu-issue", "cvtcolor-bgr2hsv": "valu-issue",
          "resize-linear-720p": "valu-issue", "resize-linear-upscale": "valu-issue", "resize-cubic-upscale": "valu-issue",
          "resize-nearest": "launch-latency", "resize-linear": "launch-latency", "empty-launch": "launch-latency"}

# The other BASELINE configurations, timed after the headline when no --workload is given.
OTHER_CONFIGS = ("resize-nearest", "resize-linear", "nv12-to-rgb", "warp-affine-varshape", "resize-cubic-4k")
MIN_GRAPH_LAUNCHES = 500


def measure(wl, torch, steps, warmup, rotate, use_graph, streams, min_seconds):
    """Times `wl` on the current device: `warmup` eager Submits, then a HIP graph of max(steps, 500) Submits
    (so that what is timed does not depend on --steps: a graph of a few dozen launches pays a graph-launch gap
    every few dozen kernels) replayed until the timed region holds at least `min_seconds` of device work.
    Returns the buffer sets and the figures."""
    nsets = rotate if rotate > 0 else max(3, math.ceil(1.5e9 / max(wl.alg_bytes, 1)) if wl.alg_bytes else 1)
    sets = [wl.make_set() for _ in range(nsets)]
    stream = torch.cuda.current_stream()
    torch.cuda.synchronize()
    for i in range(warmup):
        wl.submit(stream, sets[i % nsets])
    torch.cuda.synchronize()

    # Default: the Submits are captured once into a HIP graph (a Submit only validates on the host and launches
    # one kernel, so it is capturable) and the replay is timed; this keeps the Python call overhead (~10 us per
    # Submit) out of a ~20 us kernel's way. --no-graph times eager Submits.
    mode, graph = "eager", None
    launches = max(steps, MIN_GRAPH_LAUNCHES) if use_graph else steps
    if use_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            sides = [torch.cuda.Stream() for _ in range(streams)] if streams > 1 else []
            with torch.cuda.graph(graph):
                cap = torch.cuda.current_stream()
                for sd in sides:
                    sd.wait_stream(cap)
                for i in range(launches):
                    wl.submit(sides[i % len(sides)] if sides else cap, sets[i % nsets])
                for sd in sides:
                    cap.wait_stream(sd)
            graph.replay()  # untimed first replay
            torch.cuda.synchronize()
            mode = "hipgraph"
        except Exception as e:  # capture unsupported -> measure eagerly and say so
            sys.stderr.write("bench.py: graph capture failed (%s), timing eager submits\n" % e)
            graph, launches = None, steps
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def run_once():
        if graph is not None:
            graph.replay()
        else:
            for i in range(launches):
                wl.submit(stream, sets[i % nsets])

    # One untimed pass sizes the timed region. With a few dozen steps of a ~20 us kernel the clocks would
    # otherwise mostly see the host's launch and synchronisation latency, and the device would still be
    # ramping its memory clocks up.
    torch.cuda.synchronize()
    e0.record(stream)
    run_once()
    e1.record(stream)
    torch.cuda.synchronize()
    est_s = max(e0.elapsed_time(e1) * 1e-3, 1e-6)
    replays = max(1, min(100000, math.ceil(min_seconds / est_s)))
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(replays):
        run_once()
    e1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    timed = launches * replays
    # mean launch-to-launch duration of a step on the device over the timed region: HIP events on the stream the
    # kernels are launched on. Consecutive launches overlap the end of one kernel with the start of the next, so
    # this can be a few tenths of a microsecond below the begin-to-end duration a kernel trace shows per kernel.
    mean_kernel_ms = e0.elapsed_time(e1) / timed
    return {"sets": sets, "nsets": nsets, "graph": graph, "mode": mode, "launches": launches, "replays": replays,
            "timed": timed, "wall": wall, "mean_kernel_ms": mean_kernel_ms, "stream": stream}


def cpu_baseline(wl, seconds, single_seconds):
    """The CPU oracle on a bounded sample of the workload: all host threads (at most 16), then one thread."""
    if seconds <= 0 or wl.images <= 0:
        return None

    def leg(threads, budget):
        reps, done, tcpu = 0, 0, 0.0
        c0 = time.perf_counter()
        while reps < 2 or tcpu < budget:
            done += wl.cpu(threads)
            reps += 1
            tcpu = time.perf_counter() - c0
        return done, tcpu

    threads = min(os.cpu_count() or 1, 16)
    done, tcpu = leg(threads, seconds)
    used = wl.cpu_cores(threads) if hasattr(wl, "cpu_cores") else threads
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "")
    except OSError:
        pass
    cpu = {"value": round(done / tcpu, 1), "unit": "images/s", "cores": used, "kind": "port",
           "host": {"cpu_model": model, "logical_cpus": os.cpu_count()},
           "sample": "%d images of this workload through the CPU oracle in %.1f s, %d thread%s"
                     % (done, tcpu, used, "" if used == 1 else "s")}
    if single_seconds > 0:
        done1, tcpu1 = leg(1, single_seconds)
        cpu["single_thread"] = {"value": round(done1 / tcpu1, 1), "unit": "images/s", "cores": 1,
                                "sample": "%d images in %.1f s, 1 thread" % (done1, tcpu1)}
    return cpu


def roofline_of(wl, mean_kernel_ms):
    achieved = wl.alg_bytes / (mean_kernel_ms * 1e-3) / 1e9
    return {"bound": BOUNDS.get(wl.key, "hbm"), "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(wl.key),
            "kernel": wl.kernel, "kernel_ms_mean": round(mean_kernel_ms, 5),
            "algorithmic_bytes_per_launch": wl.alg_bytes}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default=None,
                    help="one workload only (default: the headline, fused, followed by the other BASELINE "
                         "configurations under the key `configs`)")
    ap.add_argument("--rotate", type=int, default=0,
                    help="distinct buffer sets cycled through (0 = at least 3 and enough for 1.5 GB of algorithmic bytes, 1 = cache-resident)")
    ap.add_argument("--no-graph", action="store_true", help="time eager Submits instead of a HIP-graph replay")
    ap.add_argument("--min-seconds", type=float, default=0.3,
                    help="the captured launches are replayed until the timed region holds at least this much device work")
    ap.add_argument("--cpu-seconds", type=float, default=8.0, help="time budget of the CPU-oracle leg (0 = skip)")
    ap.add_argument("--batch", type=int, default=0,
                    help="images per step for the fused and resize-nearest / resize-linear workloads (0 = the "
                         "configuration's own batch size); for fits of launch time against batch size")
    ap.add_argument("--streams", type=int, default=1,
                    help="independent streams the steps are dealt to inside the captured graph (default 1: every "
                         "step waits for the one before, as consecutive Submits on one stream do)")
    ap.add_argument("--no-check", action="store_true", help="skip the oracle spot check (kernel experiments only)")
    ap.add_argument("--no-mover", action="store_true",
                    help="skip the plain byte mover that the fused, nv12-to-rgb and resize-cubic-4k workloads time beside "
                         "the operator (roofline.dense_mover)")
    ap.add_argument("--no-configs", action="store_true",
                    help="with no --workload: time the headline only, not the other BASELINE configurations")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MiB",
                    help="after the timed region, also run a plain device copy of this many MiB three times "
                         "(a kernel of known traffic to scale hardware byte counters against)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (the path shards by batch with no exchange); "
                 "--gpus %d is not supported" % args.gpus)
    all_configs = args.workload is None and not args.no_configs and args.batch == 0
    if args.workload is None:
        args.workload = "fused"

    import numpy as np
    import torch

    root = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, root)
    import __graft_entry__ as entry

    cv = entry.load_package()
    orc = entry.load_oracle()
    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    torch.cuda.set_device(0)

    # ---- inputs resident in HBM ----------------------------------------------------------------
    if args.batch > 0:
        if args.workload.startswith("fused"):
            Fused.N = args.batch
        elif args.workload in ("resize-nearest", "resize-linear"):
            ResizeC1.N = args.batch
        else:
            sys.exit("bench.py: --batch applies to the fused and resize-nearest / resize-linear workloads")
    wl = WORKLOADS[args.workload](cv, orc, np, torch)
    m = measure(wl, torch, args.steps, args.warmup, args.rotate, not args.no_graph, args.streams, args.min_seconds)
    sets, nsets, graph, stream = m["sets"], m["nsets"], m["graph"], m["stream"]
    mean_kernel_ms = m["mean_kernel_ms"]

    # One step from Submit to the end of its work, eagerly and one at a time: what a caller that waits for every
    # result sees (the Python call, the descriptor upload of image batches, the launch, the kernel, the wake-up).
    eager = []
    for i in range(20):
        torch.cuda.synchronize()
        c0 = time.perf_counter()
        wl.submit(stream, sets[i % nsets])
        torch.cuda.synchronize()
        eager.append(time.perf_counter() - c0)
    submit_to_sync_ms = sorted(eager)[len(eager) // 2] * 1e3

    # ---- the same bytes through a kernel that only moves them (dense 16-byte loads, streaming stores, no
    # arithmetic): what the memory system gives a launch of this size, measured in this run beside the operator
    mover = None
    mover_key = getattr(wl, "mover", None)
    if mover_key and not args.no_mover and graph is not None:
        mw = StreamMix(cv, orc, np, torch, mover_key)
        msets = [mw.make_set() for _ in range(max(3, int(math.ceil(2 * 268e6 / (16 * mw.lanes * mw.reads)))))]
        msteps = MIN_GRAPH_LAUNCHES
        for i in range(len(msets)):
            mw.submit(stream, msets[i])
        torch.cuda.synchronize()
        mgraph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(mgraph):
            mcap = torch.cuda.current_stream()
            for i in range(msteps):
                mw.submit(mcap, msets[i % len(msets)])
        mgraph.replay()
        torch.cuda.synchronize()
        mreps = max(1, int(math.ceil(0.1 / max(msteps * mean_kernel_ms * 1e-3, 1e-6))))
        m0, m1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        m0.record(stream)
        for _ in range(mreps):
            mgraph.replay()
        m1.record(stream)
        torch.cuda.synchronize()
        mover_ms = m0.elapsed_time(m1) / (msteps * mreps)
        mw.check(msets[0])
        mover = {"workload": mover_key, "kernel": mw.kernel, "bytes_per_launch": mw.alg_bytes,
                 "ms_per_launch": round(mover_ms, 5), "GB/s": round(mw.alg_bytes / (mover_ms * 1e-3) / 1e9, 1),
                 "operator_over_mover": round(mean_kernel_ms / mover_ms, 4)}
        del mgraph, msets

    if args.copy_probe > 0:
        a = torch.full((args.copy_probe << 20,), 7, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        del a, b

    # ---- correctness spot check of what was just produced (set 0)
    if not args.no_check:
        wl.check(sets[0])

    # ---- CPU oracle on the same workload (bounded sample)
    cpu = cpu_baseline(wl, args.cpu_seconds, args.cpu_seconds / 2)

    out = {
        "metric": "images/sec and achieved HBM GB/s (% of roofline), 1 MI355X",
        "value": round(wl.images * m["timed"] / m["wall"], 1),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "launches_per_graph": m["launches"],
        "replays": m["replays"],
        "warmup": args.warmup,
        "ms_per_step": round(m["wall"] / m["timed"] * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl.dtype,
        "data": "synthetic",
        "config": {"workload": wl.workload, "rotate_buffer_sets": nsets, "launch": m["mode"],
                   "streams": args.streams if graph is not None else 1},
        "roofline": roofline_of(wl, mean_kernel_ms),
        "cpu_baseline": cpu,
        "submit_to_sync_ms": round(submit_to_sync_ms, 4),
    }
    if mover is not None:
        out["roofline"]["dense_mover"] = mover
    if getattr(wl, "other_bytes", None):
        # the same launch time under two other byte conventions: the whole input and output tensors (what the
        # reference's own benchmarks count), and only the pixels an output pixel refers to plus the output
        out["roofline"]["other_conventions"] = {
            k: {"bytes_per_launch": v, "GB/s": round(v / (mean_kernel_ms * 1e-3) / 1e9, 1)}
            for k, v in wl.other_bytes.items()}

    # ---- the other BASELINE configurations, each the same way on a smaller budget: HBM-cold buffer rotation,
    # at least 0.1 s of device work, an oracle spot check, the CPU oracle for about 2 s
    if all_configs:
        configs = [{"workload": wl.key, "description": wl.workload, "images_per_launch": wl.images,
                    "images_per_s": out["value"], "cpu_baseline": cpu, **out["roofline"]}]
        del sets, graph, m, wl
        for key in OTHER_CONFIGS:
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            w2 = WORKLOADS[key](cv, orc, np, torch)
            m2 = measure(w2, torch, args.steps, min(args.warmup, 50), args.rotate, not args.no_graph, 1,
                         min(args.min_seconds, 0.1))
            if not args.no_check:
                w2.check(m2["sets"][0])
            entry2 = {"workload": key, "description": w2.workload, "images_per_launch": w2.images,
                      "images_per_s": round(w2.images * m2["timed"] / m2["wall"], 1),
                      "cpu_baseline": cpu_baseline(w2, min(args.cpu_seconds, 1.5), 0.0)}
            entry2.update(roofline_of(w2, m2["mean_kernel_ms"]))
            configs.append(entry2)
            del m2, w2
        out["configs"] = configs
    print(json.dumps(out))


if __name__ == "__main__":
    main()
