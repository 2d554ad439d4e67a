// Kernels the benchmark times beside the operators (libcvamd_bench.so, not part of the operator
// libraries): an empty kernel, a plain mover of bytes in a given read : write ratio, and
// FusedCopyBound, the copy-bound twin of the fused bilinear kernel: the same grid, the same
// workgroup -> tile map, the same four 8-byte tap loads per lane and the same three streaming stores
// per lane into an f32 NCHW batch, but no blend, no conversion and no scale/offset: the stored values
// are the loaded bytes. Its launch time is what the memory system allows a kernel of this access
// pattern; the fused kernel's time is compared with it.
#include "cvcuda/FusedTiles.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>

using namespace cvamd;

namespace {

__global__ __launch_bounds__(256) void FusedCopyBound(const FusedArgs a)
{
    const TilePos tp   = LocateFusedTile(a);
    const int     n    = tp.n;
    const int     dx   = FusedColumnOf(tp.tx, a.wavesAcross);
    const int     dy0  = FusedFirstRowOf(tp.ty, a.wavesAcross);
    if (dx >= a.dstW)
    {
        return;
    }
    const SrcImage    s        = GetSource<false>(a, n);
    float            *dst      = static_cast<float *>(a.dstBase) + n * a.dstStrideN;
    const FusedColumn col      = ColumnTerms(a, s, dx);
    const int64_t     lastLoad = LastTapLoad(s);
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
    {
        const int dy = dy0 + r;
        if (dy >= a.dstH)
        {
            break;
        }
        const FusedRow row = RowTerms(a, s, dy, col.xoff);
        uint32_t       a0, a1, b0, b1;
        LoadTapPairs(s, row, lastLoad, col.twoTap, a0, a1, b0, b1);
        float *out = dst + (int64_t)dy * a.dstStrideY + dx * a.dstStrideX;
        StoreStreamThrough(__uint_as_float(a0 & 0xFFFFFFu), out + a.dstOffC[0]);
        StoreStreamThrough(__uint_as_float(b0 & 0xFFFFFFu), out + a.dstOffC[1]);
        StoreStreamThrough(__uint_as_float((a1 ^ b1) & 0xFFFFFFu), out + a.dstOffC[2]);
    }
}

__global__ void EmptyKernel() {}

// R 16-byte chunks read and W written per lane, both streams dense over the wave (chunk k of lane i is
// chunk k * lanes + i of its stream): what the memory system gives a kernel that moves bytes in this
// ratio and does nothing else. The stored values depend on every loaded one.
template<int R, int W>
__global__ __launch_bounds__(256) void StreamMix(const uint4 *src, uint4 *dst, int64_t lanes)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= lanes)
    {
        return;
    }
    uint4 v[R];
#pragma unroll
    for (int k = 0; k < R; ++k)
    {
        v[k] = src[k * lanes + i];
    }
    uint32_t x = 0, y = 0, z = 0, w = 0;
#pragma unroll
    for (int k = 0; k < R; ++k)
    {
        x ^= v[k].x;
        y ^= v[k].y;
        z ^= v[k].z;
        w ^= v[k].w;
    }
#pragma unroll
    for (int k = 0; k < W; ++k)
    {
        uint32_t *o = reinterpret_cast<uint32_t *>(dst + (k * lanes + i));
        __builtin_nontemporal_store(x + k, o + 0);
        __builtin_nontemporal_store(y, o + 1);
        __builtin_nontemporal_store(z, o + 2);
        __builtin_nontemporal_store(w, o + 3);
    }
}

template<int R, int W>
int LaunchStreamMix(hipStream_t stream, const void *src, void *dst, int64_t lanes)
{
    hipLaunchKernelGGL((StreamMix<R, W>), dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), lanes);
    return (int)hipGetLastError();
}

} // namespace

// One launch of a kernel that does nothing: the cost of a dependent launch as the benchmark's clocks see it.
extern "C" __attribute__((visibility("default"))) int cvamdBenchEmptyLaunch(hipStream_t stream)
{
    hipLaunchKernelGGL(EmptyKernel, dim3(1), dim3(64), 0, stream);
    return (int)hipGetLastError();
}

// Reads `reads` x 16 bytes and writes `writes` x 16 bytes per lane, for `lanes` lanes: src holds at least
// reads * lanes * 16 bytes, dst writes * lanes * 16, both 16-byte aligned. Ratios built: 1:1, 1:2, 4:2, 24:1.
extern "C" __attribute__((visibility("default"))) int cvamdBenchStreamMix(hipStream_t stream, const void *src, void *dst,
                                                                          int64_t lanes, int32_t reads, int32_t writes)
{
    if (lanes <= 0 || lanes > ((int64_t)1 << 31) * 256 || ((uintptr_t)src | (uintptr_t)dst) % 16 != 0)
    {
        return (int)hipErrorInvalidValue;
    }
    if (reads == 1 && writes == 1)
    {
        return LaunchStreamMix<1, 1>(stream, src, dst, lanes);
    }
    if (reads == 1 && writes == 2)
    {
        return LaunchStreamMix<1, 2>(stream, src, dst, lanes);
    }
    if (reads == 4 && writes == 2)
    {
        return LaunchStreamMix<4, 2>(stream, src, dst, lanes);
    }
    if (reads == 24 && writes == 1)
    {
        return LaunchStreamMix<24, 1>(stream, src, dst, lanes);
    }
    return (int)hipErrorInvalidValue;
}

// src: u8 NHWC batch of N images (srcW x srcH x 3, given row and sample strides in bytes); dst: packed
// f32 NCHW batch N x 3 x dstH x dstW. Geometry as cvcudaResizeCropConvertReformatSubmit computes it for a
// resize to newW x newH and a crop at (cropX, cropY). Plane 0 / 1 of the output receive the 3 bytes of
// the upper / lower row's first tap as an integer bit pattern, plane 2 the second taps' XOR.
// Returns 0 on success, a hipError_t otherwise. Shapes are the caller's responsibility: crop inside the
// resized image, images of at least 8 bytes.
extern "C" __attribute__((visibility("default"))) int cvamdBenchFusedCopyBound(
    hipStream_t stream, const void *src, int64_t srcSampleStride, int32_t srcRowStride, int32_t srcW, int32_t srcH,
    void *dst, int32_t N, int32_t dstW, int32_t dstH, int32_t newW, int32_t newH, int32_t cropX, int32_t cropY)
{
    if (N <= 0 || dstW <= 0 || dstH <= 0 || newW <= 1 || newH <= 1 || cropX < 0 || cropY < 0 || cropX + dstW > newW
        || cropY + dstH > newH || (int64_t)(srcH - 1) * srcRowStride + (int64_t)srcW * 3 < 8)
    {
        return (int)hipErrorInvalidValue;
    }
    FusedArgs a       = {};
    a.srcBase         = static_cast<const uint8_t *>(src);
    a.srcSampleStride = srcSampleStride;
    a.srcRowStride    = srcRowStride;
    a.srcW            = srcW;
    a.srcH            = srcH;
    a.dstBase         = dst;
    a.dstStrideN      = (int64_t)3 * dstH * dstW;
    a.dstStrideY      = dstW;
    a.dstStrideX      = 1;
    for (int c = 0; c < 3; ++c)
    {
        a.dstOffC[c] = (int64_t)c * dstH * dstW;
    }
    a.dstW   = dstW;
    a.dstH   = dstH;
    a.newW   = newW;
    a.newH   = newH;
    a.cropX  = cropX;
    a.cropY  = cropY;
    a.scaleX = static_cast<float>(srcW) / newW;
    a.scaleY = static_cast<float>(srcH) / newH;
    if (N > kFusedImagesPerLaunch || dstH / (int)kXcdCount >= 65535)
    {
        return (int)hipErrorInvalidValue;
    }
    const dim3 grid = SetFusedGrid(a, N);
    hipLaunchKernelGGL(FusedCopyBound, grid, dim3(256), 0, stream, a);
    return (int)hipGetLastError();
}
