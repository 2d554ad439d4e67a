// Fused resize -> crop -> scale/offset/convert -> channel reorder -> layout change.
//
// Arithmetic follows the reference's kernels (src/cvcuda/priv/OpResizeCropConvertReformat.cu:137-278)
// expression for expression in float32 without FMA contraction; validation order and status codes
// follow its operator() (:418-683).
//
// Kernel shape (gfx950, wave64): one lane per output column, each wave produces kRowsPerWave output
// rows (one: see FusedTiles.hpp), a 256-thread block covers 64 columns x 4*kRowsPerWave rows. The x-dependent terms (source column, weight)
// are computed once per lane and reused for all its rows. Source taps are two adjacent u8x3 pixels,
// i.e. 6 contiguous bytes, fetched with ONE unaligned 8-byte load per source row; consecutive lanes
// read addresses ~3*scale bytes apart, so a wave touches a dense run of cache lines and the HBM
// traffic equals the row span the output needs. Output stores are one element per lane per plane
// (planar: 256 contiguous bytes per wave).
#include "DeviceUtils.hpp"
#include "FusedTiles.hpp"
#include "LaneExchange.hpp"
#include "OpCommon.hpp"

#include <cvcuda/OpNormalize.h>
#include <cvcuda/OpResizeCropConvertReformat.h>

#include <algorithm>
#include <cmath>

namespace cvamd {

namespace {

template<class DstT, bool NORM>
__device__ __forceinline__ DstT Finish(const FusedArgs &a, float v, int c)
{
    if constexpr (NORM)
    {
        // the value an f32 fused output would hold, then the Normalize operator's expression
        const float x = a.scale * v + a.offset;
        return SaturateCast<DstT>((x - a.normBase[c]) * a.normMul[c] * a.normGlobal + a.normShift);
    }
    else
    {
        return SaturateCast<DstT>(a.scale * v + a.offset);
    }
}

// One output pixel per lane, lane l of the wave at column dx = 64 * tile + l of row `rowOut` (the row's
// first element). Streaming (non-temporal) stores: the output is written once and not read back by this
// kernel, so it should not displace source lines in L2 / the memory-side cache (on MI355X this alone
// shortens the batch-64 1080p -> 224x224 launch by ~15 %). Interleaved outputs leave as whole pixels:
// three separate element stores per lane complete every 32-byte sector in three instructions, which
// costs write traffic (f32 NHWC: 29.7 -> 24 us per batch). f32 pixels are one 12-byte store; u8 pixels
// are packed into dwords across the wave through LDS first.
template<class DstT, bool NORM, bool PLANAR = false>
__device__ __forceinline__ void StorePixel(const FusedArgs &a, DstT *rowOut, int dx, float v0, float v1, float v2)
{
    const DstT f0 = Finish<DstT, NORM>(a, v0, 0), f1 = Finish<DstT, NORM>(a, v1, 1), f2 = Finish<DstT, NORM>(a, v2, 2);
    if (PLANAR || a.interleaved == 0)
    {
        DstT *out = rowOut + dx * a.dstStrideX;
        StoreStreamThrough(f0, out + a.dstOffC[0]);
        StoreStreamThrough(f1, out + a.dstOffC[1]);
        StoreStreamThrough(f2, out + a.dstOffC[2]);
        return;
    }
    const bool rev   = a.interleaved == 2;
    const DstT o[3]  = {rev ? f2 : f0, f1, rev ? f0 : f2};
    uint8_t   *bytes = reinterpret_cast<uint8_t *>(rowOut);
    if constexpr (sizeof(DstT) == 4)
    {
        uint32_t w[3];
        __builtin_memcpy(w, o, 12);
        StoreDwordsNT<3>(bytes + (int64_t)dx * 12, w);
    }
    else
    {
        static_assert(sizeof(DstT) == 1, "outputs are u8 or f32");
        // lanes 0 .. n-1 of the wave hold the 3-byte pixels of columns x0 .. x0+n-1
        __shared__ __attribute__((aligned(4))) uint8_t stage[4][64 * 3];
        const int lane = threadIdx.x & 63, x0 = dx - lane, n = min(64, a.dstW - x0);
        uint8_t  *mine = stage[threadIdx.x >> 6];
        mine[lane * 3 + 0] = o[0];
        mine[lane * 3 + 1] = o[1];
        mine[lane * 3 + 2] = o[2];
        WaveExchangeFence();
        const int total = n * 3, dwords = total >> 2;
        uint8_t  *to    = bytes + (int64_t)x0 * 3;
        if (lane < dwords)
        {
            uint32_t w[1];
            __builtin_memcpy(w, mine + lane * 4, 4);
            StoreDwordsNT<1>(to + lane * 4, w);
        }
        // the row's last 1-3 bytes, all from lane 0: only the lanes of columns inside the output are here, and a
        // wave that holds the row's last column alone has 3 bytes to store
        if (lane == 0)
        {
            for (int i = dwords * 4; i < total; ++i)
            {
                __builtin_nontemporal_store(mine[i], to + i);
            }
        }
        WaveExchangeFence(); // the next row reuses the staging area
    }
}

template<class DstT, bool VARSHAPE, bool NORM>
__global__ __launch_bounds__(256) void FusedNearest(const FusedArgs a)
{
    const TilePos tp   = LocateFusedTile(a);
    const int     n    = tp.n;
    const int     dx   = FusedColumnOf(tp.tx, a.wavesAcross);
    const int     dy0  = FusedFirstRowOf(tp.ty, a.wavesAcross);
    if (dx >= a.dstW)
    {
        return;
    }
    const SrcImage s   = GetSource<VARSHAPE>(a, n);
    DstT          *dst = static_cast<DstT *>(a.dstBase) + n * a.dstStrideN;

    int sx = (int)floorf((dx + a.cropX + 0.5f) * s.scaleX);
    sx     = min(sx, s.w - 1);
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r)
    {
        const int dy = dy0 + r;
        if (dy >= a.dstH)
        {
            break;
        }
        int sy = (int)floorf((dy + a.cropY + 0.5f) * s.scaleY);
        sy     = min(sy, s.h - 1);
        const uint8_t *p = s.base + (int64_t)sy * s.rowStride + sx * 3;
        StorePixel<DstT, NORM>(a, dst + (int64_t)dy * a.dstStrideY, dx, (float)p[0], (float)p[1], (float)p[2]);
    }
}

// BYTEWISE=false: each source row is fetched with one unaligned 8-byte load per lane (LoadTapPairs; needs
// an image of >= 8 bytes). BYTEWISE=true: plain byte loads, used for images smaller than 8 bytes.
// PLANAR=true: the caller knows that the output is not pixel-interleaved (a.interleaved == 0), which takes the
// interleaved store paths and their branch out of the kernel.
template<class DstT, bool VARSHAPE, bool BYTEWISE, bool NORM, bool PLANAR>
__global__ __launch_bounds__(256) void FusedBilinear(const FusedArgs a)
{
    const TilePos tp   = LocateFusedTile(a);
    const int     n    = tp.n;
    const int     dx   = FusedColumnOf(tp.tx, a.wavesAcross);
    const int     dy0  = FusedFirstRowOf(tp.ty, a.wavesAcross);
    if (dx >= a.dstW)
    {
        return;
    }
    const SrcImage s   = GetSource<VARSHAPE>(a, n);
    DstT          *dst = static_cast<DstT *>(a.dstBase) + n * a.dstStrideN;

    const FusedColumn col = ColumnTerms(a, s, dx); // shared by all rows of this lane
    const float       fx = col.fx, wx0 = 1 - col.fx;
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
        const float    fy  = row.fy;

        uint32_t a0, a1, b0, b1; // bytes 0..2 of a0/b0: first tap of the upper/lower row; a1/b1: second tap
        if constexpr (BYTEWISE)
        {
            const int      x1 = col.twoTap ? 3 : 0;
            const uint8_t *p0 = s.base + row.off0, *p1 = s.base + row.off1;
            a0 = p0[0] | (p0[1] << 8) | (p0[2] << 16);
            a1 = p0[x1] | (p0[x1 + 1] << 8) | (p0[x1 + 2] << 16);
            b0 = p1[0] | (p1[1] << 8) | (p1[2] << 16);
            b1 = p1[x1] | (p1[x1 + 1] << 8) | (p1[x1 + 2] << 16);
        }
        else
        {
            LoadTapPairs(s, row, lastLoad, col.twoTap, a0, a1, b0, b1);
        }
        float v[3];
#pragma unroll
        for (int c = 0; c < 3; ++c)
        {
            const float p00 = (float)((a0 >> (8 * c)) & 0xFF);
            const float p01 = (float)((a1 >> (8 * c)) & 0xFF);
            const float p10 = (float)((b0 >> (8 * c)) & 0xFF);
            const float p11 = (float)((b1 >> (8 * c)) & 0xFF);
            float       t   = (1 - fy) * (wx0 * p00 + p01 * fx) + fy * (wx0 * p10 + p11 * fx);
            if (a.srcCast)
            {
                t = (float)SaturateCast<uint8_t>(t);
            }
            v[c] = t;
        }
        StorePixel<DstT, NORM, PLANAR>(a, dst + (int64_t)dy * a.dstStrideY, dx, v[0], v[1], v[2]);
    }
}

template<class DstT, bool VARSHAPE, bool NORM>
void LaunchKernels(FusedArgs a, int N, NVCVInterpolationType interp, bool tinyImages, hipStream_t stream)
{
    if (N == 0 || a.dstW == 0 || a.dstH == 0)
    {
        return;
    }
    if ((a.dstW + 63) / 64 > (INT32_MAX / (int)kXcdCount) || a.dstH / (int)kXcdCount >= 65535)
    {
        throw OpError(NVCV_ERROR_OVERFLOW, "Output of %d x %d needs too many tiles for one launch", a.dstW, a.dstH);
    }
    const dim3 block(256);
    for (int first = 0; first < N; first += kFusedImagesPerLaunch)
    {
        a.firstImage    = (uint32_t)first;
        const dim3 grid = SetFusedGrid(a, std::min(N - first, kFusedImagesPerLaunch));
        if (interp == NVCV_INTERP_NEAREST)
        {
            hipLaunchKernelGGL((FusedNearest<DstT, VARSHAPE, NORM>), grid, block, 0, stream, a);
            CheckLaunch("FusedNearest");
        }
        else
        {
            if (tinyImages)
            {
                hipLaunchKernelGGL((FusedBilinear<DstT, VARSHAPE, true, NORM, false>), grid, block, 0, stream, a);
            }
            else if (a.interleaved == 0)
            {
                hipLaunchKernelGGL((FusedBilinear<DstT, VARSHAPE, false, NORM, true>), grid, block, 0, stream, a);
            }
            else
            {
                hipLaunchKernelGGL((FusedBilinear<DstT, VARSHAPE, false, NORM, false>), grid, block, 0, stream, a);
            }
            CheckLaunch("FusedBilinear");
        }
    }
}

template<class DstT, bool VARSHAPE>
void Launch(const FusedArgs &a, bool normalize, int N, NVCVInterpolationType interp, bool tinyImages, hipStream_t stream)
{
    if (normalize)
    {
        LaunchKernels<DstT, VARSHAPE, true>(a, N, interp, tinyImages, stream);
    }
    else
    {
        LaunchKernels<DstT, VARSHAPE, false>(a, N, interp, tinyImages, stream);
    }
}

class ResizeCropConvertReformat final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, NVCVSize2D resizeDim,
                NVCVInterpolationType interp, int2 cropPos, NVCVChannelManip manip, float scale, float offset,
                bool srcCast, const CVCUDAXChannelNormalize *norm = nullptr) const
    {
        NVCVTensorData din, dout;
        ExportTensor(hin, din, "Input");
        ExportTensor(hout, dout, "Output");
        // Layout problems are NOT_COMPATIBLE for this operator; a tensor that is not an image batch
        // at all is reported the same way.
        ImageBatchView in  = RequireImageBatchView(din, "Input", NVCV_ERROR_NOT_COMPATIBLE);
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_NOT_COMPATIBLE);

        checkCommon(in.N, in.C, in.elem, /*srcPlanes*/ 1, out);
        if (in.layout != kLayoutNHWC)
        {
            throw OpError(NVCV_ERROR_NOT_COMPATIBLE, "Input tensor must have 'NHWC' or 'HWC' layout: Layout provided %s",
                          in.layoutName);
        }
        if (resizeDim.w <= 1 || resizeDim.h <= 1)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Invalid resize dimensions: width x hight = %d x %d dimensions must be larger than 1.",
                          resizeDim.w, resizeDim.h);
        }
        checkCrop(cropPos, out, resizeDim.w, resizeDim.h);
        if (in.bytesSpanned() > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_OVERFLOW, "Input size exceeds %d. Tensor is too large.", INT32_MAX);
        }
        checkInterp(interp);

        FusedArgs a       = makeArgs(out, resizeDim, cropPos, manip, scale, offset, srcCast, norm);
        a.srcBase         = in.base;
        a.srcSampleStride = in.strideN;
        a.srcRowStride    = (int32_t)in.strideH;
        a.srcW            = in.W;
        a.srcH            = in.H;
        a.scaleX          = static_cast<float>(in.W) / resizeDim.w;
        a.scaleY          = static_cast<float>(in.H) / resizeDim.h;
        const bool tiny = (int64_t)(in.H - 1) * in.strideH + (int64_t)in.W * 3 < 8;
        if (out.elem == kU8)
        {
            Launch<uint8_t, false>(a, norm != nullptr, in.N, interp, tiny, stream);
        }
        else
        {
            Launch<float, false>(a, norm != nullptr, in.N, interp, tiny, stream);
        }
    }

    void submit(hipStream_t stream, NVCVImageBatchHandle hin, NVCVTensorHandle hout, NVCVSize2D resizeDim,
                NVCVInterpolationType interp, int2 cropPos, NVCVChannelManip manip, float scale, float offset,
                bool srcCast, const CVCUDAXChannelNormalize *norm = nullptr) const
    {
        VarShapeView   in = ExportVarShape(hin, stream, "Input");
        NVCVTensorData dout;
        ExportTensor(hout, dout, "Output");
        if (in.uniqueFormat == NVCV_IMAGE_FORMAT_NONE)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "All input images in a batch must have the same format (including number of channels)");
        }
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_NOT_COMPATIBLE);
        FormatInfo     fi  = DecodeFormat(in.uniqueFormat);
        checkCommon(in.N, fi.channels, fi.elem, fi.planes, out);
        checkCrop(cropPos, out, std::abs(resizeDim.w), std::abs(resizeDim.h));
        checkInterp(interp);
        if (resizeDim.w <= 0 || resizeDim.h <= 0)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid resize dimensions: %d x %d", resizeDim.w, resizeDim.h);
        }
        FusedArgs a = makeArgs(out, resizeDim, cropPos, manip, scale, offset, srcCast, norm);
        a.srcList   = in.data.buffer.varShapeStrided.imageList;
        bool tiny = false;
        for (int i = 0; i < in.N; ++i)
        {
            const NVCVImagePlaneStrided &pl = in.hostList[i].planes[0];
            tiny = tiny || (int64_t)(pl.height - 1) * pl.rowStride + (int64_t)pl.width * 3 < 8;
        }
        if (out.elem == kU8)
        {
            Launch<uint8_t, true>(a, norm != nullptr, in.N, interp, tiny, stream);
        }
        else
        {
            Launch<float, true>(a, norm != nullptr, in.N, interp, tiny, stream);
        }
    }

private:
    static void checkCommon(int samples, int channels, ElemType srcElem, int srcPlanes, const ImageBatchView &out)
    {
        if (samples != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Input and output must have the same batch size (i.e., same number of images): Provided %d "
                          "input and %d output images / samples",
                          samples, out.N);
        }
        if (channels != out.C)
        {
            throw OpError(NVCV_ERROR_NOT_COMPATIBLE,
                          "Input and output must have same number of channels: Provided %d input and %d output channels",
                          channels, out.C);
        }
        if (channels != 3)
        {
            throw OpError(NVCV_ERROR_NOT_COMPATIBLE,
                          "Only three-channel input is currently supported: Provided %d input channels", channels);
        }
        if (srcElem != kU8)
        {
            throw OpError(NVCV_ERROR_NOT_COMPATIBLE, "Input must be of data type uchar.");
        }
        if (out.elem != kU8 && out.elem != kF32)
        {
            throw OpError(NVCV_ERROR_NOT_COMPATIBLE, "Output must be of data type uchar or float.");
        }
        if (srcPlanes > 1)
        {
            throw OpError(NVCV_ERROR_NOT_COMPATIBLE, "Input must be non-planar (i.e., interleaved).");
        }
    }

    static void checkCrop(int2 cropPos, const ImageBatchView &out, int newW, int newH)
    {
        if (cropPos.x < 0 || cropPos.y < 0 || cropPos.x + out.W > newW || cropPos.y + out.H > newH)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Invalid crop region: crop region(x, y, w, h) = (%d, %d, %d, %d) extends beyond bounds of "
                          "resized tensor",
                          cropPos.x, cropPos.y, out.W, out.H);
        }
    }

    static void checkInterp(NVCVInterpolationType interp)
    {
        if (interp != NVCV_INTERP_NEAREST && interp != NVCV_INTERP_LINEAR)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s",
                          interp == NVCV_INTERP_CUBIC  ? "Interpolation not implemented: NVCV_INTERP_CUBIC"
                          : interp == NVCV_INTERP_AREA ? "Interpolation not implemented: NVCV_INTERP_AREA"
                                                       : "Invalid interpolation");
        }
    }

    static FusedArgs makeArgs(const ImageBatchView &out, NVCVSize2D resizeDim, int2 cropPos, NVCVChannelManip manip,
                              float scale, float offset, bool srcCast, const CVCUDAXChannelNormalize *norm)
    {
        const int es = ElemSize(out.elem);
        if (out.strideN % es || out.strideH % es || out.strideW % es || out.strideC % es)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Output strides must be multiples of the element size");
        }
        FusedArgs a  = {};
        a.dstBase    = out.base;
        a.dstStrideN = out.strideN / es;
        a.dstStrideY = (int32_t)(out.strideH / es);
        a.dstStrideX = (int32_t)(out.strideW / es);
        for (int c = 0; c < 3; ++c)
        {
            int to       = manip == NVCV_CHANNEL_REVERSE ? 2 - c : c;
            a.dstOffC[c] = to * (out.strideC / es);
        }
        a.interleaved = (out.strideC == es && out.strideW == 3 * es) ? (manip == NVCV_CHANNEL_REVERSE ? 2 : 1) : 0;
        a.dstW        = out.W;
        a.dstH        = out.H;
        a.newW    = resizeDim.w;
        a.newH    = resizeDim.h;
        a.cropX   = cropPos.x;
        a.cropY   = cropPos.y;
        a.scale   = scale;
        a.offset  = offset;
        a.srcCast = srcCast ? 1 : 0;
        if (norm != nullptr)
        {
            if (norm->flags & ~(uint32_t)CVCUDA_NORMALIZE_SCALE_IS_STDDEV)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid normalization flags 0x%x", norm->flags);
            }
            for (int c = 0; c < 3; ++c)
            {
                // base / scale are given per OUTPUT channel; the kernel indexes by source channel
                const int   to = manip == NVCV_CHANNEL_REVERSE ? 2 - c : c;
                const float sc = norm->scale[to];
                a.normBase[c]  = norm->base[to];
                // same expression, in float32, as the Normalize operator evaluates on the device
                a.normMul[c] = (norm->flags & CVCUDA_NORMALIZE_SCALE_IS_STDDEV) ? 1.0f / std::sqrt(sc * sc + norm->epsilon)
                                                                                : sc;
            }
            a.normGlobal = norm->globalScale;
            a.normShift  = norm->shift;
        }
        return a;
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaResizeCropConvertReformatCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<ResizeCropConvertReformat>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaResizeCropConvertReformatSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                               NVCVTensorHandle in, NVCVTensorHandle out,
                                                               const NVCVSize2D            resizeDim,
                                                               const NVCVInterpolationType interpolation,
                                                               const int2 cropPos, const NVCVChannelManip manip,
                                                               const float scale, const float offset,
                                                               const bool srcCast)
{
    return Protect(
        [&]
        {
            ToOperator<ResizeCropConvertReformat>(handle).submit(stream, in, out, resizeDim, interpolation, cropPos,
                                                                 manip, scale, offset, srcCast);
        });
}

CVCUDA_PUBLIC NVCVStatus cvcudaResizeCropConvertReformatVarShapeSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVImageBatchHandle in, NVCVTensorHandle out,
    const NVCVSize2D resizeDim, const NVCVInterpolationType interpolation, const int2 cropPos,
    const NVCVChannelManip manip, const float scale, const float offset, const bool srcCast)
{
    return Protect(
        [&]
        {
            ToOperator<ResizeCropConvertReformat>(handle).submit(stream, in, out, resizeDim, interpolation, cropPos,
                                                                 manip, scale, offset, srcCast);
        });
}

CVCUDA_PUBLIC NVCVStatus cvcudaxResizeCropConvertReformatNormalizeSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in, NVCVTensorHandle out,
    const NVCVSize2D resizeDim, const NVCVInterpolationType interpolation, const int2 cropPos,
    const NVCVChannelManip manip, const float scale, const float offset, const bool srcCast,
    const CVCUDAXChannelNormalize *normalize)
{
    return Protect(
        [&]
        {
            if (normalize == nullptr)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Pointer to the normalization parameters must not be NULL");
            }
            ToOperator<ResizeCropConvertReformat>(handle).submit(stream, in, out, resizeDim, interpolation, cropPos,
                                                                 manip, scale, offset, srcCast, normalize);
        });
}

CVCUDA_PUBLIC NVCVStatus cvcudaxResizeCropConvertReformatNormalizeVarShapeSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVImageBatchHandle in, NVCVTensorHandle out,
    const NVCVSize2D resizeDim, const NVCVInterpolationType interpolation, const int2 cropPos,
    const NVCVChannelManip manip, const float scale, const float offset, const bool srcCast,
    const CVCUDAXChannelNormalize *normalize)
{
    return Protect(
        [&]
        {
            if (normalize == nullptr)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Pointer to the normalization parameters must not be NULL");
            }
            ToOperator<ResizeCropConvertReformat>(handle).submit(stream, in, out, resizeDim, interpolation, cropPos,
                                                                 manip, scale, offset, srcCast, normalize);
        });
}
}
