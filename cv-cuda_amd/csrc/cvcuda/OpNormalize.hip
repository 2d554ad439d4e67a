// Normalize: out = sat((in - base) * scale * global_scale + shift), or with SCALE_IS_STDDEV
// out = sat((in - base) * (1 / sqrt(scale^2 + epsilon)) * global_scale + shift), evaluated in float32
// left to right without FMA contraction.
//
// Follows src/cvcuda/priv/legacy/normalize.cu:35-93 (kernels) and :301-421 (validation) for tensors,
// normalize_var_shape.cu:36-68, 227-308 for var-shape batches (there the output may be u8 or f32
// whatever the input type, and base/scale are one value or one value per channel).
//
// Kernel shapes: base/scale that vary per channel only (the usual mean/stddev vectors, and always
// for var-shape batches) are read once per wave and the image is streamed in runs of 4 pixels per
// lane; base/scale with extents along N, H or W go through the generic kernel, one lane per pixel,
// which addresses them with per-dimension strides that are 0 along broadcast dimensions.
#include "DeviceUtils.hpp"
#include "OpCommon.hpp"
#include "RunIO.hpp"
#include "VarShapeTiles.hpp"

#include <cvcuda/OpNormalize.h>

#include <algorithm>

namespace cvamd {

namespace {

struct ParamView
{
    const float *ptr;
    int64_t      sN, sH, sW, sC; // strides in floats; 0 along broadcast dimensions
};

struct NormArgs
{
    const uint8_t *src;
    uint8_t       *dst;
    int64_t        srcN, dstN;
    int32_t        srcRow, dstRow;
    int32_t        W, H;
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
    ParamView base, scale;
    float     gscale, shift, eps;
    int32_t   stddev;
};

template<class T, int C>
using Vec = Packed<T, C>;

template<class TI, class TO, int C>
__device__ __forceinline__ void NormPixel(const NormArgs &a, const uint8_t *srcRow, uint8_t *dstRow, int n, int y, int x)
{
    const Vec<TI, C> in = reinterpret_cast<const Vec<TI, C> *>(srcRow)[x];
    const float     *pb = a.base.ptr + n * a.base.sN + y * a.base.sH + x * a.base.sW;
    const float     *ps = a.scale.ptr + n * a.scale.sN + y * a.scale.sH + x * a.scale.sW;
    Vec<TO, C>      *o  = reinterpret_cast<Vec<TO, C> *>(dstRow) + x;
    // parameters whose channels are adjacent come as one load per pixel (wave-uniform choice), and a pixel of whole
    // dwords leaves as one store: per channel, both were a third of the rate on 3-channel float images
    float bv[C], sv[C];
    if (a.base.sC == 1)
    {
        const Vec<float, C> t = *reinterpret_cast<const Vec<float, C> *>(pb);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            bv[c] = t.v[c];
        }
    }
    else
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            bv[c] = pb[c * a.base.sC];
        }
    }
    if (a.scale.sC == 1)
    {
        const Vec<float, C> t = *reinterpret_cast<const Vec<float, C> *>(ps);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            sv[c] = t.v[c];
        }
    }
    else
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            sv[c] = ps[c * a.scale.sC];
        }
    }
    Vec<TO, C> out;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        const float b = bv[c];
        const float s = sv[c];
        float       mul;
        if (a.stddev)
        {
            const float t = s * s + a.eps;
            mul           = 1.0f / sqrtf(t);
        }
        else
        {
            mul = s;
        }
        const float v = ((float)in.v[c] - b) * mul * a.gscale + a.shift;
        out.v[c]      = SaturateCast<TO>(v);
    }
    if constexpr (sizeof(Vec<TO, C>) % 4 == 0)
    {
        uint32_t w[sizeof(Vec<TO, C>) / 4];
        __builtin_memcpy(w, &out, sizeof(w));
        StoreDwordsNT<sizeof(Vec<TO, C>) / 4>(reinterpret_cast<uint8_t *>(o), w);
    }
    else
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            __builtin_nontemporal_store(out.v[c], &o->v[c]);
        }
    }
}

template<class TI, class TO, int C>
__global__ __launch_bounds__(256) void NormTensor(const NormArgs a)
{
    const int x = blockIdx.x * 64 + (threadIdx.x & 63);
    const int y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.W || y >= a.H)
    {
        return;
    }
    const int n = blockIdx.z;
    NormPixel<TI, TO, C>(a, a.src + n * a.srcN + (int64_t)y * a.srcRow, a.dst + n * a.dstN + (int64_t)y * a.dstRow, n, y,
                         x);
}

template<class TI, class TO, int C>
__global__ __launch_bounds__(256) void NormVarShape(const NormArgs a, const VarTiles tiles)
{
    const TileCoord              tc = LocateTile(tiles, blockIdx.x);
    const NVCVImagePlaneStrided &s  = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided &d  = a.dstList[tc.image].planes[0];
    const int                    x  = tc.tx * 64 + (threadIdx.x & 63);
    const int                    y  = tc.ty * 4 + (threadIdx.x >> 6);
    if (x >= d.width || y >= d.height)
    {
        return;
    }
    NormPixel<TI, TO, C>(a, AsGlobal(s.basePtr) + (int64_t)y * s.rowStride, AsGlobal(d.basePtr) + (int64_t)y * d.rowStride, 0, 0, x);
}

// Pixels per lane of the run kernels: kRunPixelsFor, and for single-channel images as many as make 16 bytes on the
// wider side (a lane that moves 4 bytes per instruction left the kernel at 3.3 of the 6.5 TB/s the 3-channel form
// reaches on cached inputs).
template<class TI, class TO, int C>
constexpr int kNormRunPixels = C == 1 ? 16 / (int)(sizeof(TI) > sizeof(TO) ? sizeof(TI) : sizeof(TO)) : kRunPixelsFor<TI, TO>;

// Per-channel base/scale: runs of P pixels per lane, one row per wave.
template<class TI, class TO, int C>
__device__ __forceinline__ void NormRun(const NormArgs &a, const uint8_t *srcRow, uint8_t *dstRow, int W, int x0)
{
    constexpr int P = kNormRunPixels<TI, TO, C>;
    // every uniform value is loaded before the first use, so the loads share one round trip
    float b[C], m[C];
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        b[c] = a.base.ptr[c * a.base.sC];
        m[c] = a.scale.ptr[c * a.scale.sC];
    }
    if (a.stddev)
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            const float t = m[c] * m[c] + a.eps;
            m[c]          = 1.0f / sqrtf(t);
        }
    }
    if (x0 + P <= W)
    {
        TI in[P * C];
        TO out[P * C];
        LoadRun<TI, P * C>(srcRow + (int64_t)x0 * C * sizeof(TI), in);
        if (a.gscale == 1.f && a.shift == 0.f) // wave-uniform; x * 1 + 0 == x, two operations per element saved
        {
#pragma unroll
            for (int i = 0; i < P * C; ++i)
            {
                out[i] = SaturateCast<TO>(((float)in[i] - b[i % C]) * m[i % C]);
            }
        }
        else
        {
#pragma unroll
            for (int i = 0; i < P * C; ++i)
            {
                out[i] = SaturateCast<TO>(((float)in[i] - b[i % C]) * m[i % C] * a.gscale + a.shift);
            }
        }
        // the wave's lanes 0 .. lanes-1 hold consecutive pieces of the row
        const int lane = threadIdx.x & 63, lanes = min(64, (W - (x0 - lane * P)) / P);
        StoreRowRunNT<TO, P * C>(dstRow + (int64_t)(x0 - lane * P) * C * sizeof(TO), out, lane, lanes);
    }
    else
    {
        for (int x = x0; x < W; ++x)
        {
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                const float v = ((float)reinterpret_cast<const TI *>(srcRow)[x * C + c] - b[c]) * m[c] * a.gscale + a.shift;
                reinterpret_cast<TO *>(dstRow)[x * C + c] = SaturateCast<TO>(v);
            }
        }
    }
}

template<class TI, class TO, int C>
__global__ __launch_bounds__(256) void NormRunsTensor(const NormArgs a)
{
    const int x0 = (blockIdx.x * 64 + (threadIdx.x & 63)) * kNormRunPixels<TI, TO, C>;
    const int y  = blockIdx.y * kRunTileH + (threadIdx.x >> 6);
    if (x0 >= a.W || y >= a.H)
    {
        return;
    }
    const int n = blockIdx.z;
    NormRun<TI, TO, C>(a, a.src + n * a.srcN + (int64_t)y * a.srcRow, a.dst + n * a.dstN + (int64_t)y * a.dstRow, a.W,
                       x0);
}

template<class TI, class TO, int C>
constexpr int kVarRows = kVarShapeRows<kNormRunPixels<TI, TO, C> * C * (int)sizeof(TO)>;

template<class TI, class TO, int C>
__global__ __launch_bounds__(256) void NormRunsVarShape(const NormArgs a, const VarTiles tiles)
{
    const TileCoord              tc = LocateTile(tiles, blockIdx.x);
    const NVCVImagePlaneStrided &s  = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided &d  = a.dstList[tc.image].planes[0];
    const int                    x0 = (tc.tx * 64 + (threadIdx.x & 63)) * kNormRunPixels<TI, TO, C>;
    const uint8_t *src = AsGlobal(s.basePtr);
    uint8_t       *dst = AsGlobal(d.basePtr);
    const int      W = d.width, H = d.height, srcRow = s.rowStride, dstRow = d.rowStride;
    if (x0 >= W)
    {
        return;
    }
    constexpr int R = kVarRows<TI, TO, C>;
    for (int r = 0; r < R; ++r)
    {
        const int y = (tc.ty * R + r) * kRunTileH + (threadIdx.x >> 6);
        if (y >= H)
        {
            return;
        }
        NormRun<TI, TO, C>(a, src + (int64_t)y * srcRow, dst + (int64_t)y * dstRow, W, x0);
    }
}

inline bool PerChannelOnly(const ParamView &p)
{
    return p.sN == 0 && p.sH == 0 && p.sW == 0;
}

template<class TI, class TO, int C>
void Launch(const NormArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    if (PerChannelOnly(a.base) && PerChannelOnly(a.scale))
    {
        if (dstHost == nullptr)
        {
            dim3 grid(DivUp(a.W, 64 * kNormRunPixels<TI, TO, C>), DivUp(a.H, kRunTileH), N);
            hipLaunchKernelGGL((NormRunsTensor<TI, TO, C>), grid, dim3(256), 0, stream, a);
            CheckLaunch("NormRunsTensor");
            return;
        }
        for (int first = 0; first < N; first += kMaxTileImages)
        {
            VarTiles tiles;
            int total = BuildVarTiles(tiles, dstHost, first, std::min(kMaxTileImages, N - first),
                                      64 * kNormRunPixels<TI, TO, C>, kRunTileH * kVarRows<TI, TO, C>);
            if (total > 0)
            {
                hipLaunchKernelGGL((NormRunsVarShape<TI, TO, C>), dim3(total), dim3(256), 0, stream, a, tiles);
                CheckLaunch("NormRunsVarShape");
            }
        }
        return;
    }
    if (dstHost == nullptr)
    {
        dim3 grid(DivUp(a.W, 64), DivUp(a.H, 4), N);
        hipLaunchKernelGGL((NormTensor<TI, TO, C>), grid, dim3(256), 0, stream, a);
        CheckLaunch("NormTensor");
        return;
    }
    for (int first = 0; first < N; first += kMaxTileImages)
    {
        VarTiles tiles;
        int      total = BuildVarTiles(tiles, dstHost, first, std::min(kMaxTileImages, N - first), 64, 4);
        if (total > 0)
        {
            hipLaunchKernelGGL((NormVarShape<TI, TO, C>), dim3(total), dim3(256), 0, stream, a, tiles);
            CheckLaunch("NormVarShape");
        }
    }
}

template<class TI, class TO>
void DispatchC(int C, const NormArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    switch (C)
    {
    case 1:
        Launch<TI, TO, 1>(a, N, dstHost, stream);
        break;
    case 2:
        Launch<TI, TO, 2>(a, N, dstHost, stream);
        break;
    case 3:
        Launch<TI, TO, 3>(a, N, dstHost, stream);
        break;
    case 4:
        Launch<TI, TO, 4>(a, N, dstHost, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", C);
    }
}

// out: 0 = same as input, 1 = u8, 2 = f32
template<class TI>
void DispatchOut(int outSel, int C, const NormArgs &a, int N, const NVCVImageBufferStrided *dstHost,
                 hipStream_t stream)
{
    if (outSel == 0)
    {
        DispatchC<TI, TI>(C, a, N, dstHost, stream);
    }
    else if (outSel == 1)
    {
        DispatchC<TI, uint8_t>(C, a, N, dstHost, stream);
    }
    else
    {
        DispatchC<TI, float>(C, a, N, dstHost, stream);
    }
}

void DispatchIn(ElemType in, int outSel, int C, const NormArgs &a, int N, const NVCVImageBufferStrided *dstHost,
                hipStream_t stream)
{
    if (N == 0)
    {
        return;
    }
    switch (in)
    {
    case kU8:
        DispatchOut<uint8_t>(outSel, C, a, N, dstHost, stream);
        break;
    case kS8:
        DispatchOut<int8_t>(outSel, C, a, N, dstHost, stream);
        break;
    case kU16:
        DispatchOut<uint16_t>(outSel, C, a, N, dstHost, stream);
        break;
    case kS16:
        DispatchOut<int16_t>(outSel, C, a, N, dstHost, stream);
        break;
    case kS32:
        DispatchOut<int32_t>(outSel, C, a, N, dstHost, stream);
        break;
    case kF32:
        DispatchOut<float>(outSel, C, a, N, dstHost, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
    }
}

// base / scale tensor -> broadcast view against an input of (N,H,W,C)
ParamView MakeParam(NVCVTensorHandle h, const char *what, int N, int H, int W, int C, bool varshape)
{
    NVCVTensorData d;
    ExportTensor(h, d, what);
    ImageBatchView v = RequireImageBatchView(d, what, NVCV_ERROR_INVALID_ARGUMENT);
    if (v.elem != kF32 || v.layout != kLayoutNHWC)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s tensor must hold float32 values in [N]HWC layout", what);
    }
    if (varshape)
    {
        // one value, or one per channel: of a longer vector the first C are used, as the reference reads it
        // (legacy/normalize_var_shape.cu:107-140 takes the tensor's first element as a C-vector)
        if (v.N != 1 || v.H != 1 || v.W != 1 || (v.C != 1 && v.C < C))
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s tensor must have shape [1,1,1,1] or [1,1,1,%d]", what, C);
        }
    }
    else if ((v.N != N && v.N != 1) || (v.H != H && v.H != 1) || (v.W != W && v.W != 1) || (v.C != C && v.C != 1))
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                      "%s tensor extents (%d,%d,%d,%d) must each be 1 or match the input's (%d,%d,%d,%d)", what, v.N,
                      v.H, v.W, v.C, N, H, W, C);
    }
    if (v.strideN % 4 || v.strideH % 4 || v.strideW % 4)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s tensor strides must be multiples of 4 bytes", what);
    }
    ParamView p;
    p.ptr = reinterpret_cast<const float *>(v.base);
    p.sN  = v.N == 1 ? 0 : v.strideN / 4;
    p.sH  = v.H == 1 ? 0 : v.strideH / 4;
    p.sW  = v.W == 1 ? 0 : v.strideW / 4;
    p.sC  = v.C == 1 ? 0 : 1;
    return p;
}

class Normalize final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hbase, NVCVTensorHandle hscale,
                NVCVTensorHandle hout, float gscale, float shift, float eps, uint32_t flags) const
    {
        NVCVTensorData din, dout;
        ExportTensor(hin, din, "Input");
        ExportTensor(hout, dout, "Output");
        ImageBatchView in  = RequireImageBatchView(din, "Input", NVCV_ERROR_INVALID_ARGUMENT);
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
        if (in.layout != kLayoutNHWC || out.layout != kLayoutNHWC || in.hasBatchDim != out.hasBatchDim)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Invalid DataFormat between input (%s) and output (%s): both must be \"NHWC\" or \"HWC\"",
                          in.layoutName, out.layoutName);
        }
        if (in.C > 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", in.C);
        }
        if (in.elem != out.elem || in.N != out.N || in.H != out.H || in.W != out.W || in.C != out.C)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input and output must have the same data type and shape");
        }
        if (std::max(in.bytesSpanned(), out.bytesSpanned()) > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output size exceeds %d. Tensor is too large.",
                          INT32_MAX);
        }
        NormArgs a = {};
        a.base     = MakeParam(hbase, "Base", in.N, in.H, in.W, in.C, false);
        a.scale    = MakeParam(hscale, "Scale", in.N, in.H, in.W, in.C, false);
        a.src      = in.base;
        a.dst      = out.base;
        a.srcN     = in.strideN;
        a.dstN     = out.strideN;
        a.srcRow   = (int32_t)in.strideH;
        a.dstRow   = (int32_t)out.strideH;
        a.W        = in.W;
        a.H        = in.H;
        a.gscale   = gscale;
        a.shift    = shift;
        a.eps      = eps;
        a.stddev   = (flags & CVCUDA_NORMALIZE_SCALE_IS_STDDEV) ? 1 : 0;
        if (in.W == 0 || in.H == 0)
        {
            return;
        }
        DispatchIn(in.elem, 0, in.C, a, in.N, nullptr, stream);
    }

    void submit(hipStream_t stream, NVCVImageBatchHandle hin, NVCVTensorHandle hbase, NVCVTensorHandle hscale,
                NVCVImageBatchHandle hout, float gscale, float shift, float eps, uint32_t flags) const
    {
        VarShapeView in  = ExportVarShape(hin, stream, "Input");
        VarShapeView out = ExportVarShape(hout, stream, "Output");
        if (in.N != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input and output batch sizes: %d != %d", in.N, out.N);
        }
        if (in.uniqueFormat == NVCV_IMAGE_FORMAT_NONE || out.uniqueFormat == NVCV_IMAGE_FORMAT_NONE)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images in the input (output) batch must all share one format");
        }
        FormatInfo fi = DecodeFormat(in.uniqueFormat), fo = DecodeFormat(out.uniqueFormat);
        if (fi.planes != 1 || fo.planes != 1 || fi.channels != fo.channels)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Input and output images must be single-plane with the same number of channels");
        }
        if (fo.elem != kU8 && fo.elem != kF32)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid Output DataType, must be u8 or f32");
        }
        if (fi.channels > 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", fi.channels);
        }
        for (int i = 0; i < in.N; ++i)
        {
            if (in.hostList[i].planes[0].width != out.hostList[i].planes[0].width
                || in.hostList[i].planes[0].height != out.hostList[i].planes[0].height)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Image %d: input and output sizes differ", i);
            }
        }
        NormArgs a = {};
        a.base     = MakeParam(hbase, "Base", 1, 1, 1, fi.channels, true);
        a.scale    = MakeParam(hscale, "Scale", 1, 1, 1, fi.channels, true);
        a.srcList  = in.data.buffer.varShapeStrided.imageList;
        a.dstList  = out.data.buffer.varShapeStrided.imageList;
        a.gscale   = gscale;
        a.shift    = shift;
        a.eps      = eps;
        a.stddev   = (flags & CVCUDA_NORMALIZE_SCALE_IS_STDDEV) ? 1 : 0;
        // base/scale are indexed at (0,0,0): NormVarShape passes n = y = 0 and the W stride is 0
        DispatchIn(fi.elem, fo.elem == kU8 ? 1 : 2, fi.channels, a, in.N, out.hostList, stream);
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaNormalizeCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<Normalize>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaNormalizeSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                               NVCVTensorHandle base, NVCVTensorHandle scale, NVCVTensorHandle out,
                                               float global_scale, float shift, float epsilon, uint32_t flags)
{
    return Protect(
        [&] { ToOperator<Normalize>(handle).submit(stream, in, base, scale, out, global_scale, shift, epsilon, flags); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaNormalizeVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                       NVCVImageBatchHandle in, NVCVTensorHandle base,
                                                       NVCVTensorHandle scale, NVCVImageBatchHandle out,
                                                       float global_scale, float shift, float epsilon, uint32_t flags)
{
    return Protect(
        [&] { ToOperator<Normalize>(handle).submit(stream, in, base, scale, out, global_scale, shift, epsilon, flags); });
}
}
