// CropFlipNormalizeReformat: var-shape batch -> tensor, one pass.
//
// Semantics follow src/cvcuda/priv/OpCropFlipNormalizeReformat.cu: coordinate map :165-187, zero fill
// outside the rectangle :157-161, expression and its order :73-74, scale / stddev :45-59, type tables
// :341-351 and :449-454, parameter checks :416-433, output layout :193-197.
//
// Two kernels, grid z = image; the crop rectangle, the flip code and the per-channel base / scale
// values are uniform per block and read in the prologue; streaming stores.
//  * The pipeline cases (interleaved u8 or f32 images to packed u8 / f32 NHWC or NCHW tensors): a
//    lane produces a run of 4 output pixels. Where the 4 source pixels lie inside the image they are
//    one vector load (reversed in registers for mirrored columns), otherwise they are fetched one by
//    one through the border rule; the run is stored as whole dwords, per plane for NCHW.
//  * Everything else: one lane per output pixel, source and destination addressed through
//    per-channel strides, so planar images and any destination strides run through the same code.
#include "DeviceUtils.hpp"
#include "OpCommon.hpp"
#include "RunIO.hpp"

#include <cvcuda/OpCropFlipNormalizeReformat.h>

#include <cmath>

namespace cvamd {

namespace {

struct CfnrArgs
{
    const NVCVImageBufferStrided *srcList;
    int32_t        srcPlanar;      // 1: channel c lives in plane c
    uint8_t       *dst;
    int64_t        dN, dH, dW, dC; // destination strides in bytes
    int32_t        W, H, C;        // output size
    const uint8_t *crop;           // int32[4] per image
    int64_t        cropStride;
    const uint8_t *flip;           // int32 per image
    int64_t        flipStride;
    const float   *base, *scale;   // device tensors, baseC / scaleC packed values each
    int32_t        baseC, scaleC;
    float          gscale, shift, eps;
    int32_t        stddev;
    int32_t        border;
    float          borderValue;
};

template<class TS, class TD>
__global__ __launch_bounds__(256) void CfnrKernel(const CfnrArgs a)
{
    const int x = blockIdx.x * 64 + (threadIdx.x & 63);
    const int y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.W || y >= a.H)
    {
        return;
    }
    const int      n    = blockIdx.z;
    const int32_t *rect = reinterpret_cast<const int32_t *>(a.crop + n * a.cropStride);
    const int      cx = rect[0], cy = rect[1], cw = rect[2], ch = rect[3];
    uint8_t       *d = a.dst + n * a.dN + y * a.dH + x * a.dW;
    if (x >= cw || y >= ch)
    {
        for (int c = 0; c < a.C; ++c)
        {
            __builtin_nontemporal_store((TD)0, reinterpret_cast<TD *>(d + c * a.dC));
        }
        return;
    }
    const int  code    = *reinterpret_cast<const int32_t *>(a.flip + n * a.flipStride);
    const bool mirrorX = code == 1 || code == -1, mirrorY = code == 0 || code == -1;
    int        sx = (mirrorX ? cw - 1 - x : x) + cx;
    int        sy = (mirrorY ? ch - 1 - y : y) + cy;

    const NVCVImageBufferStrided &img = a.srcList[n];
    const NVCVImagePlaneStrided  &p0  = img.planes[0];
    bool                          outside = false;
    if (sx < 0 || sx >= p0.width || sy < 0 || sy >= p0.height)
    {
        if (a.border == NVCV_BORDER_CONSTANT)
        {
            outside = true;
        }
        else
        {
            sx = BorderIndex(a.border, sx, p0.width);
            sy = BorderIndex(a.border, sy, p0.height);
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c)
    {
        if (c < a.C)
        {
            TS v;
            if (outside)
            {
                v = BorderValueAs<TS>(a.borderValue);
            }
            else if (a.srcPlanar)
            {
                const NVCVImagePlaneStrided &pl = img.planes[c];
                v = reinterpret_cast<const TS *>(AsGlobal(pl.basePtr) + (int64_t)sy * pl.rowStride)[sx];
            }
            else
            {
                v = reinterpret_cast<const TS *>(AsGlobal(p0.basePtr) + (int64_t)sy * p0.rowStride)[sx * a.C + c];
            }
            const float b = a.base[a.baseC == 1 ? 0 : c];
            const float s = a.scale[a.scaleC == 1 ? 0 : c];
            const float m = a.stddev ? 1.0f / sqrtf(s * s + a.eps) : s;
            const float r = ((float)v - b) * m * a.gscale + a.shift;
            __builtin_nontemporal_store(SaturateCast<TD>(r), reinterpret_cast<TD *>(d + c * a.dC));
        }
    }
}

// Runs of 4 output pixels per lane; interleaved source, destination rows packed (NHWC: pixel stride
// C elements, NCHW: pixel stride one element).
constexpr int kCfnrRowsPerWave = 1; // rows a wave works through (more per wave measured slower)

template<class TS, class TD, int C>
__global__ __launch_bounds__(256) void CfnrRunsKernel(const CfnrArgs a)
{
    constexpr int P  = kRunPixels;
    const int     x0 = (blockIdx.x * 64 + (threadIdx.x & 63)) * P;
    if (x0 >= a.W)
    {
        return;
    }
    const int      n    = blockIdx.z;
    const int32_t *rect = reinterpret_cast<const int32_t *>(a.crop + n * a.cropStride);
    const int      cx = rect[0], cy = rect[1], cw = rect[2], ch = rect[3];
    const int      code    = *reinterpret_cast<const int32_t *>(a.flip + n * a.flipStride);
    const bool     mirrorX = code == 1 || code == -1, mirrorY = code == 0 || code == -1;
    const NVCVImagePlaneStrided &p0 = a.srcList[n].planes[0];
    const uint8_t *srcBase = AsGlobal(p0.basePtr);
    const int      srcRow = p0.rowStride, srcW = p0.width, srcH = p0.height;
    // every uniform value is loaded before the first use, so the loads share one round trip
    float b[C], m[C];
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        b[c] = a.base[a.baseC == 1 ? 0 : c];
        m[c] = a.scale[a.scaleC == 1 ? 0 : c];
    }
    if (a.stddev)
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            m[c] = 1.0f / sqrtf(m[c] * m[c] + a.eps);
        }
    }
    const int  first  = mirrorX ? cw - 1 - (x0 + P - 1) + cx : x0 + cx; // lowest source column of the run
    const bool runIn  = x0 + P <= cw && first >= 0 && first + P <= srcW;
    const bool planar = a.dW == (int64_t)sizeof(TD) && C > 1;

#pragma unroll 2
    for (int r = 0; r < kCfnrRowsPerWave; ++r)
    {
        const int y = (blockIdx.y * kCfnrRowsPerWave + r) * kRunTileH + (threadIdx.x >> 6);
        if (y >= a.H)
        {
            break;
        }
        TD out[P * C];
#pragma unroll
        for (int i = 0; i < P * C; ++i)
        {
            out[i] = (TD)0; // outside the rectangle
        }
        if (x0 < cw && y < ch)
        {
            const int sy = (mirrorY ? ch - 1 - y : y) + cy;
            TS        in[P * C];
            if (runIn && sy >= 0 && sy < srcH)
            {
                // two branches with constant indices: a select between two indices would turn every
                // element into a chain of compares over the whole run
                TS raw[P * C];
                LoadRun<TS, P * C>(srcBase + (int64_t)sy * srcRow + (int64_t)first * C * sizeof(TS), raw);
                if (mirrorX)
                {
#pragma unroll
                    for (int k = 0; k < P; ++k)
                    {
#pragma unroll
                        for (int c = 0; c < C; ++c)
                        {
                            in[k * C + c] = raw[(P - 1 - k) * C + c];
                        }
                    }
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < P * C; ++i)
                    {
                        in[i] = raw[i];
                    }
                }
            }
            else
            {
                const int syIn = a.border == NVCV_BORDER_CONSTANT ? sy : BorderIndex(a.border, sy, srcH);
#pragma unroll
                for (int k = 0; k < P; ++k)
                {
                    int        sx      = (mirrorX ? cw - 1 - (x0 + k) : x0 + k) + cx;
                    const bool outside = a.border == NVCV_BORDER_CONSTANT && (sx < 0 || sx >= srcW || sy < 0 || sy >= srcH);
                    if (a.border != NVCV_BORDER_CONSTANT)
                    {
                        sx = BorderIndex(a.border, sx, srcW);
                    }
                    // pixels of the run beyond the rectangle are computed from a clamped column and dropped below
                    sx = outside ? 0 : min(max(sx, 0), srcW - 1);
                    const TS *px = reinterpret_cast<const TS *>(srcBase + (int64_t)(outside ? 0 : syIn) * srcRow) + sx * C;
#pragma unroll
                    for (int c = 0; c < C; ++c)
                    {
                        in[k * C + c] = outside ? BorderValueAs<TS>(a.borderValue) : px[c];
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < P; ++k)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    const float v  = ((float)in[k * C + c] - b[c]) * m[c] * a.gscale + a.shift;
                    out[k * C + c] = x0 + k < cw ? SaturateCast<TD>(v) : (TD)0;
                }
            }
        }
        uint8_t *d = a.dst + n * a.dN + y * a.dH + x0 * a.dW;
        if (x0 + P <= a.W)
        {
            if (planar)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    TD t[P];
#pragma unroll
                    for (int k = 0; k < P; ++k)
                    {
                        t[k] = out[k * C + c];
                    }
                    StoreRunNT<TD, P>(d + c * a.dC, t);
                }
            }
            else
            {
                const int lane = threadIdx.x & 63, lanes = min(64, (a.W - (x0 - lane * P)) / P);
                StoreRowRunNT<TD, P * C>(d - (int64_t)lane * P * C * sizeof(TD), out, lane, lanes);
            }
        }
        else
        {
#pragma unroll
            for (int k = 0; k < P - 1; ++k)
            {
                if (x0 + k < a.W)
                {
#pragma unroll
                    for (int c = 0; c < C; ++c)
                    {
                        *reinterpret_cast<TD *>(d + k * a.dW + c * a.dC) = out[k * C + c];
                    }
                }
            }
        }
    }
}

template<class TS, class TD>
constexpr bool kCfnrRuns = (std::is_same_v<TS, uint8_t> && (std::is_same_v<TD, uint8_t> || std::is_same_v<TD, float>))
                        || (std::is_same_v<TS, float> && std::is_same_v<TD, float>);

template<class TS, class TD>
void Launch(const CfnrArgs &a, int N, hipStream_t stream)
{
    if constexpr (kCfnrRuns<TS, TD>)
    {
        const bool nchw = a.dW == (int64_t)sizeof(TD);
        const bool nhwc = a.dC == (int64_t)sizeof(TD) && a.dW == (int64_t)(a.C * sizeof(TD));
        if (!a.srcPlanar && (nchw || nhwc))
        {
            dim3 grid(DivUp(a.W, kRunTileW), DivUp(a.H, kRunTileH * kCfnrRowsPerWave), N);
            switch (a.C)
            {
            case 1:
                hipLaunchKernelGGL((CfnrRunsKernel<TS, TD, 1>), grid, dim3(256), 0, stream, a);
                break;
            case 3:
                hipLaunchKernelGGL((CfnrRunsKernel<TS, TD, 3>), grid, dim3(256), 0, stream, a);
                break;
            default:
                hipLaunchKernelGGL((CfnrRunsKernel<TS, TD, 4>), grid, dim3(256), 0, stream, a);
                break;
            }
            CheckLaunch("CfnrRunsKernel");
            return;
        }
    }
    dim3 grid(DivUp(a.W, 64), DivUp(a.H, 4), N);
    hipLaunchKernelGGL((CfnrKernel<TS, TD>), grid, dim3(256), 0, stream, a);
    CheckLaunch("CfnrKernel");
}

template<class TS>
void DispatchDst(ElemType out, const CfnrArgs &a, int N, hipStream_t stream)
{
    switch (out)
    {
    case kU8:
        Launch<TS, uint8_t>(a, N, stream);
        break;
    case kS8:
        Launch<TS, int8_t>(a, N, stream);
        break;
    case kU16:
        Launch<TS, uint16_t>(a, N, stream);
        break;
    case kS16:
        Launch<TS, int16_t>(a, N, stream);
        break;
    case kS32:
        Launch<TS, int32_t>(a, N, stream);
        break;
    case kU32:
        Launch<TS, uint32_t>(a, N, stream);
        break;
    case kF32:
        Launch<TS, float>(a, N, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Unsupported output data type");
    }
}

void DispatchSrc(ElemType in, ElemType out, const CfnrArgs &a, int N, hipStream_t stream)
{
    switch (in)
    {
    case kU8:
        DispatchDst<uint8_t>(out, a, N, stream);
        break;
    case kS8:
        DispatchDst<int8_t>(out, a, N, stream);
        break;
    case kU16:
        DispatchDst<uint16_t>(out, a, N, stream);
        break;
    case kS16:
        DispatchDst<int16_t>(out, a, N, stream);
        break;
    case kS32:
        DispatchDst<int32_t>(out, a, N, stream);
        break;
    case kU32:
        DispatchDst<uint32_t>(out, a, N, stream);
        break;
    case kF32:
        DispatchDst<float>(out, a, N, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Unsupported input data type");
    }
}

// base / scale: float32 [N]HWC tensor whose channel count is 1 or >= C; only element (0,0,0,c) is used
void CheckParam(NVCVTensorHandle h, const char *what, int C, const float *&ptr, int32_t &channels)
{
    NVCVTensorData d;
    ExportTensor(h, d, what);
    ImageBatchView v = RequireImageBatchView(d, what, NVCV_ERROR_INVALID_ARGUMENT);
    if (v.elem != kF32 || v.layout != kLayoutNHWC)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s tensor must hold float32 values in [N]HWC layout", what);
    }
    if (!(v.C == 1 || v.C >= C))
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Channel of %s tensor must be 1 or >= input/output tensor channels",
                      what);
    }
    if (v.C > 1 && v.strideC != 4)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s tensor channels must be packed", what);
    }
    ptr      = reinterpret_cast<const float *>(v.base);
    channels = v.C;
}

class CropFlipNormalizeReformat final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVImageBatchHandle hin, NVCVTensorHandle hout, NVCVTensorHandle hcrop,
                NVCVBorderType border, float borderValue, NVCVTensorHandle hflip, NVCVTensorHandle hbase,
                NVCVTensorHandle hscale, float gscale, float shift, float eps, uint32_t flags) const
    {
        VarShapeView   in = ExportVarShape(hin, stream, "Input");
        NVCVTensorData dout;
        ExportTensor(hout, dout, "Output");
        if (in.uniqueFormat == NVCV_IMAGE_FORMAT_NONE)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images in the input batch must all have the same format");
        }
        FormatInfo fi = DecodeFormat(in.uniqueFormat);
        if (fi.channels != 1 && fi.channels != 3 && fi.channels != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", fi.channels);
        }
        if (fi.planes != 1 && fi.planes != fi.channels)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input images must be interleaved or fully planar");
        }
        if (dout.rank != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid tensor layout in output");
        }
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
        if (out.N != in.N || out.C != fi.channels)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Output must hold %d images of %d channels: provided %d images of %d channels", in.N,
                          fi.channels, out.N, out.C);
        }
        if (out.bytesSpanned() > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_OVERFLOW, "Output size exceeds %d. Tensor is too large.", INT32_MAX);
        }
        if ((int)border < NVCV_BORDER_CONSTANT || (int)border > NVCV_BORDER_REFLECT101)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Unsupported border mode");
        }

        CfnrArgs a  = {};
        a.srcList   = in.data.buffer.varShapeStrided.imageList;
        a.srcPlanar = fi.planes > 1 ? 1 : 0;
        a.dst       = out.base;
        a.dN        = out.strideN;
        a.dH        = out.strideH;
        a.dW        = out.strideW;
        a.dC        = out.strideC;
        a.W         = out.W;
        a.H         = out.H;
        a.C         = out.C;

        NVCVTensorData dcrop, dflip;
        ExportTensor(hcrop, dcrop, "Crop rectangle");
        DTypeInfo tc = DecodeDataType(dcrop.dtype);
        if (tc.elem != kS32 || tc.channels != 1 || dcrop.rank != 4 || dcrop.shape[0] < in.N || dcrop.shape[1] != 1
            || dcrop.shape[2] != 1 || dcrop.shape[3] != 4 || dcrop.buffer.strided.strides[3] != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Crop rectangle tensor must be int32 of shape [N,1,1,4], N >= %d",
                          in.N);
        }
        a.crop       = dcrop.buffer.strided.basePtr;
        a.cropStride = dcrop.buffer.strided.strides[0];

        ExportTensor(hflip, dflip, "Flip code");
        DTypeInfo tf    = DecodeDataType(dflip.dtype);
        int64_t   count = 1;
        for (int i = 0; i < dflip.rank; ++i)
        {
            count *= dflip.shape[i];
        }
        if (tf.elem != kS32 || tf.channels != 1 || dflip.rank < 1 || dflip.shape[0] != count || count < in.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Flip code tensor must hold one int32 per image (%d)", in.N);
        }
        a.flip       = dflip.buffer.strided.basePtr;
        a.flipStride = dflip.buffer.strided.strides[0];

        CheckParam(hbase, "Base", a.C, a.base, a.baseC);
        CheckParam(hscale, "Scale", a.C, a.scale, a.scaleC);
        a.gscale      = gscale;
        a.shift       = shift;
        a.eps         = eps;
        a.stddev      = flags != 0 ? 1 : 0; // the reference converts the flags word to bool
        a.border      = border;
        a.borderValue = borderValue;
        if (in.N == 0 || a.W == 0 || a.H == 0)
        {
            return;
        }
        DispatchSrc(fi.elem, out.elem, a, in.N, stream);
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaCropFlipNormalizeReformatCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<CropFlipNormalizeReformat>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaCropFlipNormalizeReformatSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVImageBatchHandle in, NVCVTensorHandle out,
    NVCVTensorHandle cropRect, NVCVBorderType borderMode, float borderValue, NVCVTensorHandle flipCode,
    NVCVTensorHandle base, NVCVTensorHandle scale, float global_scale, float shift, float epsilon, uint32_t flags)
{
    return Protect(
        [&]
        {
            ToOperator<CropFlipNormalizeReformat>(handle).submit(stream, in, out, cropRect, borderMode, borderValue,
                                                                 flipCode, base, scale, global_scale, shift, epsilon,
                                                                 flags);
        });
}
}
