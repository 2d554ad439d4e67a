// CropFlipNormalizeReformat: var-shape batch -> tensor, one pass.
//
// Semantics follow src/cvcuda/priv/OpCropFlipNormalizeReformat.cu: coordinate map :165-187, zero fill
// outside the rectangle :157-161, expression and its order :73-74, scale / stddev :45-59, type tables
// :341-351 and :449-454, parameter checks :416-433, output layout :193-197.
//
// Kernel shape: one lane per output pixel, 64 columns x 4 rows per block, grid z = image. The crop
// rectangle, the flip code and the per-channel base / scale values are uniform per block and read in
// the prologue. Source and destination are addressed through per-channel strides, so interleaved and
// planar images, NHWC and NCHW outputs all run through the same code; for an interleaved source the C
// channel loads of a lane are adjacent bytes and coalesce in the memory pipeline. Streaming stores.
#include "DeviceUtils.hpp"
#include "OpCommon.hpp"

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

template<class T>
__device__ __forceinline__ T BorderValueAs(float v)
{
    if constexpr (std::is_same_v<T, float>)
    {
        return v;
    }
    else
    {
        // truncation toward zero, saturated to the range of T
        const float lo = (float)std::numeric_limits<T>::min(), hi = (float)std::numeric_limits<T>::max();
        return (T)(int)fminf(fmaxf(truncf(v), lo), hi);
    }
}

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
                v = reinterpret_cast<const TS *>(pl.basePtr + (int64_t)sy * pl.rowStride)[sx];
            }
            else
            {
                v = reinterpret_cast<const TS *>(p0.basePtr + (int64_t)sy * p0.rowStride)[sx * a.C + c];
            }
            const float b = a.base[a.baseC == 1 ? 0 : c];
            const float s = a.scale[a.scaleC == 1 ? 0 : c];
            const float m = a.stddev ? 1.0f / sqrtf(s * s + a.eps) : s;
            const float r = ((float)v - b) * m * a.gscale + a.shift;
            __builtin_nontemporal_store(SaturateCast<TD>(r), reinterpret_cast<TD *>(d + c * a.dC));
        }
    }
}

template<class TS, class TD>
void Launch(const CfnrArgs &a, int N, hipStream_t stream)
{
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
