// ConvertTo: out = saturate_cast<out type>(alpha * in + beta), element-wise.
//
// Semantics and validation follow src/cvcuda/priv/legacy/convert_to.cu:36-47 (the expression, in
// float32 unless either side is float64, alpha/beta converted to that type first), :62-99 and
// :131-206 (checks, the 7 x 7 type table). Saturation as cuda_tools/detail/SaturateCastImpl.hpp:31-157.
//
// Kernel shape: channels play no role in an element-wise operator, so a row is W*C scalars; one lane
// converts 4 consecutive scalars, loaded and stored as whole dwords (u8 -> f32: one 4-byte load, one
// 16-byte store per lane). A wave covers 256 scalars of a row, a block 4 rows. Streaming stores.
#include "DeviceUtils.hpp"
#include "OpCommon.hpp"
#include "RunIO.hpp"

#include <cvcuda/OpConvertTo.h>

#include <algorithm>
#include <cstring>

namespace cvamd {

namespace {

struct ConvertArgs
{
    const uint8_t *src;
    uint8_t       *dst;
    int64_t        srcN, dstN;
    int32_t        srcRow, dstRow;
    int32_t        rowElems, H;
    double         alpha, beta;
};

// double -> T with round-half-to-even and saturation; NaN -> 0 for integer targets
template<class T>
__device__ __forceinline__ T SaturateCastD(double v)
{
    if constexpr (std::is_same_v<T, double>)
    {
        return v;
    }
    else if constexpr (std::is_same_v<T, float>)
    {
        return (float)v;
    }
    else
    {
        if (v != v)
        {
            return 0;
        }
        const double lo = (double)std::numeric_limits<T>::min(), hi = (double)std::numeric_limits<T>::max();
        return (T)fmin(fmax(rint(v), lo), hi);
    }
}

template<class TS, class TD>
__device__ __forceinline__ TD ConvertOne(TS s, const ConvertArgs &a)
{
    if constexpr (std::is_same_v<TS, double> || std::is_same_v<TD, double>)
    {
        return SaturateCastD<TD>(a.alpha * (double)s + a.beta);
    }
    else
    {
        const float v = (float)a.alpha * (float)s + (float)a.beta;
        if constexpr (std::is_same_v<TD, float>)
        {
            return v;
        }
        else
        {
            return SaturateCast<TD>(v);
        }
    }
}

// Scalars per lane: as many as make 16 bytes on the wider side, at least 4 (1- and 2-byte types on both sides: 16 or
// 8 scalars; with 4 a lane moved 4 bytes per instruction and 16 x 1080p x 3 u8 -> u8 took 44 us where it takes 30).
// Byte inputs widened to 4-byte outputs take 8, so that the load is 8 bytes instead of 4; their 32 output bytes per
// lane leave through the row-regrouped stores (stored directly they measured 235 us against 175 us with 4 scalars
// on 32 x 1080p x 3); 4-byte inputs narrowed to bytes take 8 as well (8 output bytes per lane: 88.4 -> 86.2 us).
template<class TS, class TD>
constexpr int kConvertRun = ((sizeof(TS) == 1 && sizeof(TD) == 4) || (sizeof(TS) == 4 && sizeof(TD) == 1))
                              ? 8
                              : (16 / (int)(sizeof(TS) > sizeof(TD) ? sizeof(TS) : sizeof(TD)) > 4
                                     ? 16 / (int)(sizeof(TS) > sizeof(TD) ? sizeof(TS) : sizeof(TD))
                                     : 4);

template<class TS, class TD>
__global__ __launch_bounds__(256) void ConvertKernel(const ConvertArgs a)
{
    constexpr int E = kConvertRun<TS, TD>;
    const int     y = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int     lane = threadIdx.x & 63, e0 = blockIdx.x * 64 * E, e = e0 + lane * E;
    if (y >= a.H || e >= a.rowElems)
    {
        return;
    }
    const int      n = blockIdx.z;
    const uint8_t *s = a.src + n * a.srcN + (int64_t)y * a.srcRow + (int64_t)e * sizeof(TS);
    uint8_t       *d = a.dst + n * a.dstN + (int64_t)y * a.dstRow + (int64_t)e * sizeof(TD);
    if (e + E <= a.rowElems)
    {
        TS in[E];
        TD out[E];
        LoadRun<TS, E>(s, in);
#pragma unroll
        for (int i = 0; i < E; ++i)
        {
            out[i] = ConvertOne<TS, TD>(in[i], a);
        }
        StoreRowRunNT<TD, E>(d - (int64_t)lane * E * sizeof(TD), out, lane, min(64, (a.rowElems - e0) / E));
    }
    else
    {
        for (int i = 0; e + i < a.rowElems; ++i)
        {
            reinterpret_cast<TD *>(d)[i] = ConvertOne<TS, TD>(reinterpret_cast<const TS *>(s)[i], a);
        }
    }
}

template<class TS, class TD>
void Launch(const ConvertArgs &a, int N, hipStream_t stream)
{
    dim3 grid(DivUp(a.rowElems, 64 * kConvertRun<TS, TD>), DivUp(a.H, 4), N);
    hipLaunchKernelGGL((ConvertKernel<TS, TD>), grid, dim3(256), 0, stream, a);
    CheckLaunch("ConvertKernel");
}

template<class TS>
void DispatchDst(ElemType out, const ConvertArgs &a, int N, hipStream_t stream)
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
    case kF64:
        Launch<TS, double>(a, N, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid Converted DataType");
    }
}

void DispatchSrc(ElemType in, ElemType out, const ConvertArgs &a, int N, hipStream_t stream)
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
    case kF64:
        DispatchDst<double>(out, a, N, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
    }
}

bool Convertible(ElemType e)
{
    return e == kU8 || e == kS8 || e == kU16 || e == kS16 || e == kS32 || e == kF32 || e == kF64;
}

class ConvertTo final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, double alpha, double beta) const
    {
        NVCVTensorData din, dout;
        ExportTensor(hin, din, "Input");
        ExportTensor(hout, dout, "Output");
        ImageBatchView in  = RequireImageBatchView(din, "Input", NVCV_ERROR_INVALID_ARGUMENT);
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
        if (in.layout != kLayoutNHWC || out.layout != kLayoutNHWC)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataFormat: input and output must be \"NHWC\" or \"HWC\"");
        }
        if (in.N != out.N || in.H != out.H || in.W != out.W || in.C != out.C)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Input (%dx%dx%dx%d) and output (%dx%dx%dx%d) shapes are different", in.N, in.H, in.W, in.C,
                          out.N, out.H, out.W, out.C);
        }
        if (in.C > 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", in.C);
        }
        if (!Convertible(in.elem))
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
        }
        if (!Convertible(out.elem))
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid Converted DataType");
        }
        if (std::max(in.bytesSpanned(), out.bytesSpanned()) > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output size exceeds %d. Tensor is too large.",
                          INT32_MAX);
        }
        // the kernel walks a row as W*C packed scalars
        if (in.strideW != (int64_t)in.C * ElemSize(in.elem) || out.strideW != (int64_t)out.C * ElemSize(out.elem)
            || (in.C > 1 && (in.strideC != ElemSize(in.elem) || out.strideC != ElemSize(out.elem))))
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Pixels of a row must be packed");
        }
        if (in.N == 0 || in.H == 0 || in.W == 0 || in.C == 0)
        {
            return;
        }
        ConvertArgs a = {in.base, out.base, in.strideN, out.strideN, (int32_t)in.strideH, (int32_t)out.strideH,
                         in.W * in.C, in.H, alpha, beta};
        DispatchSrc(in.elem, out.elem, a, in.N, stream);
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaConvertToCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<ConvertTo>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaConvertToSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                               NVCVTensorHandle out, const double alpha, const double beta)
{
    return Protect([&] { ToOperator<ConvertTo>(handle).submit(stream, in, out, alpha, beta); });
}
}
