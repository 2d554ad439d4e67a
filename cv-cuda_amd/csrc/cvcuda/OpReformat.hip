// Reformat: [N]HWC <-> [N]CHW layout change, or a pitched copy when layout and shape agree.
//
// Semantics follow src/cvcuda/priv/legacy/reformat.cu:35-70 (element (n,y,x,c) of the input goes to
// element (n,y,x,c) of the output, whatever the two memory layouts are) and its validation (:118-197).
// Only the bytes of real elements are written; row/plane padding of the output is left untouched.
//
// Kernel shapes. Packed rows of 1- and 2-byte elements (interleaved: pixel stride C elements; planar:
// pixel stride one element) move in runs of 4 pixels per lane: one vector load per lane on an
// interleaved side, one 4-element access per plane on a planar side, whole-dword streaming stores.
// Everything else: one lane per pixel, 64 columns x 4 rows per block, the interleaved side as one
// vector access, the planar side one element per lane per plane.
#include "DeviceUtils.hpp"
#include "OpCommon.hpp"
#include "RunIO.hpp"

#include <cvcuda/OpReformat.h>

namespace cvamd {

namespace {

struct ReformatArgs
{
    const uint8_t *src;
    uint8_t       *dst;
    int64_t        sN, sH, sW, sC; // source strides in bytes
    int64_t        dN, dH, dW, dC; // destination strides in bytes
    int32_t        W, H, C;
};

template<class T, int C>
using Vec = Packed<T, C>;

// C > 0: channel count known at compile time; SRC_IL / DST_IL: that side has its channels
// interleaved and packed (stride of C == element size), so the whole pixel moves as one vector.
template<class T, int C, bool SRC_IL, bool DST_IL>
__global__ __launch_bounds__(256) void ReformatKernel(const ReformatArgs a)
{
    const int x = blockIdx.x * 64 + (threadIdx.x & 63);
    const int y = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (x >= a.W || y >= a.H)
    {
        return;
    }
    const int      n = blockIdx.z;
    const uint8_t *s = a.src + n * a.sN + y * a.sH + x * a.sW;
    uint8_t       *d = a.dst + n * a.dN + y * a.dH + x * a.dW;
    if constexpr (C > 0)
    {
        Vec<T, C> px;
        if constexpr (SRC_IL)
        {
            px = *reinterpret_cast<const Vec<T, C> *>(s);
        }
        else
        {
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                px.v[c] = *reinterpret_cast<const T *>(s + c * a.sC);
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            T *o = DST_IL ? reinterpret_cast<T *>(d) + c : reinterpret_cast<T *>(d + c * a.dC);
            __builtin_nontemporal_store(px.v[c], o);
        }
    }
    else
    {
        for (int c = 0; c < a.C; ++c)
        {
            __builtin_nontemporal_store(*reinterpret_cast<const T *>(s + c * a.sC), reinterpret_cast<T *>(d + c * a.dC));
        }
    }
}

// Runs of 4 pixels per lane; SRC_IL / DST_IL: interleaved packed rows, otherwise planar packed rows.
template<class T, int C, bool SRC_IL, bool DST_IL>
__global__ __launch_bounds__(256) void ReformatRunsKernel(const ReformatArgs a)
{
    const int x0 = (blockIdx.x * 64 + (threadIdx.x & 63)) * kRunPixels;
    const int y  = blockIdx.y * kRunTileH + (threadIdx.x >> 6);
    if (x0 >= a.W || y >= a.H)
    {
        return;
    }
    const int      n = blockIdx.z;
    const uint8_t *s = a.src + n * a.sN + y * a.sH + x0 * a.sW;
    uint8_t       *d = a.dst + n * a.dN + y * a.dH + x0 * a.dW;
    if (x0 + kRunPixels > a.W)
    {
        for (int x = 0; x < a.W - x0; ++x)
        {
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                *reinterpret_cast<T *>(d + x * a.dW + c * a.dC) = *reinterpret_cast<const T *>(s + x * a.sW + c * a.sC);
            }
        }
        return;
    }
    T px[kRunPixels * C]; // pixel-major
    if constexpr (SRC_IL)
    {
        LoadRun<T, kRunPixels * C>(s, px);
    }
    else
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            T t[kRunPixels];
            LoadRun<T, kRunPixels>(s + c * a.sC, t);
#pragma unroll
            for (int k = 0; k < kRunPixels; ++k)
            {
                px[k * C + c] = t[k];
            }
        }
    }
    if constexpr (DST_IL)
    {
        // a wave's lanes 0 .. lanes-1 hold consecutive pieces of the row (pieces of 24 or 32 bytes are regrouped
        // into dense 16-byte stores there)
        const int lane = threadIdx.x & 63, lanes = min(64, (a.W - (x0 - lane * kRunPixels)) / kRunPixels);
        StoreRowRunNT<T, kRunPixels * C>(d - (int64_t)lane * kRunPixels * a.dW, px, lane, lanes);
    }
    else
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            T t[kRunPixels];
#pragma unroll
            for (int k = 0; k < kRunPixels; ++k)
            {
                t[k] = px[k * C + c];
            }
            StoreRunNT<T, kRunPixels>(d + c * a.dC, t);
        }
    }
}

template<class T, int C>
void LaunchC(const ReformatArgs &a, int N, bool srcIl, bool dstIl, hipStream_t stream)
{
    // Rows that are one dense run on both sides in the same order (packed interleaved to packed interleaved, or a
    // single channel) are copied 16 bytes per lane whatever the pixel: as rows of 4-byte pixels in runs of 4.
    {
        const int64_t rowBytes = (int64_t)a.W * C * (int64_t)sizeof(T);
        const bool    packed   = C == 1 ? (a.sW == (int64_t)sizeof(T) && a.dW == (int64_t)sizeof(T))
                                        : (srcIl && dstIl && a.sW == (int64_t)(C * sizeof(T)) && a.dW == (int64_t)(C * sizeof(T)));
        if (packed && rowBytes % 4 == 0 && (sizeof(T) < 4 || C == 1))
        {
            ReformatArgs b = a;
            b.W            = (int32_t)(rowBytes / 4);
            b.C            = 4;
            b.sW = b.dW = 4;
            b.sC = b.dC = 1;
            dim3 grid(DivUp(b.W, kRunTileW), DivUp(b.H, kRunTileH), N), block(256);
            hipLaunchKernelGGL((ReformatRunsKernel<uint8_t, 4, true, true>), grid, block, 0, stream, b);
            CheckLaunch("ReformatRunsKernel");
            return;
        }
    }
    if constexpr (sizeof(T) <= 2)
    {
        const bool srcPlanar = a.sW == (int64_t)sizeof(T), dstPlanar = a.dW == (int64_t)sizeof(T);
        const bool srcPacked = (srcIl && a.sW == (int64_t)(C * sizeof(T))) || srcPlanar;
        const bool dstPacked = (dstIl && a.dW == (int64_t)(C * sizeof(T))) || dstPlanar;
        if (srcPacked && dstPacked)
        {
            dim3 grid(DivUp(a.W, kRunTileW), DivUp(a.H, kRunTileH), N), block(256);
            // C == 1: interleaved and planar coincide
            const bool sIl = srcIl && !(C == 1), dIl = dstIl && !(C == 1);
            if (sIl && dIl)
            {
                hipLaunchKernelGGL((ReformatRunsKernel<T, C, true, true>), grid, block, 0, stream, a);
            }
            else if (sIl)
            {
                hipLaunchKernelGGL((ReformatRunsKernel<T, C, true, false>), grid, block, 0, stream, a);
            }
            else if (dIl)
            {
                hipLaunchKernelGGL((ReformatRunsKernel<T, C, false, true>), grid, block, 0, stream, a);
            }
            else
            {
                hipLaunchKernelGGL((ReformatRunsKernel<T, C, false, false>), grid, block, 0, stream, a);
            }
            CheckLaunch("ReformatRunsKernel");
            return;
        }
    }
    dim3 grid(DivUp(a.W, 64), DivUp(a.H, 4), N), block(256);
    if (srcIl && dstIl)
    {
        hipLaunchKernelGGL((ReformatKernel<T, C, true, true>), grid, block, 0, stream, a);
    }
    else if (srcIl)
    {
        hipLaunchKernelGGL((ReformatKernel<T, C, true, false>), grid, block, 0, stream, a);
    }
    else if (dstIl)
    {
        hipLaunchKernelGGL((ReformatKernel<T, C, false, true>), grid, block, 0, stream, a);
    }
    else
    {
        hipLaunchKernelGGL((ReformatKernel<T, C, false, false>), grid, block, 0, stream, a);
    }
    CheckLaunch("ReformatKernel");
}

template<class T>
void LaunchT(const ReformatArgs &a, int N, hipStream_t stream)
{
    const bool srcIl = a.sC == (int64_t)sizeof(T);
    const bool dstIl = a.dC == (int64_t)sizeof(T);
    switch (a.C)
    {
    case 1:
        LaunchC<T, 1>(a, N, srcIl, dstIl, stream);
        break;
    case 2:
        LaunchC<T, 2>(a, N, srcIl, dstIl, stream);
        break;
    case 3:
        LaunchC<T, 3>(a, N, srcIl, dstIl, stream);
        break;
    case 4:
        LaunchC<T, 4>(a, N, srcIl, dstIl, stream);
        break;
    default:
    {
        dim3 grid(DivUp(a.W, 64), DivUp(a.H, 4), N);
        hipLaunchKernelGGL((ReformatKernel<T, 0, false, false>), grid, dim3(256), 0, stream, a);
        CheckLaunch("ReformatKernel");
    }
    }
}

class Reformat final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout) const
    {
        NVCVTensorData din, dout;
        ExportTensor(hin, din, "Input");
        ExportTensor(hout, dout, "Output");
        ImageBatchView in  = RequireImageBatchView(din, "Input", NVCV_ERROR_INVALID_ARGUMENT);
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
        if (in.hasBatchDim != out.hasBatchDim)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid combination of input format %s and output format %s",
                          in.layoutName, out.layoutName);
        }
        if (in.elem != out.elem)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "DataType of input and output must be equal");
        }
        if (in.elem == kF16 || in.elem == kUnknown)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
        }
        if (in.N != out.N || in.H != out.H || in.W != out.W || in.C != out.C)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Input (%dx%dx%dx%d) and output (%dx%dx%dx%d) must hold the same N, H, W, C", in.N, in.H, in.W,
                          in.C, out.N, out.H, out.W, out.C);
        }
        if (in.bytesSpanned() > INT32_MAX || out.bytesSpanned() > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output size exceeds %d. Tensor is too large.",
                          INT32_MAX);
        }
        ReformatArgs a = {in.base,    out.base,    in.strideN,  in.strideH, in.strideW, in.strideC,
                          out.strideN, out.strideH, out.strideW, out.strideC, in.W,       in.H,
                          in.C};
        if (in.N == 0 || in.W == 0 || in.H == 0 || in.C == 0)
        {
            return;
        }
        switch (ElemSize(in.elem))
        {
        case 1:
            LaunchT<uint8_t>(a, in.N, stream);
            break;
        case 2:
            LaunchT<uint16_t>(a, in.N, stream);
            break;
        case 4:
            LaunchT<uint32_t>(a, in.N, stream);
            break;
        default:
            LaunchT<uint64_t>(a, in.N, stream);
            break;
        }
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaReformatCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<Reformat>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaReformatSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                              NVCVTensorHandle out)
{
    return Protect([&] { ToOperator<Reformat>(handle).submit(stream, in, out); });
}
}
