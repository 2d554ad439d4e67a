// CustomCrop, CenterCrop and Flip: index-mapped copies, bit-exact by construction.
//
// Semantics and validation follow src/cvcuda/priv/legacy/custom_crop.cu:35-46, 83-156,
// center_crop.cu:35-58, 74-141, flip.cu:30-196 (tensor: flipCode > 0 mirrors columns, == 0 mirrors
// rows, < 0 both) and flip_or_copy_var_shape.cu:31-62, 88-160 (per-image code from an int32 tensor:
// 1 columns, 0 rows, -1 both, anything else plain copy).
//
// Two kernels. Crops and row-mirroring flips keep the byte order inside a row, so they run as row
// copies: every lane moves 16 bytes of a row with one unaligned 16-byte load and store whatever the
// pixel type is (a wave covers 1 KiB of a row). Column-mirroring flips permute pixels: a lane reads a
// run of 4 source pixels with one vector load, reverses their order and writes them as whole dwords.
// Stores are streaming. Only the bytes of the region are written; the rest of the output is left
// untouched.
#include "DeviceUtils.hpp"
#include "OpCommon.hpp"
#include "RunIO.hpp"
#include "VarShapeTiles.hpp"

#include <cvcuda/OpCenterCrop.h>
#include <cvcuda/OpCustomCrop.h>
#include <cvcuda/OpFlip.h>

#include <algorithm>

namespace cvamd {

namespace {

struct CopyArgs
{
    const uint8_t *src;
    uint8_t       *dst;
    int64_t        srcN, dstN;
    int32_t        srcRow, dstRow;
    int32_t        w, h;       // region size in pixels
    int32_t        x0, y0;     // source pixel of region pixel (0,0) ...
    int32_t        stepX, stepY; // ... and the direction (+1 / -1) the source is walked in
    int32_t        pixelBytes;
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
    const uint8_t *codes; // var-shape flip: int32 per image
    int64_t        codeStride;
};

struct __attribute__((packed, aligned(1))) Chunk16
{
    uint32_t w[4];
};

constexpr int kChunk     = 16;
constexpr int kRowTileB  = 64 * kChunk; // bytes of a row per wave
constexpr int kRowTileH  = 4;           // rows per block (one per wave)

// dst row y, bytes [0, w*pixelBytes)  <-  src row y0 + stepY*y, bytes from x0*pixelBytes on
__global__ __launch_bounds__(256) void RowCopyKernel(const CopyArgs a)
{
    const int y = blockIdx.y * kRowTileH + (threadIdx.x >> 6);
    if (y >= a.h)
    {
        return;
    }
    const int      n      = blockIdx.z;
    const int      nbytes = a.w * a.pixelBytes;
    const int      at     = (blockIdx.x * 64 + (threadIdx.x & 63)) * kChunk;
    const uint8_t *s = a.src + n * a.srcN + (int64_t)(a.y0 + a.stepY * y) * a.srcRow + (int64_t)a.x0 * a.pixelBytes + at;
    uint8_t       *d = a.dst + n * a.dstN + (int64_t)y * a.dstRow + at;
    if (at + kChunk <= nbytes)
    {
        const Chunk16 c  = *reinterpret_cast<const Chunk16 *>(s);
        Chunk16      *dc = reinterpret_cast<Chunk16 *>(d);
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            __builtin_nontemporal_store(c.w[i], &dc->w[i]);
        }
    }
    else
    {
        for (int i = 0; at + i < nbytes; ++i)
        {
            d[i] = s[i];
        }
    }
}

template<class T, int C>
using Vec = Packed<T, C>;

template<class T, int C>
__device__ __forceinline__ void CopyPixel(const uint8_t *srcRow, uint8_t *dstRow, int sx, int dx)
{
    const Vec<T, C> px = reinterpret_cast<const Vec<T, C> *>(srcRow)[sx];
    Vec<T, C>      *o  = reinterpret_cast<Vec<T, C> *>(dstRow) + dx;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        __builtin_nontemporal_store(px.v[c], &o->v[c]);
    }
}

// Pixels per lane of the mirrored-column copies: kRunPixelsFor, and for single-channel images as many as make 16
// bytes (4 bytes per lane and instruction ran at 3.9 of the 6.3 TB/s the 3-channel form reaches on cached inputs).
template<class T, int C>
constexpr int kFlipRunPixels = C == 1 ? 16 / (int)sizeof(T) : kRunPixelsFor<T, T>;

// Runs of a row, one per lane (the wave's first run is run0): dst pixel x <- src pixel sx0 + step * x
// (step = +1 / -1, wave-uniform). Whole wave must call this; the ragged end of a row goes pixel by pixel.
// Mirrored columns: a lane loads the run that lane 63 - l will store, so the wave reads ascending
// addresses, the runs change lanes through the LDS crossbar (no memory involved) and the wave also
// writes ascending addresses; with the loads descending instead the operator ran at 0.7 of this rate.
template<class T, int C>
__device__ __forceinline__ void CopyRuns(const uint8_t *srcRow, uint8_t *dstRow, int w, int sx0, int step, int run0)
{
    constexpr int P = kFlipRunPixels<T, C>, PB = C * sizeof(T), D = P * PB / 4;
    static_assert((P * PB) % 4 == 0, "runs are whole dwords");
    const int lane = threadIdx.x & 63, lanes = min(64, max(0, w - run0 * P) / P); // lanes with a whole run
    const int dx0  = (run0 + lane) * P;
    uint8_t  *out0 = dstRow + (int64_t)run0 * P * PB; // where lane 0's run goes
    T         in[P * C];
    if (step > 0)
    {
        if (dx0 + P <= w)
        {
            LoadRun<T, P * C>(srcRow + (int64_t)(sx0 + dx0) * PB, in);
            StoreRowRunNT<T, P * C>(out0, in, lane, lanes);
            return;
        }
    }
    else
    {
        const int theirDx0 = (run0 + 63 - lane) * P;
        uint32_t  q[D]     = {};
        if (theirDx0 + P <= w)
        {
            LoadRun<T, P * C>(srcRow + (int64_t)(sx0 - theirDx0 - (P - 1)) * PB, in);
            __builtin_memcpy(q, in, sizeof(q));
        }
#pragma unroll
        for (int d = 0; d < D; ++d)
        {
            q[d] = (uint32_t)__builtin_amdgcn_ds_bpermute((63 - lane) * 4, (int)q[d]);
        }
        if (dx0 + P <= w)
        {
            __builtin_memcpy(in, q, sizeof(q));
            T out[P * C];
#pragma unroll
            for (int k = 0; k < P; ++k)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    out[k * C + c] = in[(P - 1 - k) * C + c];
                }
            }
            StoreRowRunNT<T, P * C>(out0, out, lane, lanes);
            return;
        }
    }
    for (int x = dx0; x < w; ++x)
    {
        CopyPixel<T, C>(srcRow, dstRow, sx0 + step * x, x);
    }
}

template<class T, int C>
__global__ __launch_bounds__(256) void PixelMapTensor(const CopyArgs a)
{
    const int y = blockIdx.y * kRunTileH + (threadIdx.x >> 6);
    if (y >= a.h)
    {
        return;
    }
    const int n = blockIdx.z;
    CopyRuns<T, C>(a.src + n * a.srcN + (int64_t)(a.y0 + a.stepY * y) * a.srcRow, a.dst + n * a.dstN + (int64_t)y * a.dstRow,
                   a.w, a.x0, a.stepX, blockIdx.x * 64);
}

template<class T, int C>
constexpr int kFlipVarRows = kVarShapeRows<kFlipRunPixels<T, C> * C * (int)sizeof(T)>;

template<class T, int C>
__global__ __launch_bounds__(256) void FlipVarShape(const CopyArgs a, const VarTiles tiles)
{
    const TileCoord              tc = LocateTile(tiles, blockIdx.x);
    const NVCVImagePlaneStrided &s  = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided &d  = a.dstList[tc.image].planes[0];
    const int  code    = *reinterpret_cast<const int32_t *>(a.codes + tc.image * a.codeStride);
    const bool mirrorX = code == 1 || code == -1, mirrorY = code == 0 || code == -1;
    const uint8_t *src = AsGlobal(s.basePtr);
    uint8_t       *dst = AsGlobal(d.basePtr);
    const int      W = d.width, H = d.height, srcRow = s.rowStride, dstRow = d.rowStride;
    constexpr int  R = kFlipVarRows<T, C>;
    for (int r = 0; r < R; ++r)
    {
        const int y = (tc.ty * R + r) * kRunTileH + (threadIdx.x >> 6);
        if (y >= H)
        {
            return;
        }
        const int sy = mirrorY ? H - 1 - y : y;
        CopyRuns<T, C>(src + (int64_t)sy * srcRow, dst + (int64_t)y * dstRow, W, mirrorX ? W - 1 : 0, mirrorX ? -1 : 1, tc.tx * 64);
    }
}

void LaunchRowCopy(const CopyArgs &a, int N, hipStream_t stream)
{
    if (N == 0 || a.w == 0 || a.h == 0)
    {
        return;
    }
    dim3 grid(DivUp(a.w * a.pixelBytes, kRowTileB), DivUp(a.h, kRowTileH), N);
    hipLaunchKernelGGL(RowCopyKernel, grid, dim3(256), 0, stream, a);
    CheckLaunch("RowCopyKernel");
}

template<class T, int C>
void LaunchPixelMap(const CopyArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    if (dstHost == nullptr)
    {
        dim3 grid(DivUp(a.w, 64 * kFlipRunPixels<T, C>), DivUp(a.h, kRunTileH), N);
        hipLaunchKernelGGL((PixelMapTensor<T, C>), grid, dim3(256), 0, stream, a);
        CheckLaunch("PixelMapTensor");
        return;
    }
    for (int first = 0; first < N; first += kMaxTileImages)
    {
        VarTiles tiles;
        int total = BuildVarTiles(tiles, dstHost, first, std::min(kMaxTileImages, N - first), 64 * kFlipRunPixels<T, C>,
                                  kRunTileH * kFlipVarRows<T, C>);
        if (total > 0)
        {
            hipLaunchKernelGGL((FlipVarShape<T, C>), dim3(total), dim3(256), 0, stream, a, tiles);
            CheckLaunch("FlipVarShape");
        }
    }
}

template<class T>
void DispatchPixelMapC(int C, const CopyArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    switch (C)
    {
    case 1:
        LaunchPixelMap<T, 1>(a, N, dstHost, stream);
        break;
    case 3:
        LaunchPixelMap<T, 3>(a, N, dstHost, stream);
        break;
    case 4:
        LaunchPixelMap<T, 4>(a, N, dstHost, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", C);
    }
}

void DispatchPixelMap(int elemSize, int C, const CopyArgs &a, int N, const NVCVImageBufferStrided *dstHost,
                      hipStream_t stream)
{
    if (N == 0)
    {
        return;
    }
    switch (elemSize)
    {
    case 1:
        DispatchPixelMapC<uint8_t>(C, a, N, dstHost, stream);
        break;
    case 2:
        DispatchPixelMapC<uint16_t>(C, a, N, dstHost, stream);
        break;
    default:
        DispatchPixelMapC<uint32_t>(C, a, N, dstHost, stream);
        break;
    }
}

struct CropViews
{
    ImageBatchView in, out;
};

// Checks shared by both crops (custom_crop.cu:88-127, center_crop.cu:77-118).
CropViews CheckCropTensors(NVCVTensorHandle hin, NVCVTensorHandle hout)
{
    NVCVTensorData din, dout;
    ExportTensor(hin, din, "Input");
    ExportTensor(hout, dout, "Output");
    CropViews v;
    v.in  = RequireImageBatchView(din, "Input", NVCV_ERROR_INVALID_ARGUMENT);
    v.out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
    if (v.in.layout != kLayoutNHWC || v.out.layout != kLayoutNHWC)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataFormat: both input and output must be \"NHWC\" or \"HWC\"");
    }
    if (din.dtype != dout.dtype)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input and output must have the same data type");
    }
    if (v.in.C < 1 || v.in.C > 4 || v.in.C != v.out.C)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number: input %d, output %d", v.in.C, v.out.C);
    }
    const int es = ElemSize(v.in.elem);
    if (v.in.elem == kUnknown || (es != 1 && es != 2 && es != 4 && es != 8))
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
    }
    if (v.in.N != v.out.N)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input (%d) and output (%d) must hold the same number of images",
                      v.in.N, v.out.N);
    }
    if (std::max(v.in.bytesSpanned(), v.out.bytesSpanned()) > INT32_MAX)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output size exceeds %d. Tensor is too large.", INT32_MAX);
    }
    return v;
}

CopyArgs RegionArgs(const ImageBatchView &in, const ImageBatchView &out, int x0, int y0, int w, int h)
{
    CopyArgs a   = {};
    a.src        = in.base;
    a.dst        = out.base;
    a.srcN       = in.strideN;
    a.dstN       = out.strideN;
    a.srcRow     = (int32_t)in.strideH;
    a.dstRow     = (int32_t)out.strideH;
    a.w          = w;
    a.h          = h;
    a.x0         = x0;
    a.y0         = y0;
    a.stepX      = 1;
    a.stepY      = 1;
    a.pixelBytes = in.C * ElemSize(in.elem);
    return a;
}

class CustomCrop final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, NVCVRectI roi) const
    {
        CropViews v = CheckCropTensors(hin, hout);
        if (roi.width < 0 || roi.height < 0 || roi.height > v.out.H || roi.width > v.out.W)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "ROI %d x %d larger than the output %d x %d", roi.width, roi.height,
                          v.out.W, v.out.H);
        }
        if (roi.x < 0 || roi.y < 0 || (int64_t)roi.x + roi.width > v.in.W || (int64_t)roi.y + roi.height > v.in.H)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid ROI range x %d y %d width %d height %d for a %d x %d input",
                          roi.x, roi.y, roi.width, roi.height, v.in.W, v.in.H);
        }
        LaunchRowCopy(RegionArgs(v.in, v.out, roi.x, roi.y, roi.width, roi.height), v.in.N, stream);
    }
};

class CenterCrop final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, int32_t cropW, int32_t cropH) const
    {
        CropViews v = CheckCropTensors(hin, hout);
        if (cropW < 0 || cropH < 0 || cropH > v.out.H || cropW > v.out.W)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Crop %d x %d larger than the output %d x %d", cropW, cropH,
                          v.out.W, v.out.H);
        }
        if (cropW > v.in.W || cropH > v.in.H)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Crop %d x %d larger than the input %d x %d", cropW, cropH, v.in.W,
                          v.in.H);
        }
        const int top = (v.in.H - cropH) / 2, left = (v.in.W - cropW) / 2;
        LaunchRowCopy(RegionArgs(v.in, v.out, left, top, cropW, cropH), v.in.N, stream);
    }
};

class Flip final : public IOperator
{
public:
    explicit Flip(int32_t /*maxVarShapeBatchSize: not needed, no operator-owned buffers*/) {}

    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, int32_t flipCode) const
    {
        NVCVTensorData din, dout;
        ExportTensor(hin, din, "Input");
        ExportTensor(hout, dout, "Output");
        ImageBatchView in  = RequireImageBatchView(din, "Input", NVCV_ERROR_INVALID_ARGUMENT);
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
        if (in.elem != out.elem || din.dtype != dout.dtype)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType between input and output");
        }
        if (in.layout != kLayoutNHWC || out.layout != kLayoutNHWC || in.hasBatchDim != out.hasBatchDim)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Invalid DataFormat between input (%s) and output (%s): both must be \"NHWC\" or \"HWC\"",
                          in.layoutName, out.layoutName);
        }
        if (!(in.elem == kU8 || in.elem == kU16 || in.elem == kS32 || in.elem == kF32))
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
        }
        if (in.C != 1 && in.C != 3 && in.C != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", in.C);
        }
        if (in.N != out.N || in.H != out.H || in.W != out.W || in.C != out.C)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input and output must have the same shape");
        }
        if (std::max(in.bytesSpanned(), out.bytesSpanned()) > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output size exceeds %d. Tensor is too large.",
                          INT32_MAX);
        }
        CopyArgs a = RegionArgs(in, out, 0, 0, in.W, in.H);
        if (flipCode <= 0) // rows mirrored
        {
            a.y0    = in.H - 1;
            a.stepY = -1;
        }
        if (flipCode == 0)
        {
            LaunchRowCopy(a, in.N, stream);
            return;
        }
        a.x0    = in.W - 1; // columns mirrored
        a.stepX = -1;
        if (in.W == 0 || in.H == 0)
        {
            return;
        }
        DispatchPixelMap(ElemSize(in.elem), in.C, a, in.N, nullptr, stream);
    }

    void submit(hipStream_t stream, NVCVImageBatchHandle hin, NVCVImageBatchHandle hout, NVCVTensorHandle hcodes) const
    {
        VarShapeView in  = ExportVarShape(hin, stream, "Input");
        VarShapeView out = ExportVarShape(hout, stream, "Output");
        if (in.uniqueFormat == NVCV_IMAGE_FORMAT_NONE || out.uniqueFormat == NVCV_IMAGE_FORMAT_NONE)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images in a batch must all have the same format");
        }
        FormatInfo fi = DecodeFormat(in.uniqueFormat), fo = DecodeFormat(out.uniqueFormat);
        if (fi.planes != 1 || fo.planes != 1)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images must have a single interleaved plane");
        }
        if (fi.elem != fo.elem || fi.channels != fo.channels)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "DataType of input and output must be equal");
        }
        if (!(fi.elem == kU8 || fi.elem == kU16 || fi.elem == kS16 || fi.elem == kS32 || fi.elem == kF32))
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
        }
        if (fi.channels != 1 && fi.channels != 3 && fi.channels != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", fi.channels);
        }
        if (in.N != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input and output batch sizes: %d != %d", in.N, out.N);
        }
        for (int i = 0; i < in.N; ++i)
        {
            const NVCVImagePlaneStrided &s = in.hostList[i].planes[0], &d = out.hostList[i].planes[0];
            if (s.width != d.width || s.height != d.height)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Image %d: input %d x %d and output %d x %d differ in size", i,
                              s.width, s.height, d.width, d.height);
            }
        }
        NVCVTensorData dc;
        ExportTensor(hcodes, dc, "Flip code");
        DTypeInfo dt = DecodeDataType(dc.dtype);
        int64_t   count = 1;
        for (int i = 0; i < dc.rank; ++i)
        {
            count *= dc.shape[i];
        }
        // one int32 per image: a rank-1 tensor, or any shape whose only extent above 1 is the first
        if (dt.elem != kS32 || dt.channels != 1 || dc.rank < 1 || dc.shape[0] != count || count < in.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Flip code tensor must hold one int32 per image (%d)", in.N);
        }
        CopyArgs a   = {};
        a.srcList    = in.data.buffer.varShapeStrided.imageList;
        a.dstList    = out.data.buffer.varShapeStrided.imageList;
        a.codes      = dc.buffer.strided.basePtr;
        a.codeStride = dc.buffer.strided.strides[0];
        DispatchPixelMap(ElemSize(fi.elem), fi.channels, a, in.N, out.hostList, stream);
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaCustomCropCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<CustomCrop>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaCustomCropSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                                NVCVTensorHandle out, const NVCVRectI cropRect)
{
    return Protect([&] { ToOperator<CustomCrop>(handle).submit(stream, in, out, cropRect); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaCenterCropCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<CenterCrop>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaCenterCropSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                                NVCVTensorHandle out, int32_t cropWidth, int32_t cropHeight)
{
    return Protect([&] { ToOperator<CenterCrop>(handle).submit(stream, in, out, cropWidth, cropHeight); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaFlipCreate(NVCVOperatorHandle *handle, int32_t maxVarShapeBatchSize)
{
    return CreateOperator<Flip>(handle, maxVarShapeBatchSize);
}

CVCUDA_PUBLIC NVCVStatus cvcudaFlipSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                          NVCVTensorHandle out, int32_t flipCode)
{
    return Protect([&] { ToOperator<Flip>(handle).submit(stream, in, out, flipCode); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaFlipVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVImageBatchHandle in,
                                                  NVCVImageBatchHandle out, NVCVTensorHandle flipCode)
{
    return Protect([&] { ToOperator<Flip>(handle).submit(stream, in, out, flipCode); });
}
}
