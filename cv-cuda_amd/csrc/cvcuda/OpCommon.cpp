#include "OpCommon.hpp"

#include <cvcuda/Version.h>

#include <cstring>

namespace cvamd {

void CheckCore(NVCVStatus st)
{
    if (st != NVCV_SUCCESS)
    {
        char msg[NVCV_MAX_STATUS_MESSAGE_LENGTH];
        nvcvPeekAtLastErrorMessage(msg, sizeof(msg));
        throw OpError(st, "%s", msg);
    }
}

void CheckHip(hipError_t e, const char *what)
{
    if (e != hipSuccess)
    {
        (void)hipGetLastError();
        throw OpError(NVCV_ERROR_DEVICE, "%s failed: %s", what, hipGetErrorString(e));
    }
}

void CheckLaunch(const char *kernel)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
    {
        throw OpError(NVCV_ERROR_INTERNAL, "Launch of %s failed: %s", kernel, hipGetErrorString(e));
    }
}

IOperator::~IOperator()
{
    magic = 0;
}

int ElemSize(ElemType t)
{
    switch (t)
    {
    case kU8:
    case kS8:
        return 1;
    case kU16:
    case kS16:
    case kF16:
        return 2;
    case kS32:
    case kU32:
    case kF32:
        return 4;
    case kF64:
        return 8;
    default:
        return 0;
    }
}

namespace {
ElemType ElemFrom(NVCVDataKind kind, int bits)
{
    switch (kind)
    {
    case NVCV_DATA_KIND_UNSIGNED:
        return bits == 8 ? kU8 : bits == 16 ? kU16 : bits == 32 ? kU32 : kUnknown;
    case NVCV_DATA_KIND_SIGNED:
        return bits == 8 ? kS8 : bits == 16 ? kS16 : bits == 32 ? kS32 : kUnknown;
    case NVCV_DATA_KIND_FLOAT:
        return bits == 16 ? kF16 : bits == 32 ? kF32 : bits == 64 ? kF64 : kUnknown;
    default:
        return kUnknown;
    }
}
} // namespace

DTypeInfo DecodeDataType(NVCVDataType dt)
{
    DTypeInfo    info = {kUnknown, 0};
    NVCVDataKind kind;
    int32_t      nch = 0, bits[4] = {};
    if (nvcvDataTypeGetDataKind(dt, &kind) != NVCV_SUCCESS || nvcvDataTypeGetNumChannels(dt, &nch) != NVCV_SUCCESS
        || nvcvDataTypeGetBitsPerChannel(dt, bits) != NVCV_SUCCESS || nch < 1)
    {
        return info;
    }
    for (int i = 1; i < nch; ++i)
    {
        if (bits[i] != bits[0])
        {
            return info;
        }
    }
    info.elem     = ElemFrom(kind, bits[0]);
    info.channels = nch;
    return info;
}

FormatInfo DecodeFormat(NVCVImageFormat fmt)
{
    FormatInfo   f = {0, 0, kUnknown};
    int32_t      planes = 0, channels = 0, bits[4] = {};
    NVCVDataKind kind;
    if (nvcvImageFormatGetNumPlanes(fmt, &planes) != NVCV_SUCCESS
        || nvcvImageFormatGetNumChannels(fmt, &channels) != NVCV_SUCCESS
        || nvcvImageFormatGetDataKind(fmt, &kind) != NVCV_SUCCESS)
    {
        return f;
    }
    f.planes   = planes;
    f.channels = channels;
    if (nvcvImageFormatGetBitsPerChannel(fmt, bits) == NVCV_SUCCESS)
    {
        bool same = bits[0] > 0;
        for (int i = 1; i < 4 && bits[i] != 0; ++i)
        {
            same = same && bits[i] == bits[0];
        }
        if (same)
        {
            f.elem = ElemFrom(kind, bits[0]);
        }
    }
    return f;
}

void ExportTensor(NVCVTensorHandle h, NVCVTensorData &out, const char *what)
{
    if (h == nullptr)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s tensor handle must not be NULL", what);
    }
    CheckCore(nvcvTensorExportData(h, &out));
    if (out.bufferType != NVCV_TENSOR_BUFFER_STRIDED_CUDA)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s must be a device-accessible, pitch-linear tensor", what);
    }
}

bool MakeImageBatchView(const NVCVTensorData &d, ImageBatchView &v)
{
    const NVCVTensorLayout &L = d.layout;
    int iN = -1, iC = -1, iH = -1, iW = -1;
    for (int i = 0; i < L.rank; ++i)
    {
        switch (L.data[i])
        {
        case 'N':
            iN = iN < 0 ? i : -2;
            break;
        case 'C':
            iC = iC < 0 ? i : -2;
            break;
        case 'H':
            iH = iH < 0 ? i : -2;
            break;
        case 'W':
            iW = iW < 0 ? i : -2;
            break;
        default:
            return false;
        }
    }
    if (L.rank != d.rank || iH < 0 || iW < 0 || iN == -2 || iC == -2 || iW != iH + 1)
    {
        return false;
    }
    if (iN >= 0 && iN != 0)
    {
        return false;
    }
    bool channelLast = iC < 0 || iC == L.rank - 1;
    if (!channelLast && iC != iH - 1)
    {
        return false;
    }
    DTypeInfo dt = DecodeDataType(d.dtype);
    if (dt.elem == kUnknown)
    {
        return false;
    }
    if (!channelLast && dt.channels != 1)
    {
        return false; // planar tensors of multi-component elements are not image batches
    }
    const int64_t *st = d.buffer.strided.strides;
    int            es = ElemSize(dt.elem);
    v                 = {};
    v.base            = d.buffer.strided.basePtr;
    v.elem            = dt.elem;
    v.H               = (int)d.shape[iH];
    v.W               = (int)d.shape[iW];
    v.N               = iN >= 0 ? (int)d.shape[iN] : 1;
    v.C               = (iC >= 0 ? (int)d.shape[iC] : 1) * dt.channels;
    v.strideH         = st[iH];
    v.strideW         = st[iW];
    v.strideC         = (iC >= 0 && !channelLast) ? st[iC] : es;
    v.layout          = channelLast ? kLayoutNHWC : kLayoutNCHW;
    v.hasBatchDim     = iN >= 0;
    if (iN >= 0)
    {
        v.strideN = st[iN];
    }
    else
    {
        // sample stride of a single image: extent of its outermost dimension
        v.strideN = st[0] * d.shape[0];
    }
    std::memcpy(v.layoutName, L.data, sizeof(v.layoutName));
    v.layoutName[L.rank] = '\0';
    return true;
}

ImageBatchView RequireImageBatchView(const NVCVTensorData &d, const char *what, NVCVStatus onBadLayout)
{
    ImageBatchView v;
    if (!MakeImageBatchView(d, v))
    {
        throw OpError(onBadLayout, "%s tensor must be an image batch ([N]HWC, [N]CHW or [N]HW layout of a supported "
                                   "element type): layout provided %s",
                      what, d.layout.data);
    }
    return v;
}

VarShapeView ExportVarShape(NVCVImageBatchHandle h, hipStream_t stream, const char *what)
{
    if (h == nullptr)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s image batch handle must not be NULL", what);
    }
    VarShapeView v = {};
    CheckCore(nvcvImageBatchExportData(h, stream, &v.data));
    if (v.data.bufferType != NVCV_IMAGE_BATCH_VARSHAPE_BUFFER_STRIDED_CUDA)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s data must be a device-accessible, varshape image batch", what);
    }
    int32_t n = 0;
    CheckCore(nvcvxImageBatchVarShapeGetHostImageList(h, &v.hostList, &n));
    v.N            = v.data.numImages;
    v.uniqueFormat = v.data.buffer.varShapeStrided.uniqueFormat;
    v.maxW         = v.data.buffer.varShapeStrided.maxWidth;
    v.maxH         = v.data.buffer.varShapeStrided.maxHeight;
    return v;
}

} // namespace cvamd

extern "C"
{
CVCUDA_PUBLIC void nvcvOperatorDestroy(NVCVOperatorHandle handle)
{
    if (handle != nullptr)
    {
        cvamd::IOperator *op = reinterpret_cast<cvamd::IOperator *>(handle);
        if (op->magic == cvamd::IOperator::kMagic)
        {
            delete op;
        }
    }
}

CVCUDA_PUBLIC uint32_t cvcudaGetVersion(void)
{
    return CVCUDA_VERSION;
}
}
