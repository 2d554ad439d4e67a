// Shared host-side pieces of the operator library: error transport to the NVCV per-thread status,
// operator handle plumbing, and the strided "batch of images" view of tensors and var-shape
// batches that every operator validates against.
#ifndef CVCUDA_AMD_OPCOMMON_HPP
#define CVCUDA_AMD_OPCOMMON_HPP

#include <cvcuda/Operator.h>
#include <cvcuda/Types.h>
#include <nvcv/ImageBatch.h>
#include <nvcv/Tensor.h>

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <exception>
#include <new>

namespace cvamd {

class OpError : public std::exception
{
public:
    OpError(NVCVStatus code, const char *fmt, ...) __attribute__((format(printf, 3, 4)))
        : m_code(code)
    {
        va_list va;
        va_start(va, fmt);
        vsnprintf(m_msg, sizeof(m_msg), fmt, va);
        va_end(va);
    }

    NVCVStatus code() const noexcept
    {
        return m_code;
    }

    const char *what() const noexcept override
    {
        return m_msg;
    }

private:
    NVCVStatus m_code;
    char       m_msg[NVCV_MAX_STATUS_MESSAGE_LENGTH];
};

// Runs fn; any exception becomes the calling thread's NVCV status (same contract as the core
// library's entry points; reference: src/nvcv/src/include/nvcv/Exception.hpp:209-222).
template<class F>
NVCVStatus Protect(F &&fn) noexcept
{
    try
    {
        fn();
        return NVCV_SUCCESS;
    }
    catch (const OpError &e)
    {
        nvcvSetThreadStatus(e.code(), "%s", e.what());
        return e.code();
    }
    catch (const std::bad_alloc &)
    {
        nvcvSetThreadStatus(NVCV_ERROR_OUT_OF_MEMORY, "Not enough space for resource allocation");
        return NVCV_ERROR_OUT_OF_MEMORY;
    }
    catch (const std::exception &e)
    {
        nvcvSetThreadStatus(NVCV_ERROR_INTERNAL, "%s", e.what());
        return NVCV_ERROR_INTERNAL;
    }
    catch (...)
    {
        nvcvSetThreadStatus(NVCV_ERROR_INTERNAL, "Unexpected error");
        return NVCV_ERROR_INTERNAL;
    }
}

// The bits of an enumeration argument as an int. A C caller can pass any integer where the C API names an
// enum; reading such a value THROUGH the enum type is undefined in C++ when it lies outside the range the
// enumerators span (the undefined-behaviour sanitizer reports every such read), so arguments that are
// validated - and may be invalid - are carried as plain ints from the entry point on.
template<class E>
inline int EnumBits(const E &e)
{
    static_assert(sizeof(E) == sizeof(int), "C enums of this API are int-sized");
    int v;
    __builtin_memcpy(&v, &e, sizeof(v));
    return v;
}

// A colour conversion code as callers pass it (an NVCVColorConversionCode, possibly not a valid one).
using ColorCode = int;

// Calls a core-library function and rethrows its status (with its message) as an OpError.
void CheckCore(NVCVStatus st);
void CheckHip(hipError_t e, const char *what);
// After a kernel launch: launch-configuration errors are reported as INTERNAL.
void CheckLaunch(const char *kernel);

// ---- operator handles -------------------------------------------------------------------------
// An operator handle is a plain heap object (created by cvcuda*Create, freed by nvcvOperatorDestroy),
// as in the reference (src/cvcuda/OpResize.cpp:40, Operator.cpp:26-29). Submit entry points get
// INVALID_ARGUMENT for a NULL handle and NOT_COMPATIBLE for a handle of another operator
// (src/cvcuda/priv/IOperator.hpp:56-73).
class IOperator
{
public:
    virtual ~IOperator();

    static constexpr uint64_t kMagic = 0x43564F50414D4431ull; // "CVOPAMD1"
    uint64_t                  magic  = kMagic;
};

template<class T>
T &ToOperator(NVCVOperatorHandle h)
{
    if (h == nullptr)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Operator handle must not be NULL");
    }
    IOperator *base = reinterpret_cast<IOperator *>(h);
    if (base->magic != IOperator::kMagic)
    {
        throw OpError(NVCV_ERROR_NOT_COMPATIBLE, "Handle doesn't refer to a live operator");
    }
    T *op = dynamic_cast<T *>(base);
    if (op == nullptr)
    {
        throw OpError(NVCV_ERROR_NOT_COMPATIBLE, "Handle doesn't correspond to the requested operator");
    }
    return *op;
}

template<class T, class... A>
NVCVStatus CreateOperator(NVCVOperatorHandle *handle, A &&...args)
{
    return Protect(
        [&]
        {
            if (handle == nullptr)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Pointer to NVCVOperator handle must not be NULL");
            }
            *handle = reinterpret_cast<NVCVOperatorHandle>(static_cast<IOperator *>(new T(static_cast<A &&>(args)...)));
        });
}

// ---- element types ------------------------------------------------------------------------------
// Same numbering as the reference's internal dtype enum (src/cvcuda/priv/legacy/CvCudaLegacy.h:53-63).
enum ElemType
{
    kU8      = 0,
    kS8      = 1,
    kU16     = 2,
    kS16     = 3,
    kS32     = 4,
    kF32     = 5,
    kF64     = 6,
    kF16     = 7,
    kU32     = 8, // beyond the reference's enum: CropFlipNormalizeReformat and the byte-moving operators take it
    kUnknown = -1
};

int ElemSize(ElemType t);

struct DTypeInfo
{
    ElemType elem;
    int      channels; // components packed in one tensor element
};

DTypeInfo DecodeDataType(NVCVDataType dt);

// ---- image-batch view of a tensor -----------------------------------------------------------------
// Layouts accepted: NHWC, HWC, NCHW, CHW, NHW, HW (the set the reference's
// TensorDataAccessStridedImagePlanar handles for these operators). Strides are in bytes.
enum LayoutKind
{
    kLayoutNHWC, // also HWC, NHW, HW (channels innermost or absent)
    kLayoutNCHW  // also CHW
};

struct ImageBatchView
{
    uint8_t   *base;
    int        N, H, W, C; // C counts tensor channel dim x channels packed in the dtype
    int64_t    strideN, strideH, strideW, strideC;
    ElemType   elem;
    LayoutKind layout;
    bool       hasBatchDim;
    char       layoutName[NVCV_TENSOR_MAX_RANK + 1];

    int64_t bytesSpanned() const // sampleStride * N, the quantity the reference compares with INT32_MAX
    {
        return strideN * N;
    }
};

// what: "Input" / "Output" for messages. Throws INVALID_ARGUMENT for non-device buffers.
void           ExportTensor(NVCVTensorHandle h, NVCVTensorData &out, const char *what);
// Returns false when the layout is not one of the image layouts above.
bool           MakeImageBatchView(const NVCVTensorData &d, ImageBatchView &v);
ImageBatchView RequireImageBatchView(const NVCVTensorData &d, const char *what, NVCVStatus onBadLayout);

// ---- var-shape batch view ---------------------------------------------------------------------------
struct VarShapeView
{
    NVCVImageBatchData            data;     // device lists (descriptor upload already enqueued on the stream)
    const NVCVImageBufferStrided *hostList; // host mirror of data.buffer.varShapeStrided.imageList
    int                           N;
    NVCVImageFormat               uniqueFormat;
    int                           maxW, maxH;
};

VarShapeView ExportVarShape(NVCVImageBatchHandle h, hipStream_t stream, const char *what);

struct FormatInfo
{
    int      planes;
    int      channels;
    ElemType elem; // component type of plane 0; kUnknown if components differ or are sub-byte
};

FormatInfo DecodeFormat(NVCVImageFormat fmt);

// ---- launch helpers -----------------------------------------------------------------------------------
inline int DivUp(int a, int b)
{
    return (a + b - 1) / b;
}

} // namespace cvamd

#endif // CVCUDA_AMD_OPCOMMON_HPP
