/* Tensor objects: reference-counted N-D strided arrays in device memory.
 * Replaces: src/nvcv/src/include/nvcv/Tensor.h:38-403 (entry points src/nvcv/src/Tensor.cpp:40-354,
 * stride rule src/nvcv/src/priv/Tensor.cpp:95-190, wrap validation
 * src/nvcv/src/priv/TensorWrapDataStrided.cpp:35-105). */
#ifndef NVCV_TENSOR_H
#define NVCV_TENSOR_H

#include "Export.h"
#include "Fwd.h"
#include "Image.h"
#include "ImageFormat.h"
#include "Status.h"
#include "TensorData.h"
#include "alloc/Allocator.h"
#include "alloc/Requirements.h"

#ifdef __cplusplus
extern "C"
{
#endif

typedef void (*NVCVTensorDataCleanupFunc)(void *ctx, const NVCVTensorData *data);

typedef struct NVCVTensorRequirementsRec
{
    NVCVDataType     dtype;
    NVCVTensorLayout layout;
    int32_t          rank;
    int64_t          shape[NVCV_TENSOR_MAX_RANK];
    int64_t          strides[NVCV_TENSOR_MAX_RANK]; /* bytes */
    int32_t          alignBytes;                    /* base address alignment */
    NVCVRequirements mem;
} NVCVTensorRequirements;

/* Strides for a tensor of the given shape. Alignments are powers of two, 0 = library default
 * (128-byte rows, 512-byte base). The innermost dimension is packed; for layouts ending in "WC" the
 * W and C dimensions are packed together and the dimension outside W (the row) is padded to the
 * row alignment; for any other layout the second-innermost stride is padded. */
NVCV_PUBLIC NVCVStatus nvcvTensorCalcRequirements(int32_t rank, const int64_t *shape, NVCVDataType dtype,
                                                  NVCVTensorLayout layout, int32_t baseAddrAlignment,
                                                  int32_t rowAddrAlignment, NVCVTensorRequirements *reqs);
/* Same for a batch of numImages equal images: one plane -> NHWC, planes==channels -> NCHW. */
NVCV_PUBLIC NVCVStatus nvcvTensorCalcRequirementsForImages(int32_t numImages, int32_t width, int32_t height,
                                                           NVCVImageFormat format, int32_t baseAddrAlignment,
                                                           int32_t rowAddrAlignment, NVCVTensorRequirements *reqs);

/* Allocates reqs->mem.cudaMem through `alloc` (NULL = default) and returns a handle owning one reference. */
NVCV_PUBLIC NVCVStatus nvcvTensorConstruct(const NVCVTensorRequirements *reqs, NVCVAllocatorHandle alloc,
                                           NVCVTensorHandle *handle);
/* Wraps caller-owned device memory; `cleanup` (may be NULL) runs when the last reference goes away. */
NVCV_PUBLIC NVCVStatus nvcvTensorWrapDataConstruct(const NVCVTensorData *data, NVCVTensorDataCleanupFunc cleanup,
                                                   void *ctxCleanup, NVCVTensorHandle *handle);
/* Views an image as a 1-image tensor; the tensor keeps a reference on the image. */
NVCV_PUBLIC NVCVStatus nvcvTensorWrapImageConstruct(NVCVImageHandle img, NVCVTensorHandle *handle);

NVCV_PUBLIC NVCVStatus nvcvTensorDecRef(NVCVTensorHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvTensorIncRef(NVCVTensorHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvTensorRefCount(NVCVTensorHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvTensorSetUserPointer(NVCVTensorHandle handle, void *userPtr);
NVCV_PUBLIC NVCVStatus nvcvTensorGetUserPointer(NVCVTensorHandle handle, void **outUserPtr);
NVCV_PUBLIC NVCVStatus nvcvTensorGetDataType(NVCVTensorHandle handle, NVCVDataType *type);
NVCV_PUBLIC NVCVStatus nvcvTensorGetLayout(NVCVTensorHandle handle, NVCVTensorLayout *layout);
NVCV_PUBLIC NVCVStatus nvcvTensorGetAllocator(NVCVTensorHandle handle, NVCVAllocatorHandle *alloc);
NVCV_PUBLIC NVCVStatus nvcvTensorExportData(NVCVTensorHandle handle, NVCVTensorData *data);
/* *rank: in = capacity of shape[], out = tensor rank; leading entries are filled with 1 when capacity > rank. */
NVCV_PUBLIC NVCVStatus nvcvTensorGetShape(NVCVTensorHandle handle, int32_t *rank, int64_t *shape);
/* New tensor sharing the same memory with another shape of equal volume; the source must be densely packed. */
NVCV_PUBLIC NVCVStatus nvcvTensorReshape(NVCVTensorHandle handle, int32_t rank, const int64_t *shape,
                                         NVCVTensorLayout layout, NVCVTensorHandle *out_handle);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_TENSOR_H */
