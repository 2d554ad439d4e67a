/* Variable-shape image batches: an ordered list of image handles plus a device-side array of
 * their plane descriptors, refreshed lazily on export.
 * Replaces: src/nvcv/src/include/nvcv/ImageBatch.h:40-403 (behaviour of
 * src/nvcv/src/priv/ImageBatchVarShape.cpp:38-430). */
#ifndef NVCV_IMAGEBATCH_H
#define NVCV_IMAGEBATCH_H

#include "Export.h"
#include "Fwd.h"
#include "Image.h"
#include "ImageBatchData.h"
#include "Status.h"
#include "alloc/Allocator.h"
#include "alloc/Requirements.h"

#ifdef __cplusplus
extern "C"
{
#endif

typedef enum
{
    NVCV_TYPE_IMAGEBATCH_VARSHAPE,
    NVCV_TYPE_IMAGEBATCH_TENSOR,
    NVCV_TYPE_IMAGEBATCH_TENSOR_WRAPDATA
} NVCVTypeImageBatch;

typedef void (*NVCVImageBatchDataCleanupFunc)(void *ctx, const NVCVImageBatchData *data);

typedef struct NVCVImageBatchVarShapeRequirementsRec
{
    int32_t          capacity;
    int32_t          alignBytes;
    NVCVRequirements mem;
} NVCVImageBatchVarShapeRequirements;

NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapeCalcRequirements(int32_t                             capacity,
                                                              NVCVImageBatchVarShapeRequirements *reqs);
NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapeConstruct(const NVCVImageBatchVarShapeRequirements *reqs,
                                                       NVCVAllocatorHandle alloc, NVCVImageBatchHandle *handle);
NVCV_PUBLIC NVCVStatus nvcvImageBatchDecRef(NVCVImageBatchHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvImageBatchIncRef(NVCVImageBatchHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvImageBatchRefCount(NVCVImageBatchHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvImageBatchSetUserPointer(NVCVImageBatchHandle handle, void *userPtr);
NVCV_PUBLIC NVCVStatus nvcvImageBatchGetUserPointer(NVCVImageBatchHandle handle, void **outUserPtr);
NVCV_PUBLIC NVCVStatus nvcvImageBatchGetType(NVCVImageBatchHandle handle, NVCVTypeImageBatch *type);
NVCV_PUBLIC NVCVStatus nvcvImageBatchGetCapacity(NVCVImageBatchHandle handle, int32_t *capacity);
NVCV_PUBLIC NVCVStatus nvcvImageBatchGetAllocator(NVCVImageBatchHandle handle, NVCVAllocatorHandle *alloc);
NVCV_PUBLIC NVCVStatus nvcvImageBatchGetNumImages(NVCVImageBatchHandle handle, int32_t *numImages);

/* Fills `data`; descriptors pushed since the last export are copied to the device on `stream`
 * (asynchronously, from pinned staging), so kernels launched later on that stream see them. */
NVCV_PUBLIC NVCVStatus nvcvImageBatchExportData(NVCVImageBatchHandle handle, NVCVStreamHandle stream,
                                                NVCVImageBatchData *data);

NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapeGetMaxSize(NVCVImageBatchHandle handle, int32_t *maxWidth,
                                                        int32_t *maxHeight);
NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapeGetUniqueFormat(NVCVImageBatchHandle handle, NVCVImageFormat *format);

/* Appends images (the batch takes one reference on each); exceeding the capacity -> OVERFLOW and
 * the batch is left unchanged. The callback variant appends until the callback returns NULL. */
NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapePushImages(NVCVImageBatchHandle handle, const NVCVImageHandle *images,
                                                        int32_t numImages);
typedef NVCVImageHandle (*NVCVPushImageFunc)(void *ctx);
NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapePushImagesCallback(NVCVImageBatchHandle handle,
                                                                NVCVPushImageFunc cbPushImage, void *ctxCallback);
/* Removes the last numImages images; more than present -> UNDERFLOW. */
NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapePopImages(NVCVImageBatchHandle handle, int32_t numImages);
NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapeClear(NVCVImageBatchHandle handle);
/* Copies handles [begIndex, begIndex+numImages) out, adding one reference to each. */
NVCV_PUBLIC NVCVStatus nvcvImageBatchVarShapeGetImages(NVCVImageBatchHandle handle, int32_t begIndex,
                                                       NVCVImageHandle *outImages, int32_t numImages);

/* Extension (no counterpart in the reference ABI): host-side copy of the plane descriptors, valid
 * until the batch is modified. Operators use it to size and pack their launch grids without a
 * device round trip. */
NVCV_PUBLIC NVCVStatus nvcvxImageBatchVarShapeGetHostImageList(NVCVImageBatchHandle          handle,
                                                               const NVCVImageBufferStrided **outList,
                                                               int32_t                       *outNumImages);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_IMAGEBATCH_H */
