/* Image objects: reference-counted, 1..4 pitch-linear planes in device memory.
 * Replaces: src/nvcv/src/include/nvcv/Image.h:40-295 (behaviour of src/nvcv/src/priv/Image.cpp:36-262). */
#ifndef NVCV_IMAGE_H
#define NVCV_IMAGE_H

#include "Export.h"
#include "Fwd.h"
#include "ImageData.h"
#include "ImageFormat.h"
#include "Status.h"
#include "alloc/Allocator.h"
#include "alloc/Requirements.h"

#ifdef __cplusplus
extern "C"
{
#endif

typedef enum
{
    NVCV_TYPE_IMAGE,         /* owns its memory */
    NVCV_TYPE_IMAGE_WRAPDATA /* wraps caller memory */
} NVCVTypeImage;

typedef void (*NVCVImageDataCleanupFunc)(void *ctx, const NVCVImageData *data);

typedef struct NVCVImageRequirementsRec
{
    int32_t          width, height;
    NVCVImageFormat  format;
    int32_t          planeRowStride[NVCV_MAX_PLANE_COUNT];
    int32_t          alignBytes;
    NVCVRequirements mem;
} NVCVImageRequirements;

/* Alignments are powers of two, 0 = library default (128-byte rows, 512-byte base). All planes live
 * in one allocation, each plane starting at a multiple of the base alignment. */
NVCV_PUBLIC NVCVStatus nvcvImageCalcRequirements(int32_t width, int32_t height, NVCVImageFormat format,
                                                 int32_t baseAddrAlignment, int32_t rowAddrAlignment,
                                                 NVCVImageRequirements *reqs);
NVCV_PUBLIC NVCVStatus nvcvImageConstruct(const NVCVImageRequirements *reqs, NVCVAllocatorHandle alloc,
                                          NVCVImageHandle *handle);
NVCV_PUBLIC NVCVStatus nvcvImageWrapDataConstruct(const NVCVImageData *data, NVCVImageDataCleanupFunc cleanup,
                                                  void *ctxCleanup, NVCVImageHandle *handle);
NVCV_PUBLIC NVCVStatus nvcvImageDecRef(NVCVImageHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvImageIncRef(NVCVImageHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvImageRefCount(NVCVImageHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvImageSetUserPointer(NVCVImageHandle handle, void *userPtr);
NVCV_PUBLIC NVCVStatus nvcvImageGetUserPointer(NVCVImageHandle handle, void **outUserPtr);
NVCV_PUBLIC NVCVStatus nvcvImageGetType(NVCVImageHandle handle, NVCVTypeImage *type);
NVCV_PUBLIC NVCVStatus nvcvImageGetSize(NVCVImageHandle handle, int32_t *width, int32_t *height);
NVCV_PUBLIC NVCVStatus nvcvImageGetFormat(NVCVImageHandle handle, NVCVImageFormat *fmt);
NVCV_PUBLIC NVCVStatus nvcvImageGetAllocator(NVCVImageHandle handle, NVCVAllocatorHandle *alloc);
NVCV_PUBLIC NVCVStatus nvcvImageExportData(NVCVImageHandle handle, NVCVImageData *data);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_IMAGE_H */
