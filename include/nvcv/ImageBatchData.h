/* Plain-data description of a batch of images of different sizes.
 * Replaces: src/nvcv/src/include/nvcv/ImageBatchData.h:26-111. */
#ifndef NVCV_IMAGEBATCHDATA_H
#define NVCV_IMAGEBATCHDATA_H

#include "ImageData.h"

#ifdef __cplusplus
extern "C"
{
#endif

typedef struct NVCVImageBatchVarShapeBufferStridedRec
{
    NVCVImageFormat         uniqueFormat;        /* common format, or NVCV_IMAGE_FORMAT_NONE if they differ */
    int32_t                 maxWidth, maxHeight; /* over all images */
    NVCVImageFormat        *formatList;          /* device array, one entry per image */
    const NVCVImageFormat  *hostFormatList;      /* host copy of formatList */
    NVCVImageBufferStrided *imageList;           /* device array of plane descriptors, one per image */
} NVCVImageBatchVarShapeBufferStrided;

typedef struct NVCVImageBatchTensorBufferStridedRec
{
    int64_t imgStride;
    int32_t rowStride;
    int32_t imgWidth, imgHeight;
    void   *planeBuffer[NVCV_MAX_PLANE_COUNT];
} NVCVImageBatchTensorBufferStrided;

typedef enum
{
    NVCV_IMAGE_BATCH_BUFFER_NONE = 0,
    NVCV_IMAGE_BATCH_VARSHAPE_BUFFER_STRIDED_CUDA
} NVCVImageBatchBufferType;

typedef union NVCVImageBatchBufferRec
{
    NVCVImageBatchVarShapeBufferStrided varShapeStrided;
} NVCVImageBatchBuffer;

typedef struct NVCVImageBatchDataRec
{
    int32_t                  numImages;
    NVCVImageBatchBufferType bufferType;
    NVCVImageBatchBuffer     buffer;
} NVCVImageBatchData;

#ifdef __cplusplus
}
#endif

#endif /* NVCV_IMAGEBATCHDATA_H */
