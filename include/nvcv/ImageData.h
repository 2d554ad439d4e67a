/* Plain-data description of an image: up to 6 pitch-linear planes in device memory.
 * Replaces: src/nvcv/src/include/nvcv/ImageData.h:27-129. */
#ifndef NVCV_IMAGEDATA_H
#define NVCV_IMAGEDATA_H

#include "Fwd.h"
#include "ImageFormat.h"
#include "detail/CudaFwd.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

typedef struct NVCVImagePlaneStridedRec
{
    int32_t   width;     /* pixels */
    int32_t   height;    /* rows */
    int32_t   rowStride; /* bytes between rows, >= ceil(width * bitsPerPixel / 8) */
    NVCVByte *basePtr;   /* device address of pixel (0,0) */
} NVCVImagePlaneStrided;

#define NVCV_MAX_PLANE_COUNT (6)

typedef struct NVCVImageBufferStridedRec
{
    int32_t               numPlanes;
    NVCVImagePlaneStrided planes[NVCV_MAX_PLANE_COUNT];
} NVCVImageBufferStrided;

/* Layout placeholder for the reference's texture-array variant; never produced or accepted here. */
typedef struct NVCVImageBufferCudaArrayRec
{
    int32_t     numPlanes;
    cudaArray_t planes[NVCV_MAX_PLANE_COUNT];
} NVCVImageBufferCudaArray;

typedef enum
{
    NVCV_IMAGE_BUFFER_NONE = 0,
    NVCV_IMAGE_BUFFER_STRIDED_CUDA, /* device-accessible (HBM) */
    NVCV_IMAGE_BUFFER_STRIDED_HOST,
    NVCV_IMAGE_BUFFER_CUDA_ARRAY
} NVCVImageBufferType;

typedef union NVCVImageBufferRec
{
    NVCVImageBufferStrided   strided;
    NVCVImageBufferCudaArray cudaarray;
} NVCVImageBuffer;

typedef struct NVCVImageDataRec
{
    NVCVImageFormat     format;
    NVCVImageBufferType bufferType;
    NVCVImageBuffer     buffer;
} NVCVImageData;

#ifdef __cplusplus
}
#endif

#endif /* NVCV_IMAGEDATA_H */
