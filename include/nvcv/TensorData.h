/* Plain-data description of a strided tensor in device memory.
 * Replaces: src/nvcv/src/include/nvcv/TensorData.h:31-80. */
#ifndef NVCV_TENSORDATA_H
#define NVCV_TENSORDATA_H

#include "DataType.h"
#include "Fwd.h"
#include "TensorLayout.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

typedef struct NVCVTensorBufferStridedRec
{
    int64_t   strides[NVCV_TENSOR_MAX_RANK]; /* bytes between consecutive elements of each dimension */
    NVCVByte *basePtr;                       /* device address of element [0,0,...] */
} NVCVTensorBufferStrided;

typedef enum
{
    NVCV_TENSOR_BUFFER_NONE = 0,
    NVCV_TENSOR_BUFFER_STRIDED_CUDA /* device-accessible (HBM) strided buffer */
} NVCVTensorBufferType;

typedef union NVCVTensorBufferRec
{
    NVCVTensorBufferStrided strided;
} NVCVTensorBuffer;

typedef struct NVCVTensorDataRec
{
    NVCVDataType         dtype;
    NVCVTensorLayout     layout;
    int32_t              rank;
    int64_t              shape[NVCV_TENSOR_MAX_RANK];
    NVCVTensorBufferType bufferType;
    NVCVTensorBuffer     buffer;
} NVCVTensorData;

#ifdef __cplusplus
}
#endif

#endif /* NVCV_TENSORDATA_H */
