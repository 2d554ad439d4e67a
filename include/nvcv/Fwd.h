/* Opaque handle types. Replaces: src/nvcv/src/include/nvcv/Fwd.h:29-37, alloc/Fwd.h:26-28,
 * detail/CudaFwd.h (the stream slot is a hipStream_t here). */
#ifndef NVCV_FWD_H
#define NVCV_FWD_H

#ifdef __cplusplus
extern "C"
{
#endif

typedef struct NVCVImage      *NVCVImageHandle;
typedef struct NVCVImageBatch *NVCVImageBatchHandle;
typedef struct NVCVTensor     *NVCVTensorHandle;
typedef struct NVCVAllocator  *NVCVAllocatorHandle;

typedef unsigned char NVCVByte;

/* HIP stream, declared without pulling in the HIP headers (same tag as hip_runtime_api.h). */
typedef struct ihipStream_t *NVCVStreamHandle;

#ifdef __cplusplus
}
#endif

#endif /* NVCV_FWD_H */
