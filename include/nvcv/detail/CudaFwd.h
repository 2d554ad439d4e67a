/* Forward declarations of the two device-runtime handle types the C++ wrappers name without including
 * the runtime's headers: the stream handle and the opaque array handle of NVCV_IMAGE_BUFFER_CUDA_ARRAY
 * image data (a buffer type this library never produces; the wrapper class for it only needs the name).
 * Replaces: src/nvcv/src/include/nvcv/detail/CudaFwd.h:17-24. On this platform the stream handle is HIP's. */
#ifndef NVCV_DETAIL_FWD_CUDA_H
#define NVCV_DETAIL_FWD_CUDA_H

typedef struct ihipStream_t *hipStream_t;
typedef struct ihipStream_t *CUstream;
typedef struct cudaArray    *cudaArray_t;

#endif /* NVCV_DETAIL_FWD_CUDA_H */
