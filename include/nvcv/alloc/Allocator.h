/* Resource allocators. A NULL allocator handle everywhere means "the default one":
 * hipMalloc for device memory, hipHostMalloc for pinned memory, aligned_alloc for host memory.
 * Replaces: src/nvcv/src/include/nvcv/alloc/Allocator.h:77-388 (default behaviour of
 * src/nvcv/src/priv/DefaultAllocator.cpp:29-84, retargeted from the CUDA to the HIP runtime). */
#ifndef NVCV_ALLOCATOR_H
#define NVCV_ALLOCATOR_H

#include "../Export.h"
#include "../Fwd.h"
#include "../Status.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

typedef void *(*NVCVMemAllocFunc)(void *ctx, int64_t sizeBytes, int32_t alignBytes);
typedef void (*NVCVMemFreeFunc)(void *ctx, void *ptr, int64_t sizeBytes, int32_t alignBytes);

typedef enum
{
    NVCV_RESOURCE_MEM_HOST,
    NVCV_RESOURCE_MEM_CUDA, /* device memory (HBM) */
    NVCV_RESOURCE_MEM_HOST_PINNED
} NVCVResourceType;

#define NVCV_NUM_RESOURCE_TYPES (3)

typedef struct NVCVCustomMemAllocatorRec
{
    NVCVMemAllocFunc fnAlloc;
    NVCVMemFreeFunc  fnFree;
} NVCVCustomMemAllocator;

typedef union NVCVCustomResourceAllocatorRec
{
    NVCVCustomMemAllocator mem;
} NVCVCustomResourceAllocator;

typedef struct NVCVResourceAllocatorRec NVCVResourceAllocator;
typedef void (*NVCVResourceAllocatorCleanupFunc)(void *ctx, NVCVResourceAllocator *data);

struct NVCVResourceAllocatorRec
{
    void                            *ctx;
    NVCVResourceType                 resType;
    NVCVCustomResourceAllocator      res;
    NVCVResourceAllocatorCleanupFunc cleanup; /* may be NULL; runs when the allocator object dies */
};

/* Builds an allocator from 0..3 per-resource overrides (each resource type at most once). */
NVCV_PUBLIC NVCVStatus nvcvAllocatorConstructCustom(const NVCVResourceAllocator *customAllocators,
                                                    int32_t numCustomAllocators, NVCVAllocatorHandle *handle);
NVCV_PUBLIC NVCVStatus nvcvAllocatorDecRef(NVCVAllocatorHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvAllocatorIncRef(NVCVAllocatorHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvAllocatorRefCount(NVCVAllocatorHandle handle, int *newRefCount);
NVCV_PUBLIC NVCVStatus nvcvAllocatorGet(NVCVAllocatorHandle handle, NVCVResourceType resType,
                                        NVCVResourceAllocator *result);
NVCV_PUBLIC NVCVStatus nvcvAllocatorSetUserPointer(NVCVAllocatorHandle handle, void *userPtr);
NVCV_PUBLIC NVCVStatus nvcvAllocatorGetUserPointer(NVCVAllocatorHandle handle, void **outUserPtr);

/* sizeBytes >= 0, alignBytes a power of two; failure -> OUT_OF_MEMORY. */
NVCV_PUBLIC NVCVStatus nvcvAllocatorAllocHostMemory(NVCVAllocatorHandle halloc, void **ptr, int64_t sizeBytes,
                                                    int32_t alignBytes);
NVCV_PUBLIC NVCVStatus nvcvAllocatorFreeHostMemory(NVCVAllocatorHandle halloc, void *ptr, int64_t sizeBytes,
                                                   int32_t alignBytes);
NVCV_PUBLIC NVCVStatus nvcvAllocatorAllocHostPinnedMemory(NVCVAllocatorHandle halloc, void **ptr, int64_t sizeBytes,
                                                          int32_t alignBytes);
NVCV_PUBLIC NVCVStatus nvcvAllocatorFreeHostPinnedMemory(NVCVAllocatorHandle halloc, void *ptr, int64_t sizeBytes,
                                                         int32_t alignBytes);
NVCV_PUBLIC NVCVStatus nvcvAllocatorAllocCudaMemory(NVCVAllocatorHandle halloc, void **ptr, int64_t sizeBytes,
                                                    int32_t alignBytes);
NVCV_PUBLIC NVCVStatus nvcvAllocatorFreeCudaMemory(NVCVAllocatorHandle halloc, void *ptr, int64_t sizeBytes,
                                                   int32_t alignBytes);

NVCV_PUBLIC const char *nvcvResourceTypeGetName(NVCVResourceType resource);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_ALLOCATOR_H */
