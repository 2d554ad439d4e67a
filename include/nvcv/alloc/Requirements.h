/* Memory requirements of an object, bucketed by power-of-two alignment.
 * numBlocks[i] counts blocks of 2^i bytes that must be aligned to 2^i bytes.
 * Replaces: src/nvcv/src/include/nvcv/alloc/Requirements.h:40-122 (arithmetic of
 * src/nvcv/src/priv/Requirements.cpp:49-109). */
#ifndef NVCV_REQUIREMENTS_H
#define NVCV_REQUIREMENTS_H

#include "../Export.h"
#include "../Status.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

#define NVCV_MAX_MEM_REQUIREMENTS_LOG2_BLOCK_SIZE (32)
#define NVCV_MAX_MEM_REQUIREMENTS_BLOCK_SIZE (((int64_t)1) << NVCV_MAX_MEM_REQUIREMENTS_LOG2_BLOCK_SIZE)

typedef struct NVCVMemRequirementsRec
{
    int64_t numBlocks[NVCV_MAX_MEM_REQUIREMENTS_LOG2_BLOCK_SIZE];
} NVCVMemRequirements;

typedef struct NVCVRequirementsRec
{
    NVCVMemRequirements cudaMem;       /* device memory (HBM) */
    NVCVMemRequirements hostMem;       /* pageable host memory */
    NVCVMemRequirements hostPinnedMem; /* page-locked host memory */
} NVCVRequirements;

NVCV_PUBLIC NVCVStatus nvcvRequirementsInit(NVCVRequirements *req);
NVCV_PUBLIC NVCVStatus nvcvRequirementsAdd(NVCVRequirements *reqSum, const NVCVRequirements *req);
NVCV_PUBLIC NVCVStatus nvcvMemRequirementsCalcTotalSizeBytes(const NVCVMemRequirements *memReq, int64_t *sizeBytes);
/* bufSize<0 removes blocks (never below zero); bufAlignment must be a power of two < 2^32. */
NVCV_PUBLIC NVCVStatus nvcvMemRequirementsAddBuffer(NVCVMemRequirements *memReq, int64_t bufSize,
                                                    int64_t bufAlignment);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_REQUIREMENTS_H */
