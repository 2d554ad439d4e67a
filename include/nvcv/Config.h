/* Handle-pool limits. Replaces: src/nvcv/src/include/nvcv/Config.h:48-108.
 * maxCount >= 0 fixes the pool at that many live objects, -1 makes it grow on demand (default).
 * Changing a limit while objects of that kind are alive -> INVALID_OPERATION. */
#ifndef NVCV_CONFIG_H
#define NVCV_CONFIG_H

#include "Export.h"
#include "Status.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

NVCV_PUBLIC NVCVStatus nvcvConfigSetMaxImageCount(int32_t maxCount);
NVCV_PUBLIC NVCVStatus nvcvConfigSetMaxImageBatchCount(int32_t maxCount);
NVCV_PUBLIC NVCVStatus nvcvConfigSetMaxTensorCount(int32_t maxCount);
NVCV_PUBLIC NVCVStatus nvcvConfigSetMaxAllocatorCount(int32_t maxCount);
/* Accepted for source compatibility with callers of nvcv/Config.hpp; this library has no array objects, so the
 * limit has nothing to act on. */
NVCV_PUBLIC NVCVStatus nvcvConfigSetMaxArrayCount(int32_t maxCount);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_CONFIG_H */
