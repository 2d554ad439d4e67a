/* Replaces: src/cvcuda/include/cvcuda/Version.h (cvcudaGetVersion). */
#ifndef CVCUDA_VERSION_H
#define CVCUDA_VERSION_H

#include "Operator.h"

#include <stdint.h>

#define CVCUDA_VERSION_MAJOR 0
#define CVCUDA_VERSION_MINOR 15
#define CVCUDA_VERSION_PATCH 0
#define CVCUDA_VERSION ((uint32_t)(CVCUDA_VERSION_MAJOR * 1000000 + CVCUDA_VERSION_MINOR * 10000 + CVCUDA_VERSION_PATCH * 100))

#ifdef __cplusplus
extern "C"
{
#endif
CVCUDA_PUBLIC uint32_t cvcudaGetVersion(void);
#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_VERSION_H */
