/* Replaces: src/cvcuda/include/cvcuda/Version.h (cvcudaGetVersion); the numbers themselves are in VersionDef.h. */
#ifndef CVCUDA_VERSION_H
#define CVCUDA_VERSION_H

#include "Operator.h"
#include "VersionDef.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif
/* Version of the loaded library, which may differ from CVCUDA_VERSION of the headers a program was built with. */
CVCUDA_PUBLIC uint32_t cvcudaGetVersion(void);
#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_VERSION_H */
