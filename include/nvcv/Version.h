/* Library version as one integer: major*1000000 + minor*10000 + patch*100 + tweak.
 * Replaces: src/nvcv/src/include/nvcv/Version.h:40; the numbers themselves are in VersionDef.h. */
#ifndef NVCV_VERSION_H
#define NVCV_VERSION_H

#include "Export.h"
#include "VersionDef.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

/* Version of the loaded library, which may differ from NVCV_VERSION of the headers a program was built with. */
NVCV_PUBLIC uint32_t nvcvGetVersion(void);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_VERSION_H */
