/* Library version as one integer: major*1000000 + minor*10000 + patch*100 + tweak.
 * Replaces: src/nvcv/src/include/nvcv/Version.h:40 and cmake/VersionDef.h.in:47-48. */
#ifndef NVCV_VERSION_H
#define NVCV_VERSION_H

#include "Export.h"

#include <stdint.h>

#define NVCV_VERSION_MAJOR 0
#define NVCV_VERSION_MINOR 15
#define NVCV_VERSION_PATCH 0
#define NVCV_VERSION_TWEAK 0

#define NVCV_MAKE_VERSION4(major, minor, patch, tweak) \
    ((uint32_t)((major)*1000000 + (minor)*10000 + (patch)*100 + (tweak)))
#define NVCV_VERSION \
    NVCV_MAKE_VERSION4(NVCV_VERSION_MAJOR, NVCV_VERSION_MINOR, NVCV_VERSION_PATCH, NVCV_VERSION_TWEAK)

#ifdef __cplusplus
extern "C"
{
#endif

NVCV_PUBLIC uint32_t nvcvGetVersion(void);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_VERSION_H */
