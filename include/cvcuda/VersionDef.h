/* Version numbers of the operator interface and helpers to compare against them.
 * Replaces the header the reference generates at build time from cmake/VersionDef.h.in:30-112 (installed as
 * cvcuda/VersionDef.h). A version is one integer: major*1000000 + minor*10000 + patch*100 + tweak. */
#ifndef CVCUDA_VERSIONDEF_H
#define CVCUDA_VERSIONDEF_H

#include <stdint.h>

#define CVCUDA_MAKE_VERSION4(major, minor, patch, tweak) \
    ((uint32_t)((major)*1000000 + (minor)*10000 + (patch)*100 + (tweak)))
#define CVCUDA_MAKE_VERSION3(major, minor, patch) CVCUDA_MAKE_VERSION4(major, minor, patch, 0)
#define CVCUDA_MAKE_VERSION2(major, minor) CVCUDA_MAKE_VERSION4(major, minor, 0, 0)
#define CVCUDA_MAKE_VERSION1(major) CVCUDA_MAKE_VERSION4(major, 0, 0, 0)
/* one to four components */
#define CVCUDA_DETAIL_GET_MACRO(_1, _2, _3, _4, NAME, ...) NAME
#define CVCUDA_MAKE_VERSION(...)                                                                               \
    CVCUDA_DETAIL_GET_MACRO(__VA_ARGS__, CVCUDA_MAKE_VERSION4, CVCUDA_MAKE_VERSION3, CVCUDA_MAKE_VERSION2, CVCUDA_MAKE_VERSION1) \
    (__VA_ARGS__)

#define CVCUDA_VERSION_MAJOR 0
#define CVCUDA_VERSION_MINOR 15
#define CVCUDA_VERSION_PATCH 0
#define CVCUDA_VERSION_TWEAK 0
#define CVCUDA_VERSION_SUFFIX ""
#define CVCUDA_VERSION \
    CVCUDA_MAKE_VERSION(CVCUDA_VERSION_MAJOR, CVCUDA_VERSION_MINOR, CVCUDA_VERSION_PATCH, CVCUDA_VERSION_TWEAK)
#define CVCUDA_VERSION_STRING "0.15.0"

/* The interface version a program is written against: define CVCUDA_VERSION_API before including this header to
 * pin an older minor version of the same major; by default it is this header's major.minor. */
#ifdef CVCUDA_VERSION_API
#    if CVCUDA_VERSION_API < CVCUDA_MAKE_VERSION(CVCUDA_VERSION_MAJOR) \
        || CVCUDA_VERSION_API > CVCUDA_MAKE_VERSION(CVCUDA_VERSION_MAJOR, CVCUDA_VERSION_MINOR)
#        error Selected CVCUDA API version not supported.
#    endif
#else
#    define CVCUDA_VERSION_API CVCUDA_MAKE_VERSION(CVCUDA_VERSION_MAJOR, CVCUDA_VERSION_MINOR)
#endif

#define CVCUDA_VERSION_API_IS(major, minor) (CVCUDA_MAKE_VERSION(major, minor) == CVCUDA_VERSION_API)
#define CVCUDA_VERSION_API_AT_LEAST(major, minor) (CVCUDA_MAKE_VERSION(major, minor) <= CVCUDA_VERSION_API)
#define CVCUDA_VERSION_API_AT_MOST(major, minor) (CVCUDA_MAKE_VERSION(major, minor) >= CVCUDA_VERSION_API)
#define CVCUDA_VERSION_API_IN_RANGE(min_major, min_minor, max_major, max_minor) \
    (CVCUDA_VERSION_API_AT_LEAST(min_major, min_minor) && CVCUDA_VERSION_API_AT_MOST(max_major, max_minor))

#endif /* CVCUDA_VERSIONDEF_H */
