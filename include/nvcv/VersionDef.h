/* Version numbers of the NVCV core interface and helpers to compare against them.
 * Replaces the header the reference generates at build time from cmake/VersionDef.h.in:30-112 (installed as
 * nvcv/VersionDef.h). A version is one integer: major*1000000 + minor*10000 + patch*100 + tweak. */
#ifndef NVCV_VERSIONDEF_H
#define NVCV_VERSIONDEF_H

#include <stdint.h>

#define NVCV_MAKE_VERSION4(major, minor, patch, tweak) \
    ((uint32_t)((major)*1000000 + (minor)*10000 + (patch)*100 + (tweak)))
#define NVCV_MAKE_VERSION3(major, minor, patch) NVCV_MAKE_VERSION4(major, minor, patch, 0)
#define NVCV_MAKE_VERSION2(major, minor) NVCV_MAKE_VERSION4(major, minor, 0, 0)
#define NVCV_MAKE_VERSION1(major) NVCV_MAKE_VERSION4(major, 0, 0, 0)
/* one to four components */
#define NVCV_DETAIL_GET_MACRO(_1, _2, _3, _4, NAME, ...) NAME
#define NVCV_MAKE_VERSION(...)                                                                               \
    NVCV_DETAIL_GET_MACRO(__VA_ARGS__, NVCV_MAKE_VERSION4, NVCV_MAKE_VERSION3, NVCV_MAKE_VERSION2, NVCV_MAKE_VERSION1) \
    (__VA_ARGS__)

#define NVCV_VERSION_MAJOR 0
#define NVCV_VERSION_MINOR 15
#define NVCV_VERSION_PATCH 0
#define NVCV_VERSION_TWEAK 0
#define NVCV_VERSION_SUFFIX ""
#define NVCV_VERSION \
    NVCV_MAKE_VERSION(NVCV_VERSION_MAJOR, NVCV_VERSION_MINOR, NVCV_VERSION_PATCH, NVCV_VERSION_TWEAK)
#define NVCV_VERSION_STRING "0.15.0"

/* The interface version a program is written against: define NVCV_VERSION_API before including this header to
 * pin an older minor version of the same major; by default it is this header's major.minor. */
#ifdef NVCV_VERSION_API
#    if NVCV_VERSION_API < NVCV_MAKE_VERSION(NVCV_VERSION_MAJOR) \
        || NVCV_VERSION_API > NVCV_MAKE_VERSION(NVCV_VERSION_MAJOR, NVCV_VERSION_MINOR)
#        error Selected NVCV API version not supported.
#    endif
#else
#    define NVCV_VERSION_API NVCV_MAKE_VERSION(NVCV_VERSION_MAJOR, NVCV_VERSION_MINOR)
#endif

#define NVCV_VERSION_API_IS(major, minor) (NVCV_MAKE_VERSION(major, minor) == NVCV_VERSION_API)
#define NVCV_VERSION_API_AT_LEAST(major, minor) (NVCV_MAKE_VERSION(major, minor) <= NVCV_VERSION_API)
#define NVCV_VERSION_API_AT_MOST(major, minor) (NVCV_MAKE_VERSION(major, minor) >= NVCV_VERSION_API)
#define NVCV_VERSION_API_IN_RANGE(min_major, min_minor, max_major, max_minor) \
    (NVCV_VERSION_API_AT_LEAST(min_major, min_minor) && NVCV_VERSION_API_AT_MOST(max_major, max_minor))

#endif /* NVCV_VERSIONDEF_H */
