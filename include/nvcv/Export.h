/* Symbol visibility for the NVCV core library (ELF only).
 * Replaces: src/nvcv/src/include/nvcv/Export.h:21-45 of the reference. */
#ifndef NVCV_EXPORT_H
#define NVCV_EXPORT_H

#if defined(__GNUC__) && !defined(NVCV_STATIC)
#    define NVCV_PUBLIC __attribute__((visibility("default")))
#else
#    define NVCV_PUBLIC
#endif

#ifdef __cplusplus
#    define NVCV_CONSTEXPR constexpr
#else
#    define NVCV_CONSTEXPR
#endif

#endif /* NVCV_EXPORT_H */
