/* Language-level helper macros used by the C headers and by the reference's header-only C++ wrappers
 * (the nvcv .hpp files include this file by name).
 * Replaces: src/nvcv/src/include/nvcv/detail/CompilerUtils.h:17-35. */
#ifndef NVCV_DETAIL_COMPILERUTILS_H
#define NVCV_DETAIL_COMPILERUTILS_H

#ifdef __cplusplus
#    define NVCV_CONSTEXPR constexpr
#else
#    define NVCV_CONSTEXPR
#endif

#if defined(__cplusplus) && __cplusplus >= 201703L
#    define NVCV_NODISCARD [[nodiscard]]
#    define NVCV_IF_CONSTEXPR constexpr
#else
#    define NVCV_NODISCARD
#    define NVCV_IF_CONSTEXPR
#endif

#endif /* NVCV_DETAIL_COMPILERUTILS_H */
