/* Tensor layouts: up to 15 one-letter dimension labels, e.g. "NHWC".
 * Replaces: src/nvcv/src/include/nvcv/TensorLayout.h:36-297, TensorLayoutDef.inc.
 * The struct is passed and returned by value across the ABI: 16 chars + int32 rank = 20 bytes. */
#ifndef NVCV_TENSORLAYOUT_H
#define NVCV_TENSORLAYOUT_H

#include "Export.h"
#include "Status.h"
#include "detail/CompilerUtils.h"

#include <stdint.h>
#include <string.h>

#ifdef __cplusplus
extern "C"
{
#endif

#define NVCV_TENSOR_MAX_RANK (15)

typedef struct NVCVTensorLayoutRec
{
    char    data[NVCV_TENSOR_MAX_RANK + 1]; /* NUL-terminated labels */
    int32_t rank;
} NVCVTensorLayout;

typedef enum
{
    NVCV_TLABEL_BATCH   = 'N',
    NVCV_TLABEL_CHANNEL = 'C',
    NVCV_TLABEL_FRAME   = 'F',
    NVCV_TLABEL_DEPTH   = 'D',
    NVCV_TLABEL_HEIGHT  = 'H',
    NVCV_TLABEL_WIDTH   = 'W'
} NVCVTensorLabel;

#ifdef __cplusplus
#    define NVCV_TENSOR_LAYOUT_MAKE(str) \
        NVCVTensorLayout { str, (int32_t)(sizeof(str) - 1) }
#else
#    define NVCV_TENSOR_LAYOUT_MAKE(str) \
        { .data = str, .rank = (int32_t)(sizeof(str) - 1) }
#endif

NVCV_CONSTEXPR static const NVCVTensorLayout NVCV_TENSOR_NONE = NVCV_TENSOR_LAYOUT_MAKE("");

#define NVCV_DETAIL_TLAYOUT(L) NVCV_CONSTEXPR static const NVCVTensorLayout NVCV_TENSOR_##L = NVCV_TENSOR_LAYOUT_MAKE(#L);
NVCV_DETAIL_TLAYOUT(W)
NVCV_DETAIL_TLAYOUT(WC)
NVCV_DETAIL_TLAYOUT(CW)
NVCV_DETAIL_TLAYOUT(NW)
NVCV_DETAIL_TLAYOUT(NWC)
NVCV_DETAIL_TLAYOUT(NCW)
NVCV_DETAIL_TLAYOUT(HW)
NVCV_DETAIL_TLAYOUT(NHW)
NVCV_DETAIL_TLAYOUT(FHW)
NVCV_DETAIL_TLAYOUT(NFHW)
NVCV_DETAIL_TLAYOUT(CHW)
NVCV_DETAIL_TLAYOUT(NCHW)
NVCV_DETAIL_TLAYOUT(HWC)
NVCV_DETAIL_TLAYOUT(NHWC)
NVCV_DETAIL_TLAYOUT(CFHW)
NVCV_DETAIL_TLAYOUT(FCHW)
NVCV_DETAIL_TLAYOUT(FHWC)
NVCV_DETAIL_TLAYOUT(NCFHW)
NVCV_DETAIL_TLAYOUT(NFCHW)
NVCV_DETAIL_TLAYOUT(NFHWC)
NVCV_DETAIL_TLAYOUT(DHW)
NVCV_DETAIL_TLAYOUT(NDHW)
NVCV_DETAIL_TLAYOUT(CDHW)
NVCV_DETAIL_TLAYOUT(DHWC)
NVCV_DETAIL_TLAYOUT(NCDHW)
NVCV_DETAIL_TLAYOUT(NDHWC)
NVCV_DETAIL_TLAYOUT(FDHW)
NVCV_DETAIL_TLAYOUT(NFDHW)
NVCV_DETAIL_TLAYOUT(CFDHW)
NVCV_DETAIL_TLAYOUT(FCDHW)
NVCV_DETAIL_TLAYOUT(FDHWC)
NVCV_DETAIL_TLAYOUT(NCFDHW)
NVCV_DETAIL_TLAYOUT(NFCDHW)
NVCV_DETAIL_TLAYOUT(NFDHWC)
#undef NVCV_DETAIL_TLAYOUT

/* Layout assumed for a tensor of rank r created without one (index = r). */
NVCV_CONSTEXPR static const NVCVTensorLayout NVCV_TENSOR_IMPLICIT[7] = {
    NVCV_TENSOR_LAYOUT_MAKE(""),     NVCV_TENSOR_LAYOUT_MAKE("W"),     NVCV_TENSOR_LAYOUT_MAKE("HW"),
    NVCV_TENSOR_LAYOUT_MAKE("NHW"),  NVCV_TENSOR_LAYOUT_MAKE("NCHW"),  NVCV_TENSOR_LAYOUT_MAKE("NCDHW"),
    NVCV_TENSOR_LAYOUT_MAKE("NCFDHW"),
};

/* Builders. descr==NULL yields the empty layout; more than 15 labels -> INVALID_ARGUMENT.
 * First(n<0) is Last(-n) and vice versa; SubRange clamps [beg,end) (negatives count from the end). */
NVCV_PUBLIC NVCVStatus nvcvTensorLayoutMake(const char *descr, NVCVTensorLayout *layout);
NVCV_PUBLIC NVCVStatus nvcvTensorLayoutMakeRange(const char *beg, const char *end, NVCVTensorLayout *layout);
NVCV_PUBLIC NVCVStatus nvcvTensorLayoutMakeFirst(NVCVTensorLayout in, int32_t n, NVCVTensorLayout *layout);
NVCV_PUBLIC NVCVStatus nvcvTensorLayoutMakeLast(NVCVTensorLayout in, int32_t n, NVCVTensorLayout *layout);
NVCV_PUBLIC NVCVStatus nvcvTensorLayoutMakeSubRange(NVCVTensorLayout in, int32_t beg, int32_t end,
                                                    NVCVTensorLayout *layout);

/* Index of the first `label` at or after idxStart (negative idxStart counts from the end), or -1. */
static inline int32_t nvcvTensorLayoutFindDimIndex(NVCVTensorLayout layout, char label, int idxStart)
{
    int i = idxStart < 0 ? layout.rank + idxStart : idxStart;
    for (; i >= 0 && i < layout.rank; ++i)
    {
        if (layout.data[i] == label)
        {
            return i;
        }
    }
    return -1;
}

/* The three accessors below are constant expressions in C++ (the C++ wrappers evaluate them at compile time). */
NVCV_CONSTEXPR static inline char nvcvTensorLayoutGetLabel(NVCVTensorLayout layout, int idx)
{
    return ((idx < 0 ? layout.rank + idx : idx) >= 0 && (idx < 0 ? layout.rank + idx : idx) < layout.rank)
             ? layout.data[idx < 0 ? layout.rank + idx : idx]
             : '\0';
}

NVCV_CONSTEXPR static inline int32_t nvcvTensorLayoutGetNumDim(NVCVTensorLayout layout)
{
    return layout.rank;
}

/* memcmp-style ordering: by rank first, then by labels. */
static inline int32_t nvcvTensorLayoutCompare(NVCVTensorLayout a, NVCVTensorLayout b)
{
    return a.rank != b.rank ? a.rank - b.rank : memcmp(a.data, b.data, (size_t)a.rank);
}

static inline int32_t nvcvTensorLayoutStartsWith(NVCVTensorLayout layout, NVCVTensorLayout test)
{
    return test.rank <= layout.rank && memcmp(test.data, layout.data, (size_t)test.rank) == 0;
}

static inline int32_t nvcvTensorLayoutEndsWith(NVCVTensorLayout layout, NVCVTensorLayout test)
{
    return test.rank <= layout.rank
        && memcmp(test.data, layout.data + layout.rank - test.rank, (size_t)test.rank) == 0;
}

NVCV_CONSTEXPR static inline const char *nvcvTensorLayoutGetName(const NVCVTensorLayout *layout)
{
    return layout ? layout->data : "";
}

#ifdef __cplusplus
}
#endif

#endif /* NVCV_TENSORLAYOUT_H */
