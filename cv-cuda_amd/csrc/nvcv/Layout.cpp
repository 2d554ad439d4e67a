// Tensor layout builders and shape permutation.
// Semantics follow src/nvcv/src/priv/TensorLayout.cpp:25-160 and TensorShape.cpp:25-48 of the reference.
#include "Priv.hpp"

#include <algorithm>
#include <cstring>

namespace nvcvamd {

namespace {
NVCVTensorLayout FromRange(const char *beg, const char *end)
{
    if (beg == nullptr || end == nullptr)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Range pointers must not be NULL");
    }
    if (end < beg)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Range must not have negative length");
    }
    if (end - beg > NVCV_TENSOR_MAX_RANK)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Range length %ld too large, must be <= %d", (long)(end - beg),
                    NVCV_TENSOR_MAX_RANK);
    }
    NVCVTensorLayout out = {};
    out.rank             = (int32_t)(end - beg);
    std::memcpy(out.data, beg, (size_t)out.rank);
    return out;
}

NVCVTensorLayout First(const NVCVTensorLayout &l, int n);

NVCVTensorLayout Last(const NVCVTensorLayout &l, int n)
{
    if (n < 0)
    {
        return First(l, -n);
    }
    int k = std::min(n, (int)l.rank);
    return FromRange(l.data + l.rank - k, l.data + l.rank);
}

NVCVTensorLayout First(const NVCVTensorLayout &l, int n)
{
    if (n < 0)
    {
        return Last(l, -n);
    }
    return FromRange(l.data, l.data + std::min(n, (int)l.rank));
}
} // namespace

NVCVTensorLayout MakeLayout(const char *descr)
{
    if (descr == nullptr)
    {
        return NVCVTensorLayout{};
    }
    size_t n = strnlen(descr, NVCV_TENSOR_MAX_RANK + 1);
    if (n > NVCV_TENSOR_MAX_RANK)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Tensor layout description is too big, must have at most %d labels: %.20s...",
                    NVCV_TENSOR_MAX_RANK, descr);
    }
    return FromRange(descr, descr + n);
}

NVCVTensorLayout LayoutLast(const NVCVTensorLayout &l, int n)
{
    return Last(l, n);
}

void PermuteShape(const NVCVTensorLayout &srcL, const int64_t *src, const NVCVTensorLayout &dstL, int64_t *dst)
{
    NotNull(src, "Pointer to source shape");
    NotNull(dst, "Pointer to destination shape");
    std::fill_n(dst, dstL.rank, int64_t(1));
    for (int i = 0; i < srcL.rank; ++i)
    {
        int j = nvcvTensorLayoutFindDimIndex(dstL, srcL.data[i], 0);
        if (j >= 0)
        {
            dst[j] = src[i];
        }
    }
}

} // namespace nvcvamd

using namespace nvcvamd;

extern "C"
{
NVCVStatus nvcvTensorLayoutMake(const char *descr, NVCVTensorLayout *layout)
{
    return Protect([&] { *NotNull(layout, "Pointer to output layout") = MakeLayout(descr); });
}

NVCVStatus nvcvTensorLayoutMakeRange(const char *beg, const char *end, NVCVTensorLayout *layout)
{
    return Protect([&] { *NotNull(layout, "Pointer to output layout") = FromRange(beg, end); });
}

NVCVStatus nvcvTensorLayoutMakeFirst(NVCVTensorLayout in, int32_t n, NVCVTensorLayout *layout)
{
    return Protect([&] { *NotNull(layout, "Pointer to output layout") = First(in, n); });
}

NVCVStatus nvcvTensorLayoutMakeLast(NVCVTensorLayout in, int32_t n, NVCVTensorLayout *layout)
{
    return Protect([&] { *NotNull(layout, "Pointer to output layout") = Last(in, n); });
}

NVCVStatus nvcvTensorLayoutMakeSubRange(NVCVTensorLayout in, int32_t beg, int32_t end, NVCVTensorLayout *layout)
{
    return Protect(
        [&]
        {
            NotNull(layout, "Pointer to output layout");
            int b   = beg < 0 ? std::max(0, in.rank + beg) : std::min(beg, in.rank);
            int e   = end < 0 ? std::max(0, in.rank + end) : std::min(end, in.rank);
            *layout = e > b ? FromRange(in.data + b, in.data + e) : NVCVTensorLayout{};
        });
}

NVCVStatus nvcvTensorShapePermute(NVCVTensorLayout srcLayout, const int64_t *srcShape, NVCVTensorLayout dstLayout,
                                  int64_t *dstShape)
{
    return Protect([&] { PermuteShape(srcLayout, srcShape, dstLayout, dstShape); });
}
}
