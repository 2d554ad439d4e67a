// Entry of the per-pixel colour conversion families (gray, YUV 4:4:4, HSV, RGB -> YUV 4:2:0,
// YUV 4:2:2 -> RGB / gray, YUV 4:2:0 -> gray), implemented in OpCvtColorPixel.hip and called by
// the CvtColor operator for every code its own two families do not cover.
#ifndef CVCUDA_AMD_CVTCOLORFAMILIES_HPP
#define CVCUDA_AMD_CVTCOLORFAMILIES_HPP

#include "OpCommon.hpp"

#include <cvcuda/Types.h>

namespace cvamd {

struct ColorIO
{
    // tensors: base pointers and strides in bytes; var-shape batches: device descriptor lists and the
    // host mirror of the destination list (dstHost != nullptr selects the var-shape form)
    const uint8_t *src;
    uint8_t       *dst;
    int64_t        srcN, dstN;
    int32_t        srcRow, dstRow;
    int32_t        N, srcW, srcH, srcC, dstW, dstH, dstC;
    ElemType       srcElem, dstElem;
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
    const NVCVImageBufferStrided *srcHost;
    const NVCVImageBufferStrided *dstHost;
};

// Validates and launches; false when `code` belongs to none of these families.
bool RunPixelColorFamily(ColorCode code, const ColorIO &io, hipStream_t stream);

} // namespace cvamd

#endif // CVCUDA_AMD_CVTCOLORFAMILIES_HPP
