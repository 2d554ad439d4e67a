/* Perspective warp: dst(x,y) = src(H^-1 (x,y,1)) (homogeneous divide) with NEAREST / LINEAR / CUBIC
 * sampling and a border policy.
 * Replaces: src/cvcuda/include/cvcuda/OpWarpPerspective.h:56, 130-138 (semantics of
 * src/cvcuda/priv/legacy/warp.cu:234-315, warp_var_shape.cu:33-49, 301-430, CvCudaLegacy.h:157-183).
 *
 * transMatrix is the 3x3 row-major forward map unless `flags` carries NVCV_WARP_INVERSE_MAP. The
 * var-shape variant takes an f32 tensor of shape [N,9]. Types, layouts and status codes as for
 * cvcudaWarpAffine*. */
#ifndef CVCUDA_WARP_PERSPECTIVE_H
#define CVCUDA_WARP_PERSPECTIVE_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/BorderType.h>
#include <nvcv/ImageBatch.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

typedef float NVCVPerspectiveTransform[9];

CVCUDA_PUBLIC NVCVStatus cvcudaWarpPerspectiveCreate(NVCVOperatorHandle *handle, const int32_t maxVarShapeBatchSize);
CVCUDA_PUBLIC NVCVStatus cvcudaWarpPerspectiveSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                     NVCVTensorHandle in, NVCVTensorHandle out,
                                                     const NVCVPerspectiveTransform transMatrix, const int32_t flags,
                                                     const NVCVBorderType borderMode, const float4 borderValue);
CVCUDA_PUBLIC NVCVStatus cvcudaWarpPerspectiveVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                             NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                             NVCVTensorHandle transMatrix, const int32_t flags,
                                                             const NVCVBorderType borderMode,
                                                             const float4 borderValue);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_WARP_PERSPECTIVE_H */
