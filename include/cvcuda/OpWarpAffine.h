/* Affine warp: dst(x,y) = src(M^-1 (x,y,1)) with NEAREST / LINEAR / CUBIC sampling and a border policy.
 * Replaces: src/cvcuda/include/cvcuda/OpWarpAffine.h:39, 57, 130-138 (semantics of
 * src/cvcuda/priv/legacy/warp.cu:28-232, warp_var_shape.cu:51-299, CvCudaLegacy.h:143-155).
 *
 * xform is the 2x3 row-major forward map src->dst unless `flags` carries NVCV_WARP_INVERSE_MAP, in
 * which case it is used as the dst->src map directly; the low bits of `flags` hold the interpolation.
 * in/out: [N]HWC tensors (or image batches) of u8/u16/s16/f32 with 1, 3 or 4 channels.
 * The var-shape variant takes one matrix per image from an f32 tensor of shape [N,6] and needs
 * N <= maxVarShapeBatchSize given at creation (else INVALID_ARGUMENT). The kernel reads each matrix from
 * that tensor and inverts it itself: the operator owns no device buffer, so var-shape submissions of one
 * handle may be in flight on several streams at once (the reference serialises them on an operator-owned
 * matrix buffer); the matrix tensor must stay unchanged until the submitted work has run. */
#ifndef CVCUDA_WARP_AFFINE_H
#define CVCUDA_WARP_AFFINE_H

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

typedef float NVCVAffineTransform[6];

CVCUDA_PUBLIC NVCVStatus cvcudaWarpAffineCreate(NVCVOperatorHandle *handle, const int32_t maxVarShapeBatchSize);
CVCUDA_PUBLIC NVCVStatus cvcudaWarpAffineSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                                NVCVTensorHandle out, const NVCVAffineTransform xform,
                                                const int32_t flags, const NVCVBorderType borderMode,
                                                const float4 borderValue);
CVCUDA_PUBLIC NVCVStatus cvcudaWarpAffineVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                        NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                        NVCVTensorHandle transMatrix, const int32_t flags,
                                                        const NVCVBorderType borderMode, const float4 borderValue);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_WARP_AFFINE_H */
