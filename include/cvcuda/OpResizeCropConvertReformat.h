/* Fused resize -> crop -> (scale*v+offset, dtype convert) -> channel reorder -> layout change.
 * Replaces: src/cvcuda/include/cvcuda/OpResizeCropConvertReformat.h:54, 220-228
 * (semantics of src/cvcuda/priv/OpResizeCropConvertReformat.cu:137-278, 418-683).
 *
 * in : u8, 3 interleaved channels, [N]HWC tensor or a batch of single-plane 3-channel u8 images.
 * out: u8 or f32 tensor in NHWC / HWC / NCHW / CHW, N equal to the input's; its HxW is the crop size.
 * Each source image is (virtually) resized to resizeDim with NEAREST or LINEAR sampling, the window
 * [cropPos, cropPos + out size) of the resized image is produced; v -> scale*v + offset; with
 * srcCast the interpolated value is first rounded/saturated to u8; manip REVERSE swaps channels 0/2.
 *
 * Status: INVALID_ARGUMENT for a NULL/batch-size/resizeDim<=1/crop-outside/interpolation problem,
 * NOT_COMPATIBLE for channel count != 3, dtype or layout problems, OVERFLOW when the input exceeds
 * 2 GiB - 1 bytes. */
#ifndef CVCUDA_RESIZE_CROP_CONVERT_REFORMAT_H
#define CVCUDA_RESIZE_CROP_CONVERT_REFORMAT_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/ImageBatch.h>
#include <nvcv/Size.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaResizeCropConvertReformatCreate(NVCVOperatorHandle *handle);

CVCUDA_PUBLIC NVCVStatus cvcudaResizeCropConvertReformatSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in, NVCVTensorHandle out,
    const NVCVSize2D resizeDim, const NVCVInterpolationType interpolation, const int2 cropPos,
    const NVCVChannelManip manip, const float scale, const float offset, const bool srcCast);

CVCUDA_PUBLIC NVCVStatus cvcudaResizeCropConvertReformatVarShapeSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVImageBatchHandle in, NVCVTensorHandle out,
    const NVCVSize2D resizeDim, const NVCVInterpolationType interpolation, const int2 cropPos,
    const NVCVChannelManip manip, const float scale, const float offset, const bool srcCast);

/* ---- Extension (no counterpart in the reference) -------------------------------------------------
 * The fused operator followed, in the same kernel, by a per-channel normalisation: the result is
 * what cvcudaNormalizeSubmit(base[1,1,1,3], scale[1,1,1,3], globalScale, shift, epsilon, flags)
 * gives when applied to the f32 output of the fused operator with the same scale/offset, i.e.
 *     x = scale*v + offset;  out = ((x - base[c]) * m[c]) * globalScale + shift,
 *     m[c] = scale[c], or 1/sqrt(scale[c]^2 + epsilon) with CVCUDA_NORMALIZE_SCALE_IS_STDDEV,
 * evaluated in float32 in this order, c being the OUTPUT channel (after manip). It serves the
 * "resize, crop, /255, subtract mean, divide by std, to planar f32" pre-processing in one pass over
 * the data; the reference needs three operators (fused, Normalize, Reformat) for it.
 * Status codes as for the plain entry points; INVALID_ARGUMENT for a NULL `normalize` or unknown flags. */
typedef struct CVCUDAXChannelNormalizeRec
{
    float    base[3];
    float    scale[3];
    float    globalScale;
    float    shift;
    float    epsilon;
    uint32_t flags; /* 0 or CVCUDA_NORMALIZE_SCALE_IS_STDDEV (cvcuda/OpNormalize.h) */
} CVCUDAXChannelNormalize;

CVCUDA_PUBLIC NVCVStatus cvcudaxResizeCropConvertReformatNormalizeSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in, NVCVTensorHandle out,
    const NVCVSize2D resizeDim, const NVCVInterpolationType interpolation, const int2 cropPos,
    const NVCVChannelManip manip, const float scale, const float offset, const bool srcCast,
    const CVCUDAXChannelNormalize *normalize);

CVCUDA_PUBLIC NVCVStatus cvcudaxResizeCropConvertReformatNormalizeVarShapeSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVImageBatchHandle in, NVCVTensorHandle out,
    const NVCVSize2D resizeDim, const NVCVInterpolationType interpolation, const int2 cropPos,
    const NVCVChannelManip manip, const float scale, const float offset, const bool srcCast,
    const CVCUDAXChannelNormalize *normalize);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_RESIZE_CROP_CONVERT_REFORMAT_H */
