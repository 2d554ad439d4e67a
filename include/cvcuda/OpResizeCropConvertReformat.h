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

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_RESIZE_CROP_CONVERT_REFORMAT_H */
