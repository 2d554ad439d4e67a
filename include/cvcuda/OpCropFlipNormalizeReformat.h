/* Fused pad/crop -> flip -> normalise -> convert -> layout change, from a batch of differently
 * sized images into one tensor.
 * Replaces: src/cvcuda/include/cvcuda/OpCropFlipNormalizeReformat.h:52, 171-174 (semantics of
 * src/cvcuda/priv/OpCropFlipNormalizeReformat.cu:38-470).
 *
 * in      : batch of images of one format, interleaved (one plane) or planar (one plane per channel),
 *           1, 3 or 4 channels of u8 / s8 / u16 / s16 / s32 / f32.
 * out     : rank-4 tensor, NHWC or NCHW, N = number of images, C = the images' channel count, any of the
 *           element types above; each output image is the tensor's H x W.
 * cropRect: int32 tensor [N,1,1,4] = (x, y, width, height) per image, in input pixels; x / y may be
 *           negative and the rectangle may leave the image: pixels outside come from the border mode
 *           (CONSTANT: borderValue converted to the input type).
 * flipCode: int32 tensor [N]: 1 mirrors the columns of the cropped window, 0 its rows, -1 both,
 *           anything else leaves it as is.
 * base / scale: float32 tensors [1,1,1,1] or [1,1,1,>=C].
 *
 * out(n, y, x, c) = 0 where x >= width or y >= height of the rectangle, else
 *     saturate_cast((in(n, ys, xs, c) - base[c]) * m[c] * global_scale + shift),
 *     m[c] = scale[c], or 1 / sqrt(scale[c]^2 + epsilon) when flags is non-zero
 *     (CVCUDA_NORMALIZE_SCALE_IS_STDDEV), in float32, evaluated in this order.
 * Status: INVALID_ARGUMENT for any type / layout / shape problem, OVERFLOW when the output exceeds
 * 2 GiB - 1 bytes. */
#ifndef CVCUDA_CROP_FLIP_NORMALIZE_REFORMAT_H
#define CVCUDA_CROP_FLIP_NORMALIZE_REFORMAT_H

#include "OpNormalize.h"
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

CVCUDA_PUBLIC NVCVStatus cvcudaCropFlipNormalizeReformatCreate(NVCVOperatorHandle *handle);

CVCUDA_PUBLIC NVCVStatus cvcudaCropFlipNormalizeReformatSubmit(
    NVCVOperatorHandle handle, hipStream_t stream, NVCVImageBatchHandle in, NVCVTensorHandle out,
    NVCVTensorHandle cropRect, NVCVBorderType borderMode, float borderValue, NVCVTensorHandle flipCode,
    NVCVTensorHandle base, NVCVTensorHandle scale, float global_scale, float shift, float epsilon, uint32_t flags);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_CROP_FLIP_NORMALIZE_REFORMAT_H */
