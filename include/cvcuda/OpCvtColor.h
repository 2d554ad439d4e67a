/* Colour conversion.
 * Replaces: src/cvcuda/include/cvcuda/OpCvtColor.h:52, 70-75 (semantics of
 * src/cvcuda/priv/legacy/cvt_color.cu:181-230, 514-674, 1387-1517, 1768-2006).
 *
 * Codes implemented (the set the reference implements, cvt_color.cu:1791-1995); tensors are [N]HWC:
 *   0..5     channel swizzles BGR<->RGB, BGR(A)<->RGB(A), add/drop alpha: u8/s8/u16/s16/s32/f16/f32/f64
 *   6, 7     BGR/RGB -> gray (u8, u16: 15-bit fixed point; f32), 8 gray -> BGR (any element size)
 *   40, 41, 66, 67 BGR/RGB -> HSV and 54, 55, 70, 71 HSV -> BGR/RGB(A), half (180) or full (256) hue
 *            range for u8, degrees for f32
 *   82..85   BGR/RGB <-> YUV 4:4:4 (u8, u16: 14-bit fixed point; f32)
 *   90..105  NV12 / NV21 / YV12 / I420 -> RGB/BGR(A), 106 -> gray: u8, the input is a 1-channel tensor
 *            of height H*3/2 (luma rows, then chroma rows); BT.601 limited range, 20-bit fixed point
 *   107, 108, 111, 112, 115..124 UYVY / YUY2 / YVYU -> RGB/BGR(A) or gray: u8, input 1-channel of width 2*W
 *   127..134, 140..147 RGB/BGR(A) -> I420 / YV12 / NV12 / NV21: u8, chroma from the top-left pixel of
 *            each 2x2 block
 * Image batches (VarShapeSubmit) take the same codes (src/cvcuda/priv/legacy/cvt_color_var_shape.cu:
 * 1324-1640); the 4:2:0 and 4:2:2 sides are single-plane u8 images of H*3/2 rows or 2*W columns, and
 * every image pair is checked against the shape rules above. Any other code or combination ->
 * INVALID_ARGUMENT. */
#ifndef CVCUDA_CVTCOLOR_H
#define CVCUDA_CVTCOLOR_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/ImageBatch.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaCvtColorCreate(NVCVOperatorHandle *handle);
CVCUDA_PUBLIC NVCVStatus cvcudaCvtColorSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                              NVCVTensorHandle out, NVCVColorConversionCode code);
CVCUDA_PUBLIC NVCVStatus cvcudaCvtColorVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                      NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                      NVCVColorConversionCode code);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_CVTCOLOR_H */
