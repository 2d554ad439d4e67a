/* Colour conversion.
 * Replaces: src/cvcuda/include/cvcuda/OpCvtColor.h:52, 70-75 (semantics of
 * src/cvcuda/priv/legacy/cvt_color.cu:181-230, 514-674, 1387-1517, 1768-2006).
 *
 * Codes implemented: channel swizzles BGR<->RGB, BGR(A)<->RGB(A), add/drop alpha (0..5) for
 * u8/u16/s32/f16/f32/f64 [N]HWC tensors; NV12/NV21 -> RGB/BGR/RGBA/BGRA (90..97) for u8, where the
 * input is a 1-channel tensor of height H*3/2 (luma rows followed by interleaved chroma rows) and
 * the arithmetic is BT.601 limited-range in 20-bit fixed point. Any other code -> INVALID_ARGUMENT. */
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
