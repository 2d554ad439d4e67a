/* Element-wise data type conversion with scaling: out = saturate_cast<out type>(alpha * in + beta).
 * Replaces: src/cvcuda/include/cvcuda/OpConvertTo.h:50, 116-117 (semantics of
 * src/cvcuda/priv/legacy/convert_to.cu:36-209).
 *
 * in/out: [N]HWC tensors of equal shape, up to 4 channels; element types u8, s8, u16, s16, s32, f32,
 * f64 on either side. The arithmetic runs in float32, or in float64 when either side is f64; alpha
 * and beta are converted to that type first. Conversion to an integer type rounds to nearest even
 * and saturates.
 * Status: INVALID_ARGUMENT for any type / layout / shape problem. */
#ifndef CVCUDA_CONVERT_TO_H
#define CVCUDA_CONVERT_TO_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaConvertToCreate(NVCVOperatorHandle *handle);
CVCUDA_PUBLIC NVCVStatus cvcudaConvertToSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                               NVCVTensorHandle out, const double alpha, const double beta);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_CONVERT_TO_H */
