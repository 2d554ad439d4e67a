/* Per-element normalisation: out = sat((in - base) * scale * global_scale + shift), or with
 * CVCUDA_NORMALIZE_SCALE_IS_STDDEV: out = sat((in - base) / sqrt(scale^2 + epsilon) * global_scale + shift).
 * Replaces: src/cvcuda/include/cvcuda/OpNormalize.h:43, 54, 159-166 (semantics of
 * src/cvcuda/priv/legacy/normalize.cu:35-93, 309-421 and normalize_var_shape.cu:36-308).
 *
 * in/out: [N]HWC tensors, same dtype (u8/s8/u16/s16/s32/f32), 1, 3 or 4 channels. base and scale are
 * f32 [N]HWC tensors whose N/H/W/C extents are each either 1 (broadcast) or equal to the input's. */
#ifndef CVCUDA_NORMALIZE_H
#define CVCUDA_NORMALIZE_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/ImageBatch.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

#define CVCUDA_NORMALIZE_SCALE_IS_STDDEV 1

CVCUDA_PUBLIC NVCVStatus cvcudaNormalizeCreate(NVCVOperatorHandle *handle);
CVCUDA_PUBLIC NVCVStatus cvcudaNormalizeSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                               NVCVTensorHandle base, NVCVTensorHandle scale, NVCVTensorHandle out,
                                               float global_scale, float shift, float epsilon, uint32_t flags);
CVCUDA_PUBLIC NVCVStatus cvcudaNormalizeVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                       NVCVImageBatchHandle in, NVCVTensorHandle base,
                                                       NVCVTensorHandle scale, NVCVImageBatchHandle out,
                                                       float global_scale, float shift, float epsilon,
                                                       uint32_t flags);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_NORMALIZE_H */
