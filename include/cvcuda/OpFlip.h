/* Mirror images about their axes.
 * Replaces: src/cvcuda/include/cvcuda/OpFlip.h:54, 115-116, 177-179 (semantics of
 * src/cvcuda/priv/legacy/flip.cu:30-196 and flip_or_copy_var_shape.cu:31-160).
 *
 * Tensor form: in/out [N]HWC of equal shape, u8 / u16 / s32 / f32, 1, 3 or 4 channels;
 * flipCode > 0 mirrors the columns (left-right), == 0 the rows (top-bottom), < 0 both.
 * Var-shape form: batches of single-plane images of one format (u8 / u16 / s16 / s32 / f32; 1, 3, 4
 * channels), output image i the size of input image i; flipCode is an int32 tensor with one value per
 * image: 1 columns, 0 rows, -1 both, any other value a plain copy.
 * maxVarShapeBatchSize is accepted for compatibility; the operator owns no buffers. Bit-exact.
 * Status: INVALID_ARGUMENT for any type / layout / shape / batch problem. */
#ifndef CVCUDA_FLIP_H
#define CVCUDA_FLIP_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/ImageBatch.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaFlipCreate(NVCVOperatorHandle *handle, int32_t maxVarShapeBatchSize);
CVCUDA_PUBLIC NVCVStatus cvcudaFlipSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                          NVCVTensorHandle out, int32_t flipCode);
CVCUDA_PUBLIC NVCVStatus cvcudaFlipVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                  NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                  NVCVTensorHandle flipCode);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_FLIP_H */
