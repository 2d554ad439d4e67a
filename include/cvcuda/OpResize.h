/* Resize with NEAREST / LINEAR / CUBIC / AREA sampling (half-pixel-centre mapping).
 * Replaces: src/cvcuda/include/cvcuda/OpResize.h:52, 115-120 (semantics of
 * src/cvcuda/priv/OpResize.cu:68-548 and src/cvcuda/priv/legacy/resize_var_shape.cu:92-548).
 *
 * in/out: [N]HWC tensors (or image batches) of u8 / u16 / s16 / f32 with 1, 3 or 4 channels, same
 * dtype, channel count and batch size. AREA is the box filter over the covered source rectangle
 * (tensors: cuda_tools/InterpolationWrap.hpp:668-760; image batches: the reference's separate kernel,
 * legacy/resize_var_shape.cu:236-428, whose enlargements are a bilinear variant).
 * Status: INVALID_ARGUMENT for any mismatch or unsupported interpolation. */
#ifndef CVCUDA_RESIZE_H
#define CVCUDA_RESIZE_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/ImageBatch.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaResizeCreate(NVCVOperatorHandle *handle);
CVCUDA_PUBLIC NVCVStatus cvcudaResizeSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                            NVCVTensorHandle out, const NVCVInterpolationType interpolation);
CVCUDA_PUBLIC NVCVStatus cvcudaResizeVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                    NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                    const NVCVInterpolationType interpolation);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_RESIZE_H */
