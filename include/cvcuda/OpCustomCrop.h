/* Copy of a rectangle of every image of a tensor into the top-left corner of the output.
 * Replaces: src/cvcuda/include/cvcuda/OpCustomCrop.h:51, 115-116 (semantics of
 * src/cvcuda/priv/legacy/custom_crop.cu:35-156).
 *
 * in/out: [N]HWC tensors of the same data type (element size 1, 2, 4 or 8 bytes), 1-4 channels, the
 * same N. out(n, y, x) = in(n, cropRect.y + y, cropRect.x + x) for 0 <= x < cropRect.width,
 * 0 <= y < cropRect.height; the rest of the output is left untouched. Bit-exact.
 * Status: INVALID_ARGUMENT when the rectangle leaves the input or exceeds the output, or for a
 * layout / data type / channel-count problem. */
#ifndef CVCUDA_CUSTOM_CROP_H
#define CVCUDA_CUSTOM_CROP_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/Rect.h>
#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaCustomCropCreate(NVCVOperatorHandle *handle);
CVCUDA_PUBLIC NVCVStatus cvcudaCustomCropSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                                NVCVTensorHandle out, const NVCVRectI cropRect);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_CUSTOM_CROP_H */
