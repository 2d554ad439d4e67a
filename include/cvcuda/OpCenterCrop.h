/* Copy of the centred cropWidth x cropHeight window of every image into the top-left corner of the
 * output. Replaces: src/cvcuda/include/cvcuda/OpCenterCrop.h:51, 117-118 (semantics of
 * src/cvcuda/priv/legacy/center_crop.cu:35-141).
 *
 * The window starts at ((W - cropWidth) / 2, (H - cropHeight) / 2), integer division. Tensors as for
 * cvcudaCustomCropSubmit. Bit-exact. Status: INVALID_ARGUMENT when the window exceeds the input or
 * the output, or for a layout / data type / channel-count / batch-size problem. */
#ifndef CVCUDA_CENTER_CROP_H
#define CVCUDA_CENTER_CROP_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaCenterCropCreate(NVCVOperatorHandle *handle);
CVCUDA_PUBLIC NVCVStatus cvcudaCenterCropSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                                NVCVTensorHandle out, int32_t cropWidth, int32_t cropHeight);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_CENTER_CROP_H */
