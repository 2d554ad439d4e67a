/* Layout change between [N]HWC and [N]CHW (or a pitched copy when the layouts agree).
 * Replaces: src/cvcuda/include/cvcuda/OpReformat.h:52, 112-113 (semantics of
 * src/cvcuda/priv/legacy/reformat.cu:35-197). Padding bytes of the output are never written. */
#ifndef CVCUDA_REFORMAT_H
#define CVCUDA_REFORMAT_H

#include "Operator.h"
#include "Types.h"

#include <nvcv/Status.h>
#include <nvcv/Tensor.h>

#ifdef __cplusplus
extern "C"
{
#endif

CVCUDA_PUBLIC NVCVStatus cvcudaReformatCreate(NVCVOperatorHandle *handle);
CVCUDA_PUBLIC NVCVStatus cvcudaReformatSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                              NVCVTensorHandle out);

#ifdef __cplusplus
}
#endif

#endif /* CVCUDA_REFORMAT_H */
