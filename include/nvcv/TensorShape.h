/* Shapes re-ordered from one layout to another. Replaces: src/nvcv/src/include/nvcv/TensorShape.h:45-46. */
#ifndef NVCV_TENSORSHAPE_H
#define NVCV_TENSORSHAPE_H

#include "Export.h"
#include "Status.h"
#include "TensorLayout.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

/* dstShape[j] = srcShape[i] where srcLayout[i] == dstLayout[j]; a dimension of dstLayout that srcLayout does not
 * have becomes 1, one that only srcLayout has is dropped. srcShape holds srcLayout.rank extents, dstShape room for
 * dstLayout.rank. INVALID_ARGUMENT for a NULL shape. */
NVCV_PUBLIC NVCVStatus nvcvTensorShapePermute(NVCVTensorLayout srcLayout, const int64_t *srcShape,
                                              NVCVTensorLayout dstLayout, int64_t *dstShape);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_TENSORSHAPE_H */
