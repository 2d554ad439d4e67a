/* An axis-aligned rectangle of whole pixels, the crop argument of CustomCrop and the rows of
 * CropFlipNormalizeReformat's crop tensor. Replaces: src/nvcv/src/include/nvcv/Rect.h:27-33. */
#ifndef NVCV_RECT_H
#define NVCV_RECT_H

#include <stdint.h>

typedef struct
{
    int32_t x, y;          /* top-left corner */
    int32_t width, height; /* extent */
} NVCVRectI;

#endif /* NVCV_RECT_H */
