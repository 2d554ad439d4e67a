/* Replaces: src/nvcv/src/include/nvcv/Size.h:31-34 and Rect.h:27-33. */
#ifndef NVCV_SIZE_H
#define NVCV_SIZE_H

#include <stdint.h>

typedef struct
{
    int32_t w, h;
} NVCVSize2D;

typedef struct
{
    int32_t x, y, width, height;
} NVCVRectI;

#endif /* NVCV_SIZE_H */
