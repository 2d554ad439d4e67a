/* Width and height of an image in pixels. Replaces: src/nvcv/src/include/nvcv/Size.h:31-34. */
#ifndef NVCV_SIZE_H
#define NVCV_SIZE_H

#include <stdint.h>

typedef struct
{
    int32_t w, h;
} NVCVSize2D;

#endif /* NVCV_SIZE_H */
