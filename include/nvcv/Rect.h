#ifndef NVCV_RECT_H
#define NVCV_RECT_H
#include "Size.h" /* NVCVRectI lives beside NVCVSize2D */
#endif
