#ifndef NVCV_TENSORSHAPE_H
#define NVCV_TENSORSHAPE_H
#include "TensorLayout.h" /* nvcvTensorShapePermute is declared there */
#endif
