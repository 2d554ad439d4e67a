/* Out-of-image sampling policy. Replaces: src/nvcv/src/include/nvcv/BorderType.h:36-43. */
#ifndef NVCV_BORDER_TYPE_H
#define NVCV_BORDER_TYPE_H

typedef enum
{
    NVCV_BORDER_CONSTANT   = 0, /* fixed colour                */
    NVCV_BORDER_REPLICATE  = 1, /* aaaaaa|abcdefgh|hhhhhhh     */
    NVCV_BORDER_REFLECT    = 2, /* fedcba|abcdefgh|hgfedcb     */
    NVCV_BORDER_WRAP       = 3, /* cdefgh|abcdefgh|abcdefg     */
    NVCV_BORDER_REFLECT101 = 4  /* gfedcb|abcdefgh|gfedcba     */
} NVCVBorderType;

#endif /* NVCV_BORDER_TYPE_H */
