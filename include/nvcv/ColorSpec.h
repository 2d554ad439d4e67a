/* Colour model, colour spec and chroma-subsampling codes stored inside NVCVImageFormat.
 * Replaces: src/nvcv/src/include/nvcv/ColorSpec.h:41-420 (enumerator values only; the colour-spec
 * algebra is not needed by the image pre-processing operators). */
#ifndef NVCV_FORMAT_COLORSPEC_H
#define NVCV_FORMAT_COLORSPEC_H

#include "Export.h"
#include "Status.h"
#include "detail/FormatBits.h"

#ifdef __cplusplus
extern "C"
{
#endif

typedef enum
{
    NVCV_COLOR_MODEL_UNDEFINED = 0,
    NVCV_COLOR_MODEL_YCbCr     = 1,
    NVCV_COLOR_MODEL_RGB       = 2,
    NVCV_COLOR_MODEL_RAW       = 9,
    NVCV_COLOR_MODEL_XYZ       = 10,
    NVCV_COLOR_MODEL_HSV       = 11,
    NVCV_COLOR_MODEL_CMYK      = 12,
    NVCV_COLOR_MODEL_YCCK      = 13
} NVCVColorModel;

typedef enum
{
    NVCV_COLOR_SPACE_BT601,
    NVCV_COLOR_SPACE_BT709,
    NVCV_COLOR_SPACE_BT2020,
    NVCV_COLOR_SPACE_DCIP3
} NVCVColorSpace;

typedef enum
{
    NVCV_YCbCr_ENC_UNDEFINED = 0,
    NVCV_YCbCr_ENC_BT601,
    NVCV_YCbCr_ENC_BT709,
    NVCV_YCbCr_ENC_BT2020,
    NVCV_YCbCr_ENC_BT2020c,
    NVCV_YCbCr_ENC_SMPTE240M
} NVCVYCbCrEncoding;

typedef enum
{
    NVCV_COLOR_XFER_LINEAR,
    NVCV_COLOR_XFER_sRGB,
    NVCV_COLOR_XFER_sYCC,
    NVCV_COLOR_XFER_PQ,
    NVCV_COLOR_XFER_BT709,
    NVCV_COLOR_XFER_BT2020,
    NVCV_COLOR_XFER_SMPTE240M
} NVCVColorTransferFunction;

typedef enum
{
    NVCV_COLOR_RANGE_FULL,
    NVCV_COLOR_RANGE_LIMITED
} NVCVColorRange;

typedef enum
{
    NVCV_CHROMA_LOC_BOTH = 0,
    NVCV_CHROMA_LOC_EVEN,
    NVCV_CHROMA_LOC_CENTER,
    NVCV_CHROMA_LOC_ODD
} NVCVChromaLocation;

#define NVCV_DETAIL_CSPEC(space, enc, xfer, range, loch, locv)                                             \
    NVCV_DETAIL_COLOR_SPEC_WORD(NVCV_COLOR_SPACE_##space, NVCV_YCbCr_ENC_##enc, NVCV_COLOR_XFER_##xfer, \
                                NVCV_COLOR_RANGE_##range, NVCV_CHROMA_LOC_##loch, NVCV_CHROMA_LOC_##locv)

typedef enum
{
    NVCV_COLOR_SPEC_UNDEFINED        = NVCV_DETAIL_CSPEC(BT709, UNDEFINED, LINEAR, FULL, BOTH, BOTH),
    NVCV_COLOR_SPEC_BT601            = NVCV_DETAIL_CSPEC(BT709, BT601, BT709, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT601_ER         = NVCV_DETAIL_CSPEC(BT709, BT601, BT709, FULL, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT709            = NVCV_DETAIL_CSPEC(BT709, BT709, BT709, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT709_ER         = NVCV_DETAIL_CSPEC(BT709, BT709, BT709, FULL, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT709_LINEAR     = NVCV_DETAIL_CSPEC(BT709, BT709, LINEAR, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT2020           = NVCV_DETAIL_CSPEC(BT2020, BT2020, BT2020, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT2020_ER        = NVCV_DETAIL_CSPEC(BT2020, BT2020, BT2020, FULL, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT2020_LINEAR    = NVCV_DETAIL_CSPEC(BT2020, BT2020, LINEAR, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT2020_PQ        = NVCV_DETAIL_CSPEC(BT2020, BT2020, PQ, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT2020_PQ_ER     = NVCV_DETAIL_CSPEC(BT2020, BT2020, PQ, FULL, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT2020c          = NVCV_DETAIL_CSPEC(BT2020, BT2020c, BT2020, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_BT2020c_ER       = NVCV_DETAIL_CSPEC(BT2020, BT2020c, BT2020, FULL, EVEN, EVEN),
    NVCV_COLOR_SPEC_MPEG2_BT601      = NVCV_DETAIL_CSPEC(BT709, BT601, BT709, FULL, EVEN, CENTER),
    NVCV_COLOR_SPEC_MPEG2_BT709      = NVCV_DETAIL_CSPEC(BT709, BT709, BT709, FULL, EVEN, CENTER),
    NVCV_COLOR_SPEC_MPEG2_SMPTE240M  = NVCV_DETAIL_CSPEC(BT709, SMPTE240M, SMPTE240M, FULL, EVEN, CENTER),
    NVCV_COLOR_SPEC_sRGB             = NVCV_DETAIL_CSPEC(BT709, UNDEFINED, sRGB, FULL, BOTH, BOTH),
    NVCV_COLOR_SPEC_sYCC             = NVCV_DETAIL_CSPEC(BT709, BT601, sYCC, FULL, CENTER, CENTER),
    NVCV_COLOR_SPEC_SMPTE240M        = NVCV_DETAIL_CSPEC(BT709, SMPTE240M, SMPTE240M, LIMITED, EVEN, EVEN),
    NVCV_COLOR_SPEC_DISPLAYP3        = NVCV_DETAIL_CSPEC(DCIP3, UNDEFINED, sRGB, FULL, BOTH, BOTH),
    NVCV_COLOR_SPEC_DISPLAYP3_LINEAR = NVCV_DETAIL_CSPEC(DCIP3, UNDEFINED, LINEAR, FULL, BOTH, BOTH),
    NVCV_COLOR_SPEC_FORCE32          = INT32_MAX
} NVCVColorSpec;

typedef enum
{
    NVCV_RAW_BAYER_RGGB,
    NVCV_RAW_BAYER_BGGR,
    NVCV_RAW_BAYER_GRBG,
    NVCV_RAW_BAYER_GBRG,
    NVCV_RAW_FORCE8 = UINT8_MAX
} NVCVRawPattern;

/* J:a:b notation; the R variants subsample vertically instead of horizontally. */
typedef enum
{
    NVCV_CSS_NONE = 0,
    NVCV_CSS_444  = NVCV_CSS_NONE,
    NVCV_CSS_422  = 1,
    NVCV_CSS_422R = 2,
    NVCV_CSS_411  = 3,
    NVCV_CSS_411R = 4,
    NVCV_CSS_420  = 5,
    NVCV_CSS_410  = 6,
    NVCV_CSS_410R = 7,
    NVCV_CSS_440  = NVCV_CSS_422R
} NVCVChromaSubsampling;

/* Chroma samples per 4 luma samples, horizontally and vertically. */
NVCV_PUBLIC NVCVStatus nvcvChromaSubsamplingGetNumSamples(NVCVChromaSubsampling css, int32_t *outSamplesHoriz,
                                                          int32_t *outSamplesVert);
NVCV_PUBLIC const char *nvcvColorModelGetName(NVCVColorModel cmodel);
NVCV_PUBLIC const char *nvcvChromaSubsamplingGetName(NVCVChromaSubsampling css);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_FORMAT_COLORSPEC_H */
