/* Colour model, colour spec and chroma-subsampling codes stored inside NVCVImageFormat, and the functions
 * that take a colour spec apart and put it together.
 * Replaces: src/nvcv/src/include/nvcv/ColorSpec.h:41-650. */
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
    NVCV_WHITE_POINT_D65, /* the only white point the colour spaces above use */
    NVCV_WHITE_POINT_FORCE8 = UINT8_MAX
} NVCVWhitePoint;

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

/* A user-defined colour spec as a constant expression:
 * NVCV_MAKE_COLOR_SPEC(cspace, encoding, xferFunc, range, locHoriz, locVert). */
#define NVCV_MAKE_COLOR_SPEC (NVCVColorSpec) NVCV_DETAIL_MAKE_COLOR_SPEC

/* The same at run time. No argument is range-checked: each value is truncated to its bit field. */
NVCV_PUBLIC NVCVStatus nvcvMakeColorSpec(NVCVColorSpec *outColorSpec, NVCVColorSpace cspace, NVCVYCbCrEncoding encoding,
                                         NVCVColorTransferFunction xferFunc, NVCVColorRange range,
                                         NVCVChromaLocation locHoriz, NVCVChromaLocation locVert);

typedef enum
{
    NVCV_RAW_BAYER_RGGB,
    NVCV_RAW_BAYER_BGGR,
    NVCV_RAW_BAYER_GRBG,
    NVCV_RAW_BAYER_GBRG,
    /* clear (panchromatic) filters in place of the greens, or of all but one primary */
    NVCV_RAW_BAYER_RCCB,
    NVCV_RAW_BAYER_BCCR,
    NVCV_RAW_BAYER_CRBC,
    NVCV_RAW_BAYER_CBRC,
    NVCV_RAW_BAYER_RCCC,
    NVCV_RAW_BAYER_CRCC,
    NVCV_RAW_BAYER_CCRC,
    NVCV_RAW_BAYER_CCCR,
    NVCV_RAW_BAYER_CCCC,
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

/* The subsampling with `samplesHoriz` x `samplesVert` chroma samples per 4 x 4 luma samples (each 1, 2 or 4;
 * 1 x 1 also stands for 4:4:4); INVALID_ARGUMENT for other combinations or a NULL output. */
NVCV_PUBLIC NVCVStatus nvcvMakeChromaSubsampling(NVCVChromaSubsampling *outCSS, int32_t samplesHoriz,
                                                 int32_t samplesVert);
/* Chroma samples per 4 luma samples, horizontally and vertically (either output may be NULL, not both). */
NVCV_PUBLIC NVCVStatus nvcvChromaSubsamplingGetNumSamples(NVCVChromaSubsampling css, int32_t *outSamplesHoriz,
                                                          int32_t *outSamplesVert);

/* Components of a colour spec. Getters: INVALID_ARGUMENT for a NULL output (GetChromaLoc: when both are NULL).
 * Setters: INVALID_ARGUMENT for a NULL colour spec; the new value is truncated to its bit field. */
NVCV_PUBLIC NVCVStatus nvcvColorSpecGetChromaLoc(NVCVColorSpec cspec, NVCVChromaLocation *outLocHoriz,
                                                 NVCVChromaLocation *outLocVert);
NVCV_PUBLIC NVCVStatus nvcvColorSpecSetChromaLoc(NVCVColorSpec *cspec, NVCVChromaLocation locHoriz,
                                                 NVCVChromaLocation locVert);
NVCV_PUBLIC NVCVStatus nvcvColorSpecGetColorSpace(NVCVColorSpec cspec, NVCVColorSpace *outColorSpace);
NVCV_PUBLIC NVCVStatus nvcvColorSpecSetColorSpace(NVCVColorSpec *cspec, NVCVColorSpace cspace);
NVCV_PUBLIC NVCVStatus nvcvColorSpecGetYCbCrEncoding(NVCVColorSpec cspec, NVCVYCbCrEncoding *outEncoding);
NVCV_PUBLIC NVCVStatus nvcvColorSpecSetYCbCrEncoding(NVCVColorSpec *cspec, NVCVYCbCrEncoding encoding);
NVCV_PUBLIC NVCVStatus nvcvColorSpecGetColorTransferFunction(NVCVColorSpec              cspec,
                                                             NVCVColorTransferFunction *outXferFunc);
NVCV_PUBLIC NVCVStatus nvcvColorSpecSetColorTransferFunction(NVCVColorSpec *cspec, NVCVColorTransferFunction xferFunc);
NVCV_PUBLIC NVCVStatus nvcvColorSpecGetRange(NVCVColorSpec cspec, NVCVColorRange *outColorRange);
NVCV_PUBLIC NVCVStatus nvcvColorSpecSetRange(NVCVColorSpec *cspec, NVCVColorRange range);

/* Whether formats of this colour model carry a colour spec (YCbCr and RGB do). */
NVCV_PUBLIC NVCVStatus nvcvColorModelNeedsColorspec(NVCVColorModel cmodel, int8_t *outBool);

/* Names. A predefined value gives its enumerator's name, anything else "<Type>(<number>)"; a colour spec that is
 * not predefined is spelled by its components. Pointers refer to per-thread storage that later calls reuse. */
NVCV_PUBLIC const char *nvcvColorSpecGetName(NVCVColorSpec cspec);
NVCV_PUBLIC const char *nvcvColorModelGetName(NVCVColorModel cmodel);
NVCV_PUBLIC const char *nvcvColorSpaceGetName(NVCVColorSpace cspace);
NVCV_PUBLIC const char *nvcvWhitePointGetName(NVCVWhitePoint wpoint);
NVCV_PUBLIC const char *nvcvYCbCrEncodingGetName(NVCVYCbCrEncoding enc);
NVCV_PUBLIC const char *nvcvColorTransferFunctionGetName(NVCVColorTransferFunction xfer);
NVCV_PUBLIC const char *nvcvColorRangeGetName(NVCVColorRange range);
NVCV_PUBLIC const char *nvcvChromaLocationGetName(NVCVChromaLocation loc);
NVCV_PUBLIC const char *nvcvRawPatternGetName(NVCVRawPattern raw);
/* J:a:b notation, e.g. "4:2:0", "4:2:2R" */
NVCV_PUBLIC const char *nvcvChromaSubsamplingGetName(NVCVChromaSubsampling css);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_FORMAT_COLORSPEC_H */
