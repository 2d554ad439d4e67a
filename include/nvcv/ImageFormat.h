/* Image formats: a 64-bit word describing colour model, planes, per-plane packing and swizzle.
 * Replaces: src/nvcv/src/include/nvcv/ImageFormat.h:48-1157. The named constants below are the
 * ones the image pre-processing operators and their callers use; any other format can still be
 * built with nvcvMake*ImageFormat and is decoded by the query functions. */
#ifndef NVCV_IMAGE_FORMAT_H
#define NVCV_IMAGE_FORMAT_H

#include "ColorSpec.h"
#include "DataLayout.h"
#include "DataType.h"
#include "Export.h"
#include "Status.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

typedef uint64_t NVCVImageFormat;

#define NVCV_DETAIL_FMT(model, spec, css, kind, swz, p0, p1, p2, p3)                                              \
    ((NVCVImageFormat)NVCV_DETAIL_FORMAT_WORD(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css,   \
                                              NVCV_MEM_LAYOUT_PL, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz,      \
                                              NVCV_ALPHA_ASSOCIATED, NVCV_PACKING_##p0, NVCV_PACKING_##p1,        \
                                              NVCV_PACKING_##p2, NVCV_PACKING_##p3))
/* no colour model, one plane */
#define NVCV_DETAIL_FMT_PLAIN(kind, swz, p0) NVCV_DETAIL_FMT(UNDEFINED, UNDEFINED, NONE, kind, swz, p0, 0, 0, 0)
/* RGB model */
#define NVCV_DETAIL_FMT_RGB1(kind, swz, p0) NVCV_DETAIL_FMT(RGB, UNDEFINED, NONE, kind, swz, p0, 0, 0, 0)
#define NVCV_DETAIL_FMT_RGB3(kind, swz, p) NVCV_DETAIL_FMT(RGB, UNDEFINED, NONE, kind, swz, p, p, p, 0)
#define NVCV_DETAIL_FMT_RGB4(kind, swz, p) NVCV_DETAIL_FMT(RGB, UNDEFINED, NONE, kind, swz, p, p, p, p)

#define NVCV_IMAGE_FORMAT_NONE ((NVCVImageFormat)0)

/* single channel, no colour meaning */
#define NVCV_IMAGE_FORMAT_U8 NVCV_DETAIL_FMT_PLAIN(UNSIGNED, X000, X8)
#define NVCV_IMAGE_FORMAT_S8 NVCV_DETAIL_FMT_PLAIN(SIGNED, X000, X8)
#define NVCV_IMAGE_FORMAT_U16 NVCV_DETAIL_FMT_PLAIN(UNSIGNED, X000, X16)
#define NVCV_IMAGE_FORMAT_S16 NVCV_DETAIL_FMT_PLAIN(SIGNED, X000, X16)
#define NVCV_IMAGE_FORMAT_U32 NVCV_DETAIL_FMT_PLAIN(UNSIGNED, X000, X32)
#define NVCV_IMAGE_FORMAT_S32 NVCV_DETAIL_FMT_PLAIN(SIGNED, X000, X32)
#define NVCV_IMAGE_FORMAT_F16 NVCV_DETAIL_FMT_PLAIN(FLOAT, X000, X16)
#define NVCV_IMAGE_FORMAT_F32 NVCV_DETAIL_FMT_PLAIN(FLOAT, X000, X32)
#define NVCV_IMAGE_FORMAT_F64 NVCV_DETAIL_FMT_PLAIN(FLOAT, X000, X64)
#define NVCV_IMAGE_FORMAT_2S16 NVCV_DETAIL_FMT_PLAIN(SIGNED, XY00, X16_Y16)
#define NVCV_IMAGE_FORMAT_2F32 NVCV_DETAIL_FMT_PLAIN(FLOAT, XY00, X32_Y32)

/* luma only, BT.601 limited / full range */
#define NVCV_IMAGE_FORMAT_Y8 NVCV_DETAIL_FMT(YCbCr, BT601, NONE, UNSIGNED, X000, X8, 0, 0, 0)
#define NVCV_IMAGE_FORMAT_Y8_ER NVCV_DETAIL_FMT(YCbCr, BT601_ER, NONE, UNSIGNED, X000, X8, 0, 0, 0)

/* 4:2:0 semi-planar: full-size luma plane + half-size interleaved chroma plane */
#define NVCV_IMAGE_FORMAT_NV12 NVCV_DETAIL_FMT(YCbCr, BT601, 420, UNSIGNED, XYZ0, X8, X8_Y8, 0, 0)
#define NVCV_IMAGE_FORMAT_NV12_ER NVCV_DETAIL_FMT(YCbCr, BT601_ER, 420, UNSIGNED, XYZ0, X8, X8_Y8, 0, 0)
#define NVCV_IMAGE_FORMAT_NV21 NVCV_DETAIL_FMT(YCbCr, BT601, 420, UNSIGNED, XYZ0, X8, X8_Y8, 0, 0)
#define NVCV_IMAGE_FORMAT_NV21_ER NVCV_DETAIL_FMT(YCbCr, BT601_ER, 420, UNSIGNED, XYZ0, X8, X8_Y8, 0, 0)
/* 4:2:2 packed */
#define NVCV_IMAGE_FORMAT_UYVY NVCV_DETAIL_FMT(YCbCr, BT601, 422, UNSIGNED, XYZ1, Y8_X8__Z8_X8, 0, 0, 0)
#define NVCV_IMAGE_FORMAT_YUYV NVCV_DETAIL_FMT(YCbCr, BT601, 422, UNSIGNED, XYZ1, X8_Y8__X8_Z8, 0, 0, 0)
/* 4:4:4 */
#define NVCV_IMAGE_FORMAT_YUV8 NVCV_DETAIL_FMT(YCbCr, BT601, NONE, UNSIGNED, XYZ1, X8_Y8_Z8, 0, 0, 0)
#define NVCV_IMAGE_FORMAT_YUV8p NVCV_DETAIL_FMT(YCbCr, BT601, NONE, UNSIGNED, XYZ1, X8, X8, X8, 0)

/* interleaved colour */
#define NVCV_IMAGE_FORMAT_RGB8 NVCV_DETAIL_FMT_RGB1(UNSIGNED, XYZ1, X8_Y8_Z8)
#define NVCV_IMAGE_FORMAT_BGR8 NVCV_DETAIL_FMT_RGB1(UNSIGNED, ZYX1, X8_Y8_Z8)
#define NVCV_IMAGE_FORMAT_RGBA8 NVCV_DETAIL_FMT_RGB1(UNSIGNED, XYZW, X8_Y8_Z8_W8)
#define NVCV_IMAGE_FORMAT_BGRA8 NVCV_DETAIL_FMT_RGB1(UNSIGNED, ZYXW, X8_Y8_Z8_W8)
#define NVCV_IMAGE_FORMAT_RGBf32 NVCV_DETAIL_FMT_RGB1(FLOAT, XYZ1, X32_Y32_Z32)
#define NVCV_IMAGE_FORMAT_BGRf32 NVCV_DETAIL_FMT_RGB1(FLOAT, ZYX1, X32_Y32_Z32)
#define NVCV_IMAGE_FORMAT_RGBAf32 NVCV_DETAIL_FMT_RGB1(FLOAT, XYZW, X32_Y32_Z32_W32)
#define NVCV_IMAGE_FORMAT_BGRAf32 NVCV_DETAIL_FMT_RGB1(FLOAT, ZYXW, X32_Y32_Z32_W32)
#define NVCV_IMAGE_FORMAT_RGBf16 NVCV_DETAIL_FMT_RGB1(FLOAT, XYZ1, X16_Y16_Z16)
#define NVCV_IMAGE_FORMAT_BGRf16 NVCV_DETAIL_FMT_RGB1(FLOAT, ZYX1, X16_Y16_Z16)
#define NVCV_IMAGE_FORMAT_RGBAf16 NVCV_DETAIL_FMT_RGB1(FLOAT, XYZW, X16_Y16_Z16_W16)
#define NVCV_IMAGE_FORMAT_BGRAf16 NVCV_DETAIL_FMT_RGB1(FLOAT, ZYXW, X16_Y16_Z16_W16)
#define NVCV_IMAGE_FORMAT_HSV8 NVCV_DETAIL_FMT(HSV, UNDEFINED, NONE, UNSIGNED, XYZ0, X8_Y8_Z8, 0, 0, 0)

/* planar colour */
#define NVCV_IMAGE_FORMAT_RGB8p NVCV_DETAIL_FMT_RGB3(UNSIGNED, XYZ0, X8)
#define NVCV_IMAGE_FORMAT_BGR8p NVCV_DETAIL_FMT_RGB3(UNSIGNED, ZYX1, X8)
#define NVCV_IMAGE_FORMAT_RGBA8p NVCV_DETAIL_FMT_RGB4(UNSIGNED, XYZW, X8)
#define NVCV_IMAGE_FORMAT_BGRA8p NVCV_DETAIL_FMT_RGB4(UNSIGNED, ZYXW, X8)
#define NVCV_IMAGE_FORMAT_RGBf32p NVCV_DETAIL_FMT_RGB3(FLOAT, XYZ0, X32)
#define NVCV_IMAGE_FORMAT_BGRf32p NVCV_DETAIL_FMT_RGB3(FLOAT, ZYX1, X32)
#define NVCV_IMAGE_FORMAT_RGBAf32p NVCV_DETAIL_FMT_RGB4(FLOAT, XYZW, X32)
#define NVCV_IMAGE_FORMAT_BGRAf32p NVCV_DETAIL_FMT_RGB4(FLOAT, ZYXW, X32)
#define NVCV_IMAGE_FORMAT_RGBf16p NVCV_DETAIL_FMT_RGB3(FLOAT, XYZ0, X16)
#define NVCV_IMAGE_FORMAT_BGRf16p NVCV_DETAIL_FMT_RGB3(FLOAT, ZYX1, X16)

/* Constructors. exChannelInfo may be NULL; extra channels are not supported (-> NOT_IMPLEMENTED). */
NVCV_PUBLIC NVCVStatus nvcvMakeYCbCrImageFormat(NVCVImageFormat *outFormat, NVCVColorSpec colorSpec,
                                                NVCVChromaSubsampling chromaSub, NVCVMemLayout memLayout,
                                                NVCVDataKind dataKind, NVCVSwizzle swizzle, NVCVPacking packing0,
                                                NVCVPacking packing1, NVCVPacking packing2, NVCVPacking packing3,
                                                NVCVAlphaType alphaType, const NVCVExtraChannelInfo *exChannelInfo);
NVCV_PUBLIC NVCVStatus nvcvMakeColorImageFormat(NVCVImageFormat *outFormat, NVCVColorModel colorModel,
                                                NVCVColorSpec colorSpec, NVCVMemLayout memLayout,
                                                NVCVDataKind dataKind, NVCVSwizzle swizzle, NVCVPacking packing0,
                                                NVCVPacking packing1, NVCVPacking packing2, NVCVPacking packing3,
                                                NVCVAlphaType alphaType, const NVCVExtraChannelInfo *exChannelInfo);
NVCV_PUBLIC NVCVStatus nvcvMakeNonColorImageFormat(NVCVImageFormat *outFormat, NVCVMemLayout memLayout,
                                                   NVCVDataKind dataKind, NVCVSwizzle swizzle, NVCVPacking packing0,
                                                   NVCVPacking packing1, NVCVPacking packing2, NVCVPacking packing3,
                                                   NVCVAlphaType alphaType, const NVCVExtraChannelInfo *exChannelInfo);

/* Queries. `plane` must be in [0, 4); a plane the format does not have reports packing 0 / 0 channels. */
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetNumPlanes(NVCVImageFormat fmt, int32_t *outNumPlanes);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetNumChannels(NVCVImageFormat fmt, int32_t *outNumChannels);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetBitsPerChannel(NVCVImageFormat fmt, int32_t *bits /* [4] */);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlanePacking(NVCVImageFormat fmt, int32_t plane, NVCVPacking *outPacking);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlaneNumChannels(NVCVImageFormat fmt, int32_t plane,
                                                          int32_t *outPlaneNumChannels);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlaneBitsPerPixel(NVCVImageFormat fmt, int32_t plane, int32_t *outBPP);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlanePixelStrideBytes(NVCVImageFormat fmt, int32_t plane,
                                                               int32_t *outStrideBytes);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlaneDataType(NVCVImageFormat fmt, int32_t plane, NVCVDataType *outDataType);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlaneSize(NVCVImageFormat fmt, int32_t plane, int32_t imgWidth,
                                                   int32_t imgHeight, int32_t *outPlaneWidth,
                                                   int32_t *outPlaneHeight);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetDataKind(NVCVImageFormat fmt, NVCVDataKind *outDataKind);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetSwizzle(NVCVImageFormat fmt, NVCVSwizzle *outSwizzle);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetMemLayout(NVCVImageFormat fmt, NVCVMemLayout *outMemLayout);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetColorSpec(NVCVImageFormat fmt, NVCVColorSpec *outColorSpec);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetColorModel(NVCVImageFormat fmt, NVCVColorModel *outColorModel);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetChromaSubsampling(NVCVImageFormat fmt, NVCVChromaSubsampling *outCSS);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetAlphaType(NVCVImageFormat fmt, NVCVAlphaType *outAlphaType);
NVCV_PUBLIC NVCVStatus nvcvImageFormatHasSameDataLayout(NVCVImageFormat a, NVCVImageFormat b, int8_t *outBool);
/* Printable description; the pointer stays valid until the calling thread asks for another name. */
NVCV_PUBLIC const char *nvcvImageFormatGetName(NVCVImageFormat fmt);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_IMAGE_FORMAT_H */
