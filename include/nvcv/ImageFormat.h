/* Image formats: a 64-bit word describing colour model, planes, per-plane packing and swizzle.
 * Replaces: src/nvcv/src/include/nvcv/ImageFormat.h:48-1157. Every named constant has the reference's value. */
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

/* one to four planes of the same layout; L = PL or BL memory layout */
#define NVCV_DETAIL_FMT_L(model, spec, css, L, kind, swz, alpha, p0, p1, p2, p3)                                   \
    ((NVCVImageFormat)NVCV_DETAIL_FORMAT_WORD(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css,    \
                                              NVCV_MEM_LAYOUT_##L, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz,      \
                                              NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1,            \
                                              NVCV_PACKING_##p2, NVCV_PACKING_##p3))
#define NVCV_DETAIL_FMT(model, spec, css, kind, swz, p0, p1, p2, p3) \
    NVCV_DETAIL_FMT_L(model, spec, css, PL, kind, swz, ASSOCIATED, p0, p1, p2, p3)
/* no colour model, one plane */
#define NVCV_DETAIL_FMT_PLAIN(kind, swz, p0) NVCV_DETAIL_FMT(UNDEFINED, UNDEFINED, NONE, kind, swz, p0, 0, 0, 0)
#define NVCV_DETAIL_FMT_PLAIN_BL(kind, swz, p0) \
    NVCV_DETAIL_FMT_L(UNDEFINED, UNDEFINED, NONE, BL, kind, swz, ASSOCIATED, p0, 0, 0, 0)
/* YCbCr model, BT.601 limited (spec BT601) or full (spec BT601_ER) range */
#define NVCV_DETAIL_FMT_YUV(spec, css, L, swz, p0, p1, p2) \
    NVCV_DETAIL_FMT_L(YCbCr, spec, css, L, UNSIGNED, swz, ASSOCIATED, p0, p1, p2, 0)
/* RGB model */
#define NVCV_DETAIL_FMT_RGB1(kind, swz, p0) NVCV_DETAIL_FMT(RGB, UNDEFINED, NONE, kind, swz, p0, 0, 0, 0)
#define NVCV_DETAIL_FMT_RGB3(kind, swz, p) NVCV_DETAIL_FMT(RGB, UNDEFINED, NONE, kind, swz, p, p, p, 0)
#define NVCV_DETAIL_FMT_RGB4(kind, swz, p) NVCV_DETAIL_FMT(RGB, UNDEFINED, NONE, kind, swz, p, p, p, p)
/* interleaved u8 RGB followed by `count` extra channels of `bpp` bits */
#define NVCV_DETAIL_FMT_RGB_EXTRA(swz, p0, count, bpp, exkind, extype)                                            \
    ((NVCVImageFormat)NVCV_DETAIL_FORMAT_WORD_EX(NVCV_COLOR_MODEL_RGB, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE,  \
                                                 NVCV_MEM_LAYOUT_PL, NVCV_DATA_KIND_UNSIGNED, NVCV_SWIZZLE_##swz, \
                                                 NVCV_ALPHA_ASSOCIATED, count, bpp, NVCV_DATA_KIND_##exkind,      \
                                                 NVCV_EXTRA_CHANNEL_##extype, NVCV_PACKING_##p0, 0, 0, 0))

#define NVCV_IMAGE_FORMAT_NONE ((NVCVImageFormat)0)

/* one or two channels, no colour meaning; _BL = block-linear memory layout */
#define NVCV_IMAGE_FORMAT_U8 NVCV_DETAIL_FMT_PLAIN(UNSIGNED, X000, X8)
#define NVCV_IMAGE_FORMAT_U8_BL NVCV_DETAIL_FMT_PLAIN_BL(UNSIGNED, X000, X8)
#define NVCV_IMAGE_FORMAT_S8 NVCV_DETAIL_FMT_PLAIN(SIGNED, X000, X8)
#define NVCV_IMAGE_FORMAT_U16 NVCV_DETAIL_FMT_PLAIN(UNSIGNED, X000, X16)
#define NVCV_IMAGE_FORMAT_S16 NVCV_DETAIL_FMT_PLAIN(SIGNED, X000, X16)
#define NVCV_IMAGE_FORMAT_S16_BL NVCV_DETAIL_FMT_PLAIN_BL(SIGNED, X000, X16)
#define NVCV_IMAGE_FORMAT_U32 NVCV_DETAIL_FMT_PLAIN(UNSIGNED, X000, X32)
#define NVCV_IMAGE_FORMAT_S32 NVCV_DETAIL_FMT_PLAIN(SIGNED, X000, X32)
#define NVCV_IMAGE_FORMAT_F16 NVCV_DETAIL_FMT_PLAIN(FLOAT, X000, X16)
#define NVCV_IMAGE_FORMAT_F32 NVCV_DETAIL_FMT_PLAIN(FLOAT, X000, X32)
#define NVCV_IMAGE_FORMAT_F64 NVCV_DETAIL_FMT_PLAIN(FLOAT, X000, X64)
#define NVCV_IMAGE_FORMAT_2S16 NVCV_DETAIL_FMT_PLAIN(SIGNED, XY00, X16_Y16)
#define NVCV_IMAGE_FORMAT_2S16_BL NVCV_DETAIL_FMT_PLAIN_BL(SIGNED, XY00, X16_Y16)
#define NVCV_IMAGE_FORMAT_2F16 NVCV_DETAIL_FMT_PLAIN(FLOAT, XY00, X16_Y16)
#define NVCV_IMAGE_FORMAT_2F32 NVCV_DETAIL_FMT_PLAIN(FLOAT, XY00, X32_Y32)
#define NVCV_IMAGE_FORMAT_C64 NVCV_DETAIL_FMT_PLAIN(COMPLEX, X000, X64)
#define NVCV_IMAGE_FORMAT_2C64 NVCV_DETAIL_FMT_PLAIN(COMPLEX, XY00, X64_Y64)
#define NVCV_IMAGE_FORMAT_C128 NVCV_DETAIL_FMT_PLAIN(COMPLEX, X000, X128)
#define NVCV_IMAGE_FORMAT_2C128 NVCV_DETAIL_FMT_PLAIN(COMPLEX, XY00, X128_Y128)

/* luma only, BT.601 limited / full (_ER) range */
#define NVCV_IMAGE_FORMAT_Y8 NVCV_DETAIL_FMT_YUV(BT601, NONE, PL, X000, X8, 0, 0)
#define NVCV_IMAGE_FORMAT_Y8_BL NVCV_DETAIL_FMT_YUV(BT601, NONE, BL, X000, X8, 0, 0)
#define NVCV_IMAGE_FORMAT_Y8_ER NVCV_DETAIL_FMT_YUV(BT601_ER, NONE, PL, X000, X8, 0, 0)
#define NVCV_IMAGE_FORMAT_Y8_ER_BL NVCV_DETAIL_FMT_YUV(BT601_ER, NONE, BL, X000, X8, 0, 0)
#define NVCV_IMAGE_FORMAT_Y16 NVCV_DETAIL_FMT_YUV(BT601, NONE, PL, X000, X16, 0, 0)
#define NVCV_IMAGE_FORMAT_Y16_BL NVCV_DETAIL_FMT_YUV(BT601, NONE, BL, X000, X16, 0, 0)
#define NVCV_IMAGE_FORMAT_Y16_ER NVCV_DETAIL_FMT_YUV(BT601_ER, NONE, PL, X000, X16, 0, 0)
#define NVCV_IMAGE_FORMAT_Y16_ER_BL NVCV_DETAIL_FMT_YUV(BT601_ER, NONE, BL, X000, X16, 0, 0)

/* semi-planar: full-size luma plane + interleaved chroma plane, 4:2:0 (NV12, NV21) or 4:4:4 (NV24) */
#define NVCV_IMAGE_FORMAT_NV12 NVCV_DETAIL_FMT_YUV(BT601, 420, PL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV12_BL NVCV_DETAIL_FMT_YUV(BT601, 420, BL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV12_ER NVCV_DETAIL_FMT_YUV(BT601_ER, 420, PL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV12_ER_BL NVCV_DETAIL_FMT_YUV(BT601_ER, 420, BL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV21 NVCV_DETAIL_FMT_YUV(BT601, 420, PL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV21_ER NVCV_DETAIL_FMT_YUV(BT601_ER, 420, PL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV24 NVCV_DETAIL_FMT_YUV(BT601, 444, PL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV24_BL NVCV_DETAIL_FMT_YUV(BT601, 444, BL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV24_ER NVCV_DETAIL_FMT_YUV(BT601_ER, 444, PL, XYZ0, X8, X8_Y8, 0)
#define NVCV_IMAGE_FORMAT_NV24_ER_BL NVCV_DETAIL_FMT_YUV(BT601_ER, 444, BL, XYZ0, X8, X8_Y8, 0)
/* 4:2:2 packed, two pixels per 32-bit group */
#define NVCV_IMAGE_FORMAT_UYVY NVCV_DETAIL_FMT_YUV(BT601, 422, PL, XYZ1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_UYVY_BL NVCV_DETAIL_FMT_YUV(BT601, 422, BL, XYZ1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_UYVY_ER NVCV_DETAIL_FMT_YUV(BT601_ER, 422, PL, XYZ1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_UYVY_ER_BL NVCV_DETAIL_FMT_YUV(BT601_ER, 422, BL, XYZ1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_VYUY NVCV_DETAIL_FMT_YUV(BT601, 422, PL, XZY1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_VYUY_BL NVCV_DETAIL_FMT_YUV(BT601, 422, BL, XZY1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_VYUY_ER NVCV_DETAIL_FMT_YUV(BT601_ER, 422, PL, XZY1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_VYUY_ER_BL NVCV_DETAIL_FMT_YUV(BT601_ER, 422, BL, XZY1, Y8_X8__Z8_X8, 0, 0)
#define NVCV_IMAGE_FORMAT_YUYV NVCV_DETAIL_FMT_YUV(BT601, 422, PL, XYZ1, X8_Y8__X8_Z8, 0, 0)
#define NVCV_IMAGE_FORMAT_YUYV_BL NVCV_DETAIL_FMT_YUV(BT601, 422, BL, XYZ1, X8_Y8__X8_Z8, 0, 0)
#define NVCV_IMAGE_FORMAT_YUYV_ER NVCV_DETAIL_FMT_YUV(BT601_ER, 422, PL, XYZ1, X8_Y8__X8_Z8, 0, 0)
#define NVCV_IMAGE_FORMAT_YUYV_ER_BL NVCV_DETAIL_FMT_YUV(BT601_ER, 422, BL, XYZ1, X8_Y8__X8_Z8, 0, 0)
/* 4:4:4, interleaved and planar */
#define NVCV_IMAGE_FORMAT_YUV8 NVCV_DETAIL_FMT_YUV(BT601, NONE, PL, XYZ1, X8_Y8_Z8, 0, 0)
#define NVCV_IMAGE_FORMAT_YUV8p NVCV_DETAIL_FMT_YUV(BT601, NONE, PL, XYZ1, X8, X8, X8)
#define NVCV_IMAGE_FORMAT_YUV8p_ER NVCV_DETAIL_FMT_YUV(BT601_ER, NONE, PL, XYZ1, X8, X8, X8)

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
#define NVCV_IMAGE_FORMAT_CMYK8 NVCV_DETAIL_FMT(CMYK, UNDEFINED, NONE, UNSIGNED, XYZW, X8_Y8_Z8_W8, 0, 0, 0)
#define NVCV_IMAGE_FORMAT_YCCK8 NVCV_DETAIL_FMT(YCCK, UNDEFINED, NONE, UNSIGNED, XYZW, X8_Y8_Z8_W8, 0, 0, 0)
#define NVCV_IMAGE_FORMAT_RGBA8_UNASSOCIATED_ALPHA \
    NVCV_DETAIL_FMT_L(RGB, UNDEFINED, NONE, PL, UNSIGNED, XYZW, UNASSOCIATED, X8_Y8_Z8_W8, 0, 0, 0)

/* interleaved u8 colour followed by extra channels: <count><type>_<kind><bits> */
#define NVCV_IMAGE_FORMAT_RGB8_1U_U8 NVCV_DETAIL_FMT_RGB_EXTRA(XYZ1, X8_Y8_Z8, 1, 8, UNSIGNED, U)
#define NVCV_IMAGE_FORMAT_RGB8_7U_U8 NVCV_DETAIL_FMT_RGB_EXTRA(XYZ1, X8_Y8_Z8, 7, 8, UNSIGNED, U)
#define NVCV_IMAGE_FORMAT_RGBA8_3U_U16 NVCV_DETAIL_FMT_RGB_EXTRA(XYZW, X8_Y8_Z8_W8, 3, 16, UNSIGNED, U)
#define NVCV_IMAGE_FORMAT_RGBA8_3POS3D_U32 NVCV_DETAIL_FMT_RGB_EXTRA(XYZW, X8_Y8_Z8, 3, 32, UNSIGNED, POS3D)
#define NVCV_IMAGE_FORMAT_RGB8_3D_F32 NVCV_DETAIL_FMT_RGB_EXTRA(XYZ1, X8_Y8_Z8, 3, 32, FLOAT, D)

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
#define NVCV_IMAGE_FORMAT_RGBAf16p NVCV_DETAIL_FMT_RGB4(FLOAT, XYZW, X16)
#define NVCV_IMAGE_FORMAT_BGRAf16p NVCV_DETAIL_FMT_RGB4(FLOAT, ZYXW, X16)

/* Compile-time construction of a format that has no named constant (reference: ImageFormat.h:414-590).
 * `numPlanes` is followed by exactly that many NVCVPacking values; the fourth plane may have at most 64 bits per
 * pixel. The _EXTRA_CHANNELS forms add up to 7 channels of extraChannelsBPP bits after the pixel of a single-plane
 * format. No argument is validated: use the nvcvMake*ImageFormat functions for that.
 *   NVCV_MAKE_YCbCr_IMAGE_FORMAT(colorSpec, chromaSub, memLayout, dataKind, swizzle, alphaType, numPlanes, packings...)
 *   NVCV_MAKE_COLOR_IMAGE_FORMAT(colorModel, colorSpec, memLayout, dataKind, swizzle, alphaType, numPlanes, packings...)
 *   NVCV_MAKE_NONCOLOR_IMAGE_FORMAT(memLayout, dataKind, swizzle, alphaType, numPlanes, packings...)
 *   NVCV_MAKE_RAW_IMAGE_FORMAT(rawPattern, memLayout, dataKind, swizzle, alphaType, numPlanes, packings...)
 * and in the _EXTRA_CHANNELS forms `numExtraChannels, extraChannelsBPP, extraChannelDataKind, extraChannelType`
 * between alphaType and numPlanes. */
#define NVCV_MAKE_YCbCr_IMAGE_FORMAT(colorSpec, chromaSub, memLayout, dataKind, swizzle, alphaType, ...)           \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(NVCV_COLOR_MODEL_YCbCr, colorSpec, chromaSub, memLayout, dataKind, \
                                                swizzle, alphaType, 0, 0, 0, 0, __VA_ARGS__))
#define NVCV_MAKE_YCbCr_IMAGE_EXTRA_CHANNELS_FORMAT(colorSpec, chromaSub, memLayout, dataKind, swizzle, alphaType, \
                                                    numExtraChannels, extraChannelsBPP, extraChannelDataKind,      \
                                                    extraChannelType, ...)                                         \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(NVCV_COLOR_MODEL_YCbCr, colorSpec, chromaSub, memLayout, dataKind, \
                                                swizzle, alphaType, numExtraChannels, extraChannelsBPP,            \
                                                extraChannelDataKind, extraChannelType, __VA_ARGS__))
#define NVCV_MAKE_COLOR_IMAGE_FORMAT(colorModel, colorSpec, memLayout, dataKind, swizzle, alphaType, ...)        \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(colorModel, colorSpec, NVCV_CSS_NONE, memLayout, dataKind,       \
                                                swizzle, alphaType, 0, 0, 0, 0, __VA_ARGS__))
#define NVCV_MAKE_COLOR_IMAGE_EXTRA_CHANNELS_FORMAT(colorModel, colorSpec, memLayout, dataKind, swizzle, alphaType, \
                                                    numExtraChannels, extraChannelsBPP, extraChannelDataKind,       \
                                                    extraChannelType, ...)                                          \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(colorModel, colorSpec, NVCV_CSS_NONE, memLayout, dataKind,          \
                                                swizzle, alphaType, numExtraChannels, extraChannelsBPP,             \
                                                extraChannelDataKind, extraChannelType, __VA_ARGS__))
#define NVCV_MAKE_NONCOLOR_IMAGE_FORMAT(memLayout, dataKind, swizzle, alphaType, ...)                              \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED,             \
                                                NVCV_CSS_NONE, memLayout, dataKind, swizzle, alphaType, 0, 0, 0, 0, \
                                                __VA_ARGS__))
#define NVCV_MAKE_NONCOLOR_IMAGE_EXTRA_CHANNELS_FORMAT(memLayout, dataKind, swizzle, alphaType, numExtraChannels,  \
                                                       extraChannelsBPP, extraChannelDataKind, extraChannelType,   \
                                                       ...)                                                        \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED,             \
                                                NVCV_CSS_NONE, memLayout, dataKind, swizzle, alphaType,            \
                                                numExtraChannels, extraChannelsBPP, extraChannelDataKind,          \
                                                extraChannelType, __VA_ARGS__))
#define NVCV_MAKE_RAW_IMAGE_FORMAT(rawPattern, memLayout, dataKind, swizzle, alphaType, ...)                     \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(NVCV_COLOR_MODEL_RAW, rawPattern, NVCV_CSS_NONE, memLayout,      \
                                                dataKind, swizzle, alphaType, 0, 0, 0, 0, __VA_ARGS__))
#define NVCV_MAKE_RAW_IMAGE_EXTRA_CHANNELS_FORMAT(rawPattern, memLayout, dataKind, swizzle, alphaType,           \
                                                  numExtraChannels, extraChannelsBPP, extraChannelDataKind,      \
                                                  extraChannelType, ...)                                         \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FORMAT_N(NVCV_COLOR_MODEL_RAW, rawPattern, NVCV_CSS_NONE, memLayout,      \
                                                dataKind, swizzle, alphaType, numExtraChannels,                  \
                                                extraChannelsBPP, extraChannelDataKind, extraChannelType,        \
                                                __VA_ARGS__))

/* Run-time constructors (reference: ImageFormat.h:592-730). They validate: the swizzle's channel count equals the
 * packings' channel total, plane 0 is present, planes 1/2 have at most 128 and plane 3 at most 64 bits per pixel,
 * plane 1 at most 2 channels, a colour spec only with the RGB, YCbCr, CMYK or YCCK models, chroma subsampling
 * only with YCbCr. exChannelInfo may be NULL; extra channels need a single-plane format, at most 7 channels and at
 * most 128 bits each. */
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
NVCV_PUBLIC NVCVStatus nvcvMakeRawImageFormat(NVCVImageFormat *outFormat, NVCVRawPattern rawPattern,
                                              NVCVMemLayout memLayout, NVCVDataKind dataKind, NVCVSwizzle swizzle,
                                              NVCVPacking packing0, NVCVPacking packing1, NVCVPacking packing2,
                                              NVCVPacking packing3, NVCVAlphaType alphaType,
                                              const NVCVExtraChannelInfo *exChannelInfo);
/* FourCC codes (V4L2 spelling, case-insensitive) to formats and back. The conversion to a format applies
 * `colorSpec` (when the model has one) and `memLayout`; the conversion back ignores both. */
NVCV_PUBLIC NVCVStatus nvcvMakeImageFormatFromFourCC(NVCVImageFormat *outFormat, uint32_t fourcc,
                                                     NVCVColorSpec colorSpec, NVCVMemLayout memLayout);
NVCV_PUBLIC NVCVStatus nvcvImageFormatToFourCC(NVCVImageFormat fmt, uint32_t *outFourCC);
/* One format out of up to four single-plane formats that agree in colour, layout, data kind and alpha type
 * (unused ones NVCV_IMAGE_FORMAT_NONE), and the way back: the single-plane format of one plane. */
NVCV_PUBLIC NVCVStatus nvcvMakeImageFormatFromPlanes(NVCVImageFormat *outFormat, NVCVImageFormat plane0,
                                                     NVCVImageFormat plane1, NVCVImageFormat plane2,
                                                     NVCVImageFormat plane3);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlaneFormat(NVCVImageFormat fmt, int32_t plane, NVCVImageFormat *outFormat);

/* Replace one property of *fmt (reference: ImageFormat.h:761-1157). None accepts NVCV_IMAGE_FORMAT_NONE. */
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetSwizzleAndPacking(NVCVImageFormat *fmt, NVCVSwizzle swizzle,
                                                           NVCVPacking packing0, NVCVPacking packing1,
                                                           NVCVPacking packing2, NVCVPacking packing3);
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetDataKind(NVCVImageFormat *fmt, NVCVDataKind dataKind);
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetMemLayout(NVCVImageFormat *fmt, NVCVMemLayout memLayout);
/* RGB formats drop the spec's YCbCr encoding; models without a colour spec keep theirs (undefined). */
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetColorSpec(NVCVImageFormat *fmt, NVCVColorSpec colorSpec);
/* Only YCbCr formats take a subsampling other than NVCV_CSS_NONE. */
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetChromaSubsampling(NVCVImageFormat *fmt, NVCVChromaSubsampling css);
/* Only formats of the RAW colour model have a pattern. */
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetRawPattern(NVCVImageFormat *fmt, NVCVRawPattern rawPattern);
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetRawPattern(NVCVImageFormat fmt, NVCVRawPattern *outRawPattern);
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetAlphaType(NVCVImageFormat *fmt, NVCVAlphaType alphaType);
/* Extra channels of a single-plane format; multi-planar formats and NVCV_IMAGE_FORMAT_NONE report none. */
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetExtraChannelInfo(NVCVImageFormat fmt, NVCVExtraChannelInfo *outExChannelInfo);
NVCV_PUBLIC NVCVStatus nvcvImageFormatSetExtraChannelInfo(NVCVImageFormat *fmt, const NVCVExtraChannelInfo *exChannelInfo);
/* The swizzle of one plane's own components, e.g. NV12: X000 and 0XY0. */
NVCV_PUBLIC NVCVStatus nvcvImageFormatGetPlaneSwizzle(NVCVImageFormat fmt, int32_t plane, NVCVSwizzle *outPlaneSwizzle);

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
