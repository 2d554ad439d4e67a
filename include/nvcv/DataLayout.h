/* How pixel components are laid out in memory: packing, component kind, memory layout, swizzle.
 * Replaces: src/nvcv/src/include/nvcv/DataLayout.h:36-640 (enumerator values are ABI and kept;
 * of the query functions only the ones the image pre-processing operators need are provided). */
#ifndef NVCV_FORMAT_DATALAYOUT_H
#define NVCV_FORMAT_DATALAYOUT_H

#include "Export.h"
#include "Status.h"
#include "detail/FormatUtils.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

#define NVCV_MAX_CHANNEL_COUNT (4)
#define NVCV_MAX_EXTRA_CHANNEL_COUNT (7)
#define NVCV_MAX_SWIZZLE_COUNT (57)

/* Names read LSB to MSB; "_" separates machine words, "b<N>" is N bits of padding. Within a
 * {bits-per-pixel, channel-count} family the enumerators count up from NVCV_DETAIL_PACKING_BASE. */
typedef enum
{
    NVCV_PACKING_0 = 0,

    NVCV_PACKING_X1 = NVCV_DETAIL_PACKING_BASE(1, 1),
    NVCV_PACKING_X2 = NVCV_DETAIL_PACKING_BASE(2, 1),
    NVCV_PACKING_X4 = NVCV_DETAIL_PACKING_BASE(4, 1),

    NVCV_PACKING_X8 = NVCV_DETAIL_PACKING_BASE(8, 1),
    NVCV_PACKING_b4X4,
    NVCV_PACKING_X4b4,
    NVCV_PACKING_X4Y4   = NVCV_DETAIL_PACKING_BASE(8, 2),
    NVCV_PACKING_X3Y3Z2 = NVCV_DETAIL_PACKING_BASE(8, 3),

    NVCV_PACKING_X16 = NVCV_DETAIL_PACKING_BASE(16, 1),
    NVCV_PACKING_b6X10,
    NVCV_PACKING_X10b6,
    NVCV_PACKING_b4X12,
    NVCV_PACKING_X12b4,
    NVCV_PACKING_b2X14,
    NVCV_PACKING_X14b2,
    NVCV_PACKING_X8_Y8  = NVCV_DETAIL_PACKING_BASE(16, 2),
    NVCV_PACKING_X5Y5Z6 = NVCV_DETAIL_PACKING_BASE(16, 3),
    NVCV_PACKING_X5Y6Z5,
    NVCV_PACKING_X6Y5Z5,
    NVCV_PACKING_b4X4Y4Z4,
    NVCV_PACKING_b1X5Y5Z5,
    NVCV_PACKING_X5Y5b1Z5,
    NVCV_PACKING_X1Y5Z5W5 = NVCV_DETAIL_PACKING_BASE(16, 4),
    NVCV_PACKING_X4Y4Z4W4,
    NVCV_PACKING_X5Y1Z5W5,
    NVCV_PACKING_X5Y5Z1W5,
    NVCV_PACKING_X5Y5Z5W1,
    NVCV_PACKING_X8_Y8__X8_Z8,
    NVCV_PACKING_Y8_X8__Z8_X8,

    NVCV_PACKING_X24      = NVCV_DETAIL_PACKING_BASE(24, 1),
    NVCV_PACKING_X8_Y8_Z8 = NVCV_DETAIL_PACKING_BASE(24, 3),

    NVCV_PACKING_X32 = NVCV_DETAIL_PACKING_BASE(32, 1),
    NVCV_PACKING_b12X20,
    NVCV_PACKING_X20b12,
    NVCV_PACKING_X24b8,
    NVCV_PACKING_b8X24,
    NVCV_PACKING_X16_Y16 = NVCV_DETAIL_PACKING_BASE(32, 2),
    NVCV_PACKING_X10b6_Y10b6,
    NVCV_PACKING_X12b4_Y12b4,
    NVCV_PACKING_X10Y11Z11 = NVCV_DETAIL_PACKING_BASE(32, 3),
    NVCV_PACKING_X11Y11Z10,
    NVCV_PACKING_b2X10Y10Z10,
    NVCV_PACKING_X10Y10Z10b2,
    NVCV_PACKING_X8_Y8_Z8_W8 = NVCV_DETAIL_PACKING_BASE(32, 4),
    NVCV_PACKING_X2Y10Z10W10,
    NVCV_PACKING_X10Y10Z10W2,

    NVCV_PACKING_X48         = NVCV_DETAIL_PACKING_BASE(48, 1),
    NVCV_PACKING_X16_Y16_Z16 = NVCV_DETAIL_PACKING_BASE(48, 3),

    NVCV_PACKING_X64     = NVCV_DETAIL_PACKING_BASE(64, 1),
    NVCV_PACKING_X32_Y32 = NVCV_DETAIL_PACKING_BASE(64, 2),
    NVCV_PACKING_X32_Y24b8,
    NVCV_PACKING_X16_Y16_Z16_W16 = NVCV_DETAIL_PACKING_BASE(64, 4),

    NVCV_PACKING_X96         = NVCV_DETAIL_PACKING_BASE(96, 1),
    NVCV_PACKING_X32_Y32_Z32 = NVCV_DETAIL_PACKING_BASE(96, 3),

    NVCV_PACKING_X128            = NVCV_DETAIL_PACKING_BASE(128, 1),
    NVCV_PACKING_X64_Y64         = NVCV_DETAIL_PACKING_BASE(128, 2),
    NVCV_PACKING_X32_Y32_Z32_W32 = NVCV_DETAIL_PACKING_BASE(128, 4),

    NVCV_PACKING_X192        = NVCV_DETAIL_PACKING_BASE(192, 1),
    NVCV_PACKING_X64_Y64_Z64 = NVCV_DETAIL_PACKING_BASE(192, 3),

    NVCV_PACKING_X256            = NVCV_DETAIL_PACKING_BASE(256, 1),
    NVCV_PACKING_X128_Y128       = NVCV_DETAIL_PACKING_BASE(256, 2),
    NVCV_PACKING_X64_Y64_Z64_W64 = NVCV_DETAIL_PACKING_BASE(256, 4),

    NVCV_PACKING_LIMIT32 = INT32_MAX
} NVCVPacking;

typedef enum
{
    NVCV_DATA_KIND_UNSPECIFIED = -1,
    NVCV_DATA_KIND_UNSIGNED    = 0,
    NVCV_DATA_KIND_SIGNED      = 1,
    NVCV_DATA_KIND_FLOAT       = 2,
    NVCV_DATA_KIND_COMPLEX     = 3
} NVCVDataKind;

typedef enum
{
    NVCV_MEM_LAYOUT_PITCH_LINEAR   = 0,
    NVCV_MEM_LAYOUT_BLOCK1_LINEAR  = 1,
    NVCV_MEM_LAYOUT_BLOCK2_LINEAR  = 2,
    NVCV_MEM_LAYOUT_BLOCK4_LINEAR  = 3,
    NVCV_MEM_LAYOUT_BLOCK8_LINEAR  = 4,
    NVCV_MEM_LAYOUT_BLOCK16_LINEAR = 5,
    NVCV_MEM_LAYOUT_BLOCK32_LINEAR = 6,
    NVCV_MEM_LAYOUT_BLOCK_LINEAR   = NVCV_MEM_LAYOUT_BLOCK2_LINEAR,
    NVCV_MEM_LAYOUT_PL             = NVCV_MEM_LAYOUT_PITCH_LINEAR,
    NVCV_MEM_LAYOUT_BL             = NVCV_MEM_LAYOUT_BLOCK_LINEAR
} NVCVMemLayout;

typedef enum
{
    NVCV_CHANNEL_0 = 0, /* constant zero */
    NVCV_CHANNEL_X,
    NVCV_CHANNEL_Y,
    NVCV_CHANNEL_Z,
    NVCV_CHANNEL_W,
    NVCV_CHANNEL_1, /* constant one (max value) */
    NVCV_CHANNEL_FORCE8 = UINT8_MAX
} NVCVChannel;

typedef enum
{
    NVCV_ALPHA_ASSOCIATED   = 0,
    NVCV_ALPHA_UNASSOCIATED = 1
} NVCVAlphaType;

typedef enum
{
    NVCV_EXTRA_CHANNEL_U = 0,
    NVCV_EXTRA_CHANNEL_D,
    NVCV_EXTRA_CHANNEL_POS3D
} NVCVExtraChannel;

typedef struct
{
    int32_t          numChannels;
    int32_t          bitsPerPixel;
    NVCVDataKind     datakind;
    NVCVExtraChannel channelType;
} NVCVExtraChannelInfo;

/* Swizzle codes are indices into a fixed table; the name spells the four output channels. */
typedef enum
{
    NVCV_SWIZZLE_0000, NVCV_SWIZZLE_X000, NVCV_SWIZZLE_XY00, NVCV_SWIZZLE_XYZ0, NVCV_SWIZZLE_XYZW,
    NVCV_SWIZZLE_1000, NVCV_SWIZZLE_0001, NVCV_SWIZZLE_ZYXW, NVCV_SWIZZLE_WXYZ, NVCV_SWIZZLE_WZYX,
    NVCV_SWIZZLE_YZWX, NVCV_SWIZZLE_XYZ1, NVCV_SWIZZLE_YZW1, NVCV_SWIZZLE_XXX1, NVCV_SWIZZLE_XZY1,
    NVCV_SWIZZLE_ZYX1, NVCV_SWIZZLE_ZYX0, NVCV_SWIZZLE_WZY1, NVCV_SWIZZLE_0X00, NVCV_SWIZZLE_00X0,
    NVCV_SWIZZLE_000X, NVCV_SWIZZLE_Y000, NVCV_SWIZZLE_0Y00, NVCV_SWIZZLE_00Y0, NVCV_SWIZZLE_000Y,
    NVCV_SWIZZLE_0XY0, NVCV_SWIZZLE_XXXY, NVCV_SWIZZLE_YYYX, NVCV_SWIZZLE_0YX0, NVCV_SWIZZLE_X00Y,
    NVCV_SWIZZLE_Y00X, NVCV_SWIZZLE_X001, NVCV_SWIZZLE_XY01, NVCV_SWIZZLE_0XZ0, NVCV_SWIZZLE_0ZX0,
    NVCV_SWIZZLE_XZY0, NVCV_SWIZZLE_YZX1, NVCV_SWIZZLE_ZYW1, NVCV_SWIZZLE_0YX1, NVCV_SWIZZLE_XYXZ,
    NVCV_SWIZZLE_YXZX, NVCV_SWIZZLE_XZ00, NVCV_SWIZZLE_WYXZ, NVCV_SWIZZLE_YX00, NVCV_SWIZZLE_YX01,
    NVCV_SWIZZLE_00YX, NVCV_SWIZZLE_00XY, NVCV_SWIZZLE_0XY1, NVCV_SWIZZLE_0X01, NVCV_SWIZZLE_YZXW,
    NVCV_SWIZZLE_YW00, NVCV_SWIZZLE_XYW0, NVCV_SWIZZLE_YZW0, NVCV_SWIZZLE_YZ00, NVCV_SWIZZLE_00X1,
    NVCV_SWIZZLE_0ZXY,
    NVCV_SWIZZLE_UNSUPPORTED = 63
} NVCVSwizzle;

typedef enum
{
    NVCV_ORDER_LSB,
    NVCV_ORDER_MSB
} NVCVByteOrder;

typedef struct
{
    NVCVByteOrder byteOrder;
    int32_t       alignment;
    NVCVSwizzle   swizzle;
    int32_t       bits[NVCV_MAX_CHANNEL_COUNT];
} NVCVPackingParams;

/* channels[4] receives the four NVCVChannel selectors of the swizzle. */
NVCV_PUBLIC NVCVStatus nvcvSwizzleGetChannels(NVCVSwizzle swizzle, NVCVChannel *channels);
/* Number of distinct X/Y/Z/W selectors (constants 0/1 do not count). */
NVCV_PUBLIC NVCVStatus nvcvSwizzleGetNumChannels(NVCVSwizzle swizzle, int32_t *outNumChannels);
NVCV_PUBLIC NVCVStatus nvcvMakeSwizzle(NVCVSwizzle *outSwizzle, NVCVChannel x, NVCVChannel y, NVCVChannel z,
                                       NVCVChannel w);

/* The packing with the given field widths, channel positions and byte order; a word of a single channel matches
 * either byte order, and `alignment` does not take part in the choice. INVALID_ARGUMENT when no packing fits. nvcvPackingGetParams is the way
 * back; its `bits` are the widths of the stored fields in memory order, padding included.
 * (reference: DataLayout.h:498-527) */
NVCV_PUBLIC NVCVStatus nvcvMakePacking(NVCVPacking *outPacking, const NVCVPackingParams *params);
NVCV_PUBLIC NVCVStatus nvcvPackingGetParams(NVCVPacking packing, NVCVPackingParams *outParams);
NVCV_PUBLIC NVCVStatus nvcvPackingGetNumComponents(NVCVPacking packing, int32_t *outNumComponents);
NVCV_PUBLIC NVCVStatus nvcvPackingGetBitsPerComponent(NVCVPacking packing, int32_t *outBits /* [4] */);
NVCV_PUBLIC NVCVStatus nvcvPackingGetBitsPerPixel(NVCVPacking packing, int32_t *outBPP);
NVCV_PUBLIC NVCVStatus nvcvPackingGetAlignment(NVCVPacking packing, int32_t *outAlignment);

NVCV_PUBLIC const char *nvcvDataKindGetName(NVCVDataKind kind);
NVCV_PUBLIC const char *nvcvMemLayoutGetName(NVCVMemLayout memlayout);
NVCV_PUBLIC const char *nvcvSwizzleGetName(NVCVSwizzle swizzle);
NVCV_PUBLIC const char *nvcvPackingGetName(NVCVPacking packing);
NVCV_PUBLIC const char *nvcvChannelGetName(NVCVChannel channel);
NVCV_PUBLIC const char *nvcvByteOrderGetName(NVCVByteOrder byteOrder);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_FORMAT_DATALAYOUT_H */
