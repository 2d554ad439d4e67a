/* Element type of a tensor or image plane: a 64-bit word holding {data kind, packing}.
 * Replaces: src/nvcv/src/include/nvcv/DataType.h:40-339. A data type is a format word without
 * colour model whose swizzle field holds the channel count (reference: detail/FormatUtils.h:169-175). */
#ifndef NVCV_DATA_TYPE_H
#define NVCV_DATA_TYPE_H

#include "DataLayout.h"
#include "Export.h"
#include "Status.h"

#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

typedef uint64_t NVCVDataType;

#define NVCV_DETAIL_MAKE_DATA_TYPE(kind, packing)                                                        \
    ((NVCVDataType)NVCV_DETAIL_FORMAT_WORD(0, 0, 0, NVCV_MEM_LAYOUT_PL, kind,                            \
                                           NVCV_DETAIL_BITS_GET(packing, 4, 2) + 1, NVCV_ALPHA_ASSOCIATED, \
                                           packing, 0, 0, 0))
#define NVCV_DETAIL_DATA_TYPE(kind, packing) NVCV_DETAIL_MAKE_DATA_TYPE(NVCV_DATA_KIND_##kind, NVCV_PACKING_##packing)

/* Compile-time construction of a data type without a named constant (reference: DataType.h:172-190). */
#define NVCV_MAKE_DATA_TYPE(dataKind, packing) NVCV_DETAIL_MAKE_DATA_TYPE(dataKind, packing)

#define NVCV_DATA_TYPE_NONE ((NVCVDataType)0)

/* <n><kind><bits>: n interleaved components (omitted when 1) of kind U/S/F/C with that many bits each. */
#define NVCV_DATA_TYPE_U8     NVCV_DETAIL_DATA_TYPE(UNSIGNED, X8)
#define NVCV_DATA_TYPE_2U8    NVCV_DETAIL_DATA_TYPE(UNSIGNED, X8_Y8)
#define NVCV_DATA_TYPE_3U8    NVCV_DETAIL_DATA_TYPE(UNSIGNED, X8_Y8_Z8)
#define NVCV_DATA_TYPE_4U8    NVCV_DETAIL_DATA_TYPE(UNSIGNED, X8_Y8_Z8_W8)
#define NVCV_DATA_TYPE_S8     NVCV_DETAIL_DATA_TYPE(SIGNED, X8)
#define NVCV_DATA_TYPE_2S8    NVCV_DETAIL_DATA_TYPE(SIGNED, X8_Y8)
#define NVCV_DATA_TYPE_3S8    NVCV_DETAIL_DATA_TYPE(SIGNED, X8_Y8_Z8)
#define NVCV_DATA_TYPE_4S8    NVCV_DETAIL_DATA_TYPE(SIGNED, X8_Y8_Z8_W8)
#define NVCV_DATA_TYPE_U16    NVCV_DETAIL_DATA_TYPE(UNSIGNED, X16)
#define NVCV_DATA_TYPE_2U16   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X16_Y16)
#define NVCV_DATA_TYPE_3U16   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X16_Y16_Z16)
#define NVCV_DATA_TYPE_4U16   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X16_Y16_Z16_W16)
#define NVCV_DATA_TYPE_S16    NVCV_DETAIL_DATA_TYPE(SIGNED, X16)
#define NVCV_DATA_TYPE_2S16   NVCV_DETAIL_DATA_TYPE(SIGNED, X16_Y16)
#define NVCV_DATA_TYPE_3S16   NVCV_DETAIL_DATA_TYPE(SIGNED, X16_Y16_Z16)
#define NVCV_DATA_TYPE_4S16   NVCV_DETAIL_DATA_TYPE(SIGNED, X16_Y16_Z16_W16)
#define NVCV_DATA_TYPE_F16    NVCV_DETAIL_DATA_TYPE(FLOAT, X16)
#define NVCV_DATA_TYPE_2F16   NVCV_DETAIL_DATA_TYPE(FLOAT, X16_Y16)
#define NVCV_DATA_TYPE_3F16   NVCV_DETAIL_DATA_TYPE(FLOAT, X16_Y16_Z16)
#define NVCV_DATA_TYPE_4F16   NVCV_DETAIL_DATA_TYPE(FLOAT, X16_Y16_Z16_W16)
#define NVCV_DATA_TYPE_U32    NVCV_DETAIL_DATA_TYPE(UNSIGNED, X32)
#define NVCV_DATA_TYPE_2U32   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X32_Y32)
#define NVCV_DATA_TYPE_3U32   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X32_Y32_Z32)
#define NVCV_DATA_TYPE_4U32   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X32_Y32_Z32_W32)
#define NVCV_DATA_TYPE_S32    NVCV_DETAIL_DATA_TYPE(SIGNED, X32)
#define NVCV_DATA_TYPE_2S32   NVCV_DETAIL_DATA_TYPE(SIGNED, X32_Y32)
#define NVCV_DATA_TYPE_3S32   NVCV_DETAIL_DATA_TYPE(SIGNED, X32_Y32_Z32)
#define NVCV_DATA_TYPE_4S32   NVCV_DETAIL_DATA_TYPE(SIGNED, X32_Y32_Z32_W32)
#define NVCV_DATA_TYPE_F32    NVCV_DETAIL_DATA_TYPE(FLOAT, X32)
#define NVCV_DATA_TYPE_2F32   NVCV_DETAIL_DATA_TYPE(FLOAT, X32_Y32)
#define NVCV_DATA_TYPE_3F32   NVCV_DETAIL_DATA_TYPE(FLOAT, X32_Y32_Z32)
#define NVCV_DATA_TYPE_4F32   NVCV_DETAIL_DATA_TYPE(FLOAT, X32_Y32_Z32_W32)
#define NVCV_DATA_TYPE_U64    NVCV_DETAIL_DATA_TYPE(UNSIGNED, X64)
#define NVCV_DATA_TYPE_2U64   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X64_Y64)
#define NVCV_DATA_TYPE_3U64   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X64_Y64_Z64)
#define NVCV_DATA_TYPE_4U64   NVCV_DETAIL_DATA_TYPE(UNSIGNED, X64_Y64_Z64_W64)
#define NVCV_DATA_TYPE_S64    NVCV_DETAIL_DATA_TYPE(SIGNED, X64)
#define NVCV_DATA_TYPE_2S64   NVCV_DETAIL_DATA_TYPE(SIGNED, X64_Y64)
#define NVCV_DATA_TYPE_3S64   NVCV_DETAIL_DATA_TYPE(SIGNED, X64_Y64_Z64)
#define NVCV_DATA_TYPE_4S64   NVCV_DETAIL_DATA_TYPE(SIGNED, X64_Y64_Z64_W64)
#define NVCV_DATA_TYPE_F64    NVCV_DETAIL_DATA_TYPE(FLOAT, X64)
#define NVCV_DATA_TYPE_2F64   NVCV_DETAIL_DATA_TYPE(FLOAT, X64_Y64)
#define NVCV_DATA_TYPE_3F64   NVCV_DETAIL_DATA_TYPE(FLOAT, X64_Y64_Z64)
#define NVCV_DATA_TYPE_4F64   NVCV_DETAIL_DATA_TYPE(FLOAT, X64_Y64_Z64_W64)
#define NVCV_DATA_TYPE_C64    NVCV_DETAIL_DATA_TYPE(COMPLEX, X64)
#define NVCV_DATA_TYPE_2C64   NVCV_DETAIL_DATA_TYPE(COMPLEX, X64_Y64)
#define NVCV_DATA_TYPE_3C64   NVCV_DETAIL_DATA_TYPE(COMPLEX, X64_Y64_Z64)
#define NVCV_DATA_TYPE_4C64   NVCV_DETAIL_DATA_TYPE(COMPLEX, X64_Y64_Z64_W64)
#define NVCV_DATA_TYPE_C128   NVCV_DETAIL_DATA_TYPE(COMPLEX, X128)
#define NVCV_DATA_TYPE_2C128  NVCV_DETAIL_DATA_TYPE(COMPLEX, X128_Y128)

NVCV_PUBLIC NVCVStatus nvcvMakeDataType(NVCVDataType *outDataType, NVCVDataKind dataKind, NVCVPacking packing);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetPacking(NVCVDataType type, NVCVPacking *outPacking);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetBitsPerPixel(NVCVDataType type, int32_t *outBPP);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetBitsPerChannel(NVCVDataType type, int32_t *outBits /* [4] */);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetAlignment(NVCVDataType type, int32_t *outAlignment);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetDataKind(NVCVDataType type, NVCVDataKind *outDataKind);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetNumChannels(NVCVDataType type, int32_t *outNumChannels);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetChannelType(NVCVDataType type, int32_t channel, NVCVDataType *outChannelType);
NVCV_PUBLIC NVCVStatus nvcvDataTypeGetStrideBytes(NVCVDataType type, int32_t *outStrideBytes);
/* Printable description; the pointer stays valid until the calling thread asks for another name. */
NVCV_PUBLIC const char *nvcvDataTypeGetName(NVCVDataType type);

#ifdef __cplusplus
}
#endif

#endif /* NVCV_DATA_TYPE_H */
