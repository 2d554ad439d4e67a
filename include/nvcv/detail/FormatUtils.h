/* Spellings of the format-building helper macros that code written against the reference may use
 * (reference: src/nvcv/src/include/nvcv/detail/FormatUtils.h:28-560). They are thin names over the bit helpers
 * of FormatBits.h: every value equals what the reference's macro of the same name yields.
 *
 *   NVCV_DETAIL_MAKE_<family>_FORMAT<n>(...)  full enumerators, n = 1..4 plane packings
 *   NVCV_DETAIL_MAKE_<family>_FMT<n>(...)     enumerators without their NVCV_..._ prefixes
 *   ..._EXTRA_CHANNELS_...                    the same with {count, bits, data kind, type} of extra channels
 *   the forms without <n> take the plane count as an argument followed by that many packings
 *
 * family: COLOR (model, spec), NONCOLOR, RAW (pattern), YCbCr (spec, chroma subsampling).
 * Include this header after the enumerations the abbreviated forms paste together (ImageFormat.h does). */
#ifndef NVCV_DETAIL_FORMATUTILS_H
#define NVCV_DETAIL_FORMATUTILS_H

#include "FormatBits.h"

#define NVCV_DETAIL_SET_BITFIELD(value, offset, size) NVCV_DETAIL_BITS_PUT(value, offset, size)
#define NVCV_DETAIL_GET_BITFIELD(value, offset, size) NVCV_DETAIL_BITS_GET(value, offset, size)

#define NVCV_DETAIL_MAKE_CSPC(CSpace, Encoding, XferFunc, Range, LocHoriz, LocVert)                              \
    NVCV_DETAIL_COLOR_SPEC_WORD(NVCV_COLOR_##CSpace, NVCV_YCbCr_##Encoding, NVCV_COLOR_##XferFunc,              \
                                NVCV_COLOR_##Range, NVCV_CHROMA_##LocHoriz, NVCV_CHROMA_##LocVert)

#define NVCV_DETAIL_ENCODE_BPP(bpp) NVCV_DETAIL_BPP_CODE(bpp)
#define NVCV_DETAIL_BPP_NCH(bpp, chcount) NVCV_DETAIL_PACKING_BASE(bpp, chcount)

#define NVCV_DETAIL_MAKE_SWIZZLE(x, y, z, w)                                                               \
    (NVCV_DETAIL_BITS_PUT(x, 0, 3) | NVCV_DETAIL_BITS_PUT(y, 3, 3) | NVCV_DETAIL_BITS_PUT(z, 6, 3)         \
     | NVCV_DETAIL_BITS_PUT(w, 9, 3))
#define NVCV_DETAIL_MAKE_SWZL(x, y, z, w) \
    NVCV_DETAIL_MAKE_SWIZZLE(NVCV_CHANNEL_##x, NVCV_CHANNEL_##y, NVCV_CHANNEL_##z, NVCV_CHANNEL_##w)

/* An 8-bit packing in a slot that has neither sub-code nor channel bits (plane 3) is stored as all ones. */
#define NVCV_DETAIL_ADJUST_BPP_ENCODING(PACK, BPP, PACKLEN) \
    ((PACKLEN) == 0 && (BPP) == 0 && (PACK) == 4 ? (uint64_t)-1 : (BPP))
/* note the argument order: channel bits, sub-code bits, size-code bits */
#define NVCV_DETAIL_ENCODE_PACKING(P, CHLEN, PACKLEN, BPPLEN) NVCV_DETAIL_PACKING_SLOT(P, PACKLEN, CHLEN, BPPLEN)
#define NVCV_DETAIL_EXTRACT_PACKING_CHANNELS(Packing) (NVCV_DETAIL_BITS_GET(Packing, 4, 2) + 1)
#define NVCV_DETAIL_SET_EXTRA_CHANNEL_INFO(nx, xbits, xkind, xtype) \
    NVCV_DETAIL_EXTRA_BLOCK(nx, xbits, xkind, xtype)

#define NVCV_DETAIL_MAKE_FMTTYPE(model, spec, css, layout, kind, swz, alpha, p0, p1, p2, p3, nx, xbits, xkind, xtype) \
    NVCV_DETAIL_FORMAT_WORD_EX(model, spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1, p2, p3)
#define NVCV_DETAIL_MAKE_FORMAT(model, spec, css, layout, kind, swz, alpha, p0, p1, p2, p3, nx, xbits, xkind, xtype) \
    ((NVCVImageFormat)NVCV_DETAIL_MAKE_FMTTYPE(model, spec, css, layout, kind, swz, alpha, p0, p1, p2, p3, nx,     \
                                               xbits, xkind, xtype))
#define NVCV_DETAIL_MAKE_FMT(model, spec, css, layout, kind, swz, alpha, p0, p1, p2, p3, nx, xbits, xkind, xtype)   \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css,                       \
                            NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, \
                            NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2, NVCV_PACKING_##p3, nx, xbits,  \
                            NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype)

#define NVCV_DETAIL_MAKE_PIX_TYPE(kind, packing) NVCV_DETAIL_MAKE_DATA_TYPE(NVCV_DATA_KIND_##kind, NVCV_PACKING_##packing)

/* COLOR */
#define NVCV_DETAIL_MAKE_COLOR_FORMAT1(model, spec, layout, kind, swz, alpha, p0) NVCV_DETAIL_MAKE_FORMAT(model, \
    spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, 0, 0, 0, 0, 0, NVCV_DATA_KIND_UNSPECIFIED, \
    NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_COLOR_FORMAT2(model, spec, layout, kind, swz, alpha, p0, p1) NVCV_DETAIL_MAKE_FORMAT(model, \
    spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, 0, 0, 0, 0, NVCV_DATA_KIND_UNSPECIFIED, \
    NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_COLOR_FORMAT3(model, spec, layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_FORMAT(model, spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, p2, 0, 0, 0, \
    NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_COLOR_FORMAT4(model, spec, layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_FORMAT(model, spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, p2, p3, 0, 0, \
    NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_COLOR_FORMAT(model, spec, layout, kind, swz, alpha, n, ...) \
    NVCV_DETAIL_MAKE_COLOR_FORMAT##n(model, spec, layout, kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_COLOR_FMT1(model, spec, layout, kind, swz, alpha, p0) \
    NVCV_DETAIL_MAKE_COLOR_FORMAT1(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_COLOR_FMT2(model, spec, layout, kind, swz, alpha, p0, p1) \
    NVCV_DETAIL_MAKE_COLOR_FORMAT2(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_COLOR_FMT3(model, spec, layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_COLOR_FORMAT3(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, \
    NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_COLOR_FMT4(model, spec, layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_COLOR_FORMAT4(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, \
    NVCV_PACKING_##p2, NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_COLOR_FMT(model, spec, layout, kind, swz, alpha, n, ...) \
    NVCV_DETAIL_MAKE_COLOR_FMT##n(model, spec, layout, kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT1(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, \
    xtype, p0) NVCV_DETAIL_MAKE_FORMAT(model, spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, 0, 0, 0, nx, xbits, \
    xkind, xtype)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT2(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, \
    xtype, p0, p1) NVCV_DETAIL_MAKE_FORMAT(model, spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, 0, 0, nx, \
    xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT3(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, \
    xtype, p0, p1, p2) NVCV_DETAIL_MAKE_FORMAT(model, spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, p2, 0, \
    nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT4(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, \
    xtype, p0, p1, p2, p3) NVCV_DETAIL_MAKE_FORMAT(model, spec, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, p2, \
    p3, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    n, ...) NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT##n(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, \
    xtype, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FMT1(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0) NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT1(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, \
    NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, \
    NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FMT2(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0, p1) NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT2(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, \
    NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, \
    NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FMT3(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0, p1, p2) NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT3(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, \
    NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, \
    NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FMT4(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0, p1, p2, p3) NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FORMAT4(NVCV_COLOR_MODEL_##model, NVCV_COLOR_SPEC_##spec, \
    NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, \
    NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2, \
    NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FMT(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, xtype, n, \
    ...) NVCV_DETAIL_MAKE_COLOR_EXTRA_CHANNELS_FMT##n(model, spec, layout, kind, swz, alpha, nx, xbits, xkind, \
    xtype, __VA_ARGS__)

/* NONCOLOR */
#define NVCV_DETAIL_MAKE_NONCOLOR_FORMAT1(layout, kind, swz, alpha, p0) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, kind, swz, \
    alpha, p0, 0, 0, 0, 0, 0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_NONCOLOR_FORMAT2(layout, kind, swz, alpha, p0, p1) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, kind, swz, \
    alpha, p0, p1, 0, 0, 0, 0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_NONCOLOR_FORMAT3(layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, kind, swz, \
    alpha, p0, p1, p2, 0, 0, 0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_NONCOLOR_FORMAT4(layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, kind, swz, \
    alpha, p0, p1, p2, p3, 0, 0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_NONCOLOR_FORMAT(layout, kind, swz, alpha, n, ...) \
    NVCV_DETAIL_MAKE_NONCOLOR_FORMAT##n(layout, kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_NONCOLOR_FMT1(layout, kind, swz, alpha, p0) \
    NVCV_DETAIL_MAKE_NONCOLOR_FORMAT1(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, \
    NVCV_ALPHA_##alpha, NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_NONCOLOR_FMT2(layout, kind, swz, alpha, p0, p1) \
    NVCV_DETAIL_MAKE_NONCOLOR_FORMAT2(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, \
    NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_NONCOLOR_FMT3(layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_NONCOLOR_FORMAT3(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, \
    NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_NONCOLOR_FMT4(layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_NONCOLOR_FORMAT4(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, \
    NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2, NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_NONCOLOR_FMT(layout, kind, swz, alpha, n, ...) NVCV_DETAIL_MAKE_NONCOLOR_FMT##n(layout, \
    kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT1(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, kind, swz, \
    alpha, p0, 0, 0, 0, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT2(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, kind, swz, \
    alpha, p0, p1, 0, 0, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT3(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1, \
    p2) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, kind, \
    swz, alpha, p0, p1, p2, 0, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT4(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1, \
    p2, p3) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, layout, \
    kind, swz, alpha, p0, p1, p2, p3, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT(layout, kind, swz, alpha, nx, xbits, xkind, xtype, n, ...) \
    NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT##n(layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    __VA_ARGS__)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FMT1(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0) \
    NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT1(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, \
    NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FMT2(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1) \
    NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT2(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, \
    NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FMT3(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1, p2) \
    NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT3(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, \
    NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FMT4(layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1, p2, \
    p3) NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FORMAT4(NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, \
    NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2, NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FMT(layout, kind, swz, alpha, nx, xbits, xkind, xtype, n, ...) \
    NVCV_DETAIL_MAKE_NONCOLOR_EXTRA_CHANNELS_FMT##n(layout, kind, swz, alpha, nx, xbits, xkind, xtype, __VA_ARGS__)

/* RAW */
#define NVCV_DETAIL_MAKE_RAW_FORMAT1(pattern, layout, kind, swz, alpha, p0) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, 0, 0, 0, 0, \
    0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_RAW_FORMAT2(pattern, layout, kind, swz, alpha, p0, p1) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, 0, 0, 0, \
    0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_RAW_FORMAT3(pattern, layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, p2, 0, \
    0, 0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_RAW_FORMAT4(pattern, layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, p2, p3, \
    0, 0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_RAW_FORMAT(pattern, layout, kind, swz, alpha, n, ...) \
    NVCV_DETAIL_MAKE_RAW_FORMAT##n(pattern, layout, kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_RAW_FMT1(pattern, layout, kind, swz, alpha, p0) \
    NVCV_DETAIL_MAKE_RAW_FORMAT1(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_RAW_FMT2(pattern, layout, kind, swz, alpha, p0, p1) \
    NVCV_DETAIL_MAKE_RAW_FORMAT2(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_RAW_FMT3(pattern, layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_RAW_FORMAT3(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_RAW_FMT4(pattern, layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_RAW_FORMAT4(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2, \
    NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_RAW_FMT(pattern, layout, kind, swz, alpha, n, ...) NVCV_DETAIL_MAKE_RAW_FMT##n(pattern, \
    layout, kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT1(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, 0, 0, 0, nx, \
    xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT2(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, \
    p1) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, 0, \
    0, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT3(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, \
    p1, p2) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, p1, \
    p2, 0, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT4(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, \
    p1, p2, p3) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_RAW, pattern, NVCV_CSS_NONE, layout, kind, swz, alpha, p0, \
    p1, p2, p3, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, n, \
    ...) NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT##n(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    __VA_ARGS__)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FMT1(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0) \
    NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT1(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, \
    NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FMT2(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1) \
    NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT2(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, \
    NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, \
    NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FMT3(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1, \
    p2) NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT3(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, \
    NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FMT4(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, p1, \
    p2, p3) NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FORMAT4(NVCV_RAW_##pattern, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, \
    NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2, NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FMT(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, n, ...) \
    NVCV_DETAIL_MAKE_RAW_EXTRA_CHANNELS_FMT##n(pattern, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    __VA_ARGS__)

/* YCbCr */
#define NVCV_DETAIL_MAKE_YCbCr_FORMAT1(spec, css, layout, kind, swz, alpha, p0) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, 0, 0, 0, 0, 0, \
    NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_YCbCr_FORMAT2(spec, css, layout, kind, swz, alpha, p0, p1) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, p1, 0, 0, 0, 0, \
    NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_YCbCr_FORMAT3(spec, css, layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, p1, p2, 0, 0, 0, \
    NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_YCbCr_FORMAT4(spec, css, layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, p1, p2, p3, 0, 0, \
    NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U)
#define NVCV_DETAIL_MAKE_YCbCr_FORMAT(spec, css, layout, kind, swz, alpha, n, ...) \
    NVCV_DETAIL_MAKE_YCbCr_FORMAT##n(spec, css, layout, kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_YCbCr_FMT1(spec, css, layout, kind, swz, alpha, p0) \
    NVCV_DETAIL_MAKE_YCbCr_FORMAT1(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_YCbCr_FMT2(spec, css, layout, kind, swz, alpha, p0, p1) \
    NVCV_DETAIL_MAKE_YCbCr_FORMAT2(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_YCbCr_FMT3(spec, css, layout, kind, swz, alpha, p0, p1, p2) \
    NVCV_DETAIL_MAKE_YCbCr_FORMAT3(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, \
    NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_YCbCr_FMT4(spec, css, layout, kind, swz, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_MAKE_YCbCr_FORMAT4(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, NVCV_PACKING_##p0, NVCV_PACKING_##p1, \
    NVCV_PACKING_##p2, NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_YCbCr_FMT(spec, css, layout, kind, swz, alpha, n, ...) NVCV_DETAIL_MAKE_YCbCr_FMT##n(spec, \
    css, layout, kind, swz, alpha, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT1(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, 0, 0, 0, nx, xbits, \
    xkind, xtype)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT2(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0, p1) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, p1, 0, 0, nx, \
    xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT3(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0, p1, p2) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, p1, p2, 0, \
    nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT4(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    p0, p1, p2, p3) NVCV_DETAIL_MAKE_FORMAT(NVCV_COLOR_MODEL_YCbCr, spec, css, layout, kind, swz, alpha, p0, p1, p2, \
    p3, nx, xbits, xkind, xtype)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    n, ...) NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT##n(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, \
    xtype, __VA_ARGS__)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FMT1(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0) \
    NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT1(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, NVCV_MEM_LAYOUT_##layout, \
    NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, NVCV_DATA_KIND_##xkind, \
    NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FMT2(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, \
    p1) NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT2(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, \
    NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, \
    NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FMT3(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, \
    p1, p2) NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT3(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, \
    NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, \
    NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FMT4(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, p0, \
    p1, p2, p3) NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FORMAT4(NVCV_COLOR_SPEC_##spec, NVCV_CSS_##css, \
    NVCV_MEM_LAYOUT_##layout, NVCV_DATA_KIND_##kind, NVCV_SWIZZLE_##swz, NVCV_ALPHA_##alpha, nx, xbits, \
    NVCV_DATA_KIND_##xkind, NVCV_EXTRA_CHANNEL_##xtype, NVCV_PACKING_##p0, NVCV_PACKING_##p1, NVCV_PACKING_##p2, \
    NVCV_PACKING_##p3)
#define NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FMT(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, n, \
    ...) NVCV_DETAIL_MAKE_YCbCr_EXTRA_CHANNELS_FMT##n(spec, css, layout, kind, swz, alpha, nx, xbits, xkind, xtype, \
    __VA_ARGS__)

#endif /* NVCV_DETAIL_FORMATUTILS_H */
