/* Bit layout of the 64-bit NVCVImageFormat / NVCVDataType words.
 *
 * The numeric values produced here must equal the reference's so that format constants compiled
 * into callers keep their meaning (reference layout: src/nvcv/src/include/nvcv/detail/FormatUtils.h:29-74,
 * 169-175). Field map, LSB first:
 *
 *   [ 0, 6)  swizzle code (NVCVSwizzle)            [ 6, 7)  alpha type
 *   [ 7, 8)  1 = [44,61) are plane packings           [12,15)  memory layout
 *   [16,35)  colour block: bit16==0 -> YCbCr {css [17,20), colour spec [20,35)}
 *                          all ones -> no colour model
 *                          else     -> {model-2 [17,20) (7 = escape), colour spec [20,35)}
 *   [35,44)  plane-0 packing  {sub-code:3, channels-1:2, bpp-code:4}
 *   [44,51)  plane-1 packing  {sub-code:3, channels-1:1, bpp-code:3}
 *   [51,58)  plane-2 packing  (same as plane 1)
 *   [58,61)  plane-3 packing  {bpp-code:3}, an 8-bit plane is stored as all ones
 *            with bit 7 clear, [44,56) is extra-channel info instead: {type:3, count:3, bpp-code:3, data kind:3}
 *   [61,64)  data kind
 *
 * A packing value (NVCVPacking) is {sub-code:4, channels-1:2, bpp-code:4}.
 */
#ifndef NVCV_DETAIL_FORMATBITS_H
#define NVCV_DETAIL_FORMATBITS_H

#include <stdint.h>

#define NVCV_DETAIL_BITS_PUT(v, off, len) ((((uint64_t)(v)) & ((1ULL << (len)) - 1)) << (off))
#define NVCV_DETAIL_BITS_GET(v, off, len) ((((uint64_t)(v)) >> (off)) & ((1ULL << (len)) - 1))

/* bits-per-pixel -> 4-bit size code */
#define NVCV_DETAIL_BPP_CODE(bpp) \
    ((bpp) <= 8 ? 0 : (bpp) <= 32 ? (bpp) / 8 - 1 : (bpp) <= 64 ? (bpp) / 16 + 1 : (bpp) <= 128 ? (bpp) / 32 + 3 : (bpp) / 64 + 5)

/* First packing value of the family with `bpp` bits per pixel and `nch` channels. */
#define NVCV_DETAIL_PACKING_BASE(bpp, nch)                                                    \
    (NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_BPP_CODE(bpp), 6, 4) | NVCV_DETAIL_BITS_PUT((nch)-1, 4, 2) \
     | NVCV_DETAIL_BITS_PUT((bpp) <= 2 ? (bpp) : (bpp) == 4 ? 3 : (bpp) == 8 ? 4 : 0, 0, 4))

/* Narrow a packing value into a plane slot with `nsub`, `nch`, `nbpp` bits per field. */
#define NVCV_DETAIL_PACKING_SLOT(p, nsub, nch, nbpp)                                                   \
    (NVCV_DETAIL_BITS_PUT(((nsub) == 0 && NVCV_DETAIL_BITS_GET(p, 6, 4) == 0                           \
                           && NVCV_DETAIL_BITS_GET(p, 0, 4) == 4)                                      \
                              ? ~0ULL                                                                  \
                              : NVCV_DETAIL_BITS_GET(p, 6, 4),                                         \
                          (nsub) + (nch), nbpp)                                                        \
     | NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_BITS_GET(p, 4, 2), nsub, nch)                                  \
     | NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_BITS_GET(p, 0, 4), 0, nsub))

#define NVCV_DETAIL_COLOR_SPEC_WORD(space, enc, xfer, range, loch, locv)                                      \
    (NVCV_DETAIL_BITS_PUT(space, 0, 3) | NVCV_DETAIL_BITS_PUT(xfer, 3, 4) | NVCV_DETAIL_BITS_PUT(enc, 7, 3)   \
     | NVCV_DETAIL_BITS_PUT(loch, 10, 2) | NVCV_DETAIL_BITS_PUT(locv, 12, 2) | NVCV_DETAIL_BITS_PUT(range, 14, 1))

#define NVCV_DETAIL_MAKE_COLOR_SPEC(CSpace, Encoding, XferFunc, Range, LocHoriz, LocVert) \
    NVCV_DETAIL_COLOR_SPEC_WORD(CSpace, Encoding, XferFunc, Range, LocHoriz, LocVert)

/* Colour block [16,35) for a model / spec (or raw pattern) / chroma-subsampling triple. */
#define NVCV_DETAIL_COLOR_BLOCK(model, spec, css)                                                       \
    ((model) == 1 /* YCbCr */                                                                           \
         ? (NVCV_DETAIL_BITS_PUT(spec, 20, 15) | NVCV_DETAIL_BITS_PUT(css, 17, 3))                      \
     : (model) == 0 /* undefined */                                                                     \
         ? NVCV_DETAIL_BITS_PUT((1U << 19) - 1, 16, 19)                                                 \
     : (NVCV_DETAIL_BITS_PUT(1, 16, 1)                                                                  \
        | ((model)-2 < 7 ? (NVCV_DETAIL_BITS_PUT(spec, 20, 15) | NVCV_DETAIL_BITS_PUT((model)-2, 17, 3)) \
           : (NVCV_DETAIL_BITS_PUT(7, 17, 3)                                                            \
              | ((model) == 9 /* raw */ ? NVCV_DETAIL_BITS_PUT(spec, 21, 6)                             \
                                        : (NVCV_DETAIL_BITS_PUT(1, 20, 1) | NVCV_DETAIL_BITS_PUT((model)-10, 21, 6)))))))

/* Bits [44,61) hold either the packings of planes 1..3 (bit 7 set) or, for a single-plane format with extra
 * channels (bit 7 clear), {channel type:3, count:3, bpp-code:3, data kind:3} from bit 44 up. */
#define NVCV_DETAIL_PLANES_BLOCK(p1, p2, p3)                                                                  \
    (NVCV_DETAIL_BITS_PUT(1, 7, 1) | NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_PACKING_SLOT(p1, 3, 1, 3), 44, 7)        \
     | NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_PACKING_SLOT(p2, 3, 1, 3), 51, 7)                                      \
     | NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_PACKING_SLOT(p3, 0, 0, 3), 58, 3))
#define NVCV_DETAIL_EXTRA_BLOCK(count, bpp, kind, type)                                                       \
    (NVCV_DETAIL_BITS_PUT(type, 44, 3) | NVCV_DETAIL_BITS_PUT(count, 47, 3)                                    \
     | NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_BPP_CODE(bpp), 50, 3) | NVCV_DETAIL_BITS_PUT(kind, 53, 3))

/* Whole format word. Extra channels are only representable beside a single plane: with a second plane
 * packing given they are dropped. */
#define NVCV_DETAIL_FORMAT_WORD_EX(model, spec, css, layout, kind, swizzle, alpha, exCount, exBpp, exKind, exType, \
                                   p0, p1, p2, p3)                                                                 \
    (NVCV_DETAIL_BITS_PUT(kind, 61, 3) | NVCV_DETAIL_BITS_PUT(swizzle, 0, 6) | NVCV_DETAIL_BITS_PUT(alpha, 6, 1)    \
     | NVCV_DETAIL_BITS_PUT(layout, 12, 3) | NVCV_DETAIL_COLOR_BLOCK(model, spec, css)                              \
     | NVCV_DETAIL_BITS_PUT(NVCV_DETAIL_PACKING_SLOT(p0, 3, 2, 4), 35, 9)                                           \
     | ((p1) == 0 && (exCount) > 0 ? NVCV_DETAIL_EXTRA_BLOCK(exCount, exBpp, exKind, exType)                        \
                                   : NVCV_DETAIL_PLANES_BLOCK(p1, p2, p3)))

#define NVCV_DETAIL_FORMAT_WORD(model, spec, css, layout, kind, swizzle, alpha, p0, p1, p2, p3) \
    NVCV_DETAIL_FORMAT_WORD_EX(model, spec, css, layout, kind, swizzle, alpha, 0, 0, 0, 0, p0, p1, p2, p3)

/* The public NVCV_MAKE_*_IMAGE_FORMAT macros take `numPlanes` followed by exactly that many packings. The list is
 * padded to four with zeros, and a packing at or beyond `numPlanes` reads as absent. */
#define NVCV_DETAIL_TAKE4(a, b, c, d, ...) a, b, c, d
#define NVCV_DETAIL_PAD4(...) NVCV_DETAIL_TAKE4(__VA_ARGS__, 0, 0, 0, 0)
#define NVCV_DETAIL_CALL(macro, ...) macro(__VA_ARGS__)
#define NVCV_DETAIL_FORMAT_WORD_N(model, spec, css, layout, kind, swizzle, alpha, exCount, exBpp, exKind, exType,   \
                                  numPlanes, p0, p1, p2, p3)                                                        \
    NVCV_DETAIL_FORMAT_WORD_EX(model, spec, css, layout, kind, swizzle, alpha, exCount, exBpp, exKind, exType, p0,   \
                               ((numPlanes) > 1 ? (p1) : 0), ((numPlanes) > 2 ? (p2) : 0),                          \
                               ((numPlanes) > 3 ? (p3) : 0))
#define NVCV_DETAIL_MAKE_FORMAT_N(model, spec, css, layout, kind, swizzle, alpha, exCount, exBpp, exKind, exType,   \
                                  numPlanes, ...)                                                                   \
    NVCV_DETAIL_CALL(NVCV_DETAIL_FORMAT_WORD_N, model, spec, css, layout, kind, swizzle, alpha, exCount, exBpp,     \
                     exKind, exType, numPlanes, NVCV_DETAIL_PAD4(__VA_ARGS__))

#endif /* NVCV_DETAIL_FORMATBITS_H */
