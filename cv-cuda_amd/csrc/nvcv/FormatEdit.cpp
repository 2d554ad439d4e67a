// The part of the format API that builds one format from another: property setters, per-plane formats and their
// merge, raw patterns, extra channels, FourCC codes, and the packing <-> parameters conversion. Behaviour follows
// the reference's src/nvcv/src/priv/ImageFormat.cpp:320-560, 693-1165 and DataLayout.cpp:337-545, 733-825; the
// word layout is described in nvcv/detail/FormatBits.h.
#include "Priv.hpp"

#include <cctype>
#include <cstring>

namespace nvcvamd {
namespace {

uint64_t Replace(uint64_t word, int off, int len, uint64_t value)
{
    const uint64_t mask = ((1ULL << len) - 1) << off;
    return (word & ~mask) | FieldPut(value, off, len);
}

uint64_t *Editable(NVCVImageFormat *fmt, const char *what)
{
    NotNull(fmt, "Pointer to the image format");
    if (*fmt == NVCV_IMAGE_FORMAT_NONE)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "NVCV_IMAGE_FORMAT_NONE has no %s to set", what);
    }
    return fmt;
}

// Colour spec or raw pattern, whichever the format's colour block holds.
uint32_t SpecOrRaw(uint64_t fmt)
{
    const int raw = FormatRawPattern(fmt);
    return raw >= 0 ? (uint32_t)raw : (uint32_t)EnumValue(FormatColorSpec(fmt));
}

uint64_t Rebuild(uint64_t fmt, NVCVChromaSubsampling css, NVCVSwizzle swizzle, NVCVPacking p0, NVCVPacking p1, NVCVPacking p2,
                 NVCVPacking p3, const NVCVExtraChannelInfo *ex)
{
    return MakeCheckedFormat(FormatColorModel(fmt), SpecOrRaw(fmt), css, FormatMemLayout(fmt), FormatDataKind(fmt), swizzle,
                             p0, p1, p2, p3, FormatAlphaType(fmt), ex);
}

// The swizzle of plane `plane` alone. A format's swizzle lists, position by position, which stored component each
// colour channel reads, components being numbered through the planes. The plane's own swizzle renumbers the
// components it holds from X and leaves the other positions 0; a constant-1 (opaque alpha) position stays 1.
NVCVSwizzle PlaneSwizzle(uint64_t fmt, int plane)
{
    if (FormatNumPlanes(fmt) == 1)
    {
        return plane == 0 ? FormatSwizzle(fmt) : NVCV_SWIZZLE_0000;
    }
    if (plane < 0 || plane >= 4)
    {
        return NVCV_SWIZZLE_0000;
    }
    int first = 0;
    for (int p = 0; p < plane; ++p)
    {
        first += DecodePacking(FormatPlanePacking(fmt, p)).numChannels;
    }
    int count = DecodePacking(FormatPlanePacking(fmt, plane)).numChannels;

    NVCVChannel all[4];
    SwizzleChannels(FormatSwizzle(fmt), all);
    NVCVChannel mine[4] = {NVCV_CHANNEL_0, NVCV_CHANNEL_0, NVCV_CHANNEL_0, NVCV_CHANNEL_0};
    bool        any     = false;
    for (int i = first; i < first + count && i < 4; ++i)
    {
        if (all[i] >= NVCV_CHANNEL_X && all[i] <= NVCV_CHANNEL_W)
        {
            mine[all[i] - NVCV_CHANNEL_X] = (NVCVChannel)(NVCV_CHANNEL_X + (i - first));
            any                           = true;
        }
        else if (all[i] == NVCV_CHANNEL_0)
        {
            ++count; // an unused position does not use up one of the plane's components
        }
        else
        {
            mine[i] = all[i];
            any     = true;
        }
    }
    if (any)
    {
        for (int i = 0; i < 4; ++i)
        {
            if (all[i] == NVCV_CHANNEL_1)
            {
                if (mine[i] != NVCV_CHANNEL_0)
                {
                    throw Error(NVCV_ERROR_INVALID_IMAGE_FORMAT, "Swizzle %s cannot be split over the planes",
                                nvcvSwizzleGetName(FormatSwizzle(fmt)));
                }
                mine[i] = NVCV_CHANNEL_1;
            }
        }
    }
    return MakeSwizzle(mine[0], mine[1], mine[2], mine[3]);
}

// Inverse of PlaneSwizzle: the swizzle of the format whose planes have these swizzles.
NVCVSwizzle MergeSwizzles(const NVCVSwizzle sw[4])
{
    if (sw[1] == NVCV_SWIZZLE_0000)
    {
        if (sw[2] != NVCV_SWIZZLE_0000 || sw[3] != NVCV_SWIZZLE_0000)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Plane swizzles must be given without gaps");
        }
        return sw[0];
    }
    NVCVChannel out[4] = {NVCV_CHANNEL_0, NVCV_CHANNEL_0, NVCV_CHANNEL_0, NVCV_CHANNEL_0};
    int         next   = 0;
    for (int p = 0; p < 4 && sw[p] != NVCV_SWIZZLE_0000; ++p)
    {
        NVCVChannel ch[4];
        SwizzleChannels(sw[p], ch);
        const int count = SwizzleNumChannels(sw[p]);
        int       top   = -1; // highest component the plane uses
        for (int j = 0; j < 4; ++j)
        {
            if (ch[j] >= NVCV_CHANNEL_X && ch[j] <= NVCV_CHANNEL_W)
            {
                top = ch[j] - NVCV_CHANNEL_X > top ? ch[j] - NVCV_CHANNEL_X : top;
            }
        }
        // user[c] = the position (as a channel letter) that reads component c; a constant 1 is filed after the
        // plane's last component
        NVCVChannel user[5] = {NVCV_CHANNEL_0, NVCV_CHANNEL_0, NVCV_CHANNEL_0, NVCV_CHANNEL_0, NVCV_CHANNEL_0};
        for (int j = 0; j < 4; ++j)
        {
            if (ch[j] == NVCV_CHANNEL_1)
            {
                if (top + 1 >= 4)
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "A plane swizzle that uses W cannot also hold a constant 1");
                }
                user[top + 1] = NVCV_CHANNEL_1;
            }
            else if (ch[j] >= NVCV_CHANNEL_X && ch[j] <= NVCV_CHANNEL_W)
            {
                user[ch[j] - NVCV_CHANNEL_X] = (NVCVChannel)(NVCV_CHANNEL_X + j);
            }
        }
        for (int c = 0; c < count && next + c < 4; ++c)
        {
            if (user[c] == NVCV_CHANNEL_1 && c == count - 1)
            {
                out[3] = NVCV_CHANNEL_1;
            }
            else
            {
                out[next + c] = user[c];
            }
        }
        next += count;
    }
    for (int p = 0; p < 4; ++p)
    {
        NVCVChannel ch[4];
        SwizzleChannels(sw[p], ch);
        if (ch[3] == NVCV_CHANNEL_1)
        {
            out[3] = NVCV_CHANNEL_1;
            break;
        }
    }
    return MakeSwizzle(out[0], out[1], out[2], out[3]);
}

uint64_t PlaneFormat(uint64_t fmt, int plane)
{
    if (plane < 0 || plane >= FormatNumPlanes(fmt))
    {
        return NVCV_IMAGE_FORMAT_NONE;
    }
    const NVCVExtraChannelInfo ex = FormatExtraChannels(fmt);
    return Rebuild(fmt, plane == 0 ? NVCV_CSS_NONE : FormatCSS(fmt), PlaneSwizzle(fmt, plane), FormatPlanePacking(fmt, plane),
                   NVCV_PACKING_0, NVCV_PACKING_0, NVCV_PACKING_0, &ex);
}

uint64_t FromPlanes(const uint64_t given[4])
{
    // NVCV_IMAGE_FORMAT_NONE entries are skipped wherever they stand
    uint64_t planes[4] = {};
    int      count     = 0;
    for (int i = 0; i < 4; ++i)
    {
        if (given[i] != NVCV_IMAGE_FORMAT_NONE)
        {
            planes[count++] = given[i];
        }
    }
    if (count == 0)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "At least one plane format is needed");
    }
    const uint64_t        first    = planes[0];
    NVCVChromaSubsampling css      = NVCV_CSS_NONE;
    int                   channels = 0;
    NVCVSwizzle           sw[4]    = {NVCV_SWIZZLE_0000, NVCV_SWIZZLE_0000, NVCV_SWIZZLE_0000, NVCV_SWIZZLE_0000};
    NVCVPacking           pk[4]    = {NVCV_PACKING_0, NVCV_PACKING_0, NVCV_PACKING_0, NVCV_PACKING_0};
    for (int i = 0; i < count; ++i)
    {
        const uint64_t f = planes[i];
        if (FormatNumPlanes(f) != 1)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Format of plane %d must itself have exactly one plane", i);
        }
        if (FormatAlphaType(f) != FormatAlphaType(first))
        {
            throw Error(NVCV_ERROR_INVALID_IMAGE_FORMAT, "All planes must have the same alpha type");
        }
        channels += FormatNumChannels(f);
        if (FormatColorModel(f) != FormatColorModel(first) || SpecOrRaw(f) != SpecOrRaw(first))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "All planes must have the same colour model and spec (or raw pattern)");
        }
        if (FormatMemLayout(f) != FormatMemLayout(first) || FormatDataKind(f) != FormatDataKind(first))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "All planes must have the same memory layout and data kind");
        }
        const NVCVChromaSubsampling pcss = FormatCSS(f);
        if (css == NVCV_CSS_NONE)
        {
            css = pcss;
        }
        else if (css != pcss)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Plane %d has a second kind of chroma subsampling", i);
        }
        sw[i] = FormatSwizzle(f);
        pk[i] = FormatPlanePacking(f, 0);
    }
    if (channels > 4 || channels == 0)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "The planes must hold 1 to 4 channels in total, not %d", channels);
    }
    return Rebuild(first, css, MergeSwizzles(sw), pk[0], pk[1], pk[2], pk[3], nullptr);
}

// ---- FourCC -------------------------------------------------------------------------------------------------
constexpr uint32_t Code(char a, char b, char c, char d)
{
    return (uint32_t)(uint8_t)a | (uint32_t)(uint8_t)b << 8 | (uint32_t)(uint8_t)c << 16 | (uint32_t)(uint8_t)d << 24;
}

struct FourCCRow
{
    uint32_t code;
    uint64_t fmt; // pitch-linear, undefined colour spec
};

uint64_t Rgb(NVCVSwizzle sw, NVCVPacking p)
{
    return MakeFormatWord(NVCV_COLOR_MODEL_RGB, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, NVCV_MEM_LAYOUT_PL, NVCV_DATA_KIND_UNSIGNED,
                          sw, NVCV_ALPHA_ASSOCIATED, p, NVCV_PACKING_0, NVCV_PACKING_0, NVCV_PACKING_0);
}

uint64_t Yuv(NVCVChromaSubsampling css, NVCVSwizzle sw, NVCVPacking p0, NVCVPacking p1 = NVCV_PACKING_0,
             NVCVPacking p2 = NVCV_PACKING_0)
{
    return MakeFormatWord(NVCV_COLOR_MODEL_YCbCr, NVCV_COLOR_SPEC_UNDEFINED, css, NVCV_MEM_LAYOUT_PL, NVCV_DATA_KIND_UNSIGNED, sw,
                          NVCV_ALPHA_ASSOCIATED, p0, p1, p2, NVCV_PACKING_0);
}

// V4L2 pixel-format codes the reference knows (src/nvcv/src/priv/ImageFormat.cpp:463-505), in its order: the
// first row of a format is the code the way back reports.
const FourCCRow *FourCCTable(int *count)
{
    static const FourCCRow rows[] = {
        {Code('R', 'G', 'B', '1'), Rgb(NVCV_SWIZZLE_ZYX1, NVCV_PACKING_X3Y3Z2)},
        {Code('R', '4', '4', '4'), Rgb(NVCV_SWIZZLE_XYZ1, NVCV_PACKING_b4X4Y4Z4)},
        {Code('R', 'G', 'B', '0'), Rgb(NVCV_SWIZZLE_ZYX1, NVCV_PACKING_b1X5Y5Z5)},
        {Code('R', 'G', 'B', 'P'), Rgb(NVCV_SWIZZLE_ZYX1, NVCV_PACKING_X5Y6Z5)},
        {Code('R', 'G', 'B', 'Q'), Rgb(NVCV_SWIZZLE_XYZ1, NVCV_PACKING_X5Y5b1Z5)},
        {Code('R', 'G', 'B', 'R'), Rgb(NVCV_SWIZZLE_XYZ1, NVCV_PACKING_X5Y6Z5)},
        {Code('B', 'G', 'R', '3'), Rgb(NVCV_SWIZZLE_ZYX1, NVCV_PACKING_X8_Y8_Z8)},
        {Code('R', 'G', 'B', '3'), Rgb(NVCV_SWIZZLE_XYZ1, NVCV_PACKING_X8_Y8_Z8)},
        {Code('B', 'G', 'R', '4'), Rgb(NVCV_SWIZZLE_ZYXW, NVCV_PACKING_X8_Y8_Z8_W8)},
        {Code('R', 'G', 'B', '4'), Rgb(NVCV_SWIZZLE_XYZW, NVCV_PACKING_X8_Y8_Z8_W8)},
        {Code('B', 'A', '8', '1'),
         MakeFormatWord(NVCV_COLOR_MODEL_RAW, NVCV_RAW_BAYER_BGGR, NVCV_CSS_NONE, NVCV_MEM_LAYOUT_PL, NVCV_DATA_KIND_UNSIGNED,
                        NVCV_SWIZZLE_X000, NVCV_ALPHA_ASSOCIATED, NVCV_PACKING_X8, NVCV_PACKING_0, NVCV_PACKING_0, NVCV_PACKING_0)},
        {Code('A', 'Y', 'U', 'V'), Yuv(NVCV_CSS_444, NVCV_SWIZZLE_YZWX, NVCV_PACKING_X8_Y8_Z8_W8)},
        {Code('G', 'R', 'A', 'Y'), Yuv(NVCV_CSS_444, NVCV_SWIZZLE_X000, NVCV_PACKING_X8)},
        {Code('Y', '8', ' ', ' '), Yuv(NVCV_CSS_444, NVCV_SWIZZLE_X000, NVCV_PACKING_X8)},
        {Code('Y', '8', '0', '0'), Yuv(NVCV_CSS_444, NVCV_SWIZZLE_X000, NVCV_PACKING_X8)},
        {Code('Y', '1', '6', ' '), Yuv(NVCV_CSS_444, NVCV_SWIZZLE_X000, NVCV_PACKING_X16)},
        {Code('U', 'Y', 'V', 'Y'), Yuv(NVCV_CSS_422, NVCV_SWIZZLE_XYZ1, NVCV_PACKING_Y8_X8__Z8_X8)},
        {Code('Y', 'U', 'Y', '2'), Yuv(NVCV_CSS_422, NVCV_SWIZZLE_XYZ1, NVCV_PACKING_X8_Y8__X8_Z8)},
        {Code('Y', 'U', 'Y', 'V'), Yuv(NVCV_CSS_422, NVCV_SWIZZLE_XYZ1, NVCV_PACKING_X8_Y8__X8_Z8)},
        {Code('Y', 'U', 'N', 'V'), Yuv(NVCV_CSS_422, NVCV_SWIZZLE_XYZ1, NVCV_PACKING_X8_Y8__X8_Z8)},
        {Code('Y', 'V', 'Y', 'U'), Yuv(NVCV_CSS_422, NVCV_SWIZZLE_XZY1, NVCV_PACKING_X8_Y8__X8_Z8)},
        {Code('I', '4', '2', '0'), Yuv(NVCV_CSS_420, NVCV_SWIZZLE_XYZ0, NVCV_PACKING_X8, NVCV_PACKING_X8, NVCV_PACKING_X8)},
        {Code('I', 'Y', 'U', 'V'), Yuv(NVCV_CSS_420, NVCV_SWIZZLE_XYZ0, NVCV_PACKING_X8, NVCV_PACKING_X8, NVCV_PACKING_X8)},
        {Code('N', 'V', '1', '2'), Yuv(NVCV_CSS_420, NVCV_SWIZZLE_XYZ0, NVCV_PACKING_X8, NVCV_PACKING_X8_Y8)},
        {Code('N', 'V', '2', '1'), Yuv(NVCV_CSS_420, NVCV_SWIZZLE_XZY0, NVCV_PACKING_X8, NVCV_PACKING_X8_Y8)},
        {Code('Y', 'V', '1', '2'), Yuv(NVCV_CSS_420, NVCV_SWIZZLE_XZY0, NVCV_PACKING_X8, NVCV_PACKING_X8, NVCV_PACKING_X8)},
        {Code('Y', 'V', '1', '6'), Yuv(NVCV_CSS_422, NVCV_SWIZZLE_XZY0, NVCV_PACKING_X8, NVCV_PACKING_X8, NVCV_PACKING_X8)},
    };
    *count = (int)(sizeof(rows) / sizeof(rows[0]));
    return rows;
}

uint64_t WithColorSpec(uint64_t fmt, NVCVColorSpec spec)
{
    uint32_t word = (uint32_t)EnumValue(spec);
    switch (FormatColorModel(fmt))
    {
    case NVCV_COLOR_MODEL_RGB:
        word = (uint32_t)Replace(word, 7, 3, NVCV_YCbCr_ENC_UNDEFINED); // RGB has no YCbCr encoding
        break;
    case NVCV_COLOR_MODEL_YCbCr:
        break; // an undefined encoding stays undefined (0)
    default:
        if (FormatColorSpec(fmt) != NVCV_COLOR_SPEC_UNDEFINED)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Format of colour model %s carries a colour spec it cannot have",
                        nvcvColorModelGetName(FormatColorModel(fmt)));
        }
        return fmt; // models without a colour spec ignore the request
    }
    return Replace(fmt, 20, 15, word);
}

// ---- packings -----------------------------------------------------------------------------------------------
NVCVSwizzle SwizzleOfFields(const int32_t bits[4])
{
    NVCVChannel ch[4];
    for (int i = 0; i < 4; ++i)
    {
        ch[i] = bits[i] != 0 ? (NVCVChannel)(NVCV_CHANNEL_X + i) : NVCV_CHANNEL_0;
    }
    return MakeSwizzle(ch[0], ch[1], ch[2], ch[3]);
}

// A swizzle that names fewer channels than there are fields marks a packing with padding fields; only then, and
// for the two 4:2:2 pair packings, does the swizzle take part in the match.
bool SwizzleSelects(const NVCVPackingParams &p)
{
    if (p.swizzle == NVCV_SWIZZLE_XYXZ || p.swizzle == NVCV_SWIZZLE_YXZX)
    {
        return true;
    }
    if (p.swizzle == NVCV_SWIZZLE_0000)
    {
        return false;
    }
    int fields = 0;
    for (int i = 0; i < 4; ++i)
    {
        fields += p.bits[i] != 0 ? 1 : 0;
    }
    return SwizzleNumChannels(p.swizzle) != fields;
}

NVCVPacking FindPackingByParams(const NVCVPackingParams &want)
{
    if (want.bits[0] == 0 && want.bits[1] == 0 && want.bits[2] == 0 && want.bits[3] == 0)
    {
        return NVCV_PACKING_0;
    }
    const NVCVSwizzle key = SwizzleSelects(want) ? want.swizzle : NVCV_SWIZZLE_0000;
    int               count;
    const PackingRow *rows = PackingTable(&count);
    const PackingRow *hit  = nullptr;
    for (int i = 0; i < count; ++i)
    {
        const PackingRow &r = rows[i];
        if (r.swizzle != key || std::memcmp(r.fields, want.bits, sizeof(r.fields)) != 0)
        {
            continue;
        }
        // the requested alignment never rejects a packing (nor does it in the reference, DataLayout.cpp:408-440);
        // among equal layouts the least aligned one is taken
        if (hit == nullptr || r.alignment < hit->alignment)
        {
            hit = &r;
        }
    }
    if (hit == nullptr)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "No packing has these field widths and channel positions");
    }
    // one channel reads the same in either byte order
    if (SwizzleNumChannels(want.swizzle) >= 2 && hit->order != want.byteOrder)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "The packing with these fields has the other byte order");
    }
    if (want.swizzle != NVCV_SWIZZLE_0000)
    {
        const NVCVSwizzle have = hit->swizzle != NVCV_SWIZZLE_0000 ? hit->swizzle : SwizzleOfFields(want.bits);
        if (have != want.swizzle)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "The packing with these fields places its channels as %s, not %s",
                        nvcvSwizzleGetName(have), nvcvSwizzleGetName(want.swizzle));
        }
    }
    return hit->packing;
}

} // namespace
} // namespace nvcvamd

using namespace nvcvamd;

extern "C"
{
// ---- packings -------------------------------------------------------------------------------------------------
NVCVStatus nvcvMakePacking(NVCVPacking *outPacking, const NVCVPackingParams *params)
{
    return Protect(
        [&]
        {
            NotNull(outPacking, "Pointer to output packing");
            NotNull(params, "Pointer to packing parameters");
            *outPacking = FindPackingByParams(*params);
        });
}

NVCVStatus nvcvPackingGetParams(NVCVPacking packing, NVCVPackingParams *outParams)
{
    return Protect(
        [&]
        {
            NotNull(outParams, "Pointer to output parameters");
            NVCVPackingParams p = {};
            p.byteOrder         = NVCV_ORDER_LSB;
            p.swizzle           = NVCV_SWIZZLE_0000;
            if (packing != NVCV_PACKING_0)
            {
                const PackingRow *row = FindPacking(packing);
                if (row == nullptr)
                {
                    throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Unknown packing %d", (int)packing);
                }
                p.byteOrder = row->order;
                p.alignment = row->alignment;
                std::memcpy(p.bits, row->fields, sizeof(p.bits));
                p.swizzle = row->swizzle != NVCV_SWIZZLE_0000 ? row->swizzle : SwizzleOfFields(row->fields);
            }
            *outParams = p;
        });
}

const char *nvcvPackingGetName(NVCVPacking packing)
{
    if (packing == NVCV_PACKING_0)
    {
        return "NVCV_PACKING_0";
    }
    const PackingRow *row = FindPacking(packing);
    return row != nullptr ? row->name : ThreadName("NVCVPacking(%d)", (int)packing);
}

const char *nvcvChannelGetName(NVCVChannel channel)
{
    static const char *const names[] = {"0", "X", "Y", "Z", "W", "1"};
    return EnumName(EnumValue(channel), names, 6, "NVCVChannel");
}

const char *nvcvByteOrderGetName(NVCVByteOrder byteOrder)
{
    static const char *const names[] = {"LSB", "MSB"};
    return EnumName(EnumValue(byteOrder), names, 2, "NVCVByteOrder");
}

// ---- constructors ---------------------------------------------------------------------------------------------
NVCVStatus nvcvMakeRawImageFormat(NVCVImageFormat *outFormat, NVCVRawPattern rawPattern, NVCVMemLayout memLayout,
                                  NVCVDataKind dataKind, NVCVSwizzle swizzle, NVCVPacking packing0, NVCVPacking packing1,
                                  NVCVPacking packing2, NVCVPacking packing3, NVCVAlphaType alphaType,
                                  const NVCVExtraChannelInfo *exChannelInfo)
{
    return Protect(
        [&]
        {
            NotNull(outFormat, "Pointer to output format");
            *outFormat = MakeCheckedFormat(NVCV_COLOR_MODEL_RAW, (uint32_t)EnumValue(rawPattern), NVCV_CSS_NONE, memLayout, dataKind,
                                           swizzle, packing0, packing1, packing2, packing3, alphaType, exChannelInfo);
        });
}

NVCVStatus nvcvMakeImageFormatFromFourCC(NVCVImageFormat *outFormat, uint32_t fourcc, NVCVColorSpec colorSpec,
                                         NVCVMemLayout memLayout)
{
    return Protect(
        [&]
        {
            NotNull(outFormat, "Pointer to output format");
            uint32_t upper = 0;
            for (int i = 0; i < 4; ++i)
            {
                upper |= (uint32_t)std::toupper((int)((fourcc >> (8 * i)) & 0xFF)) << (8 * i);
            }
            int              count;
            const FourCCRow *rows = FourCCTable(&count);
            for (int i = 0; i < count; ++i)
            {
                if (rows[i].code == upper)
                {
                    uint64_t     fmt   = rows[i].fmt;
                    const auto   model = FormatColorModel(fmt);
                    if (model == NVCV_COLOR_MODEL_RGB || model == NVCV_COLOR_MODEL_YCbCr)
                    {
                        fmt = WithColorSpec(fmt, colorSpec);
                    }
                    *outFormat = Replace(fmt, 12, 3, (uint64_t)EnumValue(memLayout));
                    return;
                }
            }
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "FourCC code '%c%c%c%c' is not supported", (int)(upper & 0xFF),
                        (int)((upper >> 8) & 0xFF), (int)((upper >> 16) & 0xFF), (int)(upper >> 24));
        });
}

NVCVStatus nvcvImageFormatToFourCC(NVCVImageFormat fmt, uint32_t *outFourCC)
{
    return Protect(
        [&]
        {
            NotNull(outFourCC, "Pointer to output FourCC code");
            if (fmt == NVCV_IMAGE_FORMAT_NONE)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "NVCV_IMAGE_FORMAT_NONE has no FourCC code");
            }
            const uint64_t   plain = Replace(WithColorSpec(fmt, NVCV_COLOR_SPEC_UNDEFINED), 12, 3, NVCV_MEM_LAYOUT_PL);
            int              count;
            const FourCCRow *rows = FourCCTable(&count);
            for (int i = 0; i < count; ++i)
            {
                if (rows[i].fmt == plain)
                {
                    *outFourCC = rows[i].code;
                    return;
                }
            }
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Format %s has no FourCC code", nvcvImageFormatGetName(fmt));
        });
}

NVCVStatus nvcvMakeImageFormatFromPlanes(NVCVImageFormat *outFormat, NVCVImageFormat plane0, NVCVImageFormat plane1,
                                         NVCVImageFormat plane2, NVCVImageFormat plane3)
{
    return Protect(
        [&]
        {
            NotNull(outFormat, "Pointer to output format");
            const uint64_t planes[4] = {plane0, plane1, plane2, plane3};
            *outFormat               = FromPlanes(planes);
        });
}

NVCVStatus nvcvImageFormatGetPlaneFormat(NVCVImageFormat fmt, int32_t plane, NVCVImageFormat *outFormat)
{
    return Protect([&] { *NotNull(outFormat, "Pointer to output format") = PlaneFormat(fmt, plane); });
}

NVCVStatus nvcvImageFormatGetPlaneSwizzle(NVCVImageFormat fmt, int32_t plane, NVCVSwizzle *outPlaneSwizzle)
{
    return Protect([&] { *NotNull(outPlaneSwizzle, "Pointer to output swizzle") = PlaneSwizzle(fmt, plane); });
}

// ---- setters --------------------------------------------------------------------------------------------------
NVCVStatus nvcvImageFormatSetSwizzleAndPacking(NVCVImageFormat *fmt, NVCVSwizzle swizzle, NVCVPacking packing0,
                                               NVCVPacking packing1, NVCVPacking packing2, NVCVPacking packing3)
{
    return Protect(
        [&]
        {
            uint64_t                  *f  = Editable(fmt, "swizzle and packing");
            const NVCVExtraChannelInfo ex = FormatExtraChannels(*f);
            *f                            = Rebuild(*f, FormatCSS(*f), swizzle, packing0, packing1, packing2, packing3, &ex);
        });
}

NVCVStatus nvcvImageFormatSetDataKind(NVCVImageFormat *fmt, NVCVDataKind dataKind)
{
    return Protect(
        [&]
        {
            uint64_t *f = Editable(fmt, "data kind");
            *f          = Replace(*f, 61, 3, (uint64_t)EnumValue(dataKind));
        });
}

NVCVStatus nvcvImageFormatSetMemLayout(NVCVImageFormat *fmt, NVCVMemLayout memLayout)
{
    return Protect(
        [&]
        {
            uint64_t *f = Editable(fmt, "memory layout");
            *f          = Replace(*f, 12, 3, (uint64_t)EnumValue(memLayout));
        });
}

NVCVStatus nvcvImageFormatSetColorSpec(NVCVImageFormat *fmt, NVCVColorSpec colorSpec)
{
    return Protect(
        [&]
        {
            uint64_t *f = Editable(fmt, "colour spec");
            *f          = WithColorSpec(*f, colorSpec);
        });
}

NVCVStatus nvcvImageFormatSetChromaSubsampling(NVCVImageFormat *fmt, NVCVChromaSubsampling css)
{
    return Protect(
        [&]
        {
            uint64_t *f = Editable(fmt, "chroma subsampling");
            if (FormatColorModel(*f) == NVCV_COLOR_MODEL_YCbCr)
            {
                *f = Replace(*f, 17, 3, (uint64_t)EnumValue(css));
            }
            else if (css != NVCV_CSS_NONE)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Only YCbCr formats have chroma subsampling");
            }
        });
}

NVCVStatus nvcvImageFormatSetRawPattern(NVCVImageFormat *fmt, NVCVRawPattern rawPattern)
{
    return Protect(
        [&]
        {
            uint64_t *f = Editable(fmt, "raw pattern");
            if (FormatColorModel(*f) != NVCV_COLOR_MODEL_RAW)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Only formats of the RAW colour model have a pattern, this one is %s",
                            nvcvColorModelGetName(FormatColorModel(*f)));
            }
            *f = Replace(*f, 21, 6, (uint64_t)EnumValue(rawPattern));
        });
}

NVCVStatus nvcvImageFormatGetRawPattern(NVCVImageFormat fmt, NVCVRawPattern *outRawPattern)
{
    return Protect(
        [&]
        {
            NotNull(outRawPattern, "Pointer to output raw pattern");
            const int raw = FormatRawPattern(fmt);
            if (raw < 0)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Colour model %s has no raw pattern",
                            nvcvColorModelGetName(FormatColorModel(fmt)));
            }
            *outRawPattern = (NVCVRawPattern)raw;
        });
}

NVCVStatus nvcvImageFormatSetAlphaType(NVCVImageFormat *fmt, NVCVAlphaType alphaType)
{
    return Protect(
        [&]
        {
            uint64_t *f = Editable(fmt, "alpha type");
            *f          = Replace(*f, 6, 1, (uint64_t)EnumValue(alphaType));
        });
}

NVCVStatus nvcvImageFormatGetExtraChannelInfo(NVCVImageFormat fmt, NVCVExtraChannelInfo *outExChannelInfo)
{
    return Protect([&] { *NotNull(outExChannelInfo, "Pointer to output extra-channel info") = FormatExtraChannels(fmt); });
}

NVCVStatus nvcvImageFormatSetExtraChannelInfo(NVCVImageFormat *fmt, const NVCVExtraChannelInfo *exChannelInfo)
{
    return Protect(
        [&]
        {
            uint64_t *f = Editable(fmt, "extra channels");
            NotNull(exChannelInfo, "Pointer to extra-channel info");
            if (exChannelInfo->numChannels < 0 || exChannelInfo->numChannels > NVCV_MAX_EXTRA_CHANNEL_COUNT)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Between 0 and %d extra channels, not %d", NVCV_MAX_EXTRA_CHANNEL_COUNT,
                            exChannelInfo->numChannels);
            }
            if (exChannelInfo->bitsPerPixel > 128)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Extra channels may have at most 128 bits, not %d",
                            exChannelInfo->bitsPerPixel);
            }
            if (exChannelInfo->datakind == NVCV_DATA_KIND_UNSPECIFIED)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Extra channels need a data kind");
            }
            if (FormatNumPlanes(*f) != 1)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Only single-plane formats can have extra channels");
            }
            // rebuilt rather than patched so that the marker bit that tells extra-channel info from plane packings
            // always agrees with the content
            *f = MakeFormatWord(FormatColorModel(*f), SpecOrRaw(*f), FormatCSS(*f), FormatMemLayout(*f), FormatDataKind(*f),
                                FormatSwizzle(*f), FormatAlphaType(*f), FormatPlanePacking(*f, 0), NVCV_PACKING_0, NVCV_PACKING_0,
                                NVCV_PACKING_0, exChannelInfo);
        });
}
}
