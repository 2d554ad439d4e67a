// Decoding and construction of the 64-bit format / data-type words (field map in
// nvcv/detail/FormatBits.h). Covers the queries the operators and the object layer need; follows
// the decoding rules of the reference's src/nvcv/src/priv/ImageFormat.cpp:560-860 and
// DataLayout.cpp:645-667 (channel count = distinct X/Y/Z/W selectors).
#include "Priv.hpp"

#include <cstring>

namespace nvcvamd {

namespace {

const PackingRow kPackings[] = {
#include "PackingTable.inc"
};
constexpr int kNumPackings = sizeof(kPackings) / sizeof(kPackings[0]);

const char *const kSwizzles[] = {
#include "SwizzleTable.inc"
};
constexpr int kNumSwizzles = sizeof(kSwizzles) / sizeof(kSwizzles[0]);

inline uint64_t Get(uint64_t v, int off, int len)
{
    return FieldGet(v, off, len);
}

inline uint64_t Put(uint64_t v, int off, int len)
{
    return FieldPut(v, off, len);
}

int BppFromCode(int code, int sub, int nch)
{
    switch (code)
    {
    case 0:
        return (nch == 1 && sub >= 1 && sub <= 3) ? (sub == 3 ? 4 : sub) : 8;
    case 1:
    case 2:
    case 3:
        return (code + 1) * 8;
    case 4:
    case 5:
        return (code - 1) * 16;
    case 6:
    case 7:
        return (code - 3) * 32;
    default:
        return (code - 5) * 64;
    }
}

} // namespace

const PackingRow *FindPacking(NVCVPacking p)
{
    for (const PackingRow &row : kPackings)
    {
        if (row.packing == p)
        {
            return &row;
        }
    }
    return nullptr;
}

const PackingRow *PackingTable(int *count)
{
    *count = kNumPackings;
    return kPackings;
}

PackingInfo DecodePacking(NVCVPacking p)
{
    PackingInfo info = {};
    if (p == NVCV_PACKING_0)
    {
        info.known = true;
        return info;
    }
    info.numComponents = (int)Get(p, 4, 2) + 1;
    // a 4:2:2 pixel pair stores four components for three channels (luma twice)
    info.numChannels  = (p == NVCV_PACKING_X8_Y8__X8_Z8 || p == NVCV_PACKING_Y8_X8__Z8_X8) ? 3 : info.numComponents;
    info.bitsPerPixel = BppFromCode((int)Get(p, 6, 4), (int)Get(p, 0, 4), info.numComponents);
    if (const PackingRow *row = FindPacking(p))
    {
        std::memcpy(info.bits, row->bits, sizeof(info.bits));
        info.known = true;
    }
    return info;
}

NVCVPacking FormatPlanePacking(uint64_t fmt, int plane)
{
    if (fmt == 0)
    {
        return NVCV_PACKING_0;
    }
    uint64_t sub, ch, bpp;
    switch (plane)
    {
    case 0:
        sub = Get(fmt, 35, 3);
        ch  = Get(fmt, 38, 2);
        bpp = Get(fmt, 40, 4);
        break;
    case 1:
    case 2:
        if (Get(fmt, 7, 1) == 0) // slots 1..3 hold extra-channel info instead
        {
            return NVCV_PACKING_0;
        }
        sub = Get(fmt, plane == 1 ? 44 : 51, 3);
        ch  = Get(fmt, plane == 1 ? 47 : 54, 1);
        bpp = Get(fmt, plane == 1 ? 48 : 55, 3);
        break;
    case 3:
    {
        if (Get(fmt, 7, 1) == 0)
        {
            return NVCV_PACKING_0;
        }
        uint64_t code = Get(fmt, 58, 3);
        if (code == 0)
        {
            return NVCV_PACKING_0;
        }
        if (code == 7) // an 8-bit fourth plane is stored as all ones
        {
            return NVCV_PACKING_X8;
        }
        return (NVCVPacking)Put(code, 6, 4);
    }
    default:
        return NVCV_PACKING_0;
    }
    return (NVCVPacking)(Put(bpp, 6, 4) | Put(ch, 4, 2) | Put(sub, 0, 4));
}

int FormatNumPlanes(uint64_t fmt)
{
    int n = 0;
    for (int p = 0; p < 4; ++p)
    {
        n += FormatPlanePacking(fmt, p) != NVCV_PACKING_0 ? 1 : 0;
    }
    return n;
}

NVCVSwizzle FormatSwizzle(uint64_t fmt)
{
    return (NVCVSwizzle)Get(fmt, 0, 6);
}

void SwizzleChannels(NVCVSwizzle sw, NVCVChannel out[4])
{
    if ((int)sw < 0 || (int)sw >= kNumSwizzles)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid swizzle code %d", (int)sw);
    }
    const char *s = kSwizzles[(int)sw];
    for (int i = 0; i < 4; ++i)
    {
        switch (s[i])
        {
        case 'X':
            out[i] = NVCV_CHANNEL_X;
            break;
        case 'Y':
            out[i] = NVCV_CHANNEL_Y;
            break;
        case 'Z':
            out[i] = NVCV_CHANNEL_Z;
            break;
        case 'W':
            out[i] = NVCV_CHANNEL_W;
            break;
        case '1':
            out[i] = NVCV_CHANNEL_1;
            break;
        default:
            out[i] = NVCV_CHANNEL_0;
            break;
        }
    }
}

int SwizzleNumChannels(NVCVSwizzle sw)
{
    NVCVChannel ch[4];
    SwizzleChannels(sw, ch);
    bool seen[4] = {};
    int  n       = 0;
    for (NVCVChannel c : ch)
    {
        if (c >= NVCV_CHANNEL_X && c <= NVCV_CHANNEL_W && !seen[c - NVCV_CHANNEL_X])
        {
            seen[c - NVCV_CHANNEL_X] = true;
            ++n;
        }
    }
    return n;
}

int FormatNumChannels(uint64_t fmt)
{
    return fmt == 0 ? 0 : SwizzleNumChannels(FormatSwizzle(fmt));
}

NVCVDataKind FormatDataKind(uint64_t fmt)
{
    return (NVCVDataKind)Get(fmt, 61, 3);
}

NVCVMemLayout FormatMemLayout(uint64_t fmt)
{
    return (NVCVMemLayout)Get(fmt, 12, 3);
}

NVCVColorModel FormatColorModel(uint64_t fmt)
{
    if (fmt == 0)
    {
        return NVCV_COLOR_MODEL_UNDEFINED;
    }
    if (Get(fmt, 16, 1) == 0)
    {
        return NVCV_COLOR_MODEL_YCbCr;
    }
    if (Get(fmt, 16, 19) == (1u << 19) - 1)
    {
        return NVCV_COLOR_MODEL_UNDEFINED;
    }
    uint64_t m = Get(fmt, 17, 3);
    if (m < 7)
    {
        return (NVCVColorModel)(m + 2);
    }
    if (Get(fmt, 20, 1) == 0)
    {
        return NVCV_COLOR_MODEL_RAW;
    }
    return (NVCVColorModel)(Get(fmt, 21, 6) + 10);
}

NVCVColorSpec FormatColorSpec(uint64_t fmt)
{
    NVCVColorModel m = FormatColorModel(fmt);
    if (m != NVCV_COLOR_MODEL_UNDEFINED && (int)m < 7)
    {
        return (NVCVColorSpec)Get(fmt, 20, 15);
    }
    return NVCV_COLOR_SPEC_UNDEFINED;
}

NVCVChromaSubsampling FormatCSS(uint64_t fmt)
{
    return FormatColorModel(fmt) == NVCV_COLOR_MODEL_YCbCr ? (NVCVChromaSubsampling)Get(fmt, 17, 3) : NVCV_CSS_NONE;
}

int FormatPlanePixelStrideBytes(uint64_t fmt, int plane)
{
    return (DecodePacking(FormatPlanePacking(fmt, plane)).bitsPerPixel + 7) / 8;
}

uint64_t MakeFormatWord(NVCVColorModel model, uint32_t specOrRaw, NVCVChromaSubsampling css, NVCVMemLayout layout,
                        NVCVDataKind kind, NVCVSwizzle swizzle, NVCVAlphaType alpha, NVCVPacking p0, NVCVPacking p1,
                        NVCVPacking p2, NVCVPacking p3, const NVCVExtraChannelInfo *ex)
{
    const bool extra = ex != nullptr && ex->numChannels > 0;
    return NVCV_DETAIL_FORMAT_WORD_EX((int)model, specOrRaw, (int)css, (int)layout, (int)kind, (int)swizzle, (int)alpha,
                                      extra ? ex->numChannels : 0, extra ? ex->bitsPerPixel : 0,
                                      extra ? (int)ex->datakind : 0, extra ? (int)ex->channelType : 0, (uint64_t)p0,
                                      (uint64_t)p1, (uint64_t)p2, (uint64_t)p3);
}

NVCVAlphaType FormatAlphaType(uint64_t fmt)
{
    return (NVCVAlphaType)Get(fmt, 6, 1);
}

int FormatRawPattern(uint64_t fmt)
{
    return FormatColorModel(fmt) == NVCV_COLOR_MODEL_RAW ? (int)Get(fmt, 21, 6) : -1;
}

NVCVExtraChannelInfo FormatExtraChannels(uint64_t fmt)
{
    NVCVExtraChannelInfo info = {0, 0, NVCV_DATA_KIND_UNSPECIFIED, NVCV_EXTRA_CHANNEL_U};
    // bit 7 clear = the bits above plane 0's packing describe extra channels, not planes 1..3
    if (fmt != 0 && Get(fmt, 7, 1) == 0 && Get(fmt, 47, 3) > 0)
    {
        info.numChannels  = (int32_t)Get(fmt, 47, 3);
        info.bitsPerPixel = BppFromCode((int)Get(fmt, 50, 3), 4, 2);
        info.datakind     = (NVCVDataKind)Get(fmt, 53, 3);
        info.channelType  = (NVCVExtraChannel)Get(fmt, 44, 3);
    }
    return info;
}

NVCVSwizzle MakeSwizzle(NVCVChannel x, NVCVChannel y, NVCVChannel z, NVCVChannel w)
{
    const NVCVChannel want[4] = {x, y, z, w};
    for (int i = 0; i < kNumSwizzles; ++i)
    {
        NVCVChannel have[4];
        SwizzleChannels((NVCVSwizzle)i, have);
        if (std::memcmp(have, want, sizeof(want)) == 0)
        {
            return (NVCVSwizzle)i;
        }
    }
    return NVCV_SWIZZLE_UNSUPPORTED;
}

// Argument rules of the reference's format constructors (src/nvcv/src/priv/ImageFormat.cpp:36-235).
uint64_t MakeCheckedFormat(NVCVColorModel model, uint32_t specOrRaw, NVCVChromaSubsampling css, NVCVMemLayout layout,
                           NVCVDataKind kind, NVCVSwizzle swizzle, NVCVPacking p0, NVCVPacking p1, NVCVPacking p2,
                           NVCVPacking p3, NVCVAlphaType alpha, const NVCVExtraChannelInfo *ex)
{
    const NVCVPacking pk[4] = {p0, p1, p2, p3};
    if (p0 == NVCV_PACKING_0)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Packing of the first plane must not be 0");
    }
    // plane slots keep 3 bits of the packing's sub-code (planes 0..2) or none (plane 3)
    for (int i = 0; i < 3; ++i)
    {
        if (((uint64_t)pk[i] & 8) != 0)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Packing %s cannot be stored for plane %d", nvcvPackingGetName(pk[i]), i);
        }
    }
    if (((uint64_t)p3 & 15) != 0)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Packing %s cannot be stored for plane 3", nvcvPackingGetName(p3));
    }
    int channels = 0;
    for (int i = 0; i < 4; ++i)
    {
        const PackingInfo pi = DecodePacking(pk[i]);
        if (i >= 1 && pi.bitsPerPixel > (i == 3 ? 64 : 128))
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Plane %d may have at most %d bits per pixel, not %d", i, i == 3 ? 64 : 128,
                        pi.bitsPerPixel);
        }
        if (i == 1 && pi.numChannels > 2)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Plane 1 may have at most 2 channels, not %d", pi.numChannels);
        }
        channels += pi.numChannels;
    }
    if (SwizzleNumChannels(swizzle) != channels)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Swizzle %s names %d channels, the packings hold %d", nvcvSwizzleGetName(swizzle),
                    SwizzleNumChannels(swizzle), channels);
    }
    if (model == NVCV_COLOR_MODEL_UNDEFINED && (specOrRaw != (uint32_t)NVCV_COLOR_SPEC_UNDEFINED || css != NVCV_CSS_NONE))
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Without a colour model, colour spec must be undefined and chroma subsampling NONE");
    }
    if (model != NVCV_COLOR_MODEL_RAW && model != NVCV_COLOR_MODEL_RGB && model != NVCV_COLOR_MODEL_YCbCr
        && model != NVCV_COLOR_MODEL_CMYK && model != NVCV_COLOR_MODEL_YCCK && specOrRaw != (uint32_t)NVCV_COLOR_SPEC_UNDEFINED)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Colour model %s takes no colour spec", nvcvColorModelGetName(model));
    }
    if (ex != nullptr)
    {
        if (ex->numChannels > NVCV_MAX_EXTRA_CHANNEL_COUNT)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "At most %d extra channels, not %d", NVCV_MAX_EXTRA_CHANNEL_COUNT, ex->numChannels);
        }
        if (ex->numChannels > 0 && (p1 != NVCV_PACKING_0 || p2 != NVCV_PACKING_0 || p3 != NVCV_PACKING_0))
        {
            throw Error(NVCV_ERROR_INVALID_IMAGE_FORMAT, "Extra channels need a single-plane format");
        }
        if (ex->bitsPerPixel > 128)
        {
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Extra channels may have at most 128 bits, not %d", ex->bitsPerPixel);
        }
    }
    if (model != NVCV_COLOR_MODEL_YCbCr && css != NVCV_CSS_NONE)
    {
        throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Only YCbCr formats have chroma subsampling");
    }
    return MakeFormatWord(model, specOrRaw, css, layout, kind, swizzle, alpha, p0, p1, p2, p3, ex);
}

NVCVDataType FormatPlaneDataType(uint64_t fmt, int plane)
{
    NVCVPacking p = FormatPlanePacking(fmt, plane);
    if (p == NVCV_PACKING_0)
    {
        return NVCV_DATA_TYPE_NONE;
    }
    if (p == NVCV_PACKING_X8_Y8__X8_Z8 || p == NVCV_PACKING_Y8_X8__Z8_X8)
    {
        p = NVCV_PACKING_X8_Y8; // one pixel of the pair: a luma and a chroma sample
    }
    return NVCV_DETAIL_MAKE_DATA_TYPE(FormatDataKind(fmt), (uint64_t)p);
}

void FormatPlaneSize(uint64_t fmt, int plane, int32_t w, int32_t h, int32_t *pw, int32_t *ph)
{
    int sh = 4, sv = 4; // chroma samples per 4 luma samples
    if (plane >= 1)
    {
        switch (FormatCSS(fmt))
        {
        case NVCV_CSS_444:
            break;
        case NVCV_CSS_422:
            sh = 2;
            break;
        case NVCV_CSS_422R:
            sv = 2;
            break;
        case NVCV_CSS_411:
            sh = 1;
            break;
        case NVCV_CSS_411R:
            sv = 1;
            break;
        case NVCV_CSS_420:
            sh = sv = 2;
            break;
        case NVCV_CSS_410:
            sh = 1;
            sv = 2;
            break;
        case NVCV_CSS_410R:
            sh = 2;
            sv = 1;
            break;
        }
    }
    *pw = (int32_t)(((int64_t)w * sh + 3) / 4);
    *ph = (int32_t)(((int64_t)h * sv + 3) / 4);
}

int DataTypeStrideBytes(NVCVDataType t)
{
    return (DecodePacking(DataTypePacking(t)).bitsPerPixel + 7) / 8;
}

int DataTypeAlignment(NVCVDataType t)
{
    // Machine-word size of one stored component group: for the "_"-separated packings the component size, for
    // sub-word packings the whole pixel (table column; sub-byte packings count as one byte).
    const NVCVPacking p = DataTypePacking(t);
    if (const PackingRow *row = FindPacking(p))
    {
        return row->alignment > 0 ? row->alignment : 1;
    }
    PackingInfo pi = DecodePacking(p);
    return pi.numComponents == 0 ? 1 : (int)NextPow2((pi.bitsPerPixel + 7) / 8);
}

const char *ThreadName(const char *fmt, ...)
{
    // Small ring so that a name built from other generated names does not overwrite its inputs.
    static thread_local char ring[4][512];
    static thread_local int  next = 0;
    char                    *buf  = ring[next];
    next                          = (next + 1) % 4;
    va_list va;
    va_start(va, fmt);
    vsnprintf(buf, sizeof(ring[0]), fmt, va);
    va_end(va);
    return buf;
}

const char *EnumName(int v, const char *const *names, int count, const char *type)
{
    return (v >= 0 && v < count) ? names[v] : ThreadName("%s(%d)", type, v);
}

namespace {

NVCVStatus MakeFormat(NVCVImageFormat *out, NVCVColorModel model, uint32_t spec, NVCVChromaSubsampling css,
                      NVCVMemLayout layout, NVCVDataKind kind, NVCVSwizzle swizzle, NVCVPacking p0, NVCVPacking p1,
                      NVCVPacking p2, NVCVPacking p3, NVCVAlphaType alpha, const NVCVExtraChannelInfo *ex)
{
    return Protect(
        [&]
        {
            NotNull(out, "Pointer to output format");
            *out = MakeCheckedFormat(model, spec, css, layout, kind, swizzle, p0, p1, p2, p3, alpha, ex);
        });
}

template<class E>
NVCVStatus GetSpecField(NVCVColorSpec cspec, int off, int len, E *out, const char *what)
{
    return Protect(
        [&]
        {
            NotNull(out, what);
            *out = (E)Get((uint64_t)(uint32_t)EnumValue(cspec), off, len);
        });
}

NVCVStatus SetSpecField(NVCVColorSpec *cspec, int off, int len, uint64_t value)
{
    return Protect(
        [&]
        {
            NotNull(cspec, "Pointer to input colorspec");
            const uint64_t mask = ((1ULL << len) - 1) << off;
            *cspec = (NVCVColorSpec)(int32_t)((((uint64_t)(uint32_t)EnumValue(*cspec)) & ~mask) | Put(value, off, len));
        });
}

} // namespace
} // namespace nvcvamd

using namespace nvcvamd;

extern "C"
{
// ---- swizzle / packing -------------------------------------------------------------------------
NVCVStatus nvcvSwizzleGetChannels(NVCVSwizzle swizzle, NVCVChannel *channels)
{
    return Protect([&] { SwizzleChannels(swizzle, NotNull(channels, "Pointer to output channels")); });
}

NVCVStatus nvcvSwizzleGetNumChannels(NVCVSwizzle swizzle, int32_t *outNumChannels)
{
    return Protect([&] { *NotNull(outNumChannels, "Pointer to output") = SwizzleNumChannels(swizzle); });
}

NVCVStatus nvcvMakeSwizzle(NVCVSwizzle *outSwizzle, NVCVChannel x, NVCVChannel y, NVCVChannel z, NVCVChannel w)
{
    return Protect(
        [&]
        {
            NotNull(outSwizzle, "Pointer to output swizzle");
            const NVCVSwizzle sw = MakeSwizzle(x, y, z, w);
            if (sw != NVCV_SWIZZLE_UNSUPPORTED)
            {
                *outSwizzle = sw;
                return;
            }
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Channel combination has no swizzle code");
        });
}

NVCVStatus nvcvPackingGetNumComponents(NVCVPacking packing, int32_t *outNumComponents)
{
    return Protect([&] { *NotNull(outNumComponents, "Pointer to output") = DecodePacking(packing).numComponents; });
}

NVCVStatus nvcvPackingGetBitsPerComponent(NVCVPacking packing, int32_t *outBits)
{
    return Protect(
        [&]
        {
            NotNull(outBits, "Pointer to output");
            PackingInfo pi = DecodePacking(packing);
            if (!pi.known)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Unknown packing value %d", (int)packing);
            }
            std::memcpy(outBits, pi.bits, sizeof(pi.bits));
        });
}

NVCVStatus nvcvPackingGetBitsPerPixel(NVCVPacking packing, int32_t *outBPP)
{
    return Protect([&] { *NotNull(outBPP, "Pointer to output") = DecodePacking(packing).bitsPerPixel; });
}

NVCVStatus nvcvPackingGetAlignment(NVCVPacking packing, int32_t *outAlignment)
{
    return Protect(
        [&]
        {
            *NotNull(outAlignment, "Pointer to output")
                = DataTypeAlignment(NVCV_DETAIL_MAKE_DATA_TYPE(NVCV_DATA_KIND_UNSIGNED, (uint64_t)packing));
        });
}

const char *nvcvDataKindGetName(NVCVDataKind kind)
{
    static const char *const names[] = {"NVCV_DATA_KIND_UNSPECIFIED", "NVCV_DATA_KIND_UNSIGNED", "NVCV_DATA_KIND_SIGNED",
                                        "NVCV_DATA_KIND_FLOAT", "NVCV_DATA_KIND_COMPLEX"};
    const int v = EnumValue(kind);
    return (v >= -1 && v <= 3) ? names[v + 1] : ThreadName("NVCVDataKind(%d)", v);
}

const char *nvcvMemLayoutGetName(NVCVMemLayout memlayout)
{
    static const char *const names[] = {"NVCV_MEM_LAYOUT_PITCH_LINEAR",   "NVCV_MEM_LAYOUT_BLOCK1_LINEAR", "NVCV_MEM_LAYOUT_BLOCK2_LINEAR",
                                        "NVCV_MEM_LAYOUT_BLOCK4_LINEAR",  "NVCV_MEM_LAYOUT_BLOCK8_LINEAR", "NVCV_MEM_LAYOUT_BLOCK16_LINEAR",
                                        "NVCV_MEM_LAYOUT_BLOCK32_LINEAR"};
    return EnumName(EnumValue(memlayout), names, 7, "NVCVMemLayout");
}

// The four channel selectors spelled out, e.g. "XYZ1".
const char *nvcvSwizzleGetName(NVCVSwizzle swizzle)
{
    const int v = EnumValue(swizzle);
    return (v >= 0 && v < kNumSwizzles) ? kSwizzles[v] : ThreadName("NVCVSwizzle(%d)", v);
}

// ---- colour spec -------------------------------------------------------------------------------
NVCVStatus nvcvChromaSubsamplingGetNumSamples(NVCVChromaSubsampling css, int32_t *outSamplesHoriz,
                                              int32_t *outSamplesVert)
{
    return Protect(
        [&]
        {
            if (outSamplesHoriz == nullptr && outSamplesVert == nullptr)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "At least one of the two sample-count outputs must be non-NULL");
            }
            const int code = EnumValue(css);
            if (code < 0 || code > 7)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid chroma subsampling: %d", code);
            }
            // Evaluate the plane-size rule on a 4x4 luma block of a synthetic YCbCr format.
            uint64_t fmt = MakeFormatWord(NVCV_COLOR_MODEL_YCbCr, NVCV_COLOR_SPEC_BT601, (NVCVChromaSubsampling)code, NVCV_MEM_LAYOUT_PL,
                                          NVCV_DATA_KIND_UNSIGNED, NVCV_SWIZZLE_XYZ0, NVCV_ALPHA_ASSOCIATED,
                                          NVCV_PACKING_X8, NVCV_PACKING_X8_Y8, NVCV_PACKING_0, NVCV_PACKING_0);
            int32_t  w, h;
            FormatPlaneSize(fmt, 1, 4, 4, &w, &h);
            if (outSamplesHoriz)
            {
                *outSamplesHoriz = w;
            }
            if (outSamplesVert)
            {
                *outSamplesVert = h;
            }
        });
}

const char *nvcvColorModelGetName(NVCVColorModel cmodel)
{
    const int value = EnumValue(cmodel);
    switch (value)
    {
    case NVCV_COLOR_MODEL_UNDEFINED:
        return "NVCV_COLOR_MODEL_UNDEFINED";
    case NVCV_COLOR_MODEL_YCbCr:
        return "NVCV_COLOR_MODEL_YCbCr";
    case NVCV_COLOR_MODEL_RGB:
        return "NVCV_COLOR_MODEL_RGB";
    case NVCV_COLOR_MODEL_RAW:
        return "NVCV_COLOR_MODEL_RAW";
    case NVCV_COLOR_MODEL_XYZ:
        return "NVCV_COLOR_MODEL_XYZ";
    case NVCV_COLOR_MODEL_HSV:
        return "NVCV_COLOR_MODEL_HSV";
    case NVCV_COLOR_MODEL_CMYK:
        return "NVCV_COLOR_MODEL_CMYK";
    case NVCV_COLOR_MODEL_YCCK:
        return "NVCV_COLOR_MODEL_YCCK";
    }
    return ThreadName("NVCVColorModel(%d)", value);
}

const char *nvcvChromaSubsamplingGetName(NVCVChromaSubsampling css)
{
    // J:a:b notation (reference: src/nvcv/src/priv/ColorSpec.cpp:447-478)
    static const char *const names[] = {"4:4:4", "4:2:2", "4:2:2R", "4:1:1", "4:1:1R", "4:2:0", "4:1:0", "4:1:0R"};
    return EnumName(EnumValue(css), names, 8, "NVCVChromaSubsampling");
}

NVCVStatus nvcvMakeChromaSubsampling(NVCVChromaSubsampling *outCSS, int32_t samplesHoriz, int32_t samplesVert)
{
    return Protect(
        [&]
        {
            NotNull(outCSS, "Pointer to output chroma subsampling");
            // samples per 4 luma samples -> code (reference: priv/ColorSpec.cpp:99-143); 1 x 1 is 4:4:4 as well
            static const struct
            {
                int                   h, v;
                NVCVChromaSubsampling css;
            } table[] = {{4, 4, NVCV_CSS_444}, {4, 2, NVCV_CSS_422R}, {4, 1, NVCV_CSS_411R}, {2, 4, NVCV_CSS_422},
                         {2, 2, NVCV_CSS_420}, {2, 1, NVCV_CSS_410R}, {1, 1, NVCV_CSS_444},  {1, 2, NVCV_CSS_410},
                         {1, 4, NVCV_CSS_411}};
            for (const auto &e : table)
            {
                if (e.h == samplesHoriz && e.v == samplesVert)
                {
                    *outCSS = e.css;
                    return;
                }
            }
            throw Error(NVCV_ERROR_INVALID_ARGUMENT,
                        "%d horizontal and %d vertical samples doesn't correspond to any supported chroma subsampling scheme",
                        samplesHoriz, samplesVert);
        });
}

// Colour spec word: space [0,3) xfer [3,7) encoding [7,10) horizontal / vertical chroma location [10,12) [12,14)
// range [14,15) (reference: detail/FormatUtils.h:34-37, priv/ColorSpec.cpp:41-95). No value is range-checked,
// here or there: components are truncated to their fields.
NVCVStatus nvcvMakeColorSpec(NVCVColorSpec *outColorSpec, NVCVColorSpace cspace, NVCVYCbCrEncoding encoding,
                             NVCVColorTransferFunction xferFunc, NVCVColorRange range, NVCVChromaLocation locHoriz,
                             NVCVChromaLocation locVert)
{
    return Protect(
        [&]
        {
            NotNull(outColorSpec, "Pointer to output colorspec");
            *outColorSpec = (NVCVColorSpec)(int32_t)NVCV_DETAIL_COLOR_SPEC_WORD(
                EnumValue(cspace), EnumValue(encoding), EnumValue(xferFunc), EnumValue(range), EnumValue(locHoriz),
                EnumValue(locVert));
        });
}

NVCVStatus nvcvColorSpecGetChromaLoc(NVCVColorSpec cspec, NVCVChromaLocation *outLocHoriz, NVCVChromaLocation *outLocVert)
{
    return Protect(
        [&]
        {
            if (outLocHoriz == nullptr && outLocVert == nullptr)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT,
                            "Pointer to output horizontal and vertical chroma location cannot both be NULL");
            }
            const uint64_t w = (uint32_t)EnumValue(cspec);
            if (outLocHoriz != nullptr)
            {
                *outLocHoriz = (NVCVChromaLocation)Get(w, 10, 2);
            }
            if (outLocVert != nullptr)
            {
                *outLocVert = (NVCVChromaLocation)Get(w, 12, 2);
            }
        });
}

NVCVStatus nvcvColorSpecSetChromaLoc(NVCVColorSpec *cspec, NVCVChromaLocation locHoriz, NVCVChromaLocation locVert)
{
    return SetSpecField(cspec, 10, 4, Put((uint64_t)EnumValue(locHoriz), 0, 2) | Put((uint64_t)EnumValue(locVert), 2, 2));
}

NVCVStatus nvcvColorSpecGetColorSpace(NVCVColorSpec cspec, NVCVColorSpace *outColorSpace)
{
    return GetSpecField(cspec, 0, 3, outColorSpace, "Pointer to output color space");
}

NVCVStatus nvcvColorSpecSetColorSpace(NVCVColorSpec *cspec, NVCVColorSpace cspace)
{
    return SetSpecField(cspec, 0, 3, (uint64_t)EnumValue(cspace));
}

NVCVStatus nvcvColorSpecGetYCbCrEncoding(NVCVColorSpec cspec, NVCVYCbCrEncoding *outEncoding)
{
    return GetSpecField(cspec, 7, 3, outEncoding, "Pointer to output YCbCr encoding");
}

NVCVStatus nvcvColorSpecSetYCbCrEncoding(NVCVColorSpec *cspec, NVCVYCbCrEncoding encoding)
{
    return SetSpecField(cspec, 7, 3, (uint64_t)EnumValue(encoding));
}

NVCVStatus nvcvColorSpecGetColorTransferFunction(NVCVColorSpec cspec, NVCVColorTransferFunction *outXferFunc)
{
    return GetSpecField(cspec, 3, 4, outXferFunc, "Pointer to output color transfer function");
}

NVCVStatus nvcvColorSpecSetColorTransferFunction(NVCVColorSpec *cspec, NVCVColorTransferFunction xferFunc)
{
    return SetSpecField(cspec, 3, 4, (uint64_t)EnumValue(xferFunc));
}

NVCVStatus nvcvColorSpecGetRange(NVCVColorSpec cspec, NVCVColorRange *outColorRange)
{
    return GetSpecField(cspec, 14, 1, outColorRange, "Pointer to output color range");
}

NVCVStatus nvcvColorSpecSetRange(NVCVColorSpec *cspec, NVCVColorRange range)
{
    return SetSpecField(cspec, 14, 1, (uint64_t)EnumValue(range));
}

NVCVStatus nvcvColorModelNeedsColorspec(NVCVColorModel cmodel, int8_t *outBool)
{
    return Protect(
        [&]
        {
            NotNull(outBool, "Pointer to output boolean");
            switch (EnumValue(cmodel))
            {
            case NVCV_COLOR_MODEL_YCbCr:
            case NVCV_COLOR_MODEL_RGB:
                *outBool = 1;
                return;
            case NVCV_COLOR_MODEL_UNDEFINED:
            case NVCV_COLOR_MODEL_RAW:
            case NVCV_COLOR_MODEL_XYZ:
            case NVCV_COLOR_MODEL_HSV:
            case NVCV_COLOR_MODEL_CMYK:
            case NVCV_COLOR_MODEL_YCCK:
                *outBool = 0;
                return;
            }
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Invalid color model: %d", EnumValue(cmodel));
        });
}

const char *nvcvColorSpaceGetName(NVCVColorSpace cspace)
{
    static const char *const n[] = {"NVCV_COLOR_SPACE_BT601", "NVCV_COLOR_SPACE_BT709", "NVCV_COLOR_SPACE_BT2020",
                                    "NVCV_COLOR_SPACE_DCIP3"};
    return EnumName(EnumValue(cspace), n, 4, "NVCVColorSpace");
}

const char *nvcvWhitePointGetName(NVCVWhitePoint wpoint)
{
    static const char *const n[] = {"NVCV_WHITE_POINT_D65"};
    return EnumName(EnumValue(wpoint), n, 1, "NVCVWhitePoint");
}

const char *nvcvYCbCrEncodingGetName(NVCVYCbCrEncoding enc)
{
    static const char *const n[] = {"NVCV_YCbCr_ENC_UNDEFINED", "NVCV_YCbCr_ENC_BT601",   "NVCV_YCbCr_ENC_BT709",
                                    "NVCV_YCbCr_ENC_BT2020",    "NVCV_YCbCr_ENC_BT2020c", "NVCV_YCbCr_ENC_SMPTE240M"};
    return EnumName(EnumValue(enc), n, 6, "NVCVYCbCrEncoding");
}

const char *nvcvColorTransferFunctionGetName(NVCVColorTransferFunction xfer)
{
    static const char *const n[] = {"NVCV_COLOR_XFER_LINEAR", "NVCV_COLOR_XFER_sRGB",  "NVCV_COLOR_XFER_sYCC",
                                    "NVCV_COLOR_XFER_PQ",     "NVCV_COLOR_XFER_BT709", "NVCV_COLOR_XFER_BT2020",
                                    "NVCV_COLOR_XFER_SMPTE240M"};
    return EnumName(EnumValue(xfer), n, 7, "NVCVColorTransferFunction");
}

const char *nvcvColorRangeGetName(NVCVColorRange range)
{
    static const char *const n[] = {"NVCV_COLOR_RANGE_FULL", "NVCV_COLOR_RANGE_LIMITED"};
    return EnumName(EnumValue(range), n, 2, "NVCVColorRange");
}

const char *nvcvChromaLocationGetName(NVCVChromaLocation loc)
{
    static const char *const n[] = {"NVCV_CHROMA_LOC_BOTH", "NVCV_CHROMA_LOC_EVEN", "NVCV_CHROMA_LOC_CENTER",
                                    "NVCV_CHROMA_LOC_ODD"};
    return EnumName(EnumValue(loc), n, 4, "NVCVChromaLocation");
}

const char *nvcvRawPatternGetName(NVCVRawPattern raw)
{
    static const char *const n[]
        = {"NVCV_RAW_BAYER_RGGB", "NVCV_RAW_BAYER_BGGR", "NVCV_RAW_BAYER_GRBG", "NVCV_RAW_BAYER_GBRG", "NVCV_RAW_BAYER_RCCB",
           "NVCV_RAW_BAYER_BCCR", "NVCV_RAW_BAYER_CRBC", "NVCV_RAW_BAYER_CBRC", "NVCV_RAW_BAYER_RCCC", "NVCV_RAW_BAYER_CRCC",
           "NVCV_RAW_BAYER_CCRC", "NVCV_RAW_BAYER_CCCR", "NVCV_RAW_BAYER_CCCC"};
    return EnumName(EnumValue(raw), n, 13, "NVCVRawPattern");
}

const char *nvcvColorSpecGetName(NVCVColorSpec cspec)
{
    // predefined specs by name; anything else by its components with the enumerators' common prefixes
    // shortened (reference: priv/ColorSpec.cpp:179-262). The reserved all-ones value gets both.
    static const struct
    {
        NVCVColorSpec spec;
        const char   *name;
    } predefined[] = {
#define CVAMD_SPEC(x) {x, #x}
        CVAMD_SPEC(NVCV_COLOR_SPEC_UNDEFINED),     CVAMD_SPEC(NVCV_COLOR_SPEC_MPEG2_BT601),
        CVAMD_SPEC(NVCV_COLOR_SPEC_MPEG2_BT709),   CVAMD_SPEC(NVCV_COLOR_SPEC_MPEG2_SMPTE240M),
        CVAMD_SPEC(NVCV_COLOR_SPEC_BT601),         CVAMD_SPEC(NVCV_COLOR_SPEC_BT601_ER),
        CVAMD_SPEC(NVCV_COLOR_SPEC_BT709),         CVAMD_SPEC(NVCV_COLOR_SPEC_BT709_ER),
        CVAMD_SPEC(NVCV_COLOR_SPEC_BT709_LINEAR),  CVAMD_SPEC(NVCV_COLOR_SPEC_BT2020),
        CVAMD_SPEC(NVCV_COLOR_SPEC_BT2020_ER),     CVAMD_SPEC(NVCV_COLOR_SPEC_BT2020_LINEAR),
        CVAMD_SPEC(NVCV_COLOR_SPEC_BT2020_PQ),     CVAMD_SPEC(NVCV_COLOR_SPEC_BT2020_PQ_ER),
        CVAMD_SPEC(NVCV_COLOR_SPEC_BT2020c),       CVAMD_SPEC(NVCV_COLOR_SPEC_BT2020c_ER),
        CVAMD_SPEC(NVCV_COLOR_SPEC_SMPTE240M),     CVAMD_SPEC(NVCV_COLOR_SPEC_sRGB),
        CVAMD_SPEC(NVCV_COLOR_SPEC_sYCC),          CVAMD_SPEC(NVCV_COLOR_SPEC_DISPLAYP3),
        CVAMD_SPEC(NVCV_COLOR_SPEC_DISPLAYP3_LINEAR),
#undef CVAMD_SPEC
    };
    const int value = EnumValue(cspec);
    for (const auto &e : predefined)
    {
        if ((int)e.spec == value)
        {
            return e.name;
        }
    }
    const uint64_t w = (uint32_t)value;
    auto           part = [](const char *full, const char *prefix, const char *shortened)
    {
        const size_t n = strlen(prefix);
        return strncmp(full, prefix, n) == 0 ? ThreadName("%s%s", shortened, full + n) : full;
    };
    // the ring behind ThreadName holds fewer strings than are needed here at once: copy each part
    char space[64], enc[64], xfer[64], range[64], loch[64], locv[64];
    snprintf(space, sizeof(space), "%s", part(nvcvColorSpaceGetName((NVCVColorSpace)Get(w, 0, 3)), "NVCV_COLOR_SPACE_", "SPACE_"));
    snprintf(enc, sizeof(enc), "%s", part(nvcvYCbCrEncodingGetName((NVCVYCbCrEncoding)Get(w, 7, 3)), "NVCV_YCbCr_", ""));
    snprintf(xfer, sizeof(xfer), "%s",
             part(nvcvColorTransferFunctionGetName((NVCVColorTransferFunction)Get(w, 3, 4)), "NVCV_COLOR_XFER_", "XFER_"));
    snprintf(range, sizeof(range), "%s", part(nvcvColorRangeGetName((NVCVColorRange)Get(w, 14, 1)), "NVCV_COLOR_RANGE_", "RANGE_"));
    snprintf(loch, sizeof(loch), "%s", part(nvcvChromaLocationGetName((NVCVChromaLocation)Get(w, 10, 2)), "NVCV_CHROMA_LOC_", "LOC_"));
    snprintf(locv, sizeof(locv), "%s", part(nvcvChromaLocationGetName((NVCVChromaLocation)Get(w, 12, 2)), "NVCV_CHROMA_LOC_", "LOC_"));
    return ThreadName("%sNVCVColorSpec(%s,%s,%s,%s,%s,%s)", value == (int)NVCV_COLOR_SPEC_FORCE32 ? "NVCVColorSpec(invalid)" : "",
                      space, enc, xfer, range, loch, locv);
}

// ---- data type ---------------------------------------------------------------------------------
NVCVStatus nvcvMakeDataType(NVCVDataType *outDataType, NVCVDataKind dataKind, NVCVPacking packing)
{
    return Protect([&]
                   { *NotNull(outDataType, "Pointer to output data type") = NVCV_DETAIL_MAKE_DATA_TYPE(dataKind, (uint64_t)packing); });
}

NVCVStatus nvcvDataTypeGetPacking(NVCVDataType type, NVCVPacking *outPacking)
{
    return Protect([&] { *NotNull(outPacking, "Pointer to output packing") = DataTypePacking(type); });
}

NVCVStatus nvcvDataTypeGetBitsPerPixel(NVCVDataType type, int32_t *outBPP)
{
    return Protect([&] { *NotNull(outBPP, "Pointer to output") = DecodePacking(DataTypePacking(type)).bitsPerPixel; });
}

NVCVStatus nvcvDataTypeGetBitsPerChannel(NVCVDataType type, int32_t *outBits)
{
    return nvcvPackingGetBitsPerComponent(DataTypePacking(type), outBits);
}

NVCVStatus nvcvDataTypeGetAlignment(NVCVDataType type, int32_t *outAlignment)
{
    return Protect([&] { *NotNull(outAlignment, "Pointer to output") = DataTypeAlignment(type); });
}

NVCVStatus nvcvDataTypeGetDataKind(NVCVDataType type, NVCVDataKind *outDataKind)
{
    return Protect([&] { *NotNull(outDataKind, "Pointer to output") = FormatDataKind(type); });
}

NVCVStatus nvcvDataTypeGetNumChannels(NVCVDataType type, int32_t *outNumChannels)
{
    return Protect([&]
                   { *NotNull(outNumChannels, "Pointer to output") = DecodePacking(DataTypePacking(type)).numChannels; });
}

NVCVStatus nvcvDataTypeGetChannelType(NVCVDataType type, int32_t channel, NVCVDataType *outChannelType)
{
    // reference: src/nvcv/src/priv/DataType.cpp:51-78. The type of one channel is the one-channel packing of that
    // many bits (10-, 12-, 14- and 20-bit channels: the form padded to the next word, X10b6 ...); a width no
    // one-channel packing has is an error, a channel the type does not have is NVCV_DATA_TYPE_NONE.
    return Protect(
        [&]
        {
            NotNull(outChannelType, "Pointer to output");
            if (channel < 0)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Channel must be >= 0, not %d", channel);
            }
            const PackingInfo pi   = DecodePacking(DataTypePacking(type));
            const int         bits = channel < 4 ? pi.bits[channel] : 0;
            if (bits == 0)
            {
                *outChannelType = NVCV_DATA_TYPE_NONE;
                return;
            }
            const int pad = (bits == 10 || bits == 12 || bits == 14) ? 16 - bits : bits == 20 ? 12 : 0;
            int       count;
            const PackingRow *rows = PackingTable(&count);
            for (int i = 0; i < count; ++i)
            {
                const PackingRow &r = rows[i];
                if (r.fields[0] == bits && r.fields[1] == pad && r.fields[2] == 0 && r.fields[3] == 0 && r.bits[0] == bits
                    && r.bits[1] == 0)
                {
                    *outChannelType = NVCV_DETAIL_MAKE_DATA_TYPE(FormatDataKind(type), (uint64_t)r.packing);
                    return;
                }
            }
            throw Error(NVCV_ERROR_INVALID_ARGUMENT, "No data type has one channel of %d bits", bits);
        });
}

NVCVStatus nvcvDataTypeGetStrideBytes(NVCVDataType type, int32_t *outStrideBytes)
{
    return Protect([&] { *NotNull(outStrideBytes, "Pointer to output") = DataTypeStrideBytes(type); });
}

const char *nvcvDataTypeGetName(NVCVDataType type)
{
    // the types the reference names (src/nvcv/src/priv/DataType.cpp:83-160); any other is spelled out
    static const struct
    {
        NVCVDataType type;
        const char  *name;
    } known[] = {
#define T(x) {NVCV_DATA_TYPE_##x, "NVCV_DATA_TYPE_" #x}
        T(NONE), T(U8),  T(2U8),  T(3U8),  T(4U8),  T(S8),  T(2S8),  T(3S8),  T(4S8),  T(U16), T(2U16), T(3U16), T(4U16),
        T(S16),  T(2S16), T(3S16), T(4S16), T(U32), T(2U32), T(3U32), T(4U32), T(S32), T(2S32), T(3S32), T(4S32), T(F16),
        T(2F16), T(3F16), T(4F16), T(F32), T(2F32), T(3F32), T(4F32), T(U64), T(2U64), T(3U64), T(4U64), T(S64), T(2S64),
        T(3S64), T(4S64), T(F64), T(2F64), T(3F64), T(4F64), T(C64), T(2C64), T(3C64), T(4C64), T(C128), T(2C128),
#undef T
    };
    for (const auto &k : known)
    {
        if (k.type == type)
        {
            return k.name;
        }
    }
    const char *kind = nvcvDataKindGetName(FormatDataKind(type));
    const char *pack = nvcvPackingGetName(DataTypePacking(type));
    // enumerator names without their common prefixes
    kind = std::strncmp(kind, "NVCV_DATA_KIND_", 15) == 0 ? kind + 15 : kind;
    pack = std::strncmp(pack, "NVCV_PACKING_", 13) == 0 ? pack + 13 : pack;
    return ThreadName("NVCVDataType(%s,%s)", kind, pack);
}

// ---- image format ------------------------------------------------------------------------------
NVCVStatus nvcvMakeYCbCrImageFormat(NVCVImageFormat *outFormat, NVCVColorSpec colorSpec,
                                    NVCVChromaSubsampling chromaSub, NVCVMemLayout memLayout, NVCVDataKind dataKind,
                                    NVCVSwizzle swizzle, NVCVPacking packing0, NVCVPacking packing1,
                                    NVCVPacking packing2, NVCVPacking packing3, NVCVAlphaType alphaType,
                                    const NVCVExtraChannelInfo *exChannelInfo)
{
    return MakeFormat(outFormat, NVCV_COLOR_MODEL_YCbCr, colorSpec, chromaSub, memLayout, dataKind, swizzle, packing0,
                      packing1, packing2, packing3, alphaType, exChannelInfo);
}

NVCVStatus nvcvMakeColorImageFormat(NVCVImageFormat *outFormat, NVCVColorModel colorModel, NVCVColorSpec colorSpec,
                                    NVCVMemLayout memLayout, NVCVDataKind dataKind, NVCVSwizzle swizzle,
                                    NVCVPacking packing0, NVCVPacking packing1, NVCVPacking packing2,
                                    NVCVPacking packing3, NVCVAlphaType alphaType,
                                    const NVCVExtraChannelInfo *exChannelInfo)
{
    if (colorModel == NVCV_COLOR_MODEL_RAW)
    {
        return Protect([&] { throw Error(NVCV_ERROR_INVALID_ARGUMENT, "Raw formats are made by nvcvMakeRawImageFormat"); });
    }
    return MakeFormat(outFormat, colorModel, colorSpec, NVCV_CSS_NONE, memLayout, dataKind, swizzle, packing0,
                      packing1, packing2, packing3, alphaType, exChannelInfo);
}

NVCVStatus nvcvMakeNonColorImageFormat(NVCVImageFormat *outFormat, NVCVMemLayout memLayout, NVCVDataKind dataKind,
                                       NVCVSwizzle swizzle, NVCVPacking packing0, NVCVPacking packing1,
                                       NVCVPacking packing2, NVCVPacking packing3, NVCVAlphaType alphaType,
                                       const NVCVExtraChannelInfo *exChannelInfo)
{
    return MakeFormat(outFormat, NVCV_COLOR_MODEL_UNDEFINED, NVCV_COLOR_SPEC_UNDEFINED, NVCV_CSS_NONE, memLayout, dataKind, swizzle, packing0,
                      packing1, packing2, packing3, alphaType, exChannelInfo);
}

NVCVStatus nvcvImageFormatGetNumPlanes(NVCVImageFormat fmt, int32_t *outNumPlanes)
{
    return Protect([&] { *NotNull(outNumPlanes, "Pointer to output") = FormatNumPlanes(fmt); });
}

NVCVStatus nvcvImageFormatGetNumChannels(NVCVImageFormat fmt, int32_t *outNumChannels)
{
    return Protect([&] { *NotNull(outNumChannels, "Pointer to output") = FormatNumChannels(fmt); });
}

NVCVStatus nvcvImageFormatGetBitsPerChannel(NVCVImageFormat fmt, int32_t *bits)
{
    return Protect(
        [&]
        {
            NotNull(bits, "Pointer to output");
            int n = 0;
            for (int p = 0; p < 4; ++p)
            {
                NVCVPacking pk = FormatPlanePacking(fmt, p);
                PackingInfo pi = DecodePacking(pk);
                if (!pi.known)
                {
                    throw Error(NVCV_ERROR_INVALID_IMAGE_FORMAT, "Plane %d has an unknown packing", p);
                }
                if (pk == NVCV_PACKING_X8_Y8__X8_Z8 || pk == NVCV_PACKING_Y8_X8__Z8_X8)
                {
                    pi.bits[3] = 0; // the luma sample stored twice counts once
                }
                for (int c = 0; c < 4 && pi.bits[c] != 0; ++c)
                {
                    if (n >= 4)
                    {
                        throw Error(NVCV_ERROR_INVALID_IMAGE_FORMAT, "Planes hold more than 4 channels in total");
                    }
                    bits[n++] = pi.bits[c];
                }
            }
            for (; n < 4; ++n)
            {
                bits[n] = 0;
            }
        });
}

NVCVStatus nvcvImageFormatGetPlanePacking(NVCVImageFormat fmt, int32_t plane, NVCVPacking *outPacking)
{
    return Protect(
        [&]
        {
            *NotNull(outPacking, "Pointer to output") = FormatPlanePacking(fmt, plane);
        });
}

NVCVStatus nvcvImageFormatGetPlaneNumChannels(NVCVImageFormat fmt, int32_t plane, int32_t *outPlaneNumChannels)
{
    return Protect(
        [&]
        {
            *NotNull(outPlaneNumChannels, "Pointer to output") = DecodePacking(FormatPlanePacking(fmt, plane)).numChannels;
        });
}

NVCVStatus nvcvImageFormatGetPlaneBitsPerPixel(NVCVImageFormat fmt, int32_t plane, int32_t *outBPP)
{
    return Protect(
        [&]
        {
            *NotNull(outBPP, "Pointer to output") = DecodePacking(FormatPlanePacking(fmt, plane)).bitsPerPixel;
        });
}

NVCVStatus nvcvImageFormatGetPlanePixelStrideBytes(NVCVImageFormat fmt, int32_t plane, int32_t *outStrideBytes)
{
    return Protect(
        [&]
        {
            *NotNull(outStrideBytes, "Pointer to output") = FormatPlanePixelStrideBytes(fmt, plane);
        });
}

NVCVStatus nvcvImageFormatGetPlaneDataType(NVCVImageFormat fmt, int32_t plane, NVCVDataType *outDataType)
{
    return Protect(
        [&]
        {
            *NotNull(outDataType, "Pointer to output") = FormatPlaneDataType(fmt, plane);
        });
}

NVCVStatus nvcvImageFormatGetPlaneSize(NVCVImageFormat fmt, int32_t plane, int32_t imgWidth, int32_t imgHeight,
                                       int32_t *outPlaneWidth, int32_t *outPlaneHeight)
{
    return Protect(
        [&]
        {
            if (outPlaneWidth == nullptr && outPlaneHeight == nullptr)
            {
                throw Error(NVCV_ERROR_INVALID_ARGUMENT, "At least one of the two size outputs must be non-NULL");
            }
            int32_t w, h;
            FormatPlaneSize(fmt, plane, imgWidth, imgHeight, &w, &h);
            if (outPlaneWidth)
            {
                *outPlaneWidth = w;
            }
            if (outPlaneHeight)
            {
                *outPlaneHeight = h;
            }
        });
}

NVCVStatus nvcvImageFormatGetDataKind(NVCVImageFormat fmt, NVCVDataKind *outDataKind)
{
    return Protect([&] { *NotNull(outDataKind, "Pointer to output") = FormatDataKind(fmt); });
}

NVCVStatus nvcvImageFormatGetSwizzle(NVCVImageFormat fmt, NVCVSwizzle *outSwizzle)
{
    return Protect([&] { *NotNull(outSwizzle, "Pointer to output") = FormatSwizzle(fmt); });
}

NVCVStatus nvcvImageFormatGetMemLayout(NVCVImageFormat fmt, NVCVMemLayout *outMemLayout)
{
    return Protect([&] { *NotNull(outMemLayout, "Pointer to output") = FormatMemLayout(fmt); });
}

NVCVStatus nvcvImageFormatGetColorSpec(NVCVImageFormat fmt, NVCVColorSpec *outColorSpec)
{
    return Protect([&] { *NotNull(outColorSpec, "Pointer to output") = FormatColorSpec(fmt); });
}

NVCVStatus nvcvImageFormatGetColorModel(NVCVImageFormat fmt, NVCVColorModel *outColorModel)
{
    return Protect([&] { *NotNull(outColorModel, "Pointer to output") = FormatColorModel(fmt); });
}

NVCVStatus nvcvImageFormatGetChromaSubsampling(NVCVImageFormat fmt, NVCVChromaSubsampling *outCSS)
{
    return Protect([&] { *NotNull(outCSS, "Pointer to output") = FormatCSS(fmt); });
}

NVCVStatus nvcvImageFormatGetAlphaType(NVCVImageFormat fmt, NVCVAlphaType *outAlphaType)
{
    return Protect([&] { *NotNull(outAlphaType, "Pointer to output") = (NVCVAlphaType)NVCV_DETAIL_BITS_GET(fmt, 6, 1); });
}

NVCVStatus nvcvImageFormatHasSameDataLayout(NVCVImageFormat a, NVCVImageFormat b, int8_t *outBool)
{
    return Protect(
        [&]
        {
            NotNull(outBool, "Pointer to output");
            bool same = FormatNumPlanes(a) == FormatNumPlanes(b) && FormatCSS(a) == FormatCSS(b)
                     && FormatMemLayout(a) == FormatMemLayout(b) && FormatDataKind(a) == FormatDataKind(b);
            for (int p = 0; same && p < 4; ++p)
            {
                same = FormatPlanePacking(a, p) == FormatPlanePacking(b, p);
            }
            *outBool = same ? 1 : 0;
        });
}

const char *nvcvImageFormatGetName(NVCVImageFormat fmt)
{
    // The formats the reference names (src/nvcv/src/priv/ImageFormat.cpp:1218-1290); every other value, other named
    // constants included, is spelled out field by field.
    static const struct
    {
        NVCVImageFormat fmt;
        const char     *name;
    } known[] = {
#define F(x) {NVCV_IMAGE_FORMAT_##x, "NVCV_IMAGE_FORMAT_" #x}
        F(NONE),       F(U8),         F(U8_BL),      F(S8),         F(U16),        F(S16),      F(S16_BL),
        F(U32),        F(S32),        F(Y8),         F(Y8_BL),      F(Y8_ER),      F(Y8_ER_BL), F(Y16),
        F(Y16_BL),     F(Y16_ER),     F(Y16_ER_BL),  F(NV12),       F(NV12_BL),    F(NV12_ER),  F(NV12_ER_BL),
        F(NV24),       F(NV24_BL),    F(NV24_ER),    F(NV24_ER_BL), F(RGB8),       F(RGBA8),    F(BGR8),
        F(BGRA8),      F(F32),        F(F64),        F(2S16),       F(2S16_BL),    F(2F32),     F(C64),
        F(2C64),       F(C128),       F(2C128),      F(UYVY),       F(UYVY_BL),    F(UYVY_ER),  F(UYVY_ER_BL),
        F(VYUY),       F(VYUY_BL),    F(VYUY_ER),    F(VYUY_ER_BL), F(YUYV),       F(YUYV_BL),  F(YUYV_ER),
        F(YUYV_ER_BL), F(YUV8p),      F(YUV8p_ER),   F(RGB8_1U_U8), F(RGB8_7U_U8), F(RGBA8_3U_U16),
        F(RGBA8_3POS3D_U32), F(RGB8_3D_F32), F(YCCK8), F(CMYK8),   F(HSV8),       F(RGBAf32),  F(RGBAf32p),
#undef F
    };
    for (const auto &k : known)
    {
        if (k.fmt == fmt)
        {
            return k.name;
        }
    }
    std::string          text  = "NVCVImageFormat(";
    const NVCVColorModel model = FormatColorModel(fmt);
    text += nvcvColorModelGetName(model);
    text += ",";
    if (model == NVCV_COLOR_MODEL_RAW)
    {
        text += nvcvRawPatternGetName((NVCVRawPattern)FormatRawPattern(fmt));
        text += ",";
    }
    else if (model != NVCV_COLOR_MODEL_UNDEFINED)
    {
        text += nvcvColorSpecGetName(FormatColorSpec(fmt));
        text += ",";
        if (model == NVCV_COLOR_MODEL_YCbCr)
        {
            text += nvcvChromaSubsamplingGetName(FormatCSS(fmt));
            text += ",";
        }
    }
    text += nvcvMemLayoutGetName(FormatMemLayout(fmt));
    text += ",";
    text += nvcvDataKindGetName(FormatDataKind(fmt));
    text += ",";
    text += nvcvSwizzleGetName(FormatSwizzle(fmt));
    text += FormatAlphaType(fmt) == NVCV_ALPHA_ASSOCIATED ? ",ASSOCIATED" : ",UNASSOCIATED";
    const NVCVExtraChannelInfo ex = FormatExtraChannels(fmt);
    if (ex.numChannels > 0)
    {
        static const char *const types[] = {"U", "D", "POS3D"};
        text += "," + std::to_string(ex.numChannels) + "," + std::to_string(ex.bitsPerPixel) + ",";
        text += nvcvDataKindGetName(ex.datakind);
        text += ",";
        text += EnumName((int)ex.channelType, types, 3, "NVCVExtraChannel");
    }
    for (int p = 0; p < FormatNumPlanes(fmt); ++p)
    {
        text += ",";
        text += nvcvPackingGetName(FormatPlanePacking(fmt, p));
    }
    text += ")";
    // enumerator names appear without their common prefixes
    for (const char *prefix : {"NVCV_RAW_", "NVCV_COLOR_MODEL_", "NVCV_COLOR_SPEC_", "NVCV_CSS_", "NVCV_MEM_LAYOUT_", "NVCV_DATA_KIND_",
                               "NVCV_PACKING_", "NVCV_CHROMA_", "NVCV_YCbCr_", "NVCV_COLOR_", "NVCV_ALPHA_", "NVCV_EXTRA_CHANNEL_"})
    {
        const size_t n = std::strlen(prefix);
        for (size_t at = text.find(prefix); at != std::string::npos; at = text.find(prefix, at))
        {
            text.erase(at, n);
        }
    }
    return ThreadName("%s", text.c_str());
}
}
