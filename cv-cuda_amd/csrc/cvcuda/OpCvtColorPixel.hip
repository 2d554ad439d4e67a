// Per-pixel colour conversion families of CvtColor.
//
// Arithmetic follows the reference's device functions in src/cvcuda/priv/legacy/cvt_color.cu, in
// float32 without FMA contraction where it is floating point:
//   gray       :34-43, 250-274 (15-bit fixed point for integers), gray -> BGR :232-248
//   YUV 4:4:4  :45-62, 276-301 and :324-346 (14-bit fixed point, delta = half range)
//   HSV        :368-413 (u8: 12-bit reciprocal tables computed on the fly; f32: FLT_EPSILON in the
//              denominators) and :436-503
//   RGB -> YUV 4:2:0 :70-78, 598-615 (chroma taken from the top-left pixel of each 2x2 block), layout :567-596
//   YUV 4:2:2 -> RGB / gray :676-759
// Validation follows the corresponding host functions (:855-1360, 1551-1766); every failure is
// INVALID_ARGUMENT.
//
// Kernel shape: one lane per work item, 64 items x 4 rows per block; an item is one pixel, or the
// 2x1 / 2x2 pixel group that shares chroma in the subsampled formats. Whole pixels move as one
// vector access, streaming stores. Var-shape batches use the packed tile grid.
#include "CvtColorFamilies.hpp"
#include "DeviceUtils.hpp"
#include "RunIO.hpp"
#include "VarShapeTiles.hpp"

#include <algorithm>
#include <cfloat>

namespace cvamd {

namespace {

struct PixArgs
{
    const uint8_t *src;
    uint8_t       *dst;
    int64_t        srcN, dstN;
    int32_t        srcRow, dstRow;
    int32_t        W, H; // size of the colour image in pixels (tensor form)
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
    int32_t bidx, uidx, yidx, full;
};

template<class T, int C>
using Px = Packed<T, C>;

template<class T, int C>
__device__ __forceinline__ void StorePx(uint8_t *row, int x, const Px<T, C> &p)
{
    Px<T, C> *o = reinterpret_cast<Px<T, C> *>(row) + x;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        __builtin_nontemporal_store(p.v[c], &o->v[c]);
    }
}

template<class T>
__device__ __forceinline__ T AlphaOf()
{
    if constexpr (std::is_floating_point_v<T>)
    {
        return (T)1;
    }
    else
    {
        return std::numeric_limits<T>::max();
    }
}

__device__ __forceinline__ int Descale(int x, int n)
{
    return (x + (1 << (n - 1))) >> n;
}

template<class T>
__device__ __forceinline__ T SatInt(int v)
{
    return (T)min(max(v, 0), (int)std::numeric_limits<T>::max());
}

// ---- image view handed to the operations -----------------------------------------------------------
struct View
{
    const uint8_t *src;
    uint8_t       *dst;
    int32_t        srcRow, dstRow;
    int32_t        W, H; // pixels of the colour image
};

// ---- operations: Op::kItemW x Op::kItemH pixels per work item -----------------------------------------
template<class T, int SCH>
struct GrayFromBgr
{
    static constexpr int kItemW = 1, kItemH = 1;
    using Src = Px<T, SCH>;

    static __device__ __forceinline__ auto Map(const Src &s, const PixArgs &a)
    {
        const T          b = a.bidx ? s.v[2] : s.v[0], g = s.v[1], r = a.bidx ? s.v[0] : s.v[2];
        Px<T, 1>         o;
        if constexpr (std::is_integral_v<T>)
        {
            o.v[0] = (T)Descale((int)b * 3735 + (int)g * 19235 + (int)r * 9798, 15);
        }
        else
        {
            o.v[0] = b * 0.114f + g * 0.587f + r * 0.299f;
        }
        return o;
    }
};

template<class T, int DCH>
struct BgrFromGray
{
    static constexpr int kItemW = 1, kItemH = 1;
    using Src = Px<T, 1>;

    static __device__ __forceinline__ auto Map(const Src &s, const PixArgs &)
    {
        const T    g = s.v[0];
        Px<T, DCH> o;
#pragma unroll
        for (int c = 0; c < DCH; ++c)
        {
            o.v[c] = g;
        }
        return o;
    }
};

template<class T>
struct YuvFromBgr
{
    static constexpr int kItemW = 1, kItemH = 1;
    using Src = Px<T, 3>;

    static __device__ __forceinline__ auto Map(const Src &s, const PixArgs &a)
    {
        Px<T, 3>       o;
        if constexpr (std::is_integral_v<T>)
        {
            constexpr int delta = ((int)(std::numeric_limits<T>::max() / 2 + 1)) << 14;
            const int     B = a.bidx ? s.v[2] : s.v[0], G = s.v[1], R = a.bidx ? s.v[0] : s.v[2];
            const int     Y  = Descale(R * 4899 + G * 9617 + B * 1868, 14);
            const int     Cr = Descale((R - Y) * 14369 + delta, 14);
            const int     Cb = Descale((B - Y) * 8061 + delta, 14);
            o.v[0]           = SatInt<T>(Y);
            o.v[1]           = SatInt<T>(Cb);
            o.v[2]           = SatInt<T>(Cr);
        }
        else
        {
            const float B = a.bidx ? s.v[2] : s.v[0], G = s.v[1], R = a.bidx ? s.v[0] : s.v[2];
            const float Y = R * 0.299f + G * 0.587f + B * 0.114f;
            o.v[0]        = Y;
            o.v[2]        = (R - Y) * 0.877f + 0.5f;
            o.v[1]        = (B - Y) * 0.492f + 0.5f;
        }
        return o;
    }
};

template<class T>
struct BgrFromYuv
{
    static constexpr int kItemW = 1, kItemH = 1;
    using Src = Px<T, 3>;

    static __device__ __forceinline__ auto Map(const Src &s, const PixArgs &a)
    {
        Px<T, 3>       o;
        T              b, g, r;
        if constexpr (std::is_integral_v<T>)
        {
            constexpr int delta = (int)(std::numeric_limits<T>::max() / 2 + 1);
            const int     Y = s.v[0], Cb = s.v[1], Cr = s.v[2];
            b = SatInt<T>(Y + Descale((Cb - delta) * 33292, 14));
            g = SatInt<T>(Y + Descale((Cb - delta) * -6472 + (Cr - delta) * -9519, 14));
            r = SatInt<T>(Y + Descale((Cr - delta) * 18678, 14));
        }
        else
        {
            const float Y = s.v[0], Cb = s.v[1], Cr = s.v[2];
            b = Y + (Cb - 0.5f) * 2.032f;
            g = Y + (Cb - 0.5f) * -0.395f + (Cr - 0.5f) * -0.581f;
            r = Y + (Cr - 0.5f) * 1.140f;
        }
        o.v[0] = a.bidx ? r : b;
        o.v[1] = g;
        o.v[2] = a.bidx ? b : r;
        return o;
    }
};

// The two quotients of the integer HSV formula, (hrange << 12) / (6 i) and (255 << 12) / i for i in [0, 256),
// rounded to nearest: a table in the reference (cvt_color.cu:232-270, filled on the host). Here each block
// fills its own copy in LDS, one entry of each per thread, so a pixel costs two LDS reads instead of two
// float divisions (which are a dozen instructions each).
// a * b + c for factors of at most 24 significant bits (sign included) whose product fits 32 bits: one full-rate
// instruction. The compiler picks it by itself only where it can see the factors' ranges, which it cannot for
// values read from a table; its 32-bit multiply-add issues at a quarter of the rate.
__device__ __forceinline__ int MulAdd24(int a, int b, int c)
{
    int r;
    asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

__device__ __forceinline__ int32_t *HsvDivTable()
{
    __shared__ int32_t table[512];
    return table;
}

// RED_FIRST: the source pixel is R, G, B (the order is a template parameter: chosen per pixel it cost two selects
// and two masks of the 42 instructions an 8-bit pixel takes).
template<class T, bool RED_FIRST = false>
struct HsvFromBgr
{
    static constexpr int kItemW = 1, kItemH = 1;
    using Src = Px<T, 3>;
    static constexpr bool kBlockPrepare = std::is_integral_v<T>;

    // called by every thread of a 256-thread block before any of them returns
    static __device__ __forceinline__ void Prepare(const PixArgs &a)
    {
        if constexpr (kBlockPrepare)
        {
            const int hrange = a.full ? 256 : 180;
            const int i      = threadIdx.x;
            int32_t  *t      = HsvDivTable();
            t[i]             = i == 0 ? 0 : SaturateCast<int32_t>((float)(255 << 12) / (float)i);
            t[256 + i]       = i == 0 ? 0 : SaturateCast<int32_t>((float)(hrange << 12) / (6.f * i));
            __syncthreads();
        }
    }

    static __device__ __forceinline__ auto Map(const Src &s, const PixArgs &a)
    {
        Px<T, 3>       o;
        if constexpr (std::is_integral_v<T>)
        {
            const int hrange = a.full ? 256 : 180;
            const int b = RED_FIRST ? s.v[2] : s.v[0], g = s.v[1], r = RED_FIRST ? s.v[0] : s.v[2];
            const int vmin = min(b, min(g, r));
            const int val  = max(b, max(g, r));
            const int diff = val - vmin;
            const int vr = val == r ? -1 : 0, vg = val == g ? -1 : 0;
            const int32_t *table = HsvDivTable();
            const int      hdiv  = table[256 + diff];
            const int      sdiv  = table[val];
            // both products have factors of under 24 bits (|h| <= 5 * 255, quotients <= 255 << 12) and fit 32 bits:
            // the 24-bit multiply is exact here and issues at full rate, the 32-bit one at a quarter of it
            const int sat  = (MulAdd24(diff, sdiv, 1 << 11)) >> 12;
            int       h    = (vr & (g - b)) + (~vr & ((vg & (b - r + 2 * diff)) + ((~vg) & (r - g + 4 * diff))));
            h              = (MulAdd24(h, hdiv, 1 << 11)) >> 12;
            h += h < 0 ? hrange : 0;
            o.v[0] = SatInt<T>(h);
            o.v[1] = (T)sat;
            o.v[2] = (T)val;
        }
        else
        {
            const float b = RED_FIRST ? s.v[2] : s.v[0], g = s.v[1], r = RED_FIRST ? s.v[0] : s.v[2];
            const float vmin = fminf(r, fminf(g, b));
            const float val  = fmaxf(r, fmaxf(g, b));
            float       diff = val - vmin;
            const float sat  = diff / (fabsf(val) + FLT_EPSILON);
            diff             = 60.f / (diff + FLT_EPSILON);
            float h;
            if (val == r)
            {
                h = (g - b) * diff;
            }
            else if (val == g)
            {
                h = (b - r) * diff + 120.f;
            }
            else
            {
                h = (r - g) * diff + 240.f;
            }
            if (h < 0.f)
            {
                h += 360.f;
            }
            o.v[0] = h;
            o.v[1] = sat;
            o.v[2] = val;
        }
        return o;
    }
};

__device__ __forceinline__ float Select4(float t0, float t1, float t2, float t3, int idx)
{
    float out = idx == 1 ? t1 : t0;
    out       = idx == 2 ? t2 : out;
    out       = idx == 3 ? t3 : out;
    return out;
}

__device__ __forceinline__ void HsvToBgrFloat(float h, float s, float v, float &b, float &g, float &r)
{
    // the three constants say which of the four candidates each channel takes in each of the six hue
    // sectors, 4 bits per sector; zero saturation gives grey whatever the hue
    h += 6 * (h < 0);
    int idx = (int)h; // sector
    h -= idx;         // fraction inside the sector
    idx = (idx % 6) << 2;
    const float t0 = v, t1 = v * (1 - s), t2 = v * (1 - s * h), t3 = v * (1 - s * (1 - h));
    const bool  grey = s == 0;
    b = grey ? v : Select4(t0, t1, t2, t3, (0x00200311 >> idx) & 0xf);
    g = grey ? v : Select4(t0, t1, t2, t3, (0x00112003 >> idx) & 0xf);
    r = grey ? v : Select4(t0, t1, t2, t3, (0x00031120 >> idx) & 0xf);
}

template<class T, int DCH>
struct BgrFromHsv
{
    static constexpr int kItemW = 1, kItemH = 1;
    using Src = Px<T, 3>;

    static __device__ __forceinline__ auto Map(const Src &s, const PixArgs &a)
    {
        Px<T, DCH>     o;
        T              b, g, r;
        if constexpr (std::is_integral_v<T>)
        {
            const float scaleH = a.full ? (6.0f / 256.0f) : (6.0f / 180.0f);
            float       bf, gf, rf;
            HsvToBgrFloat((float)s.v[0] * scaleH, s.v[1] * (1.0f / 255.0f), s.v[2] * (1.0f / 255.0f), bf, gf, rf);
            b = SaturateCast<T>(bf * 255.0f);
            g = SaturateCast<T>(gf * 255.0f);
            r = SaturateCast<T>(rf * 255.0f);
        }
        else
        {
            HsvToBgrFloat(s.v[0] * (6.0f / 360.0f), s.v[1], s.v[2], b, g, r);
        }
        o.v[0] = a.bidx ? r : b;
        o.v[1] = g;
        o.v[2] = a.bidx ? b : r;
        if constexpr (DCH == 4)
        {
            o.v[3] = AlphaOf<T>();
        }
        return o;
    }
};

// u8 RGB(A) -> Y, U, V of BT.601 limited range in 20-bit fixed point
__device__ __forceinline__ void BgrToYuv420(int b, int g, int r, uint8_t &Y, uint8_t &U, uint8_t &V)
{
    const int half = 1 << 19;
    const int yy   = 269484 * r + 528482 * g + 102760 * b + half + (16 << 20);
    const int uu   = -155188 * r + -305135 * g + 460324 * b + half + (128 << 20);
    const int vv   = 460324 * r + -385875 * g + -74448 * b + half + (128 << 20);
    Y              = SatInt<uint8_t>(yy >> 20);
    U              = SatInt<uint8_t>(uu >> 20);
    V              = SatInt<uint8_t>(vv >> 20);
}

// one work item = a 2x2 pixel block: four lumas, chroma of its top-left pixel
template<int SCH, bool SEMIPLANAR>
struct Yuv420FromBgr
{
    static constexpr int  kItemW = 2, kItemH = 2;
    static constexpr bool kSizeFromSrc = true; // the colour image is the input

    static __device__ __forceinline__ void Run(const View &v, const PixArgs &a, int ix, int iy)
    {
        const int x = ix * 2, y = iy * 2;
        uint8_t   U = 0, V = 0;
#pragma unroll
        for (int r = 0; r < 2; ++r)
        {
            const Px<uint8_t, 2 * SCH> s
                = *reinterpret_cast<const Px<uint8_t, 2 * SCH> *>(v.src + (int64_t)(y + r) * v.srcRow + x * SCH);
            uint8_t Y0, Y1, u, w;
            BgrToYuv420(a.bidx ? s.v[2] : s.v[0], s.v[1], a.bidx ? s.v[0] : s.v[2], Y0, u, w);
            if (r == 0)
            {
                U = u;
                V = w;
            }
            BgrToYuv420(a.bidx ? s.v[SCH + 2] : s.v[SCH], s.v[SCH + 1], a.bidx ? s.v[SCH] : s.v[SCH + 2], Y1, u, w);
            __builtin_nontemporal_store((uint16_t)(Y0 | (Y1 << 8)),
                                        reinterpret_cast<uint16_t *>(v.dst + (int64_t)(y + r) * v.dstRow + x));
        }
        if constexpr (SEMIPLANAR)
        {
            uint8_t *uv = v.dst + (int64_t)(v.H + iy) * v.dstRow + x;
            const uint32_t pair = a.uidx == 0 ? (U | (V << 8)) : (V | (U << 8));
            __builtin_nontemporal_store((uint16_t)pair, reinterpret_cast<uint16_t *>(uv));
        }
        else
        {
            // each chroma plane is (H/2) x (W/2), stored as H/4 rows of W bytes after the luma rows
            const int h4  = v.H >> 2;
            const int uvx = ix + ((v.W >> 1) & -(iy & 1));
            v.dst[(int64_t)(v.H + (y >> 2) + h4 * a.uidx) * v.dstRow + uvx]       = U;
            v.dst[(int64_t)(v.H + (y >> 2) + h4 * (a.uidx ^ 1)) * v.dstRow + uvx] = V;
        }
    }

    // kGroup blocks side by side: 8 x 2 pixels, whole-dword stores on every plane
    static constexpr int kGroup = 4;

    static __device__ __forceinline__ void RunGroup(const View &v, const PixArgs &a, int ix, int iy)
    {
        constexpr int P = 2 * kGroup;
        const int     x = ix * 2, y = iy * 2;
        uint8_t       U[kGroup], V[kGroup];
#pragma unroll
        for (int r = 0; r < 2; ++r)
        {
            uint8_t  s[P * SCH], Y[P];
            uint32_t w[P * SCH / 4];
            LoadDwords<P * SCH / 4>(v.src + (int64_t)(y + r) * v.srcRow + x * SCH, w);
            __builtin_memcpy(s, w, sizeof(s));
#pragma unroll
            for (int k = 0; k < P; ++k)
            {
                uint8_t u, w;
                BgrToYuv420(a.bidx ? s[k * SCH + 2] : s[k * SCH], s[k * SCH + 1], a.bidx ? s[k * SCH] : s[k * SCH + 2],
                            Y[k], u, w);
                if (r == 0 && (k & 1) == 0)
                {
                    U[k >> 1] = u;
                    V[k >> 1] = w;
                }
            }
            StoreRunNT<uint8_t, P>(v.dst + (int64_t)(y + r) * v.dstRow + x, Y);
        }
        if constexpr (SEMIPLANAR)
        {
            uint8_t uv[P];
#pragma unroll
            for (int k = 0; k < kGroup; ++k)
            {
                uv[2 * k]     = a.uidx == 0 ? U[k] : V[k];
                uv[2 * k + 1] = a.uidx == 0 ? V[k] : U[k];
            }
            StoreRunNT<uint8_t, P>(v.dst + (int64_t)(v.H + iy) * v.dstRow + x, uv);
        }
        else
        {
            const int h4  = v.H >> 2;
            const int uvx = ix + ((v.W >> 1) & -(iy & 1));
            StoreRunNT<uint8_t, kGroup>(v.dst + (int64_t)(v.H + (y >> 2) + h4 * a.uidx) * v.dstRow + uvx, U);
            StoreRunNT<uint8_t, kGroup>(v.dst + (int64_t)(v.H + (y >> 2) + h4 * (a.uidx ^ 1)) * v.dstRow + uvx, V);
        }
    }
};

__device__ __forceinline__ void Yuv42xToBgr(int Y, int U, int V, uint8_t &b, uint8_t &g, uint8_t &r)
{
    const int yy = max(0, Y - 16) * 1220542, uu = U - 128, vv = V - 128;
    r            = SatInt<uint8_t>(Descale(yy + 1673527 * vv, 20));
    g            = SatInt<uint8_t>(Descale(yy + -852492 * vv + -409993 * uu, 20));
    b            = SatInt<uint8_t>(Descale(yy + 2116026 * uu, 20));
}

// one work item = 2 pixels = 4 source bytes (Y0 U Y1 V in some order)
template<int DCN>
struct BgrFromYuv422
{
    static constexpr int  kItemW = 2, kItemH = 1;
    static constexpr bool kSizeFromSrc = false;

    // the 2 pixels of source dword q to o[0 .. 2 * DCN)
    static __device__ __forceinline__ void Convert(uint32_t q, const PixArgs &a, uint8_t *o)
    {
        const int Y0 = (q >> (8 * a.yidx)) & 0xFF, Y1 = (q >> (8 * (a.yidx + 2))) & 0xFF;
        const int U = (q >> (8 * ((a.yidx ^ 1) + a.uidx))) & 0xFF, V = (q >> (8 * ((a.yidx ^ 1) + (a.uidx ^ 2)))) & 0xFF;
#pragma unroll
        for (int k = 0; k < 2; ++k)
        {
            uint8_t b, g, r;
            Yuv42xToBgr(k == 0 ? Y0 : Y1, U, V, b, g, r);
            o[k * DCN + 0] = a.bidx ? r : b;
            o[k * DCN + 1] = g;
            o[k * DCN + 2] = a.bidx ? b : r;
            if constexpr (DCN == 4)
            {
                o[k * DCN + 3] = 255;
            }
        }
    }

    static __device__ __forceinline__ void Run(const View &v, const PixArgs &a, int ix, int y)
    {
        const uint32_t       q = *reinterpret_cast<const uint32_t *>(v.src + (int64_t)y * v.srcRow + ix * 4);
        Px<uint8_t, 2 * DCN> o;
        Convert(q, a, o.v);
        StorePx<uint8_t, 2 * DCN>(v.dst + (int64_t)y * v.dstRow, ix, o);
    }

    // 8 pixels: 16 source bytes in one load, 24 or 32 bytes out. Pieces that long are regrouped over the wave
    // so that every store instruction writes one dense span (4 pixels per lane, 8 bytes in and 12 out as
    // they are, ran at 0.57 of the memory rate).
    static constexpr int  kGroup    = 4;
    static constexpr bool kRowStore = true;

    // lanes 0 .. lanes-1 of the wave hold consecutive groups of row y, this one is `lane`. The chroma terms
    // of Yuv42xToBgr's three sums and its rounding constant are formed once per chroma pair, already in output
    // channel order; integer addition is associative, so the results are the same.
    static __device__ __forceinline__ void RunGroupInRow(const View &v, const PixArgs &a, int ix, int y, int lane, int lanes)
    {
        uint32_t q[kGroup];
        LoadDwords<kGroup>(v.src + (int64_t)y * v.srcRow + ix * 4, q);
        uint8_t   o[kGroup * 2 * DCN];
        const int shY = 8 * a.yidx, shU = 8 * ((a.yidx ^ 1) + a.uidx), shV = 8 * ((a.yidx ^ 1) + (a.uidx ^ 2));
#pragma unroll
        for (int g = 0; g < kGroup; ++g)
        {
            const int uu = (int)((q[g] >> shU) & 0xFF) - 128, vv = (int)((q[g] >> shV) & 0xFF) - 128;
            const int rC = 1673527 * vv + (1 << 19), bC = 2116026 * uu + (1 << 19);
            const int c0 = a.bidx ? rC : bC, c1 = -852492 * vv - 409993 * uu + (1 << 19), c2 = a.bidx ? bC : rC;
#pragma unroll
            for (int k = 0; k < 2; ++k)
            {
                const int t  = max(0, (int)((q[g] >> (shY + 16 * k)) & 0xFF) - 16) * 1220542;
                uint8_t  *px = o + (g * 2 + k) * DCN;
                px[0]        = (uint8_t)min(max((t + c0) >> 20, 0), 255);
                px[1]        = (uint8_t)min(max((t + c1) >> 20, 0), 255);
                px[2]        = (uint8_t)min(max((t + c2) >> 20, 0), 255);
                if constexpr (DCN == 4)
                {
                    px[3] = 255;
                }
            }
        }
        StoreRowRunNT<uint8_t, kGroup * 2 * DCN>(v.dst + (int64_t)y * v.dstRow + (int64_t)(ix - lane * kGroup) * 2 * DCN, o,
                                                 lane, lanes);
    }
};

struct GrayFromYuv422
{
    static constexpr int  kItemW = 2, kItemH = 1;
    static constexpr bool kSizeFromSrc = false;

    static __device__ __forceinline__ void Run(const View &v, const PixArgs &a, int ix, int y)
    {
        const uint32_t q = *reinterpret_cast<const uint32_t *>(v.src + (int64_t)y * v.srcRow + ix * 4);
        const uint32_t o = ((q >> (8 * a.yidx)) & 0xFF) | (((q >> (8 * (a.yidx + 2))) & 0xFF) << 8);
        __builtin_nontemporal_store((uint16_t)o, reinterpret_cast<uint16_t *>(v.dst + (int64_t)y * v.dstRow) + ix);
    }

    // 8 pixels: 16 source bytes in, 8 bytes out
    static constexpr int kGroup = 4;

    static __device__ __forceinline__ void RunGroup(const View &v, const PixArgs &a, int ix, int y)
    {
        uint32_t q[kGroup];
        LoadDwords<kGroup>(v.src + (int64_t)y * v.srcRow + ix * 4, q);
        uint8_t o[2 * kGroup];
#pragma unroll
        for (int g = 0; g < kGroup; ++g)
        {
            o[2 * g]     = (uint8_t)(q[g] >> (8 * a.yidx));
            o[2 * g + 1] = (uint8_t)(q[g] >> (8 * (a.yidx + 2)));
        }
        StoreRunNT<uint8_t, 2 * kGroup>(v.dst + (int64_t)y * v.dstRow + ix * 2, o);
    }
};

// the luma rows of a 4:2:0 image are its gray image; 2 pixels per item (widths are even)
struct GrayFromYuv420
{
    static constexpr int  kItemW = 2, kItemH = 1;
    static constexpr bool kSizeFromSrc = false;

    static __device__ __forceinline__ void Run(const View &v, const PixArgs &, int ix, int y)
    {
        const uint16_t q = reinterpret_cast<const uint16_t *>(v.src + (int64_t)y * v.srcRow)[ix];
        __builtin_nontemporal_store(q, reinterpret_cast<uint16_t *>(v.dst + (int64_t)y * v.dstRow) + ix);
    }

    // 16 pixels: a 16-byte copy
    static constexpr int kGroup = 8;

    static __device__ __forceinline__ void RunGroup(const View &v, const PixArgs &, int ix, int y)
    {
        uint8_t q[2 * kGroup];
        LoadRun<uint8_t, 2 * kGroup>(v.src + (int64_t)y * v.srcRow + ix * 2, q);
        StoreRunNT<uint8_t, 2 * kGroup>(v.dst + (int64_t)y * v.dstRow + ix * 2, q);
    }
};

// ---- kernels -----------------------------------------------------------------------------------------
// Pixels per lane of a one-in, one-out operation. Byte pixels on both sides take runs of 8: measured
// against 4 on 32 x 1080p, BGR2GRAY 53 -> 47 us (half as many of the narrow 1-byte-pixel stores), BGR2HSV
// 82 -> 76 us, BGR2YUV 75 -> 73 us, swizzle-like maps unchanged; 16 and 32 were no better.
template<class Op>
constexpr int MapRunPixels()
{
    using S = typename Op::Src;
    using D = decltype(Op::Map(S{}, PixArgs{}));
    if (sizeof(typename D::Elem) == 1 && sizeof(typename S::Elem) == 1)
    {
        return 8;
    }
    return kRunPixelsFor<typename S::Elem, typename D::Elem>;
}

template<class Op>
constexpr int kMapRun = MapRunPixels<Op>();

// One pixel in, one pixel out (Op::Map): runs of kMapRun<Op> pixels per lane, one row per wave.
template<class Op>
__device__ __forceinline__ void MapRun(const uint8_t *srcRow, uint8_t *dstRow, int W, int x0, const PixArgs &a)
{
    using S  = typename Op::Src;
    using D  = decltype(Op::Map(S{}, a));
    using TS = typename S::Elem;
    using TD = typename D::Elem;
    constexpr int P = kMapRun<Op>;
    if (x0 + P > W)
    {
        for (int x = x0; x < W; ++x)
        {
            reinterpret_cast<D *>(dstRow)[x] = Op::Map(reinterpret_cast<const S *>(srcRow)[x], a);
        }
        return;
    }
    TS in[P * S::kC];
    TD out[P * D::kC];
    LoadRun<TS, P * S::kC>(srcRow + (int64_t)x0 * sizeof(S), in);
#pragma unroll
    for (int k = 0; k < P; ++k)
    {
        S s;
#pragma unroll
        for (int c = 0; c < S::kC; ++c)
        {
            s.v[c] = in[k * S::kC + c];
        }
        const D d = Op::Map(s, a);
#pragma unroll
        for (int c = 0; c < D::kC; ++c)
        {
            out[k * D::kC + c] = d.v[c];
        }
    }
    // the wave's lanes 0 .. lanes-1 hold consecutive pieces of this row (the ragged run returned above)
    const int lane = threadIdx.x & 63, lanes = min(64, (W - (x0 - lane * P)) / P);
    StoreRowRunNT<TD, P * D::kC>(dstRow + (int64_t)(x0 - lane * P) * sizeof(D), out, lane, lanes);
}

template<class Op, class = void>
struct HasBlockPrepare : std::false_type
{
};

template<class Op>
struct HasBlockPrepare<Op, std::enable_if_t<Op::kBlockPrepare>> : std::true_type
{
};

template<class Op>
__global__ __launch_bounds__(256) void MapTensor(const PixArgs a)
{
    if constexpr (HasBlockPrepare<Op>::value)
    {
        Op::Prepare(a);
    }
    const int x0 = (blockIdx.x * 64 + (threadIdx.x & 63)) * kMapRun<Op>;
    const int y  = blockIdx.y * kRunTileH + (threadIdx.x >> 6);
    if (x0 >= a.W || y >= a.H)
    {
        return;
    }
    const int n = blockIdx.z;
    MapRun<Op>(a.src + n * a.srcN + (int64_t)y * a.srcRow, a.dst + n * a.dstN + (int64_t)y * a.dstRow, a.W, x0, a);
}

template<class Op>
constexpr int MapPieceBytes()
{
    using S = typename Op::Src;
    using D = decltype(Op::Map(S{}, PixArgs{}));
    return kMapRun<Op> * (int)sizeof(D);
}

template<class Op>
constexpr int kMapVarRows = kVarShapeRows<MapPieceBytes<Op>()>;

// var-shape: the size comes from the destination image
template<class Op>
__global__ __launch_bounds__(256) void MapVarShape(const PixArgs a, const VarTiles tiles)
{
    if constexpr (HasBlockPrepare<Op>::value)
    {
        Op::Prepare(a);
    }
    const TileCoord              tc = LocateTile(tiles, blockIdx.x);
    const NVCVImagePlaneStrided &s  = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided &d  = a.dstList[tc.image].planes[0];
    const int                    x0 = (tc.tx * 64 + (threadIdx.x & 63)) * kMapRun<Op>;
    const uint8_t *src = AsGlobal(s.basePtr);
    uint8_t       *dst = AsGlobal(d.basePtr);
    const int      W = d.width, H = d.height, srcRow = s.rowStride, dstRow = d.rowStride;
    if (x0 >= W)
    {
        return;
    }
    constexpr int R = kMapVarRows<Op>;
    for (int r = 0; r < R; ++r)
    {
        const int y = (tc.ty * R + r) * kRunTileH + (threadIdx.x >> 6);
        if (y >= H)
        {
            return;
        }
        MapRun<Op>(src + (int64_t)y * srcRow, dst + (int64_t)y * dstRow, W, x0, a);
    }
}

template<class Op, class = void>
struct HasRowStore : std::false_type
{
};

template<class Op>
struct HasRowStore<Op, std::enable_if_t<Op::kRowStore>> : std::true_type
{
};

// Subsampled formats: Op::kGroup work items (each Op::kItemW x Op::kItemH pixels) side by side per lane,
// so that loads and stores are whole dwords; the items of a row's last, partial group go one by one.
// Lane (tx, lane) of wave `ty` within the image whose view is v.
template<class Op>
__device__ __forceinline__ void RunItems(const View &v, const PixArgs &a, int tx, int ty)
{
    const int itemsW = v.W / Op::kItemW, itemsH = v.H / Op::kItemH;
    const int x0 = (tx * 64 + (threadIdx.x & 63)) * Op::kGroup;
    const int y  = ty * 4 + (threadIdx.x >> 6);
    if (x0 >= itemsW || y >= itemsH)
    {
        return;
    }
    if (x0 + Op::kGroup <= itemsW)
    {
        if constexpr (HasRowStore<Op>::value)
        {
            const int lane = threadIdx.x & 63;
            Op::RunGroupInRow(v, a, x0, y, lane, min(64, (itemsW - (x0 - lane * Op::kGroup)) / Op::kGroup));
        }
        else
        {
            Op::RunGroup(v, a, x0, y);
        }
        return;
    }
    for (int x = x0; x < itemsW; ++x)
    {
        Op::Run(v, a, x, y);
    }
}

template<class Op>
__global__ __launch_bounds__(256) void PixelTensor(const PixArgs a)
{
    const int  n = blockIdx.z;
    const View v = {a.src + n * a.srcN, a.dst + n * a.dstN, a.srcRow, a.dstRow, a.W, a.H};
    RunItems<Op>(v, a, blockIdx.x, blockIdx.y);
}

// Image batches: the size of the colour image comes from the input (Op::kSizeFromSrc) or the output.
template<class Op>
__global__ __launch_bounds__(256) void PixelVarShape(const PixArgs a, const VarTiles tiles)
{
    const TileCoord             tc = LocateTile(tiles, blockIdx.x);
    const NVCVImagePlaneStrided s  = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided d  = a.dstList[tc.image].planes[0];
    const View v = {AsGlobal(s.basePtr), AsGlobal(d.basePtr), s.rowStride, d.rowStride,
                    Op::kSizeFromSrc ? s.width : d.width, Op::kSizeFromSrc ? s.height : d.height};
    RunItems<Op>(v, a, tc.tx, tc.ty);
}

PixArgs MakeArgs(const ColorIO &io, int W, int H)
{
    PixArgs a = {};
    a.src     = io.src;
    a.dst     = io.dst;
    a.srcN    = io.srcN;
    a.dstN    = io.dstN;
    a.srcRow  = io.srcRow;
    a.dstRow  = io.dstRow;
    a.W       = W;
    a.H       = H;
    a.srcList = io.srcList;
    a.dstList = io.dstList;
    return a;
}

template<class Op>
void Launch(const ColorIO &io, PixArgs a, hipStream_t stream)
{
    if (io.N == 0)
    {
        return;
    }
    if constexpr (Op::kItemW == 1 && Op::kItemH == 1)
    {
        if (io.dstHost == nullptr)
        {
            if (a.W == 0 || a.H == 0)
            {
                return;
            }
            dim3 grid(DivUp(a.W, 64 * kMapRun<Op>), DivUp(a.H, kRunTileH), io.N);
            hipLaunchKernelGGL((MapTensor<Op>), grid, dim3(256), 0, stream, a);
            CheckLaunch("MapTensor");
            return;
        }
        for (int first = 0; first < io.N; first += kMaxTileImages)
        {
            VarTiles tiles;
            int      total = BuildVarTiles(tiles, io.dstHost, first, std::min(kMaxTileImages, io.N - first),
                                           64 * kMapRun<Op>, kRunTileH * kMapVarRows<Op>);
            if (total > 0)
            {
                hipLaunchKernelGGL((MapVarShape<Op>), dim3(total), dim3(256), 0, stream, a, tiles);
                CheckLaunch("MapVarShape");
            }
        }
    }
    else
    {
        constexpr int tileW = 64 * Op::kGroup * Op::kItemW, tileH = 4 * Op::kItemH; // pixels of the colour image
        if (io.dstHost != nullptr)
        {
            const NVCVImageBufferStrided *sizes = Op::kSizeFromSrc ? io.srcHost : io.dstHost;
            for (int first = 0; first < io.N; first += kMaxTileImages)
            {
                VarTiles tiles;
                int      total = BuildVarTiles(tiles, sizes, first, std::min(kMaxTileImages, io.N - first), tileW, tileH);
                if (total > 0)
                {
                    hipLaunchKernelGGL((PixelVarShape<Op>), dim3(total), dim3(256), 0, stream, a, tiles);
                    CheckLaunch("PixelVarShape");
                }
            }
            return;
        }
        if (a.W < Op::kItemW || a.H < Op::kItemH)
        {
            return;
        }
        dim3 grid(DivUp(a.W, tileW), DivUp(a.H, tileH), io.N);
        hipLaunchKernelGGL((PixelTensor<Op>), grid, dim3(256), 0, stream, a);
        CheckLaunch("PixelTensor");
    }
}

[[noreturn]] void Bad(const char *msg)
{
    throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "%s", msg);
}

// same size for every (input, output) image pair; tensors: one size
void RequireSameSize(const ColorIO &io)
{
    if (io.dstHost == nullptr)
    {
        if (io.srcW != io.dstW || io.srcH != io.dstH)
        {
            Bad("Shape mismatch -- output tensor shape doesn't match input tensor shape");
        }
        return;
    }
    for (int i = 0; i < io.N; ++i)
    {
        const NVCVImagePlaneStrided &s = io.srcHost[i].planes[0], &d = io.dstHost[i].planes[0];
        if (s.width != d.width || s.height != d.height)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Image %d: input and output sizes differ", i);
        }
    }
}

void RequireChannels(const ColorIO &io, int sch, int dch)
{
    if (io.srcC != sch)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input channel number %d -- expecting %d", io.srcC, sch);
    }
    if (io.dstC != dch)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid output channel number %d -- expecting %d", io.dstC, dch);
    }
}

void RequireSameType(const ColorIO &io)
{
    if (io.srcElem != io.dstElem)
    {
        Bad("Mismatched input / output DataTypes");
    }
}

// check(srcW, srcH, dstW, dstH) on the tensor pair, or on every (input, output) image pair of a batch
template<class F>
void ForEachSizePair(const ColorIO &io, F check)
{
    if (io.dstHost == nullptr)
    {
        check(io.srcW, io.srcH, io.dstW, io.dstH);
        return;
    }
    for (int i = 0; i < io.N; ++i)
    {
        const NVCVImagePlaneStrided &s = io.srcHost[i].planes[0], &d = io.dstHost[i].planes[0];
        check(s.width, s.height, d.width, d.height);
    }
}

void RequireU8(const ColorIO &io)
{
    if (io.srcElem != kU8 || io.dstElem != kU8)
    {
        Bad("Unsupported input/output DataType, must be 8-bit unsigned");
    }
}

} // namespace

bool RunPixelColorFamily(ColorCode code, const ColorIO &io, hipStream_t stream)
{
    const int c = (int)code;
    PixArgs   a = MakeArgs(io, io.dstW, io.dstH);

    // ---- BGR / RGB -> gray (6, 7) ---------------------------------------------------------------------
    if (code == NVCV_COLOR_BGR2GRAY || code == NVCV_COLOR_RGB2GRAY)
    {
        RequireChannels(io, 3, 1);
        RequireSameType(io);
        RequireSameSize(io);
        a.bidx = code == NVCV_COLOR_RGB2GRAY ? 2 : 0;
        switch (io.srcElem)
        {
        case kU8:
            Launch<GrayFromBgr<uint8_t, 3>>(io, a, stream);
            break;
        case kU16:
            Launch<GrayFromBgr<uint16_t, 3>>(io, a, stream);
            break;
        case kF32:
            Launch<GrayFromBgr<float, 3>>(io, a, stream);
            break;
        default:
            Bad("Unsupported DataType");
        }
        return true;
    }
    // ---- gray -> BGR (8) ------------------------------------------------------------------------------
    if (code == NVCV_COLOR_GRAY2BGR)
    {
        RequireChannels(io, 1, 3);
        RequireSameType(io);
        RequireSameSize(io);
        switch (ElemSize(io.srcElem))
        {
        case 1:
            Launch<BgrFromGray<uint8_t, 3>>(io, a, stream);
            break;
        case 2:
            Launch<BgrFromGray<uint16_t, 3>>(io, a, stream);
            break;
        case 4:
            Launch<BgrFromGray<uint32_t, 3>>(io, a, stream);
            break;
        case 8:
            Launch<BgrFromGray<uint64_t, 3>>(io, a, stream);
            break;
        default:
            Bad("Unsupported DataType");
        }
        return true;
    }
    // ---- BGR / RGB <-> YUV 4:4:4 (82 - 85) --------------------------------------------------------------
    if (c >= NVCV_COLOR_BGR2YUV && c <= NVCV_COLOR_YUV2RGB)
    {
        RequireChannels(io, 3, 3);
        RequireSameType(io);
        RequireSameSize(io);
        const bool toYuv = code == NVCV_COLOR_BGR2YUV || code == NVCV_COLOR_RGB2YUV;
        a.bidx           = (code == NVCV_COLOR_BGR2YUV || code == NVCV_COLOR_YUV2BGR) ? 0 : 2;
        switch (io.srcElem)
        {
        case kU8:
            toYuv ? Launch<YuvFromBgr<uint8_t>>(io, a, stream) : Launch<BgrFromYuv<uint8_t>>(io, a, stream);
            break;
        case kU16:
            toYuv ? Launch<YuvFromBgr<uint16_t>>(io, a, stream) : Launch<BgrFromYuv<uint16_t>>(io, a, stream);
            break;
        case kF32:
            toYuv ? Launch<YuvFromBgr<float>>(io, a, stream) : Launch<BgrFromYuv<float>>(io, a, stream);
            break;
        default:
            Bad("Unsupported DataType");
        }
        return true;
    }
    // ---- BGR / RGB -> HSV (40, 41, 66, 67) --------------------------------------------------------------
    if (code == NVCV_COLOR_BGR2HSV || code == NVCV_COLOR_RGB2HSV || code == NVCV_COLOR_BGR2HSV_FULL
        || code == NVCV_COLOR_RGB2HSV_FULL)
    {
        RequireChannels(io, 3, 3);
        RequireSameType(io);
        RequireSameSize(io);
        a.full = (code == NVCV_COLOR_BGR2HSV_FULL || code == NVCV_COLOR_RGB2HSV_FULL) ? 1 : 0;
        a.bidx = (code == NVCV_COLOR_BGR2HSV || code == NVCV_COLOR_BGR2HSV_FULL) ? 0 : 2;
        switch (io.srcElem)
        {
        case kU8:
            a.bidx ? Launch<HsvFromBgr<uint8_t, true>>(io, a, stream) : Launch<HsvFromBgr<uint8_t, false>>(io, a, stream);
            break;
        case kF32:
            a.bidx ? Launch<HsvFromBgr<float, true>>(io, a, stream) : Launch<HsvFromBgr<float, false>>(io, a, stream);
            break;
        default:
            Bad("Unsupported DataType");
        }
        return true;
    }
    // ---- HSV -> BGR / RGB (54, 55, 70, 71) --------------------------------------------------------------
    if (code == NVCV_COLOR_HSV2BGR || code == NVCV_COLOR_HSV2RGB || code == NVCV_COLOR_HSV2BGR_FULL
        || code == NVCV_COLOR_HSV2RGB_FULL)
    {
        if (io.dstC != 3 && io.dstC != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid output channel number %d", io.dstC);
        }
        RequireChannels(io, 3, io.dstC);
        RequireSameType(io);
        RequireSameSize(io);
        a.full = (code == NVCV_COLOR_HSV2BGR_FULL || code == NVCV_COLOR_HSV2RGB_FULL) ? 1 : 0;
        a.bidx = (code == NVCV_COLOR_HSV2BGR || code == NVCV_COLOR_HSV2BGR_FULL) ? 0 : 2;
        if (io.srcElem == kU8)
        {
            io.dstC == 3 ? Launch<BgrFromHsv<uint8_t, 3>>(io, a, stream) : Launch<BgrFromHsv<uint8_t, 4>>(io, a, stream);
        }
        else if (io.srcElem == kF32)
        {
            io.dstC == 3 ? Launch<BgrFromHsv<float, 3>>(io, a, stream) : Launch<BgrFromHsv<float, 4>>(io, a, stream);
        }
        else
        {
            Bad("Unsupported DataType");
        }
        return true;
    }
    // ---- YUV 4:2:0 -> gray (106) ------------------------------------------------------------------------
    if (code == NVCV_COLOR_YUV2GRAY_420)
    {
        RequireChannels(io, 1, 1);
        RequireU8(io);
        ForEachSizePair(io,
                        [](int sw, int sh, int dw, int dh)
                        {
                            if (sh % 3 != 0 || sw % 2 != 0)
                            {
                                Bad("Invalid input shape: height must be a multiple of 3 and width a multiple of 2");
                            }
                            if (dh != sh * 2 / 3 || dw != sw)
                            {
                                Bad("Invalid output shape");
                            }
                        });
        Launch<GrayFromYuv420>(io, a, stream);
        return true;
    }
    // ---- YUV 4:2:2 -> BGR / RGB / gray (107, 108, 111, 112, 115 - 124) ------------------------------------
    if (c >= NVCV_COLOR_YUV2RGB_UYVY && c <= NVCV_COLOR_YUV2GRAY_YUY2)
    {
        switch (c)
        {
        case 109: // the VYUY codes are not implemented by the reference either
        case 110:
        case 113:
        case 114:
            return false;
        default:
            break;
        }
        RequireU8(io);
        const bool gray = code == NVCV_COLOR_YUV2GRAY_UYVY || code == NVCV_COLOR_YUV2GRAY_YUY2;
        if (io.srcC != 1)
        {
            Bad("Invalid input channel number -- input must have 1 channel");
        }
        if (!(gray && io.dstC == 1) && io.dstC != 3 && io.dstC != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid output channel number %d", io.dstC);
        }
        ForEachSizePair(io,
                        [](int sw, int sh, int dw, int dh)
                        {
                            if (sw % 4 != 0)
                            {
                                Bad("Invalid input shape -- width must be a multiple of 4");
                            }
                            if (dh != sh || 2 * dw != sw)
                            {
                                Bad("Invalid output shape");
                            }
                        });
        const bool bgrOrder = code == NVCV_COLOR_YUV2BGR_YUY2 || code == NVCV_COLOR_YUV2BGRA_YUY2
                           || code == NVCV_COLOR_YUV2BGR_YVYU || code == NVCV_COLOR_YUV2BGRA_YVYU
                           || code == NVCV_COLOR_YUV2BGR_UYVY || code == NVCV_COLOR_YUV2BGRA_UYVY;
        const bool lumaFirst = (c >= NVCV_COLOR_YUV2RGB_YUY2 && c <= NVCV_COLOR_YUV2BGRA_YVYU)
                            || code == NVCV_COLOR_YUV2GRAY_YUY2;
        const bool uFirst = code == NVCV_COLOR_YUV2BGR_YUY2 || code == NVCV_COLOR_YUV2BGRA_YUY2
                         || code == NVCV_COLOR_YUV2RGB_YUY2 || code == NVCV_COLOR_YUV2RGBA_YUY2
                         || code == NVCV_COLOR_YUV2BGR_UYVY || code == NVCV_COLOR_YUV2BGRA_UYVY
                         || code == NVCV_COLOR_YUV2RGB_UYVY || code == NVCV_COLOR_YUV2RGBA_UYVY;
        a.bidx = bgrOrder ? 0 : 2;
        a.yidx = lumaFirst ? 0 : 1;
        a.uidx = uFirst ? 0 : 2;
        if (gray && io.dstC == 1)
        {
            Launch<GrayFromYuv422>(io, a, stream);
        }
        else if (gray)
        {
            Bad("Invalid output channel number -- expecting 1");
        }
        else
        {
            io.dstC == 3 ? Launch<BgrFromYuv422<3>>(io, a, stream) : Launch<BgrFromYuv422<4>>(io, a, stream);
        }
        return true;
    }
    // ---- BGR / RGB (A) -> YUV 4:2:0 (127 - 134, 140 - 147) ------------------------------------------------
    if ((c >= NVCV_COLOR_RGB2YUV_I420 && c <= NVCV_COLOR_BGRA2YUV_YV12)
        || (c >= NVCV_COLOR_RGB2YUV_NV12 && c <= NVCV_COLOR_BGRA2YUV_NV21))
    {
        const bool planar = c <= NVCV_COLOR_BGRA2YUV_YV12;
        const bool bgrOrder
            = code == NVCV_COLOR_BGR2YUV_NV12 || code == NVCV_COLOR_BGRA2YUV_NV12 || code == NVCV_COLOR_BGR2YUV_NV21
           || code == NVCV_COLOR_BGRA2YUV_NV21 || code == NVCV_COLOR_BGR2YUV_YV12 || code == NVCV_COLOR_BGRA2YUV_YV12
           || code == NVCV_COLOR_BGR2YUV_IYUV || code == NVCV_COLOR_BGRA2YUV_IYUV;
        const bool uFirst
            = code == NVCV_COLOR_BGR2YUV_NV12 || code == NVCV_COLOR_BGRA2YUV_NV12 || code == NVCV_COLOR_RGB2YUV_NV12
           || code == NVCV_COLOR_RGBA2YUV_NV12 || code == NVCV_COLOR_BGR2YUV_IYUV || code == NVCV_COLOR_BGRA2YUV_IYUV
           || code == NVCV_COLOR_RGB2YUV_IYUV || code == NVCV_COLOR_RGBA2YUV_IYUV;
        if (io.srcC != 3 && io.srcC != 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input channel number %d", io.srcC);
        }
        RequireU8(io);
        if (io.dstC != 1)
        {
            Bad("Invalid output shape");
        }
        ForEachSizePair(io,
                        [planar](int sw, int sh, int dw, int dh)
                        {
                            if (sh % 2 != 0 || sw % 2 != 0)
                            {
                                Bad("Invalid input shape: width and height must be even");
                            }
                            if (planar && sh % 4 != 0)
                            {
                                Bad("Invalid input shape: to convert to YUV 420 planar formats, the input height must "
                                    "be a multiple of 4");
                            }
                            if (dh != sh / 2 * 3 || dw != sw)
                            {
                                Bad("Invalid output shape");
                            }
                        });
        a      = MakeArgs(io, io.srcW, io.srcH);
        a.bidx = bgrOrder ? 0 : 2;
        a.uidx = uFirst ? 0 : 1;
        if (planar)
        {
            io.srcC == 3 ? Launch<Yuv420FromBgr<3, false>>(io, a, stream) : Launch<Yuv420FromBgr<4, false>>(io, a, stream);
        }
        else
        {
            io.srcC == 3 ? Launch<Yuv420FromBgr<3, true>>(io, a, stream) : Launch<Yuv420FromBgr<4, true>>(io, a, stream);
        }
        return true;
    }
    return false;
}

} // namespace cvamd
