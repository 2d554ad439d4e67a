// WarpAffine and WarpPerspective, tensors and var-shape batches.
//
// Coordinates, sampling and border handling follow the reference in float32 without FMA
// contraction (the bilinear sum in the association of the reference's golden, tap * (wx * wy),
// tests/cvcuda/system/TestOpWarpAffine.cpp:159-170, so integer results equal the golden's bit for bit): destination->source map src/cvcuda/priv/legacy/CvCudaLegacy.h:143-183, matrix
// inversion warp.cu:139-150 (affine) and cuda_tools/math/LinAlg.hpp:1446-1450, 1640-1654 (3x3),
// samplers cuda_tools/InterpolationWrap.hpp:83-104, 332-339, 429-447, 535-565, border index maps
// cuda_tools/BorderWrap.hpp:62-121. Validation follows warp.cu:152-232 and warp_var_shape.cu:194-299.
//
// Differences by design: the var-shape kernels read each image's matrix straight from the caller's
// [N,6] / [N,9] tensor and invert it in the block prologue (a few scalar operations), so the operator
// owns no device buffer and launches no separate inversion kernel; several var-shape submissions of
// one operator handle may therefore be in flight at once. Var-shape batches run on a packed tile grid.
//
// Kernel shape. A 256-thread block produces a 64 x 16 pixel tile of the destination; each of its four
// waves works on its own 32 x 8 part, no LDS and no barrier.
// Gather: the cost of the gather is set by how many distinct cache lines one wave-wide load touches,
// and under a rotation every source row a wave's footprint crosses is another line; so a wave samples
// compact 8 x 8 pixel patches (one lane per pixel, ~10 source rows per load where a 64 x 1 strip would
// cross ~20), four patches side by side per wave, i.e. kPxPerLane = 4 independent samples per lane
// whose loads are in flight together. Taps that lie inside the source image - nearly all of them -
// skip the border logic and fetch the horizontally adjacent taps of a row with one load (u8x3: the 6
// bytes of two pixels from an aligned 12-byte window).
// Store: a 4x4 transpose inside every group of 4 lanes (cross-lane moves) turns "one pixel in each of 4
// patches" into "4 consecutive pixels of one row in one patch", which the lane writes as whole dwords;
// single-byte stores scattered over 8 rows are several times slower.
#include "DeviceUtils.hpp"
#include "FixedPointBlend.hpp"
#include "LaneExchange.hpp"
#include "OpCommon.hpp"
#include "VarShapeTiles.hpp"

#include <cvcuda/OpWarpAffine.h>
#include <cvcuda/OpWarpPerspective.h>

#include <algorithm>
#include <cmath>

namespace cvamd {

namespace {

constexpr int kPatch     = 8;  // gather granule: a wave samples kPatch x kPatch pixels per step
constexpr int kPxPerLane = 4;  // steps per wave
constexpr int kTileW     = 64; // = 8 patches
constexpr int kTileH     = 16; // = 2 patches; 16 patches / 4 waves = kPxPerLane
constexpr int kPatchesX  = kTileW / kPatch;
constexpr int kThreads   = kTileW * kTileH / kPxPerLane;

struct WarpArgs
{
    const uint8_t *src;
    uint8_t       *dst;
    int64_t        srcN, dstN;
    int32_t        srcRow, dstRow;
    int32_t        srcW, srcH, dstW, dstH;
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
    // matrix: tensor path -> m[] already maps dst->src; var-shape -> rows of `xforms`
    float          m[9];
    const uint8_t *xforms;
    int64_t        xformStride; // bytes between matrices
    int32_t        inverseGiven; // var-shape: 1 = matrices already map dst->src
    int32_t        perspective;
    int32_t        border;
    float          bval[4];
};

template<class T, int C>
using Vec = Packed<T, C>;

struct Img
{
    const uint8_t *base;
    int32_t        row, w, h;
};

template<class T, int C>
__device__ __forceinline__ void Fetch(const Img &im, const WarpArgs &a, int x, int y, float (&out)[C])
{
    if (a.border == NVCV_BORDER_CONSTANT)
    {
        if (x < 0 || x >= im.w || y < 0 || y >= im.h)
        {
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                out[c] = (float)BorderValueAs<T>(a.bval[c]);
            }
            return;
        }
    }
    else
    {
        x = BorderIndex(a.border, x, im.w);
        y = BorderIndex(a.border, y, im.h);
    }
    const Vec<T, C> px = reinterpret_cast<const Vec<T, C> *>(im.base + (int64_t)y * im.row)[x];
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        out[c] = (float)px.v[c];
    }
}

__device__ __forceinline__ void CubicCoeffs(float d, float (&w)[4])
{
    w[0] = -.5f;
    w[0] = w[0] * d + 1.f;
    w[0] = w[0] * d - .5f;
    w[0] = w[0] * d;
    w[1] = 1.5f;
    w[1] = w[1] * d - 2.5f;
    w[1] = w[1] * d;
    w[1] = w[1] * d + 1.f;
    w[2] = -1.5f;
    w[2] = w[2] * d + 2.f;
    w[2] = w[2] * d + .5f;
    w[2] = w[2] * d;
    w[3] = 1 - w[0] - w[1] - w[2];
}

// float -> int index like the reference's round-down conversion; huge / non-finite coordinates
// saturate instead of invoking undefined behaviour
__device__ __forceinline__ int FloorToInt(float v)
{
    return (int)fminf(fmaxf(floorf(v), -1073741824.f), 1073741824.f);
}

// 8-bit bilinear: the blend of FixedPointBlend.hpp; the fractions are ax = trunc(fx * 2^15) with
// fx = sx - floor(sx) in float32. Integer and quarter-step maps (the reference's own exact-equality table)
// give weights that are exact in both arithmetics, hence the same results as the reference's golden.
template<class T, int INTERP>
constexpr bool kFixedPoint = std::is_same_v<T, uint8_t> && INTERP == NVCV_INTERP_LINEAR;

// 8-bit bicubic: the four horizontal weights (the reference's float32 polynomials) are rounded to
// multiples of 2^-14 with the last one taking the remainder, so that they add up to exactly 1; a row's
// four taps are combined in integers (exact), the four row sums in float32 with the vertical weights.
// Every horizontal weight is within 2^-15 of the float32 one (the last within 2^-14): the result is
// within 0.05 of the float32 expression's, i.e. at most 1 from the reference's golden.
template<class T, int INTERP>
constexpr bool kFixedPointCubic = std::is_same_v<T, uint8_t> && INTERP == NVCV_INTERP_CUBIC;

// The kernels that blend in fixed point work on coordinates in units of 2^-15 pixel: the first two rows
// of their destination -> source matrix arrive multiplied by 2^15 (exact: a power of two), so floor and
// fraction of a coordinate are the two halves of one float -> integer conversion.
template<class T, int INTERP>
constexpr float kCoordScale = kFixedPoint<T, INTERP> ? 32768.f : 1.f;

// floor and 15-bit fraction of a coordinate; NaN and infinite coordinates give fraction 0
__device__ __forceinline__ uint32_t FractionQ15(float v)
{
    const float f = v - floorf(v);
    return f >= 0.f ? (uint32_t)(int)(f * 32768.f) : 0u;
}

// CubicCoeffs times `scale` (a power of two, so every step scales exactly) with the polynomials evaluated
// by fused multiply-adds; used where the weights are quantised afterwards anyway.
__device__ __forceinline__ void CubicCoeffsFused(float d, float scale, float (&w)[4])
{
    w[0] = __builtin_fmaf(-.5f * scale, d, scale);
    w[0] = __builtin_fmaf(w[0], d, -.5f * scale);
    w[0] = w[0] * d;
    w[1] = __builtin_fmaf(1.5f * scale, d, -2.5f * scale);
    w[1] = w[1] * d;
    w[1] = __builtin_fmaf(w[1], d, scale);
    w[2] = __builtin_fmaf(-1.5f * scale, d, 2.f * scale);
    w[2] = __builtin_fmaf(w[2], d, .5f * scale);
    w[2] = w[2] * d;
    w[3] = scale - w[0] - w[1] - w[2];
}

// u8x3 taps are fetched through aligned dword windows (8 bytes for one pixel, 12 for two), which
// read up to 6 bytes = 2 pixels past them. Inside the image that is harmless; taps within 2 pixels
// of the end of the last row, after which the image ends, are kept off this path by TapsInside.
template<class T, int C>
constexpr bool kWideTapLoads = std::is_same_v<T, uint8_t> && C == 3;

// One pixel at base + off, known to be inside the image.
template<class T, int C>
__device__ __forceinline__ void LoadPixelInside(const uint8_t *base, uint32_t off, T (&out)[C])
{
    if constexpr (kWideTapLoads<T, C>)
    {
        const uint32_t q = LoadU32Window(base, off);
        out[0]           = (uint8_t)q;
        out[1]           = (uint8_t)(q >> 8);
        out[2]           = (uint8_t)(q >> 16);
    }
    else
    {
        const Vec<T, C> v = *reinterpret_cast<const Vec<T, C> *>(base + off);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out[c] = v.v[c];
        }
    }
}

// Two horizontally adjacent pixels starting at base + off, both known to be inside the image.
template<class T, int C>
__device__ __forceinline__ void LoadPairInside(const uint8_t *base, uint32_t off, float (&p0)[C], float (&p1)[C])
{
    if constexpr (kWideTapLoads<T, C>)
    {
        const uint64_t q  = LoadU64Window(base, off);
        const uint32_t lo = (uint32_t)q, hi = (uint32_t)(q >> 32);
        p0[0] = (float)(lo & 0xFF);
        p0[1] = (float)((lo >> 8) & 0xFF);
        p0[2] = (float)((lo >> 16) & 0xFF);
        p1[0] = (float)(lo >> 24);
        p1[1] = (float)(hi & 0xFF);
        p1[2] = (float)((hi >> 8) & 0xFF);
    }
    else
    {
        const Vec<T, 2 * C> v = *reinterpret_cast<const Vec<T, 2 * C> *>(base + off);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            p0[c] = (float)v.v[c];
            p1[c] = (float)v.v[C + c];
        }
    }
}

// Byte offset of pixel (x, y), both inside the image. Image planes are below 2 GiB. Uses the 24-bit
// multiply (full rate; the 32-bit one runs at a quarter): images whose row pitch or height does not
// fit 23 bits never take the path that calls this.
template<int PIXEL_BYTES>
__device__ __forceinline__ uint32_t PixelOffset(const Img &im, int x, int y)
{
    return (uint32_t)__mul24(y, im.row) + (uint32_t)x * PIXEL_BYTES;
}

template<bool PERSPECTIVE>
__device__ __forceinline__ void MapCoord(const float (&m)[9], int dx, int dy, float &sx, float &sy)
{
    if constexpr (PERSPECTIVE)
    {
        const float coeff = 1.0f / (m[6] * dx + m[7] * dy + m[8]);
        sx                = coeff * (m[0] * dx + m[1] * dy + m[2]);
        sy                = coeff * (m[3] * dx + m[4] * dy + m[5]);
    }
    else
    {
        sx = m[0] * dx + m[1] * dy + m[2];
        sy = m[3] * dx + m[4] * dy + m[5];
    }
}

// One destination pixel sampled at (sx, sy) with every tap going through the border logic. The tap
// loops are deliberately not unrolled: this path runs only for the few waves that straddle the image
// border, and one copy of the border code keeps the kernel small.
template<class T, int C, int INTERP>
__device__ __forceinline__ void SampleWithBorder(const Img &im, const WarpArgs &a, float sx, float sy, T (&out)[C])
{
    float acc[C];
    if constexpr (INTERP == NVCV_INTERP_NEAREST)
    {
        Fetch<T, C>(im, a, FloorToInt(sx + .5f), FloorToInt(sy + .5f), acc);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out[c] = (T)acc[c]; // the tap itself (exactly representable), no rounding involved
        }
        return;
    }
    else if constexpr (kFixedPoint<T, INTERP>)
    {
        const int      x1 = FloorToInt(sx), y1 = FloorToInt(sy);
        const uint32_t ax = FractionQ15(sx), ay = FractionQ15(sy);
        const uint32_t w11 = (ax * ay + (kQ15 >> 1)) >> 15;
        uint32_t       sum[C];
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            sum[c] = 0;
        }
#pragma nounroll
        for (int i = 0; i < 4; ++i) // taps (x1,y1) (x2,y1) (x1,y2) (x2,y2)
        {
            float t[C];
            Fetch<T, C>(im, a, x1 + (i & 1), y1 + (i >> 1), t);
            const uint32_t w = i == 0 ? kQ15 - ax - ay + w11 : (i == 1 ? ax - w11 : (i == 2 ? ay - w11 : w11));
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                sum[c] += (uint32_t)t[c] * w;
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out[c] = RoundQ15(sum[c]);
        }
        return;
    }
    else if constexpr (INTERP == NVCV_INTERP_LINEAR)
    {
        const int x1 = FloorToInt(sx), y1 = FloorToInt(sy);
        const int x2 = x1 + 1, y2 = y1 + 1;
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            acc[c] = 0.f;
        }
#pragma nounroll
        for (int i = 0; i < 4; ++i) // taps (x1,y1) (x2,y1) (x1,y2) (x2,y2) in this order
        {
            float t[C];
            Fetch<T, C>(im, a, x1 + (i & 1), y1 + (i >> 1), t);
            const float wx = (i & 1) ? (sx - x1) : (x2 - sx);
            const float wy = (i >> 1) ? (sy - y1) : (y2 - sy);
            const float w  = wx * wy;
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                acc[c] += t[c] * w;
            }
        }
    }
    else if constexpr (kFixedPointCubic<T, INTERP>)
    {
        const int ix = FloorToInt(sx), iy = FloorToInt(sy);
        float     wx[4], wy[4];
        CubicCoeffsFused(sx - floorf(sx), 16384.f, wx);
        CubicCoeffsFused(sy - floorf(sy), 1.f / 16384.f, wy);
        int wq[4];
        CubicWeightsQ14(wx, wq);
#pragma nounroll
        for (int cy = 0; cy < 4; ++cy)
        {
            int h[C];
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                h[c] = 0;
            }
#pragma nounroll
            for (int cx = 0; cx < 4; ++cx)
            {
                float t[C];
                Fetch<T, C>(im, a, ix + cx - 1, iy + cy - 1, t);
                const int w = cx == 0 ? wq[0] : (cx == 1 ? wq[1] : (cx == 2 ? wq[2] : wq[3]));
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    h[c] += (int)t[c] * w;
                }
            }
            const float v = cy == 0 ? wy[0] : (cy == 1 ? wy[1] : (cy == 2 ? wy[2] : wy[3]));
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                acc[c] = cy == 0 ? (float)h[c] * v : __builtin_fmaf((float)h[c], v, acc[c]);
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out[c] = SaturateCast<T>(acc[c]);
        }
        return;
    }
    else
    {
        const int ix = FloorToInt(sx), iy = FloorToInt(sy);
        float     wx[4], wy[4];
        CubicCoeffs(sx - ix, wx);
        CubicCoeffs(sy - iy, wy);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            acc[c] = 0.f;
        }
#pragma unroll
        for (int cy = 0; cy < 4; ++cy)
        {
#pragma unroll
            for (int cx = 0; cx < 4; ++cx)
            {
                float t[C];
                Fetch<T, C>(im, a, ix + cx - 1, iy + cy - 1, t);
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    acc[c] += t[c] * (wx[cx] * wy[cy]);
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        out[c] = SaturateCast<T>(acc[c]);
    }
}

// True when every tap of the sample at (sx, sy) lies inside the image (and, with WIDE loads, none of
// them is among the image's last two columns: the window loads read 2 pixels past a tap pair, which
// must not run off the end of the last row). limX / limY come from InsideLimits. For an integer k,
// floor(v) < k <=> v < k, so the test is 0 <= v - lo < lim per axis, done as ONE unsigned comparison
// of the float's bit pattern: non-negative floats order like their bits, negative ones and NaNs have
// patterns above every finite positive limit (-0.0 fails too and takes the generic path, which
// computes the same result).
// The test runs on a lane's kPxPerLane samples at once: the largest bit pattern per axis against the limit.
template<int INTERP>
__device__ __forceinline__ bool TapsInside(float limX, float limY, const float (&sx)[kPxPerLane],
                                           const float (&sy)[kPxPerLane])
{
    // taps span [floor(v) - lo, floor(v) + hi] per axis; NEAREST takes floor(v + .5)
    constexpr float lo = INTERP == NVCV_INTERP_CUBIC ? 1.f : (INTERP == NVCV_INTERP_NEAREST ? -.5f : 0.f);
    uint32_t        ux = 0, uy = 0;
#pragma unroll
    for (int k = 0; k < kPxPerLane; ++k)
    {
        ux = max(ux, __float_as_uint(sx[k] - lo));
        uy = max(uy, __float_as_uint(sy[k] - lo));
    }
    return (ux < __float_as_uint(limX)) & (uy < __float_as_uint(limY)); // bitwise on purpose: no branch
}

// Exclusive upper limit of floor(v) - lo along an axis of `size` pixels; 0 (no sample passes) when the
// image is smaller than the tap span.
template<int INTERP>
__device__ __forceinline__ float InsideLimit(int size, bool wide)
{
    constexpr int lo = INTERP == NVCV_INTERP_CUBIC ? 1 : 0;
    constexpr int hi = INTERP == NVCV_INTERP_CUBIC ? 2 : (INTERP == NVCV_INTERP_LINEAR ? 1 : 0);
    return (float)max(size - hi - lo - (wide ? 2 : 0), 0);
}

// Same arithmetic as SampleWithBorder for a sample whose taps are all inside the image: no border
// logic, adjacent taps fetched together, no branches (so the loads of several pixels can be in flight
// at once). floorf(v) is used directly where the generic path converts floor(v) to int and back.
// O = T, or float for the unrounded sums (not for NEAREST).
template<class O, int C, int INTERP, class T = O>
__device__ __forceinline__ void SampleInside(const Img &im, float sx, float sy, O (&out)[C])
{
    constexpr int PB = C * sizeof(T);
    float         acc[C];
    if constexpr (INTERP == NVCV_INTERP_NEAREST)
    {
        const int x = (int)floorf(sx + .5f), y = (int)floorf(sy + .5f);
        LoadPixelInside<T, C>(im.base, PixelOffset<PB>(im, x, y), out);
        return;
    }
    else if constexpr (INTERP == NVCV_INTERP_LINEAR)
    {
        const float fx = floorf(sx), fy = floorf(sy);
        const float wx1 = sx - fx, wx0 = (fx + 1.f) - sx;
        const float wy1 = sy - fy, wy0 = (fy + 1.f) - sy;
        const uint32_t o = PixelOffset<PB>(im, (int)fx, (int)fy);
        float          t[4][C];
        LoadPairInside<T, C>(im.base, o, t[0], t[1]);
        LoadPairInside<T, C>(im.base, o + (uint32_t)im.row, t[2], t[3]);
        const float w00 = wx0 * wy0, w01 = wx1 * wy0, w10 = wx0 * wy1, w11 = wx1 * wy1;
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            float v = t[0][c] * w00;
            v += t[1][c] * w01;
            v += t[2][c] * w10;
            v += t[3][c] * w11;
            acc[c] = v;
        }
    }
    else
    {
        const float fx = floorf(sx), fy = floorf(sy);
        float       wx[4], wy[4];
        CubicCoeffs(sx - fx, wx);
        CubicCoeffs(sy - fy, wy);
        uint32_t o = PixelOffset<PB>(im, (int)fx - 1, (int)fy - 1);
        float    t[4][4][C];
#pragma unroll
        for (int cy = 0; cy < 4; ++cy)
        {
            LoadPairInside<T, C>(im.base, o, t[cy][0], t[cy][1]);
            LoadPairInside<T, C>(im.base, o + 2 * PB, t[cy][2], t[cy][3]);
            o += (uint32_t)im.row;
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            acc[c] = 0.f;
        }
#pragma unroll
        for (int cy = 0; cy < 4; ++cy)
        {
#pragma unroll
            for (int cx = 0; cx < 4; ++cx)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    acc[c] += t[cy][cx][c] * (wx[cx] * wy[cy]);
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        if constexpr (std::is_same_v<O, T>)
        {
            out[c] = SaturateCast<T>(acc[c]);
        }
        else
        {
            out[c] = acc[c];
        }
    }
}

// Four horizontally adjacent u8 pixels at base + off (all inside the image) as raw bytes in C dwords.
// u8x3: one aligned 16-byte window, funnel-shifted (see LoadU64Window); reads up to 3 bytes before and
// 4 bytes after the 12.
template<int C>
__device__ __forceinline__ void LoadQuadBytes(const uint8_t *base, uint32_t off, uint32_t (&r)[C])
{
    if constexpr (kWideTapLoads<uint8_t, C>)
    {
        struct alignas(4) W4
        {
            uint32_t d[4];
        };
        const uint32_t mis = (uint32_t)reinterpret_cast<uintptr_t>(base) & 3u;
        const uint32_t o   = off + mis;
        const W4       w   = *reinterpret_cast<const W4 *>((base - mis) + (o & ~3u));
        r[0]               = __builtin_amdgcn_alignbyte(w.d[1], w.d[0], o);
        r[1]               = __builtin_amdgcn_alignbyte(w.d[2], w.d[1], o);
        r[2]               = __builtin_amdgcn_alignbyte(w.d[3], w.d[2], o);
    }
    else
    {
        const Vec<uint8_t, 4 * C> v = *reinterpret_cast<const Vec<uint8_t, 4 * C> *>(base + off);
        __builtin_memcpy(r, &v, 4 * C);
    }
}

// The fixed-point bicubic sum (see kFixedPointCubic) of the 4 x 4 taps in r (row j, 4 pixels as raw bytes).
template<int C>
__device__ __forceinline__ uint32_t BlendCubicQ14(const uint32_t (&r)[4][C], float sx, float sy)
{
    float wx[4], wy[4];
    CubicCoeffsFused(sx - floorf(sx), 16384.f, wx);
    CubicCoeffsFused(sy - floorf(sy), 1.f / 16384.f, wy);
    uint32_t p01, p23;
    CubicWeightPairsQ14(wx, p01, p23);
    uint32_t q = 0;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            int h = Dot2I16(BytePair(r[j], c, c + C), p01);
            h     = Dot2I16(BytePair(r[j], c + 2 * C, c + 3 * C), p23, h);
            acc   = j == 0 ? (float)h * wy[0] : __builtin_fmaf((float)h, wy[j], acc);
        }
        q = __builtin_amdgcn_cvt_pk_u8_f32(acc, c, q);
    }
    return q;
}

// The same for a sample whose 16 taps are inside the image.
template<int C>
__device__ __forceinline__ uint32_t SampleInsideCubicQ14(const Img &im, float sx, float sy)
{
    uint32_t o = PixelOffset<C>(im, (int)floorf(sx) - 1, (int)floorf(sy) - 1);
    uint32_t r[4][C];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        LoadQuadBytes<C>(im.base, o, r[j]);
        o += (uint32_t)im.row;
    }
    return BlendCubicQ14<C>(r, sx, sy);
}

// The two horizontally adjacent u8 pixels at base + off (both inside the image) as raw bytes: byte i of
// the 64-bit value {w[1]:w[0]} is channel i % C of pixel i / C.
template<int C>
__device__ __forceinline__ void LoadPairBytes(const uint8_t *base, uint32_t off, uint32_t (&w)[2])
{
    if constexpr (kWideTapLoads<uint8_t, C>)
    {
        const uint64_t q = LoadU64Window(base, off);
        w[0]             = (uint32_t)q;
        w[1]             = (uint32_t)(q >> 32);
    }
    else
    {
        const Vec<uint8_t, 2 * C> v = *reinterpret_cast<const Vec<uint8_t, 2 * C> *>(base + off);
        w[0] = w[1] = 0;
        __builtin_memcpy(w, &v, 2 * C);
    }
}

// SampleWithBorder's fixed-point bilinear sum for a sample whose taps are all inside the image, whose
// coordinates are not negative and below 2^16, given in units of 2^-15 pixel: floor and fraction come
// from one float -> integer conversion, the taps of a row from one window, the two taps of a channel
// from one byte permute. Returns the pixel's dword.
template<int C>
__device__ __forceinline__ uint32_t SampleInsideQ15(const Img &im, float sx, float sy)
{
    const uint32_t X = (uint32_t)(int)sx, Y = (uint32_t)(int)sy;
    uint32_t       top, bottom;
    WeightPairsQ15(X & (kQ15 - 1), Y & (kQ15 - 1), top, bottom);
    const uint32_t o = PixelOffset<C>(im, (int)(X >> 15), (int)(Y >> 15));
    uint32_t       r0[2], r1[2];
    LoadPairBytes<C>(im.base, o, r0);
    LoadPairBytes<C>(im.base, o + (uint32_t)im.row, r1);
    uint32_t q = 0;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        // bytes c and c + C of the row's 8 -> (left | right << 16); selector 0x0c gives a zero byte
        const uint32_t sel = 0x0c000c00u | (uint32_t)c | ((uint32_t)(c + C) << 16);
        q = BlendQ15(__builtin_amdgcn_perm(r0[1], r0[0], sel), __builtin_amdgcn_perm(r1[1], r1[0], sel), top, bottom, c, q);
    }
    return q;
}

// SampleWithBorder's fixed-point bilinear sum for the two border modes that need no division - a constant
// colour (`constant`: borderPx, channel c in byte c) or the nearest pixel of the image -, straight-line: the
// four taps are fetched at coordinates clamped into the image and, for the constant border, replaced where the
// unclamped coordinate is outside. sx, sy in units of 2^-15 pixel, below 2^30 in magnitude. Same weights, same
// exact sum and the same single rounding as the generic path, so which path a sample takes does not show.
// The border modes' index maps for coordinates no farther than one image size outside the image (-(s - 1) .. 2s - 2
// for an axis of s pixels), where each is a single fold: index = c inside, k * c + lo in front, k * c + hi behind,
// with wave-uniform k, lo, hi per mode (DeviceUtils.hpp:BorderIndex for any coordinate, with its divisions):
//   constant, replicate  0 * c + 0      | 0 * c + s - 1     (the nearest pixel; the constant colour replaces it later)
//   reflect             -1 * c - 1      | -1 * c + 2s - 1
//   wrap                 1 * c + s      |  1 * c - s
//   reflect101          -1 * c          | -1 * c + 2s - 2
struct BorderFold
{
    int k, lo, hi, size;
};

__device__ __forceinline__ BorderFold MakeBorderFold(int border, int s)
{
    BorderFold f = {0, 0, s - 1, s};
    if (border == NVCV_BORDER_REFLECT)
    {
        f = {-1, -1, 2 * s - 1, s};
    }
    else if (border == NVCV_BORDER_WRAP)
    {
        f = {1, s, -s, s};
    }
    else if (border == NVCV_BORDER_REFLECT101)
    {
        f = {-1, 0, 2 * s - 2, s};
    }
    return f;
}

__device__ __forceinline__ int Fold(const BorderFold &f, int c)
{
    const int kc = f.k * c;
    return c < 0 ? kc + f.lo : (c >= f.size ? kc + f.hi : c);
}

// Pixel (x, y) of an 8-bit image, inside it, as a dword (channel c in byte c, the rest is not looked at): one
// 4-byte load, moved back where it would run past the image's last byte.
template<int C>
__device__ __forceinline__ uint32_t LoadPixelGuarded(const Img &im, uint32_t rowOffset, int x)
{
    const uint32_t lastLoad = (uint32_t)__mul24(im.h - 1, im.row) + (uint32_t)im.w * C - 4;
    const uint32_t at = rowOffset + (uint32_t)x * C, from = min(at, lastLoad);
    return LoadU32Unaligned(im.base + from) >> (8 * (at - from));
}

template<int C>
__device__ __forceinline__ uint32_t SampleNearBorderQ15(const Img &im, const BorderFold &fx, const BorderFold &fy, bool constant,
                                                        uint32_t borderPx, float sx, float sy)
{
    const int X = __float2int_rd(sx), Y = __float2int_rd(sy);
    const int x0 = X >> 15, y0 = Y >> 15;
    const int cx0 = Fold(fx, x0), cx1 = Fold(fx, x0 + 1);
    const uint32_t r0 = (uint32_t)__mul24(Fold(fy, y0), im.row), r1 = (uint32_t)__mul24(Fold(fy, y0 + 1), im.row);
    uint32_t p00 = LoadPixelGuarded<C>(im, r0, cx0), p01 = LoadPixelGuarded<C>(im, r0, cx1);
    uint32_t p10 = LoadPixelGuarded<C>(im, r1, cx0), p11 = LoadPixelGuarded<C>(im, r1, cx1);
    if (constant) // uniform
    {
        const bool inX0 = (uint32_t)x0 < (uint32_t)im.w, inX1 = (uint32_t)(x0 + 1) < (uint32_t)im.w;
        const bool inY0 = (uint32_t)y0 < (uint32_t)im.h, inY1 = (uint32_t)(y0 + 1) < (uint32_t)im.h;
        p00             = inX0 && inY0 ? p00 : borderPx;
        p01             = inX1 && inY0 ? p01 : borderPx;
        p10             = inX0 && inY1 ? p10 : borderPx;
        p11             = inX1 && inY1 ? p11 : borderPx;
    }
    return BilinearQ15<C>(p00, p01, p10, p11, (uint32_t)X & (kQ15 - 1), (uint32_t)Y & (kQ15 - 1));
}

// The same for the fixed-point bicubic sum: the 4 x 4 taps fetched at clamped coordinates (replaced by the colour
// where the unclamped one is outside), put together as the rows BlendCubicQ14 takes. |sx|, |sy| below 2^24.
template<int C>
__device__ __forceinline__ uint32_t SampleNearBorderCubicQ14(const Img &im, const BorderFold &fx, const BorderFold &fy,
                                                             bool constant, uint32_t borderPx, float sx, float sy)
{
    const int ix = (int)floorf(sx) - 1, iy = (int)floorf(sy) - 1;
    int       cx[4];
    bool      inX[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        cx[i]  = Fold(fx, ix + i);
        inX[i] = (uint32_t)(ix + i) < (uint32_t)im.w;
    }
    uint32_t r[4][C];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const uint32_t rowOffset = (uint32_t)__mul24(Fold(fy, iy + j), im.row);
        const bool     inY       = (uint32_t)(iy + j) < (uint32_t)im.h;
        uint32_t       p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            p[i] = LoadPixelGuarded<C>(im, rowOffset, cx[i]);
            if (constant) // uniform
            {
                p[i] = inX[i] && inY ? p[i] : borderPx;
            }
        }
        if constexpr (C == 3)
        {
            r[j][0] = __builtin_amdgcn_perm(p[1], p[0], 0x04020100u);
            r[j][1] = __builtin_amdgcn_perm(p[2], p[1], 0x05040201u);
            r[j][2] = __builtin_amdgcn_perm(p[3], p[2], 0x06050402u);
        }
        else if constexpr (C == 4)
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                r[j][i] = p[i];
            }
        }
        else
        {
            r[j][0] = __builtin_amdgcn_perm(__builtin_amdgcn_perm(p[3], p[2], 0x04000c0cu), __builtin_amdgcn_perm(p[1], p[0], 0x0c0c0400u),
                                            0x07060100u);
        }
    }
    return BlendCubicQ14<C>(r, sx, sy);
}

// And for the nearest pixel.
template<int C>
__device__ __forceinline__ uint32_t SampleNearBorderNearest(const Img &im, const BorderFold &fx, const BorderFold &fy,
                                                            bool constant, uint32_t borderPx, float sx, float sy)
{
    const int      x = FloorToInt(sx + .5f), y = FloorToInt(sy + .5f);
    const uint32_t p = LoadPixelGuarded<C>(im, (uint32_t)__mul24(Fold(fy, y), im.row), Fold(fx, x));
    // (the bytes above the pixel's must be 0: the stores merge neighbouring pixels' dwords)
    return constant && !((uint32_t)x < (uint32_t)im.w && (uint32_t)y < (uint32_t)im.h) ? borderPx : p & (0xffffffffu >> (32 - 8 * C));
}

// The dwords of the pixel that SampleInside gives. u8 channels are rounded, saturated and placed into
// their byte by one instruction each (v_cvt_pk_u8_f32 with a byte select and the dword so far), where
// packing converted bytes takes as many shifts and merges again.
template<class T, int C, int INTERP>
__device__ __forceinline__ void SampleInsidePacked(const Img &im, float sx, float sy, uint32_t (&w)[(C * sizeof(T) + 3) / 4])
{
    if constexpr (kFixedPoint<T, INTERP>)
    {
        w[0] = SampleInsideQ15<C>(im, sx, sy);
    }
    else if constexpr (kFixedPointCubic<T, INTERP>)
    {
        w[0] = SampleInsideCubicQ14<C>(im, sx, sy);
    }
    else if constexpr (std::is_same_v<T, uint8_t> && INTERP != NVCV_INTERP_NEAREST)
    {
        float acc[C];
        SampleInside<float, C, INTERP, T>(im, sx, sy, acc);
        uint32_t q = 0;
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            q = __builtin_amdgcn_cvt_pk_u8_f32(acc[c], c, q);
        }
        w[0] = q;
    }
    else
    {
        T v[C];
        SampleInside<T, C, INTERP>(im, sx, sy, v);
#pragma unroll
        for (int d = 0; d < (int)((C * sizeof(T) + 3) / 4); ++d)
        {
            w[d] = 0;
        }
        __builtin_memcpy(w, v, C * sizeof(T));
    }
}

// True when every tap of the sample at (sx, sy) lies outside the image. For an integer k,
// floor(v) < k <=> v < k and floor(v) >= k <=> v >= k; NaN coordinates fail every comparison.
template<int INTERP>
__device__ __forceinline__ bool TapsOutside(const Img &im, float sx, float sy)
{
    if constexpr (INTERP == NVCV_INTERP_NEAREST)
    {
        // the tap is floor(v + .5)
        return (sx + .5f < 0.f) | (sx + .5f >= (float)im.w) | (sy + .5f < 0.f) | (sy + .5f >= (float)im.h);
    }
    constexpr float lo = INTERP == NVCV_INTERP_CUBIC ? 1.f : 0.f;
    constexpr float hi = INTERP == NVCV_INTERP_CUBIC ? 2.f : 1.f;
    return (sx < -hi) | (sx >= (float)im.w + lo) | (sy < -hi) | (sy >= (float)im.h + lo);
}

// SampleWithBorder for a sample whose taps all lie outside the image under NVCV_BORDER_CONSTANT: every tap is
// the border value, the weights and the order of the sum are the general sampler's, nothing is loaded.
template<class T, int C, int INTERP>
__device__ __forceinline__ void SampleAllOutside(const WarpArgs &a, float sx, float sy, T (&out)[C])
{
    float t[C], acc[C];
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        t[c]   = (float)BorderValueAs<T>(a.bval[c]);
        acc[c] = 0.f;
    }
    if constexpr (INTERP == NVCV_INTERP_NEAREST || kFixedPoint<T, INTERP>)
    {
        // the tap itself; in fixed point the weights add up to exactly 1
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out[c] = (T)t[c];
        }
        return;
    }
    else if constexpr (INTERP == NVCV_INTERP_LINEAR)
    {
        const int x1 = FloorToInt(sx), y1 = FloorToInt(sy);
        const int x2 = x1 + 1, y2 = y1 + 1;
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            const float wx = (i & 1) ? (sx - x1) : (x2 - sx);
            const float wy = (i >> 1) ? (sy - y1) : (y2 - sy);
            const float w  = wx * wy;
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                acc[c] += t[c] * w;
            }
        }
    }
    else if constexpr (kFixedPointCubic<T, INTERP>)
    {
        // every row sum is the border value times 2^14: the horizontal weights add up to exactly 1
        float wy[4];
        CubicCoeffsFused(sy - floorf(sy), 1.f / 16384.f, wy);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            const float h = t[c] * 16384.f;
            float       v = h * wy[0];
            v             = __builtin_fmaf(h, wy[1], v);
            v             = __builtin_fmaf(h, wy[2], v);
            v             = __builtin_fmaf(h, wy[3], v);
            out[c]        = SaturateCast<T>(v);
        }
        return;
    }
    else
    {
        const int ix = FloorToInt(sx), iy = FloorToInt(sy);
        float     wx[4], wy[4];
        CubicCoeffs(sx - ix, wx);
        CubicCoeffs(sy - iy, wy);
#pragma unroll
        for (int cy = 0; cy < 4; ++cy)
        {
#pragma unroll
            for (int cx = 0; cx < 4; ++cx)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    acc[c] += t[c] * (wx[cx] * wy[cy]);
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        out[c] = SaturateCast<T>(acc[c]);
    }
}

// 8-bit pixels of 1, 3 or 4 channels have straight-line samplers for samples next to the image's edge.
template<class T, int C>
constexpr bool kNearBorderForms = std::is_same_v<T, uint8_t> && (C == 1 || C == 3 || C == 4);

// Whether a lane's samples can take them: an image of 4 bytes or more within the 24-bit offsets (the caller's test),
// every coordinate small enough for the sampler's integer conversion (bilinear: times 2^15 below 2^30; bicubic:
// below 2^24; nearest: any) and, for the three modes that mirror or repeat the image, every tap no farther than one
// image size outside it (BorderFold; with a margin of two pixels for the widest tap window).
template<class T, int C, int INTERP>
__device__ __forceinline__ bool NearBorderForm(const Img &im, const WarpArgs &a, const float (&sx)[kPxPerLane],
                                               const float (&sy)[kPxPerLane])
{
    if constexpr (!kNearBorderForms<T, C>)
    {
        return false;
    }
    else
    {
        constexpr float kScale = kCoordScale<T, INTERP>;
        uint32_t        u = 0;
        float           minX = sx[0], maxX = sx[0], minY = sy[0], maxY = sy[0];
#pragma unroll
        for (int k = 0; k < kPxPerLane; ++k)
        {
            u    = max(u, max(__float_as_uint(sx[k]) & 0x7fffffffu, __float_as_uint(sy[k]) & 0x7fffffffu));
            minX = fminf(minX, sx[k]);
            maxX = fmaxf(maxX, sx[k]);
            minY = fminf(minY, sy[k]);
            maxY = fmaxf(maxY, sy[k]);
        }
        const uint32_t limit = INTERP == NVCV_INTERP_LINEAR ? 0x4e800000u : (INTERP == NVCV_INTERP_CUBIC ? 0x4b800000u : 0x7f800000u);
        bool           ok = u < limit && __mul24(im.h - 1, im.row) + im.w * C >= 4;
        if (a.border > NVCV_BORDER_REPLICATE) // wave-uniform
        {
            // taps reach from floor(v) - 1 to floor(v) + 2 at most: all of them within -(s - 1) .. 2s - 2
            ok = ok && minX >= (float)(2 - im.w) * kScale && maxX < (float)(2 * im.w - 4) * kScale
              && minY >= (float)(2 - im.h) * kScale && maxY < (float)(2 * im.h - 4) * kScale;
        }
        return ok;
    }
}

// One 64 x 16 tile of the destination image `dst` (tile coordinates tx, ty), all 256 threads.
template<class T, int C, int INTERP, bool PERSP>
__device__ __forceinline__ void WarpTile(const Img &im, const WarpArgs &a, const float (&m)[9], uint8_t *dst, int dstRow,
                                         int dstW, int dstH, int tx, int ty)
{
    constexpr int PB = C * sizeof(T), D = (PB + 3) / 4;

    // ---- gather: lane (lx, ly) of wave w samples its pixel in patches 4w .. 4w+3 (side by side: a
    // wave covers 32 columns x 8 rows)
    const int wave = threadIdx.x >> 6, lx = threadIdx.x & (kPatch - 1), ly = (threadIdx.x >> 3) & (kPatch - 1);
    // m maps to source coordinates times kCoordScale; so do sx, sy and the limits
    constexpr float kScale = kCoordScale<T, INTERP>;
    const float     limX = InsideLimit<INTERP>(im.w, kWideTapLoads<T, C>) * kScale, limY = InsideLimit<INTERP>(im.h, false) * kScale;
    float       sx[kPxPerLane], sy[kPxPerLane];
    uint32_t    q[D][kPxPerLane]; // q[d][k]: dword d of this lane's pixel in patch k
    // rows too long or too many for 24-bit offset arithmetic go through the generic path
    // (and, in fixed point, coordinates too large for coordinate * 2^15 in 31 bits)
    const bool fits = (im.row | im.h) < (1 << 23) && (!kFixedPoint<T, INTERP> || (im.w | im.h) < (1 << 16));
    bool       allInside = fits;
#pragma unroll
    for (int k = 0; k < kPxPerLane; ++k)
    {
        const int patch = wave * kPxPerLane + k;
        const int px = (patch % kPatchesX) * kPatch + lx, py = (patch / kPatchesX) * kPatch + ly;
        // pixels of the tile beyond the image edge repeat the edge pixel's sample; they are never stored
        const int dx = min(tx * kTileW + px, dstW - 1), dy = min(ty * kTileH + py, dstH - 1);
        MapCoord<PERSP>(m, dx, dy, sx[k], sy[k]);
    }
    allInside = allInside & TapsInside<INTERP>(limX, limY, sx, sy);
    if (allInside)
    {
        uint32_t w[kPxPerLane][D];
#pragma unroll
        for (int k = 0; k < kPxPerLane; ++k)
        {
            SampleInsidePacked<T, C, INTERP>(im, sx[k], sy[k], w[k]);
        }
#pragma unroll
        for (int k = 0; k < kPxPerLane; ++k)
        {
#pragma unroll
            for (int d = 0; d < D; ++d)
            {
                q[d][k] = w[k][d];
            }
        }
    }
    else if (fits && NearBorderForm<T, C, INTERP>(im, a, sx, sy))
    {
        // 8-bit pixels under a constant or replicating border: the border logic as selects, all four samples in
        // flight (the generic loop below costs a wave that straddles the image's edge about 4 times as much)
        if constexpr (kNearBorderForms<T, C>)
        {
            uint32_t borderPx = 0;
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                borderPx |= (uint32_t)BorderValueAs<T>(a.bval[c]) << (8 * c);
            }
            // under a constant border a lane whose samples lie outside with all their taps needs no pixel: whole
            // waves in the corners a rotation leaves empty
            const bool       constant = a.border == NVCV_BORDER_CONSTANT;
            const BorderFold foldX = MakeBorderFold(a.border, im.w), foldY = MakeBorderFold(a.border, im.h);
            bool             outside = constant;
#pragma unroll
            for (int k = 0; k < kPxPerLane; ++k)
            {
                outside &= TapsOutside<INTERP>(im, sx[k] * (1.f / kScale), sy[k] * (1.f / kScale));
            }
            if (outside)
            {
#pragma unroll
                for (int k = 0; k < kPxPerLane; ++k)
                {
                    if constexpr (INTERP == NVCV_INTERP_CUBIC)
                    {
                        T v[C];
                        SampleAllOutside<T, C, INTERP>(a, sx[k], sy[k], v);
                        q[0][k] = 0;
                        __builtin_memcpy(&q[0][k], v, C);
                    }
                    else
                    {
                        q[0][k] = borderPx; // the tap itself, or taps whose weights add up to exactly 1
                    }
                }
            }
            else
            {
#pragma unroll
                for (int k = 0; k < kPxPerLane; ++k)
                {
                    if constexpr (INTERP == NVCV_INTERP_LINEAR)
                    {
                        q[0][k] = SampleNearBorderQ15<C>(im, foldX, foldY, constant, borderPx, sx[k], sy[k]);
                    }
                    else if constexpr (INTERP == NVCV_INTERP_CUBIC)
                    {
                        q[0][k] = SampleNearBorderCubicQ14<C>(im, foldX, foldY, constant, borderPx, sx[k], sy[k]);
                    }
                    else
                    {
                        q[0][k] = SampleNearBorderNearest<C>(im, foldX, foldY, constant, borderPx, sx[k], sy[k]);
                    }
                }
            }
        }
    }
    else
    {
#pragma nounroll
        for (int k = 0; k < kPxPerLane; ++k)
        {
            // position and coordinates recomputed rather than indexed, results placed by selects: a
            // run-time index would put the arrays in scratch memory
            const int patch = wave * kPxPerLane + k;
            const int px = (patch % kPatchesX) * kPatch + lx, py = (patch / kPatchesX) * kPatch + ly;
            const int dx = min(tx * kTileW + px, dstW - 1), dy = min(ty * kTileH + py, dstH - 1);
            float     bx, by;
            MapCoord<PERSP>(m, dx, dy, bx, by);
            bx *= 1.f / kScale;
            by *= 1.f / kScale;
            T v[C];
            if (a.border == NVCV_BORDER_CONSTANT && TapsOutside<INTERP>(im, bx, by))
            {
                SampleAllOutside<T, C, INTERP>(a, bx, by, v);
            }
            else
            {
                SampleWithBorder<T, C, INTERP>(im, a, bx, by, v);
            }
            uint32_t w[D] = {};
            __builtin_memcpy(w, v, PB);
#pragma unroll
            for (int d = 0; d < D; ++d)
            {
#pragma unroll
                for (int j = 0; j < kPxPerLane; ++j)
                {
                    q[d][j] = k == j ? w[d] : q[d][j];
                }
            }
        }
    }

    // ---- store. Pixels of 12 and 16 bytes go out as they are: the 8 lanes of a patch row write 96 or 128
    // contiguous bytes per instruction (gathering 4 pixels per lane first would spread each lane's 48 or 64 bytes
    // over 3 or 4 instructions that each write every 3rd or 4th 16-byte piece: 16 x 1280 x 720 f32x4 NEAREST took
    // 201 us that way and takes 71 us this way)
    if constexpr (PB >= 12)
    {
#pragma unroll
        for (int k = 0; k < kPxPerLane; ++k)
        {
            const int patch = wave * kPxPerLane + k;
            const int px = (patch % kPatchesX) * kPatch + lx, py = (patch / kPatchesX) * kPatch + ly;
            const int dx = tx * kTileW + px, dy = ty * kTileH + py;
            if (dx < dstW && dy < dstH)
            {
                uint32_t w[D];
#pragma unroll
                for (int d = 0; d < D; ++d)
                {
                    w[d] = q[d][k];
                }
                StoreDwordsNT<D>(dst + (int64_t)dy * dstRow + (int64_t)dx * PB, w);
            }
        }
        return;
    }
    // Smaller pixels: the 4 lanes lx & ~3 .. | 3 hold columns 4g .. 4g+3 (g = lx >> 2) of row ly in each of the
    // wave's 4 patches; after a 4x4 transpose lane i = lx & 3 holds those 4 columns of patch 4w + i
#pragma unroll
    for (int d = 0; d < D; ++d)
    {
        QuadTranspose(q[d], lx & 3);
    }
    const int patch = wave * kPxPerLane + (lx & 3);
    const int px0 = (patch % kPatchesX) * kPatch + (lx & 4), py = (patch / kPatchesX) * kPatch + ly;
    const int dy = ty * kTileH + py, dx0 = tx * kTileW + px0;
    if (dy >= dstH || dx0 >= dstW)
    {
        return;
    }
    uint8_t *to = dst + (int64_t)dy * dstRow + (int64_t)dx0 * PB;
    if (dx0 + 4 <= dstW)
    {
        uint32_t w[PB];
        PackQuad<PB>(q, w);
        StoreDwordsNT<PB>(to, w); // 4 pixels = PB dwords
    }
    else
    {
#pragma unroll
        for (int k = 0; k < 3; ++k)
        {
            if (dx0 + k < dstW)
            {
                uint32_t w[D];
#pragma unroll
                for (int d = 0; d < D; ++d)
                {
                    w[d] = q[d][k];
                }
                Vec<T, C> px;
                __builtin_memcpy(&px, w, PB);
                reinterpret_cast<Vec<T, C> *>(to)[k] = px;
            }
        }
    }
}

// Loads image `image`'s matrix from the caller's tensor and, unless it already maps destination to
// source, inverts it (uniform per block). The first two rows come out multiplied by `scale` (a power of
// two: scaling commutes with every rounding of the products and sums that form a coordinate, so
// coordinates computed from the scaled rows are the scaled coordinates bit for bit).
template<bool PERSP>
__device__ __forceinline__ void LoadMatrix(const WarpArgs &a, int image, float scale, float (&m)[9])
{
    const float *p = reinterpret_cast<const float *>(a.xforms + image * a.xformStride);
    float        f[9];
#pragma unroll
    for (int i = 0; i < 9; ++i)
    {
        f[i] = i < (PERSP ? 9 : 6) ? p[i] : 0.f;
    }
    if (a.inverseGiven != 0)
    {
        m[0] = f[0] * scale;
        m[1] = f[1] * scale;
        m[2] = f[2] * scale;
        m[3] = f[3] * scale;
        m[4] = f[4] * scale;
        m[5] = f[5] * scale;
        m[6] = f[6];
        m[7] = f[7];
        m[8] = f[8];
    }
    else if constexpr (!PERSP)
    {
        // affine inverse (reference: warp.cu:139-150, 1/det evaluated in double and rounded to float32, which
        // is what the correctly rounded float32 quotient gives; 1e-5 there is a double: for a float32
        // operand, greater than it means greater than the float32 just below it)
        float den = f[0] * f[4] - f[1] * f[3];
        den       = (fabsf(den) > 9.99999974738e-06f ? 1.f / den : 0.f) * scale;
        m[0]      = f[4] * den;
        m[1]      = -f[1] * den;
        m[2]      = (f[1] * f[5] - f[4] * f[2]) * den;
        m[3]      = -f[3] * den;
        m[4]      = f[0] * den;
        m[5]      = (f[3] * f[2] - f[0] * f[5]) * den;
        m[6] = m[7] = m[8] = 0.f;
    }
    else
    {
        // 3x3 inverse by cofactors (reference: cuda_tools/math/LinAlg.hpp:1446-1450, 1640-1654); a singular
        // matrix is left as given, like the reference's failed in-place inverse
        const float d = f[0] * (f[4] * f[8] - f[5] * f[7]) + f[1] * (f[5] * f[6] - f[3] * f[8])
                      + f[2] * (f[3] * f[7] - f[4] * f[6]);
        const bool  ok = d != 0;
        m[0]           = (ok ? (f[4] * f[8] - f[5] * f[7]) / d : f[0]) * scale;
        m[1]           = (ok ? -(f[1] * f[8] - f[2] * f[7]) / d : f[1]) * scale;
        m[2]           = (ok ? (f[1] * f[5] - f[2] * f[4]) / d : f[2]) * scale;
        m[3]           = (ok ? -(f[3] * f[8] - f[5] * f[6]) / d : f[3]) * scale;
        m[4]           = (ok ? (f[0] * f[8] - f[2] * f[6]) / d : f[4]) * scale;
        m[5]           = (ok ? -(f[0] * f[5] - f[2] * f[3]) / d : f[5]) * scale;
        m[6]           = ok ? (f[3] * f[7] - f[4] * f[6]) / d : f[6];
        m[7]           = ok ? -(f[0] * f[7] - f[1] * f[6]) / d : f[7];
        m[8]           = ok ? (f[0] * f[4] - f[1] * f[3]) / d : f[8];
    }
}

template<class T, int C, int INTERP, bool PERSP>
__global__ __launch_bounds__(kThreads) void WarpTensor(const WarpArgs a)
{
    const int n  = blockIdx.z;
    const Img im = {a.src + n * a.srcN, a.srcRow, a.srcW, a.srcH};
    float     m[9];
#pragma unroll
    for (int i = 0; i < 9; ++i)
    {
        m[i] = a.m[i];
    }
    WarpTile<T, C, INTERP, PERSP>(im, a, m, a.dst + n * a.dstN, a.dstRow, a.dstW, a.dstH, blockIdx.x, blockIdx.y);
}

template<class T, int C, int INTERP, bool PERSP>
__global__ __launch_bounds__(kThreads) void WarpVarShape(const WarpArgs a, const VarTiles tiles)
{
    const TileCoord tc = LocateTile(tiles, blockIdx.x);
    // descriptors and matrix depend on the image index only: read by value here, ahead of the matrix
    // arithmetic, so that all of these loads share one memory round trip
    const NVCVImagePlaneStrided s = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided d = a.dstList[tc.image].planes[0];
    float                       m[9];
    LoadMatrix<PERSP>(a, tc.image, kCoordScale<T, INTERP>, m);
    const Img im = {AsGlobal(s.basePtr), s.rowStride, s.width, s.height};
    WarpTile<T, C, INTERP, PERSP>(im, a, m, AsGlobal(d.basePtr), d.rowStride, d.width, d.height, tc.tx, tc.ty);
}

template<class T, int C, int INTERP, bool PERSP>
void LaunchMap(const WarpArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    if (dstHost == nullptr)
    {
        dim3 grid(DivUp(a.dstW, kTileW), DivUp(a.dstH, kTileH), N);
        hipLaunchKernelGGL((WarpTensor<T, C, INTERP, PERSP>), grid, dim3(kThreads), 0, stream, a);
        CheckLaunch("WarpTensor");
        return;
    }
    for (int first = 0; first < N; first += kMaxTileImages)
    {
        VarTiles tiles;
        int      total = BuildVarTiles(tiles, dstHost, first, std::min(kMaxTileImages, N - first), kTileW, kTileH);
        if (total > 0)
        {
            hipLaunchKernelGGL((WarpVarShape<T, C, INTERP, PERSP>), dim3(total), dim3(kThreads), 0, stream, a, tiles);
            CheckLaunch("WarpVarShape");
        }
    }
}

template<class T, int C, int INTERP>
void Launch(const WarpArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    if (a.perspective)
    {
        LaunchMap<T, C, INTERP, true>(a, N, dstHost, stream);
    }
    else
    {
        LaunchMap<T, C, INTERP, false>(a, N, dstHost, stream);
    }
}

template<class T, int C>
void DispatchInterp(int interp, const WarpArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    switch (interp)
    {
    case NVCV_INTERP_NEAREST:
        Launch<T, C, NVCV_INTERP_NEAREST>(a, N, dstHost, stream);
        break;
    case NVCV_INTERP_LINEAR:
        Launch<T, C, NVCV_INTERP_LINEAR>(a, N, dstHost, stream);
        break;
    case NVCV_INTERP_CUBIC:
        Launch<T, C, NVCV_INTERP_CUBIC>(a, N, dstHost, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid interpolation (supported: NEAREST, LINEAR, CUBIC)");
    }
}

template<class T>
void DispatchC(int C, int interp, const WarpArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    switch (C)
    {
    case 1:
        DispatchInterp<T, 1>(interp, a, N, dstHost, stream);
        break;
    case 3:
        DispatchInterp<T, 3>(interp, a, N, dstHost, stream);
        break;
    case 4:
        DispatchInterp<T, 4>(interp, a, N, dstHost, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", C);
    }
}

void DispatchType(ElemType e, int C, int interp, const WarpArgs &a, int N, const NVCVImageBufferStrided *dstHost,
                  hipStream_t stream)
{
    if (N == 0)
    {
        return;
    }
    switch (e)
    {
    case kU8:
        DispatchC<uint8_t>(C, interp, a, N, dstHost, stream);
        break;
    case kU16:
        DispatchC<uint16_t>(C, interp, a, N, dstHost, stream);
        break;
    case kS16:
        DispatchC<int16_t>(C, interp, a, N, dstHost, stream);
        break;
    case kF32:
        DispatchC<float>(C, interp, a, N, dstHost, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid DataType");
    }
}

void CheckBorder(NVCVBorderType b)
{
    if ((int)b < NVCV_BORDER_CONSTANT || (int)b > NVCV_BORDER_REFLECT101)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid border mode %d", (int)b);
    }
}

void InvertAffineHost(const float *M, float *out)
{
    float den = M[0] * M[4] - M[1] * M[3];
    den       = std::abs(den) > 1e-5 ? 1. / den : .0;
    out[0]    = (float)M[4] * den;
    out[1]    = (float)-M[1] * den;
    out[2]    = (float)(M[1] * M[5] - M[4] * M[2]) * den;
    out[3]    = (float)-M[3] * den;
    out[4]    = (float)M[0] * den;
    out[5]    = (float)(M[3] * M[2] - M[0] * M[5]) * den;
    out[6] = out[7] = out[8] = 0.f;
}

void InvertPerspectiveHost(const float *f, float *m)
{
    const float d
        = f[0] * (f[4] * f[8] - f[5] * f[7]) + f[1] * (f[5] * f[6] - f[3] * f[8]) + f[2] * (f[3] * f[7] - f[4] * f[6]);
    if (d == 0)
    {
        std::copy_n(f, 9, m);
        return;
    }
    m[0] = (f[4] * f[8] - f[5] * f[7]) / d;
    m[1] = -(f[1] * f[8] - f[2] * f[7]) / d;
    m[2] = (f[1] * f[5] - f[2] * f[4]) / d;
    m[3] = -(f[3] * f[8] - f[5] * f[6]) / d;
    m[4] = (f[0] * f[8] - f[2] * f[6]) / d;
    m[5] = -(f[0] * f[5] - f[2] * f[3]) / d;
    m[6] = (f[3] * f[7] - f[4] * f[6]) / d;
    m[7] = -(f[0] * f[7] - f[1] * f[6]) / d;
    m[8] = (f[0] * f[4] - f[1] * f[3]) / d;
}

class Warp : public IOperator
{
public:
    Warp(bool perspective, int32_t maxVarShapeBatchSize)
        : m_perspective(perspective)
        , m_maxBatch(maxVarShapeBatchSize)
    {
        if (maxVarShapeBatchSize < 0)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "maxVarShapeBatchSize must be >= 0");
        }
    }

    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, const float *xform, int32_t flags,
                NVCVBorderType border, float4 bval) const
    {
        if (xform == nullptr)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Transformation matrix must not be NULL");
        }
        NVCVTensorData din, dout;
        ExportTensor(hin, din, "Input");
        ExportTensor(hout, dout, "Output");
        ImageBatchView in  = RequireImageBatchView(din, "Input", NVCV_ERROR_INVALID_ARGUMENT);
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
        if (in.layout != kLayoutNHWC || out.layout != kLayoutNHWC || in.hasBatchDim != out.hasBatchDim)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Invalid DataFormat between input (%s) and output (%s): both must be \"NHWC\" or \"HWC\"",
                          in.layoutName, out.layoutName);
        }
        if (in.C > 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", in.C);
        }
        if (in.elem != out.elem || in.C != out.C || in.N != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Input and output must have the same data type, channel count and batch size");
        }
        if (std::max(in.bytesSpanned(), out.bytesSpanned()) > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output size exceeds %d. Tensor is too large.",
                          INT32_MAX);
        }
        CheckBorder(border);
        WarpArgs a = makeArgs(border, bval);
        if (flags & NVCV_WARP_INVERSE_MAP)
        {
            for (int i = 0; i < 9; ++i)
            {
                a.m[i] = i < (m_perspective ? 9 : 6) ? xform[i] : 0.f;
            }
        }
        else if (m_perspective)
        {
            InvertPerspectiveHost(xform, a.m);
        }
        else
        {
            InvertAffineHost(xform, a.m);
        }
        if (in.elem == kU8 && (flags & NVCV_INTERP_MAX) == NVCV_INTERP_LINEAR)
        {
            for (int i = 0; i < 6; ++i)
            {
                a.m[i] *= kCoordScale<uint8_t, NVCV_INTERP_LINEAR>; // see kCoordScale
            }
        }
        a.src    = in.base;
        a.dst    = out.base;
        a.srcN   = in.strideN;
        a.dstN   = out.strideN;
        a.srcRow = (int32_t)in.strideH;
        a.dstRow = (int32_t)out.strideH;
        a.srcW   = in.W;
        a.srcH   = in.H;
        a.dstW   = out.W;
        a.dstH   = out.H;
        if (out.W == 0 || out.H == 0 || in.W == 0 || in.H == 0)
        {
            return;
        }
        DispatchType(in.elem, in.C, flags & NVCV_INTERP_MAX, a, in.N, nullptr, stream);
    }

    void submit(hipStream_t stream, NVCVImageBatchHandle hin, NVCVImageBatchHandle hout, NVCVTensorHandle hxform,
                int32_t flags, NVCVBorderType border, float4 bval) const
    {
        if (m_maxBatch <= 0)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Operator was not created for var-shape use, maxVarShapeBatchSize: %d", m_maxBatch);
        }
        VarShapeView in  = ExportVarShape(hin, stream, "Input");
        VarShapeView out = ExportVarShape(hout, stream, "Output");
        if (in.N > m_maxBatch)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid number of images, it should not exceed %d", m_maxBatch);
        }
        if (in.N != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input and output batch sizes: %d != %d", in.N, out.N);
        }
        if (in.uniqueFormat == NVCV_IMAGE_FORMAT_NONE || in.uniqueFormat != out.uniqueFormat)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Images in the input and output varshape must all have the same format");
        }
        FormatInfo fi = DecodeFormat(in.uniqueFormat);
        if (fi.planes != 1)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images must have a single interleaved plane");
        }
        if (fi.channels > 4)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid channel number %d", fi.channels);
        }
        CheckBorder(border);
        NVCVTensorData dx;
        ExportTensor(hxform, dx, "Transformation matrix");
        const int  cols = m_perspective ? 9 : 6;
        DTypeInfo  dt   = DecodeDataType(dx.dtype);
        const bool ok   = dt.elem == kF32 && dt.channels == 1 && dx.rank == 2 && dx.shape[0] >= in.N
                     && dx.shape[1] == cols && dx.buffer.strided.strides[1] == 4;
        if (!ok)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "Transformation matrix tensor must be float32 of shape [N,%d] with packed rows, N >= %d", cols,
                          in.N);
        }
        WarpArgs a     = makeArgs(border, bval);
        a.srcList      = in.data.buffer.varShapeStrided.imageList;
        a.dstList      = out.data.buffer.varShapeStrided.imageList;
        a.xforms       = dx.buffer.strided.basePtr;
        a.xformStride  = dx.buffer.strided.strides[0];
        a.inverseGiven = (flags & NVCV_WARP_INVERSE_MAP) ? 1 : 0;
        DispatchType(fi.elem, fi.channels, flags & NVCV_INTERP_MAX, a, in.N, out.hostList, stream);
    }

private:
    WarpArgs makeArgs(NVCVBorderType border, float4 bval) const
    {
        WarpArgs a    = {};
        a.perspective = m_perspective ? 1 : 0;
        a.border      = (int32_t)border;
        a.bval[0]     = bval.x;
        a.bval[1]     = bval.y;
        a.bval[2]     = bval.z;
        a.bval[3]     = bval.w;
        return a;
    }

    bool    m_perspective;
    int32_t m_maxBatch;
};

class WarpAffine final : public Warp
{
public:
    explicit WarpAffine(int32_t maxBatch)
        : Warp(false, maxBatch)
    {
    }
};

class WarpPerspective final : public Warp
{
public:
    explicit WarpPerspective(int32_t maxBatch)
        : Warp(true, maxBatch)
    {
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaWarpAffineCreate(NVCVOperatorHandle *handle, const int32_t maxVarShapeBatchSize)
{
    return CreateOperator<WarpAffine>(handle, maxVarShapeBatchSize);
}

CVCUDA_PUBLIC NVCVStatus cvcudaWarpAffineSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                                NVCVTensorHandle out, const NVCVAffineTransform xform,
                                                const int32_t flags, const NVCVBorderType borderMode,
                                                const float4 borderValue)
{
    return Protect([&] { ToOperator<WarpAffine>(handle).submit(stream, in, out, xform, flags, borderMode, borderValue); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaWarpAffineVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                        NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                        NVCVTensorHandle transMatrix, const int32_t flags,
                                                        const NVCVBorderType borderMode, const float4 borderValue)
{
    return Protect(
        [&] { ToOperator<WarpAffine>(handle).submit(stream, in, out, transMatrix, flags, borderMode, borderValue); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaWarpPerspectiveCreate(NVCVOperatorHandle *handle, const int32_t maxVarShapeBatchSize)
{
    return CreateOperator<WarpPerspective>(handle, maxVarShapeBatchSize);
}

CVCUDA_PUBLIC NVCVStatus cvcudaWarpPerspectiveSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                                     NVCVTensorHandle out, const NVCVPerspectiveTransform transMatrix,
                                                     const int32_t flags, const NVCVBorderType borderMode,
                                                     const float4 borderValue)
{
    return Protect(
        [&] { ToOperator<WarpPerspective>(handle).submit(stream, in, out, transMatrix, flags, borderMode, borderValue); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaWarpPerspectiveVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                             NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                             NVCVTensorHandle transMatrix, const int32_t flags,
                                                             const NVCVBorderType borderMode, const float4 borderValue)
{
    return Protect(
        [&]
        { ToOperator<WarpPerspective>(handle).submit(stream, in, out, transMatrix, flags, borderMode, borderValue); });
}
}
