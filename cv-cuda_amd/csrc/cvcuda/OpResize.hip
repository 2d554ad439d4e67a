// Resize with nearest / bilinear / bicubic / area sampling, tensors and var-shape batches.
//
// Index maps and weights follow the reference kernels expression for expression in float32
// (src/cvcuda/priv/OpResize.cu:142-164 nearest, 177-330 bilinear, 334-388 bicubic;
// src/cvcuda/priv/legacy/resize_var_shape.cu:92-231 for the var-shape association of the sums).
// The nearest-neighbour source index uses the single-multiply form floor((d+.5f)*scale) of the
// reference's CPU golden (tests/cvcuda/system/ResizeUtils.cpp:206-221) for every pixel, so results
// are bit-exact against it also where the coordinate lands on an integer. 8-bit pixels are blended in fixed
// point on those indices and weights (bilinear: FixedPointBlend.hpp; bicubic: kFixedCubic; box filter:
// kAreaFixed), at most 1 from the reference's goldens.
//
// Six kernel shapes, all with streaming stores, var-shape batches on a packed tile grid:
//  * pixels of up to 8 bytes: wave patches (64 columns x 4 rows per wave; adjacent taps in one load,
//    row terms computed once per wave, 4x4 lane transposes so that every lane stores whole dwords);
//  * 8-bit bilinear at horizontal scales up to 2: a lane owns 2 columns x 4 rows (image batches x 2; 4 x 8 when
//    enlarging by 1.5 or more) and fetches each source row once for all its columns and rows, lane pairs swap a
//    pixel pair each;
//    nearest neighbour takes the same strips when enlarging by 1.5 or more;
//  * 8-bit bicubic tensors of 3 and 4 channels at vertical scales of 1/2 to 2, large launches: a wave owns 64 columns
//    x 16 rows and forms every source row's sums once, adding them to the output rows in flight;
//  * bicubic reductions >= 2x of 12/16-byte pixels: tap-major loads exchanged through LDS;
//  * AREA of 8-bit pixels at reductions of up to 3: fixed-point row sums, a wave owns 64 columns x 16 rows and
//    produces vertically adjacent rows in pairs from the source rows they share;
//  * everything else (12/16-byte pixels, other AREA): one lane per output pixel, a 256-thread block covers
//    64 columns x 4 rows, pixels moved as whole C-channel vectors.
#include "DeviceUtils.hpp"
#include "FixedPointBlend.hpp"
#include "LaneExchange.hpp"
#include "OpCommon.hpp"
#include "RunIO.hpp"
#include "VarShapeTiles.hpp"

#include <cvcuda/OpResize.h>

#include <algorithm>
#include <type_traits>

namespace cvamd {

namespace {

constexpr int kTileW = 64;
constexpr int kTileH = 4;

template<class T, int C>
using Pixel = Packed<T, C>;

struct ResizeArgs
{
    // tensors
    const uint8_t *srcBase;
    uint8_t       *dstBase;
    int64_t        srcSampleStride, dstSampleStride;
    int32_t        srcRowStride, dstRowStride;
    int32_t        srcW, srcH, dstW, dstH;
    float          scaleX, scaleY; // srcW / dstW, srcH / dstH in float32 (var-shape: per image, in the kernel)
    // var-shape
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
};

struct Plane
{
    const uint8_t *src;
    uint8_t       *dst;
    int32_t        srcRow, dstRow, srcW, srcH, dstW, dstH;
    float          scaleX, scaleY;
};

template<bool VARSHAPE>
__device__ __forceinline__ Plane GetPlanes(const ResizeArgs &a, int n)
{
    Plane p;
    if constexpr (VARSHAPE)
    {
        const NVCVImagePlaneStrided &s = a.srcList[n].planes[0];
        const NVCVImagePlaneStrided &d = a.dstList[n].planes[0];
        p = {AsGlobal(s.basePtr),
             AsGlobal(d.basePtr),
             s.rowStride,
             d.rowStride,
             s.width,
             s.height,
             d.width,
             d.height,
             static_cast<float>(s.width) / d.width,
             static_cast<float>(s.height) / d.height};
    }
    else
    {
        p = {a.srcBase + n * a.srcSampleStride,
             a.dstBase + n * a.dstSampleStride,
             a.srcRowStride,
             a.dstRowStride,
             a.srcW,
             a.srcH,
             a.dstW,
             a.dstH,
             a.scaleX,
             a.scaleY};
    }
    return p;
}

template<class T, int C>
__device__ __forceinline__ Pixel<T, C> LoadPx(const uint8_t *row, int x)
{
    return reinterpret_cast<const Pixel<T, C> *>(row)[x];
}

template<class T, int C>
__device__ __forceinline__ void StorePx(uint8_t *row, int x, const Pixel<T, C> &px)
{
    Pixel<T, C> *p = reinterpret_cast<Pixel<T, C> *>(row) + x;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        __builtin_nontemporal_store(px.v[c], &p->v[c]);
    }
}

// N horizontally adjacent pixels at byte offset `xoff` of source row `row` (all inside the image).
// u8x3: 1 or 2 pixels are fetched with a 4- or 8-byte load that reads 1-2 bytes past them, harmless
// except behind the image's last row (`lastRow`, wave-uniform), where the load is moved back to end
// with the row's `rowBytes` and the value shifted; rows shorter than the load are read byte by byte.
template<class T, int C, int N>
__device__ __forceinline__ void LoadTaps(const uint8_t *row, int xoff, bool lastRow, int rowBytes, float (&t)[N][C])
{
    if constexpr (std::is_same_v<T, uint8_t> && C == 3 && N == 1)
    {
        uint32_t q;
        if (lastRow && rowBytes < 4) // a 1-pixel-wide image: moving the load back would leave the row (and a 1 x 1 image)
        {
            q = row[xoff] | (row[xoff + 1] << 8) | (row[xoff + 2] << 16);
        }
        else if (lastRow)
        {
            const int back = max(0, xoff - (rowBytes - 4));
            q              = LoadU32Unaligned(row + (xoff - back)) >> (8 * back);
        }
        else
        {
            q = LoadU32Unaligned(row + xoff);
        }
        t[0][0] = (float)(q & 0xFF);
        t[0][1] = (float)((q >> 8) & 0xFF);
        t[0][2] = (float)((q >> 16) & 0xFF);
    }
    else if constexpr (std::is_same_v<T, uint8_t> && C == 3 && N == 2)
    {
        uint64_t q;
        if (lastRow && rowBytes < 8) // a 2-pixel-wide image (the two taps are all of the row)
        {
            q = 0;
#pragma unroll
            for (int i = 0; i < 6; ++i)
            {
                q |= (uint64_t)row[xoff + i] << (8 * i);
            }
        }
        else if (lastRow)
        {
            const int back = max(0, xoff - (rowBytes - 8));
            q              = LoadU64Unaligned(row + (xoff - back)) >> (8 * back);
        }
        else
        {
            q = LoadU64Unaligned(row + xoff);
        }
        const uint32_t lo = (uint32_t)q, hi = (uint32_t)(q >> 32);
        t[0][0] = (float)(lo & 0xFF);
        t[0][1] = (float)((lo >> 8) & 0xFF);
        t[0][2] = (float)((lo >> 16) & 0xFF);
        t[1][0] = (float)(lo >> 24);
        t[1][1] = (float)(hi & 0xFF);
        t[1][2] = (float)((hi >> 8) & 0xFF);
    }
    else
    {
        const Pixel<T, N *C> v = *reinterpret_cast<const Pixel<T, N * C> *>(row + xoff);
#pragma unroll
        for (int i = 0; i < N; ++i)
        {
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                t[i][c] = (float)v.v[i * C + c];
            }
        }
    }
}

// Two horizontally adjacent 8-bit pixels as raw bytes (byte i of {w[1]:w[0]} = channel i % C of pixel i / C);
// the same loads as LoadTaps<uint8_t, C, 2>.
template<int C>
__device__ __forceinline__ void LoadTapPairBytes(const uint8_t *row, int xoff, bool lastRow, int rowBytes, uint32_t (&w)[2])
{
    if constexpr (C == 3)
    {
        uint64_t q;
        if (lastRow && rowBytes < 8)
        {
            q = 0;
#pragma unroll
            for (int i = 0; i < 6; ++i)
            {
                q |= (uint64_t)row[xoff + i] << (8 * i);
            }
        }
        else if (lastRow)
        {
            const int back = max(0, xoff - (rowBytes - 8));
            q              = LoadU64Unaligned(row + (xoff - back)) >> (8 * back);
        }
        else
        {
            q = LoadU64Unaligned(row + xoff);
        }
        w[0] = (uint32_t)q;
        w[1] = (uint32_t)(q >> 32);
    }
    else
    {
        const Pixel<uint8_t, 2 * C> v = *reinterpret_cast<const Pixel<uint8_t, 2 * C> *>(row + xoff);
        w[0] = w[1] = 0;
        __builtin_memcpy(w, &v, 2 * C);
    }
}

// Four horizontally adjacent 8-bit pixels as raw bytes (the box filter's and the bicubic blend's row window): the
// D dwords that hold the 4 pixels at byte offset `at` + `shift` of the row (shift 0 .. 3; 4 channels: none),
// brought to the front: pixel k, channel c in byte k * C + c.
template<int C, bool GUARDED>
__device__ __forceinline__ void LoadQuadWindow(const uint8_t *row, uint32_t at, uint32_t shift, bool lastRow, uint32_t rowBytes,
                                               uint32_t (&r)[C])
{
    constexpr int D = C == 4 ? 4 : C + 1;
    struct __attribute__((packed, aligned(1))) Window
    {
        uint32_t d[D];
    };
    if constexpr (C == 4)
    {
        const Window w = *reinterpret_cast<const Window *>(row + at);
        __builtin_memcpy(r, &w, 16);
    }
    else
    {
        // the load runs up to 4 bytes past the window, harmless except behind the image's last row, where it is
        // moved back to end with the row (GUARDED: the rows passed may include that one)
        bool whole = false;
        if (GUARDED && lastRow)
        {
            const uint32_t back = min(at, rowBytes - 4 * D);
            shift += at - back; // up to 4
            at    = back;
            whole = shift == 4;
            shift = whole ? 0 : shift;
        }
        const Window w = *reinterpret_cast<const Window *>(row + at);
#pragma unroll
        for (int i = 0; i < C; ++i)
        {
            r[i] = __builtin_amdgcn_alignbyte(w.d[i + 1], w.d[i], shift);
            if constexpr (GUARDED)
            {
                r[i] = whole ? w.d[i + 1] : r[i];
            }
        }
    }
}

// Channel c of pixels ka and ka + 1 of such a window as (first | second << 16).
template<int C>
__device__ __forceinline__ uint32_t QuadTapPair(const uint32_t (&r)[C], int ka, int c)
{
    const int      b0 = ka * C + c, b1 = b0 + C, j = b0 / 4;
    const uint32_t sel = 0x0c000c00u | (uint32_t)(b0 - 4 * j) | ((uint32_t)(b1 - 4 * j) << 16);
    return __builtin_amdgcn_perm(r[j + 1 < C ? j + 1 : C - 1], r[j], sel);
}

__device__ __forceinline__ void CubicCoeffs(float d, float (&w)[4])
{
    constexpr float A = -0.75f;
    w[0]              = ((A * (d + 1) - 5 * A) * (d + 1) + 8 * A) * (d + 1) - 4 * A;
    w[1]              = ((A + 2) * d - (A + 3)) * d * d + 1;
    w[2]              = ((A + 2) * (1 - d) - (A + 3)) * (1 - d) * (1 - d) + 1;
    w[3]              = 1.f - w[0] - w[1] - w[2];
}

// 8-bit pixels are blended bilinearly in 15-bit fixed point (FixedPointBlend.hpp), tensors and image
// batches alike, whichever kernel form a shape takes: the weight of the second tap along an axis (0 .. 1,
// the reference's float32 expression) is cut to a multiple of 2^-15.
template<class T>
constexpr bool kFixedLinear = std::is_same_v<T, uint8_t>;

// 8-bit pixels are blended bicubically with the four horizontal weights (the reference's float32 polynomials)
// rounded to multiples of 2^-14, the last one taking the remainder so that they add up to exactly 1; a row's four
// taps are combined in integers (exact), the four row sums in float32 with the vertical weights, ascending, by
// fused multiply-adds; the magnitude is rounded once. Tensors and image batches alike, whichever kernel form a
// shape takes. Within 0.05 of the float32 expression, i.e. at most 1 from the reference's golden.
template<class T>
constexpr bool kFixedCubic = std::is_same_v<T, uint8_t>;

__device__ __forceinline__ uint32_t FractionQ15(float w)
{
    return (uint32_t)(w * 32768.f);
}

template<class T, int C, int INTERP, bool VARSHAPE>
__device__ __forceinline__ Pixel<T, C> ResizeValue(const Plane &p, int dx, int dy)
{
    const float scaleX = p.scaleX, scaleY = p.scaleY;
    Pixel<T, C> out;

    if constexpr (INTERP == NVCV_INTERP_NEAREST)
    {
        const int sx = min((int)floorf(scaleX * (dx + 0.5f)), p.srcW - 1);
        const int sy = min((int)floorf(scaleY * (dy + 0.5f)), p.srcH - 1);
        out          = LoadPx<T, C>(p.src + (int64_t)sy * p.srcRow, sx);
    }
    else if constexpr (INTERP == NVCV_INTERP_LINEAR)
    {
        const float fx = (dx + .5f) * scaleX - .5f;
        const float fy = (dy + .5f) * scaleY - .5f;
        int         sx = (int)floorf(fx);
        int         sy = (int)floorf(fy);
        const float wx = (sx < 0) ? 0.f : ((sx > p.srcW - 2) ? 1.f : fx - sx);
        const float wy = (sy < 0) ? 0.f : ((sy > p.srcH - 2) ? 1.f : fy - sy);
        sx             = max(0, min(sx, p.srcW - 2));
        sy             = max(0, min(sy, p.srcH - 2));
        // a 1-pixel-wide (or -high) source has no second tap: reuse the first (its weight is then 0 or
        // multiplies an equal value)
        const int sx1 = min(sx + 1, p.srcW - 1);
        sx            = max(sx, 0);
        const uint8_t *r0 = p.src + (int64_t)max(sy, 0) * p.srcRow;
        const uint8_t *r1 = p.src + (int64_t)min(sy + 1, p.srcH - 1) * p.srcRow;
        const Pixel<T, C> p00 = LoadPx<T, C>(r0, sx), p01 = LoadPx<T, C>(r0, sx1);
        const Pixel<T, C> p10 = LoadPx<T, C>(r1, sx), p11 = LoadPx<T, C>(r1, sx1);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            if constexpr (kFixedLinear<T>)
            {
                out.v[c] = BilinearQ15Scalar(p00.v[c], p01.v[c], p10.v[c], p11.v[c], FractionQ15(wx), FractionQ15(wy));
                continue;
            }
            float v;
            if constexpr (VARSHAPE)
            {
                v = (1.0f - wx) * ((float)p00.v[c] * (1.0f - wy) + (float)p10.v[c] * wy)
                  + wx * ((float)p01.v[c] * (1.0f - wy) + (float)p11.v[c] * wy);
            }
            else
            {
                v = (float)p00.v[c] * ((1.f - wx) * (1.f - wy)) + (float)p01.v[c] * (wx * (1.f - wy))
                  + (float)p10.v[c] * ((1.f - wx) * wy) + (float)p11.v[c] * (wx * wy);
            }
            out.v[c] = SaturateCast<T>(v);
        }
    }
    else if constexpr (INTERP == NVCV_INTERP_AREA)
    {
        // box filter over the source rectangle the output pixel covers, partial pixels weighted by
        // their covered fraction; taps outside the image read 0 (reference:
        // cuda_tools/InterpolationWrap.hpp:668-760, accumulation order kept)
        const float fsx1 = dx * scaleX, fsy1 = dy * scaleY;
        const float fsx2 = fsx1 + scaleX, fsy2 = fsy1 + scaleY;
        const int   xmin = (int)ceilf(fsx1), xmax = (int)floorf(fsx2);
        const int   ymin = (int)ceilf(fsy1), ymax = (int)floorf(fsy2);
        float       sum[C];
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            sum[c] = 0.f;
        }
        // pixels [xa, xb) of row y, each with weight w, in ascending order; what lies outside the image
        // contributes nothing, so the range is clipped once instead of testing every tap
        auto addRun = [&](int xa, int xb, int y, float w)
        {
            if (y < 0 || y >= p.srcH)
            {
                return;
            }
            // small pixels are fetched G at a time (one load of up to 16 bytes) and added in the same order
            constexpr int  PB  = (int)sizeof(Pixel<T, C>), G = PB <= 4 ? 4 : (PB <= 8 ? 2 : 1);
            const uint8_t *row = p.src + (int64_t)y * p.srcRow;
            xb                 = min(xb, p.srcW);
            int x              = max(xa, 0);
            if constexpr (G > 1)
            {
                for (; x + G <= xb; x += G)
                {
                    float t[G][C];
                    LoadTaps<T, C, G>(row, x * PB, y == p.srcH - 1, p.srcW * PB, t);
#pragma unroll
                    for (int k = 0; k < G; ++k)
                    {
#pragma unroll
                        for (int c = 0; c < C; ++c)
                        {
                            sum[c] += t[k][c] * w;
                        }
                    }
                }
            }
            for (; x < xb; ++x)
            {
                float t[1][C];
                LoadTaps<T, C, 1>(row, x * PB, y == p.srcH - 1, p.srcW * PB, t);
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    sum[c] += t[0][c] * w;
                }
            }
        };
        auto add = [&](int x, int y, float w) { addRun(x, x + 1, y, w); };
        // u8 pixels of 1, 3 or 4 channels at horizontal scales up to 2: the taps of one source row (a partial pixel on
        // the left, up to 2 whole ones, a partial one on the right) lie within 4 pixels, one load of 4 pixels instead
        // of one per tap (u8x3: a 2- and a 1-byte load per tap before; 226 -> 151 us per 32 x 1080p -> 720p). Which taps exist differs from lane to
        // lane, their order in the sums does not. The kernel is bound by the bytes its lanes ask for, not by
        // latency: with the windows of the 4 rows from ymin - 1 on all loaded before the first sum (4 loads
        // where 2 or 3 are needed) it took 208 us. Rows before the image's last one only: a load may read up
        // to 3 pixels past its taps.
        bool windowed = false;
        if constexpr (std::is_same_v<T, uint8_t> && (C == 1 || C == 3 || C == 4))
        {
            windowed = scaleX <= 2.f && p.srcW >= 4 && ymax < p.srcH - 1;
        }
        const bool hasLeft = xmin > fsx1, hasRight = xmax < fsx2;
        const int  winX = xmin - (hasLeft ? 1 : 0), innerN = min(xmax, p.srcW) - xmin, rightI = xmax - winX;
        [[maybe_unused]] auto loadWindow = [&](int y, uint32_t (&px)[4])
        {
            // 4 pixels of C bytes, pixel k to px[k] (channel c in byte c; higher bytes are not looked at)
            uint32_t w[C];
            LoadDwords<C>(p.src + (int64_t)y * p.srcRow + winX * C, w);
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                if constexpr (C == 1)
                {
                    px[k] = w[0] >> (8 * k);
                }
                else if constexpr (C == 4)
                {
                    px[k] = w[k];
                }
                else
                {
                    px[k] = k == 0 ? w[0]
                          : k == 1 ? __builtin_amdgcn_alignbit(w[C > 1 ? 1 : 0], w[0], 24)
                          : k == 2 ? __builtin_amdgcn_alignbit(w[C > 2 ? 2 : 0], w[C > 1 ? 1 : 0], 16)
                                   : w[C > 2 ? 2 : 0] >> 8;
                }
            }
        };
        [[maybe_unused]] auto addPx = [&](uint32_t q, float w)
        {
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                sum[c] += (float)((q >> (8 * c)) & 0xFF) * w;
            }
        };
        [[maybe_unused]] auto addInner = [&](const uint32_t (&px)[4], float w) // pixels [xmin, xmax) of the row
        {
#pragma unroll
            for (int k = 0; k < 2; ++k)
            {
                if (k < innerN)
                {
                    addPx(hasLeft ? px[k + 1] : px[k], w);
                }
            }
        };
        [[maybe_unused]] auto addLeft  = [&](const uint32_t (&px)[4], float w) { addPx(px[0], w); }; // pixel xmin - 1
        [[maybe_unused]] auto addRight = [&](const uint32_t (&px)[4], float w)                        // pixel xmax
        {
            if (xmax < p.srcW)
            {
                addPx(rightI == 0 ? px[0] : rightI == 1 ? px[1] : rightI == 2 ? px[2] : px[3], w);
            }
        };
        // the rows between the partial ones: whole pixels, then the partial ones left and right
        [[maybe_unused]] auto addInnerRows = [&](float scale, bool partials)
        {
            for (int cy = ymin; cy < ymax; ++cy)
            {
                uint32_t px[4];
                loadWindow(cy, px);
                addInner(px, scale);
                if (partials && hasLeft)
                {
                    addLeft(px, (xmin - fsx1) * scale);
                }
                if (partials && hasRight)
                {
                    addRight(px, (fsx2 - xmax) * scale);
                }
            }
        };
        if (windowed && VARSHAPE && scaleX >= 1.0f && scaleY >= 1.0f)
        {
            const int iscaleX = SaturateCast<int32_t>(scaleX), iscaleY = SaturateCast<int32_t>(scaleY);
            if (scaleX == (float)iscaleX && scaleY == (float)iscaleY)
            {
                addInnerRows(1.f / (scaleX * scaleY), false);
            }
            else
            {
                // whole pixels of both partial rows, then the corners (top left, top right, bottom right, bottom left)
                const float scale = 1.f / (fminf(scaleX, p.srcW - fsx1) * fminf(scaleY, p.srcH - fsy1));
                addInnerRows(scale, true);
                uint32_t top[4] = {}, bot[4] = {};
                if (ymin > fsy1)
                {
                    loadWindow(ymin - 1, top);
                    addInner(top, (ymin - fsy1) * scale);
                }
                if (ymax < fsy2)
                {
                    loadWindow(ymax, bot);
                    addInner(bot, (fsy2 - ymax) * scale);
                }
                if (ymin > fsy1 && hasLeft)
                {
                    addLeft(top, (ymin - fsy1) * (xmin - fsx1) * scale);
                }
                if (ymin > fsy1 && hasRight)
                {
                    addRight(top, (ymin - fsy1) * (fsx2 - xmax) * scale);
                }
                if (ymax < fsy2 && hasRight)
                {
                    addRight(bot, (fsy2 - ymax) * (fsx2 - xmax) * scale);
                }
                if (ymax < fsy2 && hasLeft)
                {
                    addLeft(bot, (fsy2 - ymax) * (xmin - fsx1) * scale);
                }
            }
        }
        else if (windowed && !VARSHAPE)
        {
            if (ceilf(scaleX) == scaleX && ceilf(scaleY) == scaleY)
            {
                addInnerRows(1.f / (scaleX * scaleY), false);
            }
            else
            {
                const float scale = 1.f / (fminf(scaleX, p.srcW - fsx1) * fminf(scaleY, p.srcH - fsy1));
                addInnerRows(scale, true);
                if (ymin > fsy1)
                {
                    uint32_t px[4];
                    loadWindow(ymin - 1, px);
                    addInner(px, (ymin - fsy1) * scale);
                    if (hasLeft)
                    {
                        addLeft(px, (ymin - fsy1) * (xmin - fsx1) * scale);
                    }
                    if (hasRight)
                    {
                        addRight(px, (ymin - fsy1) * (fsx2 - xmax) * scale);
                    }
                }
                if (ymax < fsy2)
                {
                    uint32_t px[4];
                    loadWindow(ymax, px);
                    addInner(px, (fsy2 - ymax) * scale);
                    if (hasRight)
                    {
                        addRight(px, (fsy2 - ymax) * (fsx2 - xmax) * scale);
                    }
                    if (hasLeft)
                    {
                        addLeft(px, (fsy2 - ymax) * (xmin - fsx1) * scale);
                    }
                }
            }
        }
        else if constexpr (VARSHAPE)
        {
            // image batches follow the reference's separate kernel (legacy/resize_var_shape.cu:236-428):
            // same sums for reductions, corners added last; enlargements are a bilinear variant whose
            // fractions come from the inverse scale in double
            const int  iscaleX = SaturateCast<int32_t>(scaleX), iscaleY = SaturateCast<int32_t>(scaleY);
            const bool fast    = scaleX == (float)iscaleX && scaleY == (float)iscaleY;
            if (scaleX >= 1.0f && scaleY >= 1.0f)
            {
                if (fast)
                {
                    const float scale = 1.f / (scaleX * scaleY);
                    for (int cy = ymin; cy < ymax; ++cy)
                    {
                        addRun(xmin, xmax, cy, scale);
                    }
                }
                else
                {
                    const float scale = 1.f / (fminf(scaleX, p.srcW - fsx1) * fminf(scaleY, p.srcH - fsy1));
                    for (int cy = ymin; cy < ymax; ++cy)
                    {
                        addRun(xmin, xmax, cy, scale);
                        if (xmin > fsx1)
                        {
                            add(xmin - 1, cy, (xmin - fsx1) * scale);
                        }
                        if (xmax < fsx2)
                        {
                            add(xmax, cy, (fsx2 - xmax) * scale);
                        }
                    }
                    if (ymin > fsy1)
                    {
                        addRun(xmin, xmax, ymin - 1, (ymin - fsy1) * scale);
                    }
                    if (ymax < fsy2)
                    {
                        addRun(xmin, xmax, ymax, (fsy2 - ymax) * scale);
                    }
                    if (ymin > fsy1 && xmin > fsx1)
                    {
                        add(xmin - 1, ymin - 1, (ymin - fsy1) * (xmin - fsx1) * scale);
                    }
                    if (ymin > fsy1 && xmax < fsx2)
                    {
                        add(xmax, ymin - 1, (ymin - fsy1) * (fsx2 - xmax) * scale);
                    }
                    if (ymax < fsy2 && xmax < fsx2)
                    {
                        add(xmax, ymax, (fsy2 - ymax) * (fsx2 - xmax) * scale);
                    }
                    if (ymax < fsy2 && xmin > fsx1)
                    {
                        add(xmin - 1, ymax, (fsy2 - ymax) * (xmin - fsx1) * scale);
                    }
                }
            }
            else
            {
                const double invX = 1. / scaleX, invY = 1. / scaleY;
                int          sy = (int)floorf(dy * scaleY);
                float        fy = (float)((dy + 1) - (sy + 1) * invY);
                fy              = fy <= 0 ? 0.f : fy - (int)floorf(fy);
                int   sx = (int)floorf(dx * scaleX);
                float fx = (float)((dx + 1) - (sx + 1) * invX);
                fx       = fx < 0 ? 0.f : fx - (int)floorf(fx);
                if (sx < 0)
                {
                    fx = 0, sx = 0;
                }
                if (sx >= p.srcW - 1)
                {
                    fx = 0, sx = p.srcW - 2;
                }
                if (sy >= p.srcH - 1)
                {
                    sy = p.srcH - 2;
                }
                // sources of one row or column: the reference indexes outside the image; taps clamped here
                const int      x0 = max(sx, 0), x1 = min(sx + 1, p.srcW - 1), y0 = max(sy, 0), y1 = min(sy + 1, p.srcH - 1);
                const uint8_t *r0 = p.src + (int64_t)y0 * p.srcRow, *r1 = p.src + (int64_t)y1 * p.srcRow;
                const Pixel<T, C> p00 = LoadPx<T, C>(r0, x0), p10 = LoadPx<T, C>(r1, x0);
                const Pixel<T, C> p01 = LoadPx<T, C>(r0, x1), p11 = LoadPx<T, C>(r1, x1);
                const float       cx0 = 1.f - fx, cx1 = fx, cy0 = 1.f - fy, cy1 = fy;
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    sum[c] = (float)p00.v[c] * cx0 * cy0 + (float)p10.v[c] * cx0 * cy1 + (float)p01.v[c] * cx1 * cy0
                           + (float)p11.v[c] * cx1 * cy1;
                }
            }
        }
        else if (ceilf(scaleX) == scaleX && ceilf(scaleY) == scaleY)
        {
            const float scale = 1.f / (scaleX * scaleY);
            for (int cy = ymin; cy < ymax; ++cy)
            {
                addRun(xmin, xmax, cy, scale);
            }
        }
        else
        {
            const float scale = 1.f / (fminf(scaleX, p.srcW - fsx1) * fminf(scaleY, p.srcH - fsy1));
            for (int cy = ymin; cy < ymax; ++cy)
            {
                addRun(xmin, xmax, cy, scale);
                if (xmin > fsx1)
                {
                    add(xmin - 1, cy, (xmin - fsx1) * scale);
                }
                if (xmax < fsx2)
                {
                    add(xmax, cy, (fsx2 - xmax) * scale);
                }
            }
            if (ymin > fsy1)
            {
                addRun(xmin, xmax, ymin - 1, (ymin - fsy1) * scale);
                if (xmin > fsx1)
                {
                    add(xmin - 1, ymin - 1, (ymin - fsy1) * (xmin - fsx1) * scale);
                }
                if (xmax < fsx2)
                {
                    add(xmax, ymin - 1, (ymin - fsy1) * (fsx2 - xmax) * scale);
                }
            }
            if (ymax < fsy2)
            {
                addRun(xmin, xmax, ymax, (fsy2 - ymax) * scale);
                if (xmax < fsx2)
                {
                    add(xmax, ymax, (fsy2 - ymax) * (fsx2 - xmax) * scale);
                }
                if (xmin > fsx1)
                {
                    add(xmin - 1, ymax, (fsy2 - ymax) * (xmin - fsx1) * scale);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out.v[c] = SaturateCast<T>(sum[c]);
        }
    }
    else // cubic
    {
        const float cx = (dx + .5f) * scaleX - .5f;
        const float cy = (dy + .5f) * scaleY - .5f;
        int         sx = (int)floorf(cx);
        int         sy = (int)floorf(cy);
        float       fx = cx - sx;
        const float fy = cy - sy;
        fx             = (sx < 1 || sx >= p.srcW - 3) ? 0.f : fx;
        sy             = max(1, min(sy, p.srcH - 3));
        sx             = max(1, min(sx, p.srcW - 3));
        float wx[4], wy[4];
        CubicCoeffs(fx, wx);
        CubicCoeffs(fy, wy);
        float sum[C];
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            sum[c] = 0.f;
        }
        [[maybe_unused]] int wq[4];
        if constexpr (kFixedCubic<T>)
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                wx[i] *= 16384.f;
                wy[i] *= 1.f / 16384.f;
            }
            CubicWeightsQ14(wx, wq);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            // sources narrower/lower than 4 pixels: clamp the taps into the image
            const int      yy  = max(0, min(sy - 1 + j, p.srcH - 1));
            const uint8_t *row = p.src + (int64_t)yy * p.srcRow;
            Pixel<T, C>    t[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                t[i] = LoadPx<T, C>(row, max(0, min(sx - 1 + i, p.srcW - 1)));
            }
            if constexpr (kFixedCubic<T>)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    const int h = (int)t[0].v[c] * wq[0] + (int)t[1].v[c] * wq[1] + (int)t[2].v[c] * wq[2] + (int)t[3].v[c] * wq[3];
                    sum[c]      = j == 0 ? (float)h * wy[0] : fmaf((float)h, wy[j], sum[c]);
                }
                continue;
            }
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                if constexpr (VARSHAPE)
                {
                    sum[c] += wy[j]
                            * (wx[0] * (float)t[0].v[c] + wx[1] * (float)t[1].v[c] + wx[2] * (float)t[2].v[c]
                               + wx[3] * (float)t[3].v[c]);
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        sum[c] += (float)t[i].v[c] * (wx[i] * wy[j]);
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out.v[c] = SaturateCast<T>(fabsf(sum[c]));
        }
    }
    return out;
}

template<class T, int C, int INTERP, bool VARSHAPE>
__device__ __forceinline__ void ResizePixel(const Plane &p, int dx, int dy)
{
    StorePx<T, C>(p.dst + (int64_t)dy * p.dstRow, dx, ResizeValue<T, C, INTERP, VARSHAPE>(p, dx, dy));
}

template<class T, int C, int INTERP>
__global__ __launch_bounds__(256) void ResizeTensorKernel(const ResizeArgs a, const int flat)
{
    // a block is 64 columns x 4 rows, or (flat) its four waves side by side on one row
    const int dx = flat ? blockIdx.x * (kTileW * kTileH) + threadIdx.x : blockIdx.x * kTileW + (threadIdx.x & 63);
    const int dy = flat ? blockIdx.y : blockIdx.y * kTileH + (threadIdx.x >> 6);
    if (dx >= a.dstW || dy >= a.dstH)
    {
        return;
    }
    const Plane p = GetPlanes<false>(a, blockIdx.z);
    ResizePixel<T, C, INTERP, false>(p, dx, dy);
}

template<class T, int C, int INTERP>
__global__ __launch_bounds__(256) void ResizeVarShapeKernel(const ResizeArgs a, const VarTiles tiles)
{
    const TileCoord tc = LocateTile(tiles, blockIdx.x);
    const Plane     p  = GetPlanes<true>(a, tc.image);
    const int       dx = tc.tx * kTileW + (threadIdx.x & 63);
    const int       dy = tc.ty * kTileH + (threadIdx.x >> 6);
    if (dx >= p.dstW || dy >= p.dstH)
    {
        return;
    }
    ResizePixel<T, C, INTERP, true>(p, dx, dy);
}

// ---------------------------------------------------------------------------------------------
// Wave-patch form for small pixels. The per-pixel form above issues one load per tap and one store
// per channel (8 tap loads and 3 byte stores per u8x3 bilinear pixel) and is bound by the number of
// memory instructions, not by bytes or arithmetic. Here the horizontally adjacent taps of a sample
// (2 for bilinear, 4 for bicubic) come from one load, and lanes exchange results so that each
// stores 4 consecutive pixels as whole dwords. Arithmetic: the expressions of ResizeValue, term for
// term.

// Per-column and per-row terms of a sample: source index and weights, the expressions of
// ResizeValue. W = number of weights (0 nearest, 1 linear, 4 cubic); sources are >= 4 pixels wide.
template<int W>
struct AxisTerms
{
    int   s;                // nearest: source index; linear: first tap; cubic: second tap
    float w[W > 0 ? W : 1]; // linear: weight of the second tap
};

template<int INTERP>
constexpr int kWeights = INTERP == NVCV_INTERP_NEAREST ? 0 : (INTERP == NVCV_INTERP_LINEAR ? 1 : 4);

template<int INTERP>
__device__ __forceinline__ AxisTerms<kWeights<INTERP>> Axis(float scale, int d, int srcSize)
{
    AxisTerms<kWeights<INTERP>> a;
    if constexpr (INTERP == NVCV_INTERP_NEAREST)
    {
        a.s = min((int)floorf(scale * (d + 0.5f)), srcSize - 1);
    }
    else if constexpr (INTERP == NVCV_INTERP_LINEAR)
    {
        const float f = (d + .5f) * scale - .5f;
        const int   s = (int)floorf(f);
        a.w[0]        = (s < 0) ? 0.f : ((s > srcSize - 2) ? 1.f : f - s);
        a.s           = max(0, min(s, srcSize - 2));
    }
    else
    {
        const float c = (d + .5f) * scale - .5f;
        const int   s = (int)floorf(c);
        float       f = c - s;
        a.s           = s;
        a.w[0]        = f; // finished by the caller: the two axes treat the fraction differently
    }
    return a;
}

// Lane `from` (constant) of every field, as wave-uniform values.
template<int W>
__device__ __forceinline__ AxisTerms<W> FromLane(const AxisTerms<W> &a, int from)
{
    AxisTerms<W> r;
    r.s = __builtin_amdgcn_readlane(a.s, from);
#pragma unroll
    for (int i = 0; i < (W > 0 ? W : 1); ++i)
    {
        r.w[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(a.w[i]), from));
    }
    return r;
}

__device__ __forceinline__ float ReadLane(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// The 8-bit bicubic sum of one output pixel per lane: rows y0 .. y0 + 3 (clamped into the image), their windows of 4
// pixels at `at` + `shift`, the packed horizontal weights and the vertical ones times 2^-14 (wave-uniform). All four
// windows are requested before the first sum.
template<int C, bool GUARDED>
__device__ __forceinline__ uint32_t CubicRowsQ14(const Plane &p, int y0, uint32_t at, uint32_t shift, uint32_t rowBytes,
                                                 uint32_t w01, uint32_t w23, const float (&wy)[4])
{
    uint32_t       r[4][C];
    const uint8_t *first = p.src + (int64_t)y0 * p.srcRow;
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const int      yy   = GUARDED ? max(0, min(y0 + j, p.srcH - 1)) : y0 + j;
        const uint8_t *line = GUARDED ? p.src + (int64_t)yy * p.srcRow : first + (int64_t)j * p.srcRow;
        LoadQuadWindow<C, GUARDED>(line, at, shift, yy == p.srcH - 1, rowBytes, r[j]);
    }
    float acc[C];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        const float w = wy[j];
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            const int h = Dot2I16(QuadTapPair<C>(r[j], 2, c), w23, Dot2I16(QuadTapPair<C>(r[j], 0, c), w01));
            acc[c]      = j == 0 ? (float)h * w : fmaf((float)h, w, acc[c]);
        }
    }
    uint32_t q = 0;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        q = __builtin_amdgcn_cvt_pk_u8_f32(fabsf(acc[c]), c, q);
    }
    return q;
}

// The same for TWO vertically adjacent output pixels per lane whose 4-row windows start `N - 4` rows apart (0 .. 2) and
// lie inside the image, clear of its last row: the N source rows from y0 on are loaded once, each row's sums are
// formed once, and each pixel adds its own four in ascending order - the sums and their order are those of
// CubicRowsQ14, so the result is the same bit for bit. At scale 1.5 that is 5 or 6 row sums where two pixels took 8.
template<int C, int N>
__device__ __forceinline__ void CubicRowPairQ14(const Plane &p, int y0, uint32_t at, uint32_t shift, uint32_t rowBytes,
                                                uint32_t w01, uint32_t w23, const float (&wyA)[4], const float (&wyB)[4],
                                                uint32_t (&out)[2])
{
    uint32_t       r[N][C];
    const uint8_t *first = p.src + (int64_t)y0 * p.srcRow;
#pragma unroll
    for (int j = 0; j < N; ++j)
    {
        LoadQuadWindow<C, false>(first + (int64_t)j * p.srcRow, at, shift, false, rowBytes, r[j]);
    }
    float accA[C], accB[C];
#pragma unroll
    for (int j = 0; j < N; ++j)
    {
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            const float h = (float)Dot2I16(QuadTapPair<C>(r[j], 2, c), w23, Dot2I16(QuadTapPair<C>(r[j], 0, c), w01));
            if (j < 4)
            {
                accA[c] = j == 0 ? h * wyA[0] : fmaf(h, wyA[j], accA[c]);
            }
            if (j >= N - 4)
            {
                accB[c] = j == N - 4 ? h * wyB[0] : fmaf(h, wyB[j - (N - 4)], accB[c]);
            }
        }
    }
    out[0] = out[1] = 0;
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        out[0] = __builtin_amdgcn_cvt_pk_u8_f32(fabsf(accA[c]), c, out[0]);
        out[1] = __builtin_amdgcn_cvt_pk_u8_f32(fabsf(accB[c]), c, out[1]);
    }
}

// The part of the 8-bit bicubic sum that depends on the output column only.
struct CubicColumnQ14
{
    uint32_t w01, w23;  // horizontal weights in units of 2^-14, packed in pairs
    uint32_t at, shift; // the window load's byte offset in a row and the window's position in it
};

template<int C>
__device__ __forceinline__ CubicColumnQ14 CubicColumn(const AxisTerms<4> &col)
{
    CubicColumnQ14 q;
    float          wx[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        wx[i] = col.w[i] * 16384.f;
    }
    CubicWeightPairsQ14(wx, q.w01, q.w23);
    const uint32_t off = (uint32_t)(col.s - 1) * C;
    q.at               = C == 4 ? off : off & ~3u;
    q.shift            = off & 3u;
    return q;
}

// A lane's 4 output pixels (rows k = 0 .. 3 of a wave patch, row terms in lanes 0 .. 3 of `rows`, vertical weights
// already in units of 2^-14) of the 8-bit bicubic form, clear of the image's last row: output rows in pairs that
// share the source rows between their windows (wave-uniform choice by how far the windows are apart; farther than
// 2: one by one).
template<int C>
__device__ __forceinline__ void CubicPatchPairsQ14(const Plane &p, const AxisTerms<4> &col, const AxisTerms<4> &rows,
                                                   uint32_t (&q)[4])
{
    const CubicColumnQ14 cq = CubicColumn<C>(col);
    const uint32_t       rb = (uint32_t)p.srcW * C;
#pragma unroll
    for (int k = 0; k < 4; k += 2)
    {
        const auto rowA = FromLane(rows, k), rowB = FromLane(rows, k + 1);
        const int  apart = rowB.s - rowA.s;
        uint32_t   two[2];
        if (apart == 1)
        {
            CubicRowPairQ14<C, 5>(p, rowA.s - 1, cq.at, cq.shift, rb, cq.w01, cq.w23, rowA.w, rowB.w, two);
        }
        else if (apart == 2)
        {
            CubicRowPairQ14<C, 6>(p, rowA.s - 1, cq.at, cq.shift, rb, cq.w01, cq.w23, rowA.w, rowB.w, two);
        }
        else if (apart == 0)
        {
            CubicRowPairQ14<C, 4>(p, rowA.s - 1, cq.at, cq.shift, rb, cq.w01, cq.w23, rowA.w, rowB.w, two);
        }
        else
        {
            two[0] = CubicRowsQ14<C, false>(p, rowA.s - 1, cq.at, cq.shift, rb, cq.w01, cq.w23, rowA.w);
            two[1] = CubicRowsQ14<C, false>(p, rowB.s - 1, cq.at, cq.shift, rb, cq.w01, cq.w23, rowB.w);
        }
        q[k]     = two[0];
        q[k + 1] = two[1];
    }
}

// One output pixel from its column terms (per lane) and row terms (wave-uniform). GUARDED: the image's last row may
// be among the rows read, so every tap load tests for it (its loads must not run past the image's end); the caller
// settles that once per wave patch, because a wave-uniform test in front of a load keeps the compiler from requesting
// the next load before this one has returned.
template<class T, int C, int INTERP, bool VARSHAPE, bool GUARDED>
__device__ __forceinline__ Pixel<T, C> SampleWide(const Plane &p, const AxisTerms<kWeights<INTERP>> &col,
                                                  const AxisTerms<kWeights<INTERP>> &row)
{
    constexpr int PB       = sizeof(Pixel<T, C>);
    const int     rowBytes = p.srcW * PB;
    Pixel<T, C>   out;
    if constexpr (INTERP == NVCV_INTERP_NEAREST)
    {
        float t[1][C];
        LoadTaps<T, C, 1>(p.src + (int64_t)row.s * p.srcRow, col.s * PB, GUARDED && row.s == p.srcH - 1, rowBytes, t);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out.v[c] = (T)t[0][c]; // exact: the value came from a T
        }
    }
    else if constexpr (INTERP == NVCV_INTERP_LINEAR)
    {
        const int   y0 = row.s, y1 = min(row.s + 1, p.srcH - 1);
        const float wx = col.w[0], wy = row.w[0];
        if constexpr (kFixedLinear<T>)
        {
            uint32_t r0[2], r1[2], top, bottom, q = 0;
            LoadTapPairBytes<C>(p.src + (int64_t)y0 * p.srcRow, col.s * PB, GUARDED && y0 == p.srcH - 1, rowBytes, r0);
            LoadTapPairBytes<C>(p.src + (int64_t)y1 * p.srcRow, col.s * PB, GUARDED && y1 == p.srcH - 1, rowBytes, r1);
            WeightPairsQ15(FractionQ15(wx), FractionQ15(wy), top, bottom);
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                const uint32_t sel = 0x0c000c00u | (uint32_t)c | ((uint32_t)(c + C) << 16);
                q = BlendQ15(__builtin_amdgcn_perm(r0[1], r0[0], sel), __builtin_amdgcn_perm(r1[1], r1[0], sel), top, bottom, c, q);
            }
            __builtin_memcpy(&out, &q, PB);
            return out;
        }
        float       t0[2][C], t1[2][C];
        LoadTaps<T, C, 2>(p.src + (int64_t)y0 * p.srcRow, col.s * PB, GUARDED && y0 == p.srcH - 1, rowBytes, t0);
        LoadTaps<T, C, 2>(p.src + (int64_t)y1 * p.srcRow, col.s * PB, GUARDED && y1 == p.srcH - 1, rowBytes, t1);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            float v;
            if constexpr (VARSHAPE)
            {
                v = (1.0f - wx) * (t0[0][c] * (1.0f - wy) + t1[0][c] * wy)
                  + wx * (t0[1][c] * (1.0f - wy) + t1[1][c] * wy);
            }
            else
            {
                v = t0[0][c] * ((1.f - wx) * (1.f - wy)) + t0[1][c] * (wx * (1.f - wy)) + t1[0][c] * ((1.f - wx) * wy)
                  + t1[1][c] * (wx * wy);
            }
            out.v[c] = SaturateCast<T>(v);
        }
    }
    else if constexpr (kFixedCubic<T>)
    {
        // (the column's part of this does not depend on the row and is computed once per lane)
        const CubicColumnQ14 cq = CubicColumn<C>(col);
        // rows row.s - 1 .. row.s + 2, inside the image for sources of 4 rows and more; four windows together
        const uint32_t q = CubicRowsQ14<C, GUARDED>(p, row.s - 1, cq.at, cq.shift, (uint32_t)rowBytes, cq.w01, cq.w23, row.w);
        __builtin_memcpy(&out, &q, PB);
    }
    else
    {
        float sum[C];
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            sum[c] = 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int yy = max(0, min(row.s - 1 + j, p.srcH - 1));
            float     t[4][C];
            LoadTaps<T, C, 4>(p.src + (int64_t)yy * p.srcRow, (col.s - 1) * PB, GUARDED && yy == p.srcH - 1, rowBytes, t);
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                if constexpr (VARSHAPE)
                {
                    sum[c] += row.w[j] * (col.w[0] * t[0][c] + col.w[1] * t[1][c] + col.w[2] * t[2][c] + col.w[3] * t[3][c]);
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        sum[c] += t[i][c] * (col.w[i] * row.w[j]);
                    }
                }
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out.v[c] = SaturateCast<T>(fabsf(sum[c]));
        }
    }
    return out;
}

// Column (horizontal == true) or row terms of output index d, finished for sampling.
template<int INTERP>
__device__ __forceinline__ AxisTerms<kWeights<INTERP>> FinishedAxis(float scale, int d, int srcSize, bool horizontal)
{
    AxisTerms<kWeights<INTERP>> a = Axis<INTERP>(scale, d, srcSize);
    if constexpr (INTERP == NVCV_INTERP_CUBIC)
    {
        // the reference zeroes the horizontal fraction next to the image border, not the vertical one
        float f = a.w[0];
        f       = (horizontal && (a.s < 1 || a.s >= srcSize - 3)) ? 0.f : f;
        a.s     = max(1, min(a.s, srcSize - 3));
        CubicCoeffs(f, a.w);
    }
    return a;
}

// Stores a wave's 64-column x 4-row patch at (x0, y0): q[d][k] is dword d of the pixel (x0 + lane, y0 + k). After
// the 4x4 transposes lane l owns row y0 + (l & 3), columns x0 + 4 * (l >> 2) .. + 3, written as whole dwords.
template<class T, int C>
__device__ __forceinline__ void StoreWavePatch(const Plane &p, int x0, int y0, int lane,
                                               uint32_t (&q)[(sizeof(Pixel<T, C>) + 3) / 4][4])
{
    constexpr int PB = sizeof(Pixel<T, C>), D = (PB + 3) / 4;
#pragma unroll
    for (int d = 0; d < D; ++d)
    {
        QuadTranspose(q[d], lane & 3);
    }
    const int dy = y0 + (lane & 3), dx0 = x0 + 4 * (lane >> 2);
    if (dy >= p.dstH || dx0 >= p.dstW)
    {
        return;
    }
    uint8_t *to = p.dst + (int64_t)dy * p.dstRow + (int64_t)dx0 * PB;

    if (dx0 + 4 <= p.dstW)
    {
        uint32_t w[PB];
        PackQuad<PB>(q, w);
        StoreDwordsNT<PB>(to, w);
    }
    else
    {
#pragma unroll
        for (int k = 0; k < 3; ++k)
        {
            if (dx0 + k < p.dstW)
            {
                uint32_t w[D];
#pragma unroll
                for (int d = 0; d < D; ++d)
                {
                    w[d] = q[d][k];
                }
                Pixel<T, C> px;
                __builtin_memcpy(&px, w, PB);
                reinterpret_cast<Pixel<T, C> *>(to)[k] = px;
            }
        }
    }
}

// One wave resizes a 64-column x 4-row patch of the output whose top left pixel is (x0, y0), both
// wave-uniform. Sampling: lane l owns column x0 + l and computes its 4 rows (the column terms are
// shared; neighbouring lanes read neighbouring source pixels whatever the scale). Storing: after
// the 4x4 transposes lane l owns row y0 + (l & 3), columns x0 + 4 * (l >> 2) .. + 3.
template<class T, int C, int INTERP, bool VARSHAPE>
__device__ __forceinline__ void ResizeWavePatch(const Plane &p, int x0, int y0)
{
    constexpr int PB = sizeof(Pixel<T, C>), D = (PB + 3) / 4;
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    const int   lane   = threadIdx.x & 63;
    const float scaleX = p.scaleX, scaleY = p.scaleY;
    // uniform per image (the 8-bit bicubic form loads whole dwords around 4 pixels: rows of 16 bytes or more, 8 for
    // one channel)
    const bool wide = p.srcW >= 4 && (INTERP != NVCV_INTERP_CUBIC || !kFixedCubic<T> || p.srcW * C >= (C == 1 ? 8 : 16));
    // columns and rows past the output compute a duplicate of the last one: every lane takes part in
    // the transposes
    const int dx = min(x0 + lane, p.dstW - 1);
    uint32_t  q[D][4];
    if (wide)
    {
        const auto col = FinishedAxis<INTERP>(scaleX, dx, p.srcW, true);
        // the 4 rows' terms are computed side by side (lane l: row l & 3) and then read as uniform values
        auto rows = FinishedAxis<INTERP>(scaleY, min(y0 + (lane & 3), p.dstH - 1), p.srcH, false);
        if constexpr (INTERP == NVCV_INTERP_CUBIC && kFixedCubic<T>)
        {
            // the vertical weights go with row sums in units of 2^-14
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                rows.w[i] *= 1.f / 16384.f;
            }
        }
        // the last source row the patch reads (row indices ascend with the output row; bilinear reads one more, bicubic
        // two): only a patch that reaches the image's last row needs the guarded loads (wave-uniform)
        constexpr int reach = INTERP == NVCV_INTERP_NEAREST ? 0 : (INTERP == NVCV_INTERP_LINEAR ? 1 : 2);
        auto          sample = [&](auto guarded)
        {
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const Pixel<T, C> out  = SampleWide<T, C, INTERP, VARSHAPE, decltype(guarded)::value>(p, col, FromLane(rows, k));
                uint32_t          w[D] = {};
                __builtin_memcpy(w, &out, PB);
#pragma unroll
                for (int d = 0; d < D; ++d)
                {
                    q[d][k] = w[d];
                }
            }
        };
        if (__builtin_amdgcn_readlane(rows.s, 3) + reach >= p.srcH - 1)
        {
            sample(std::true_type{});
        }
        else if constexpr (INTERP == NVCV_INTERP_CUBIC && kFixedCubic<T>)
        {
            CubicPatchPairsQ14<C>(p, col, rows, q[0]);
        }
        else
        {
            sample(std::false_type{});
        }
    }
    else
    {
#pragma unroll 1
        for (int k = 0; k < 4; ++k)
        {
            const Pixel<T, C> out  = ResizeValue<T, C, INTERP, VARSHAPE>(p, dx, min(y0 + k, p.dstH - 1));
            uint32_t          w[D] = {};
            __builtin_memcpy(w, &out, PB);
#pragma unroll
            for (int d = 0; d < D; ++d)
            {
                q[d][0] = k == 0 ? w[d] : q[d][0];
                q[d][1] = k == 1 ? w[d] : q[d][1];
                q[d][2] = k == 2 ? w[d] : q[d][2];
                q[d][3] = k == 3 ? w[d] : q[d][3];
            }
        }
    }
    StoreWavePatch<T, C>(p, x0, y0, lane, q);
}

// ---- the 8-bit bicubic form over strips of 16 output rows per wave

constexpr int kCubicStripRows = 16;

// A row window as LoadQuadWindow reads it, in two steps: a strip requests the rows of its next output row before it
// works on the current one.
template<int C>
struct RawQuadWindow
{
    uint32_t d[C == 4 ? 4 : C + 1];
};

// (row: wave-uniform; at: the lane's byte offset in it - the load then takes the row as its scalar base and the
// lane needs no address arithmetic)
template<int C>
__device__ __forceinline__ RawQuadWindow<C> RequestQuadWindow(const uint8_t *row, uint32_t at)
{
    struct __attribute__((packed, aligned(1))) Window
    {
        uint32_t d[C == 4 ? 4 : C + 1];
    };
    const Window     w = *reinterpret_cast<const Window *>(row + at);
    RawQuadWindow<C> r;
    __builtin_memcpy(&r, &w, sizeof(r));
    return r;
}

// The row's sums of 4 taps times the horizontal weights (units of 2^-14), as CubicRowsQ14 forms them.
template<int C>
__device__ __forceinline__ void CubicRowSumsQ14(const RawQuadWindow<C> &w, uint32_t shift, uint32_t w01, uint32_t w23,
                                                float (&h)[C])
{
    uint32_t r[C];
#pragma unroll
    for (int i = 0; i < C; ++i)
    {
        if constexpr (C == 4)
        {
            r[i] = w.d[i];
        }
        else
        {
            r[i] = __builtin_amdgcn_alignbyte(w.d[i + 1], w.d[i], shift);
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        h[c] = (float)Dot2I16(QuadTapPair<C>(r, 2, c), w23, Dot2I16(QuadTapPair<C>(r, 0, c), w01));
    }
}

// One wave resizes 64 columns x 16 rows whose top left pixel is (x0, y0), both wave-uniform; lane l owns column
// x0 + l. The windows of consecutive output rows overlap (reducing by 1.5 they advance by 1 or 2 source rows,
// enlarging by 0 or 1), so the strip walks down the source rows once: a row's sums are formed once and added, times
// the row's weight in each, to the output pixels whose windows can hold it - the current output row and the S - 1
// after it. S = 4 when reducing (all of them while windows advance by at least one row), S = 8 when enlarging (all
// of them while the window 8 rows down starts 4 or more source rows later: enlargements up to 2). The S running
// pixels live in fixed registers (output row r in slot r mod S, S steps unrolled); a row outside a pixel's window
// is added with weight 0, which changes nothing, so the instruction stream does not depend on the scale. An output
// row is finished when the last row of its window has been added, its slot then starts the pixel S rows down.
// Every pixel adds its four row sums in ascending order (the first to a zero, which gives the product), as
// CubicRowsQ14 does: the same result bit for bit. Per output pixel 1.5 row sums when reducing by 1.5 where the patch
// form takes 2.75, 0.67 when enlarging by 1.5 where it takes 2.25, and the column terms once per 16 rows.
// The rows a step can add (reducing: two, enlarging: one) are requested two steps ahead, needed or not (no test in
// front of a load).
// A strip takes this form when its windows advance as said from each output row to the next and stay clear of the
// image's last row; others (the image's top and bottom, other scales) go one output row at a time with guarded
// loads. The launch requires sources wide enough for the window loads (16 bytes a row, 8 for one channel).
template<int C, int S>
__device__ __forceinline__ void ResizeCubicStripU8(const Plane &p, int x0, int y0)
{
    static_assert(S == 4 || S == 8);
    constexpr bool kReducing = S == 4;
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    constexpr int R    = kCubicStripRows;
    const int     lane = threadIdx.x & 63;
    const int     dx   = min(x0 + lane, p.dstW - 1); // columns past the output compute a duplicate of the last one
    const auto    col  = FinishedAxis<NVCV_INTERP_CUBIC>(p.scaleX, dx, p.srcW, true);
    // lane 4 r + t holds the second tap's row of output row y0 + r and its weight for tap t, in units of 2^-14
    // (the row sums' unit)
    const auto  rows  = FinishedAxis<NVCV_INTERP_CUBIC>(p.scaleY, min(y0 + (lane >> 2), p.dstH - 1), p.srcH, false);
    const int   t     = lane & 3;
    const float wLane = (t == 0 ? rows.w[0] : t == 1 ? rows.w[1] : t == 2 ? rows.w[2] : rows.w[3]) * (1.f / 16384.f);
    const int   apartLane = __shfl_down(rows.s, 4) - rows.s;
    bool        regular   = lane >= 4 * (R - 1) || (apartLane >= (kReducing ? 1 : 0) && apartLane <= (kReducing ? 2 : 1));
    if constexpr (!kReducing)
    {
        // (every lane takes part in the exchange: a lane that has left reads as 0)
        const int farLane = __shfl_down(rows.s, 4 * S) - rows.s;
        regular           = regular & ((lane >= 4 * (R - S)) | (farLane >= 4));
    }
    const CubicColumnQ14 cq = CubicColumn<C>(col);
    auto second = [&](int r) { return __builtin_amdgcn_readlane(rows.s, 4 * min(r, R - 1)); }; // the row of output row r's second tap
    if (y0 + R > p.dstH || __builtin_amdgcn_ballot_w64(!regular) != 0 || second(R - 1) + 2 >= p.srcH - 1) // wave-uniform
    {
        // one output row at a time, every window load guarded against the image's last row
#pragma unroll 1
        for (int g = 0; g < R && y0 + g < p.dstH; g += 4)
        {
            uint32_t q[1][4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                const int   r     = g + k;
                const float wy[4] = {ReadLane(wLane, 4 * r), ReadLane(wLane, 4 * r + 1), ReadLane(wLane, 4 * r + 2),
                                     ReadLane(wLane, 4 * r + 3)};
                q[0][k] = CubicRowsQ14<C, true>(p, second(r) - 1, cq.at, cq.shift, (uint32_t)p.srcW * C, cq.w01, cq.w23, wy);
            }
            StoreWavePatch<uint8_t, C>(p, x0, y0 + g, lane, q);
        }
        return;
    }
    auto request = [&](int row) { return RequestQuadWindow<C>(p.src + (int64_t)row * p.srcRow, cq.at); };

    float acc[S][C] = {};
    // The weight of source row j in output row r, whose second tap is row sr: tap j - (sr - 1) where that is 0 .. 3,
    // else 0. Output rows past the strip (r >= 16, terms of row 15) collect sums that are never stored. The lane is
    // read either way (no branch; the instruction takes the lane number modulo 64) and the choice is written as scalar
    // instructions, which the compiler otherwise turns into a move and a select on the vector unit per weight.
    // always: the tap is known to be one of the four, nothing to choose.
    auto weight = [&](int j, int sr, int r, bool always)
    {
        const int tap = j - sr + 1;
        const int w   = __builtin_amdgcn_readlane(__float_as_int(wLane), 4 * r + tap);
        if (always)
        {
            return __int_as_float(w);
        }
        int chosen;
        asm("s_cmp_lt_u32 %1, 4\n\ts_cselect_b32 %0, %2, 0" : "=s"(chosen) : "s"(tap), "s"(w) : "scc");
        return __int_as_float(chosen);
    };
    // Source row j, whose window is w, into the output rows r .. r + outputs - 1 (slots K .. ; K is a constant once
    // unrolled), whose second taps are rows sr[0 ..]; the first `sure` of them hold the row for certain.
    auto add = [&](int K, const RawQuadWindow<C> &w, int j, int r, const int (&sr)[S], int outputs, int sure)
    {
        float h[C];
        CubicRowSumsQ14<C>(w, cq.shift, cq.w01, cq.w23, h);
#pragma unroll
        for (int i = 0; i < S; ++i)
        {
            if (i >= outputs)
            {
                break;
            }
            // taps fall with i: from the first pixel whose window starts below the row on, nothing is added (tested
            // where it pays: once for pixels 4 - 5 and once for 6 - 7 of the enlarging form; wave-uniform)
            if ((i == 4 || i == 6) && j - sr[i] + 1 < 0)
            {
                break;
            }
            const float wi = weight(j, sr[i], r + i, i < sure);
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                acc[(K + i) & (S - 1)][c] = fmaf(h[c], wi, acc[(K + i) & (S - 1)][c]);
            }
        }
    };
    int sr[S];
#pragma unroll
    for (int i = 0; i < S; ++i)
    {
        sr[i] = second(i);
    }
    // output row 0's window but for its last row
    {
        const RawQuadWindow<C> w0 = request(sr[0] - 1), w1 = request(sr[0]), w2 = request(sr[0] + 1);
        add(0, w0, sr[0] - 1, 0, sr, S, 1);
        add(0, w1, sr[0], 0, sr, S, 1);
        add(0, w2, sr[0] + 1, 0, sr, S, 1);
    }
    // The step to output row r adds row sr + 2 if the window advanced, and before it row sr + 1 if it advanced by 2.
    // They are requested two steps ahead (even steps use one set of registers, odd steps the other).
    constexpr int    M = kReducing ? 2 : 1;
    RawQuadWindow<C> ahead[2][M];
#pragma unroll
    for (int e = 0; e < 2; ++e)
    {
#pragma unroll
        for (int m = 0; m < M; ++m)
        {
            ahead[e][m] = request(sr[e] + 2 - (M - 1 - m));
        }
    }
    int apart = 1; // the rows before sr[0] + 2 are in already
#pragma unroll 1
    for (int g = 0; g < R; g += S)
    {
        uint32_t q[1][4];
#pragma unroll
        for (int k = 0; k < S; ++k)
        {
            const int        r = g + k;
            RawQuadWindow<C> now[M];
#pragma unroll
            for (int m = 0; m < M; ++m)
            {
                now[m]           = ahead[k & 1][m];
                ahead[k & 1][m] = request(sr[2] + 2 - (M - 1 - m));
            }
            if constexpr (kReducing)
            {
                if (apart == 2)
                {
                    add(k, now[0], sr[0] + 1, r, sr, 3, 2); // the row above the window's last is in none of output row r + 3's
                }
                add(k, now[1], sr[0] + 2, r, sr, 4, 2);
            }
            else
            {
                if (apart == 1)
                {
                    add(k, now[0], sr[0] + 2, r, sr, S, 1);
                }
            }
            apart = sr[1] - sr[0];
#pragma unroll
            for (int i = 0; i + 1 < S; ++i)
            {
                sr[i] = sr[i + 1];
            }
            sr[S - 1] = second(r + S);
            q[0][k & 3] = 0;
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                q[0][k & 3] = __builtin_amdgcn_cvt_pk_u8_f32(fabsf(acc[k][c]), c, q[0][k & 3]);
                acc[k][c]   = 0.f;
            }
            if ((k & 3) == 3)
            {
                StoreWavePatch<uint8_t, C>(p, x0, y0 + r - 3, lane, q);
            }
        }
    }
}

// 8-bit bilinear at horizontal scales up to 2. The cost of the wave-patch form there is the number
// of tap loads (the texture addresser is busy 76-90 % of the time). The taps of two neighbouring
// output columns lie within 4 source pixels, so here a lane owns 2 columns x 2 rows and fetches each
// source row once for both columns (one 4-, 12- or 16-byte load): half the loads. A wave covers 128
// columns x 2 rows; lanes 2j and 2j+1 then swap a pixel pair each, so that lane 2j stores columns
// 4j .. 4j+3 of the first row and lane 2j+1 those of the second. Arithmetic as in SampleWide.
// Pixels travel as one dword each (channel c in byte c; higher bytes are don't-care).
template<int C>
struct __attribute__((packed, aligned(1))) TapWindow
{
    uint32_t w[C]; // 4 pixels of C bytes
};

// Pixel k (0 .. 3) of a window.
template<int C>
__device__ __forceinline__ uint32_t WindowPixel(const TapWindow<C> &t, int k)
{
    if constexpr (C == 4)
    {
        return t.w[k];
    }
    else if constexpr (C == 1)
    {
        return t.w[0] >> (8 * k);
    }
    else
    {
        static_assert(C == 3);
        return k == 0 ? t.w[0]
             : k == 1 ? __builtin_amdgcn_alignbit(t.w[1], t.w[0], 24)
             : k == 2 ? __builtin_amdgcn_alignbit(t.w[2], t.w[1], 16)
                      : t.w[2] >> 8;
    }
}

// The 4 pixels that start at `at` (rows before the image's last one only: the load may read past the row), in two
// steps so that a caller can request several windows before it touches the first.
// u8x3: the aligned 16 bytes that hold the window's 12, funnel-shifted into place. The texture path takes a
// 12-byte load that is not dword aligned apart into about three times as many cache accesses (counters:
// 63 against 20 per wave-load), and these kernels wait for that unit: 1080p -> 720p 61.5 -> 59.9 us,
// 720p -> 1080p 117 -> 101 us. Reads at most 3 bytes before and 4 after the window.
template<int C>
struct RawTapWindow
{
    uint32_t d[C == 3 ? 4 : C];
    uint32_t mis;
};

template<int C>
__device__ __forceinline__ RawTapWindow<C> RequestTapWindow(const uint8_t *at)
{
    RawTapWindow<C> r;
    if constexpr (C == 3)
    {
        struct alignas(4) W4
        {
            uint32_t d[4];
        };
        r.mis      = (uint32_t)reinterpret_cast<uintptr_t>(at) & 3u;
        const W4 w = *reinterpret_cast<const W4 *>(at - r.mis);
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            r.d[i] = w.d[i];
        }
    }
    else
    {
        r.mis                = 0;
        const TapWindow<C> t = *reinterpret_cast<const TapWindow<C> *>(at);
#pragma unroll
        for (int i = 0; i < C; ++i)
        {
            r.d[i] = t.w[i];
        }
    }
    return r;
}

template<int C>
__device__ __forceinline__ TapWindow<C> FinishTapWindow(const RawTapWindow<C> &r)
{
    TapWindow<C> t;
    if constexpr (C == 3)
    {
        t.w[0] = __builtin_amdgcn_alignbyte(r.d[1], r.d[0], r.mis);
        t.w[1] = __builtin_amdgcn_alignbyte(r.d[2], r.d[1], r.mis);
        t.w[2] = __builtin_amdgcn_alignbyte(r.d[3], r.d[2], r.mis);
    }
    else
    {
#pragma unroll
        for (int i = 0; i < C; ++i)
        {
            t.w[i] = r.d[i];
        }
    }
    return t;
}

template<int C>
__device__ __forceinline__ TapWindow<C> LoadTapWindowAt(const uint8_t *at)
{
    return FinishTapWindow<C>(RequestTapWindow<C>(at));
}

template<int C>
__device__ __forceinline__ TapWindow<C> LoadTapWindow(const Plane &p, int y, int xs)
{
    return LoadTapWindowAt<C>(p.src + (int64_t)y * p.srcRow + xs * C);
}

// One pixel from its four taps (a dword each, channel c in byte c) and the float32 weights of the second taps.
template<int C>
__device__ __forceinline__ uint32_t BilinearU8(uint32_t p00, uint32_t p01, uint32_t p10, uint32_t p11, float wx, float wy)
{
    return BilinearQ15<C>(p00, p01, p10, p11, FractionQ15(wx), FractionQ15(wy));
}

template<int C, bool VARSHAPE>
__device__ __forceinline__ void ResizeLinearPairsU8(const Plane &p, int x0, int y0)
{
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    const int  lane = threadIdx.x & 63;
    const bool odd  = (lane & 1) != 0;
    // columns and rows past the output compute a duplicate of the last one: every lane takes part in the swap
    const auto colA  = Axis<NVCV_INTERP_LINEAR>(p.scaleX, min(x0 + 2 * lane, p.dstW - 1), p.srcW);
    const auto colB  = Axis<NVCV_INTERP_LINEAR>(p.scaleX, min(x0 + 2 * lane + 1, p.dstW - 1), p.srcW);
    const int  delta = colB.s - colA.s; // 0 .. 2 at scales up to 2
    // the 2 rows' terms are computed side by side (even lanes the first, odd lanes the second)
    const auto rows = Axis<NVCV_INTERP_LINEAR>(p.scaleY, min(y0 + (lane & 1), p.dstH - 1), p.srcH);
    uint32_t   pxA[2], pxB[2];
    const auto row0 = FromLane(rows, 0), row1 = FromLane(rows, 1);
    // taps of source row y for both columns: A's two, then B's
    auto fetchLast = [&](int y, uint32_t (&t)[4]) // the image's last row: nothing may be read past its end
    {
        const uint8_t *line = p.src + (int64_t)y * p.srcRow;
        float          a[2][C], b[2][C];
        LoadTaps<uint8_t, C, 2>(line, colA.s * C, true, p.srcW * C, a);
        LoadTaps<uint8_t, C, 2>(line, colB.s * C, true, p.srcW * C, b);
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            t[i] = 0;
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            t[0] |= (uint32_t)a[0][c] << (8 * c);
            t[1] |= (uint32_t)a[1][c] << (8 * c);
            t[2] |= (uint32_t)b[0][c] << (8 * c);
            t[3] |= (uint32_t)b[1][c] << (8 * c);
        }
    };
    auto window = [&](int y) { return LoadTapWindow<C>(p, y, colA.s); };
    auto unpack = [&](const TapWindow<C> &win, uint32_t (&t)[4])
    {
        const uint32_t k0 = WindowPixel<C>(win, 0), k1 = WindowPixel<C>(win, 1), k2 = WindowPixel<C>(win, 2),
                       k3 = WindowPixel<C>(win, 3);
        t[0] = k0;
        t[1] = k1;
        t[2] = delta == 0 ? k0 : (delta == 1 ? k1 : k2);
        t[3] = delta == 0 ? k1 : (delta == 1 ? k2 : k3);
    };
    const int ya0 = row0.s, yb0 = min(row0.s + 1, p.srcH - 1), ya1 = row1.s, yb1 = min(row1.s + 1, p.srcH - 1);
    uint32_t  top[2][4], bot[2][4];
    if (max(yb0, yb1) < p.srcH - 1) // wave-uniform; the usual case: all four window loads go out together
    {
        // All four windows are requested before anything else (a load behind one of the tests below would wait for
        // the loads before it); the two output rows often share source rows (always when enlarging), whose taps
        // are taken apart once.
        auto request = [&](int y) { return RequestTapWindow<C>(p.src + (int64_t)y * p.srcRow + colA.s * C); };
        const RawTapWindow<C> r0 = request(ya0), r1 = request(yb0), r2 = request(ya1), r3 = request(yb1);
        // a use the compiler cannot move (without it the last two loads sink into the branches that need them) behind
        // a line the instruction scheduler does not cross (or it starts on the first window between the loads)
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::"v"(r0.d[0]), "v"(r1.d[0]), "v"(r2.d[0]), "v"(r3.d[0]));
        const TapWindow<C> w0 = FinishTapWindow<C>(r0), w1 = FinishTapWindow<C>(r1), w2 = FinishTapWindow<C>(r2),
                           w3 = FinishTapWindow<C>(r3);
        unpack(w0, top[0]);
        unpack(w1, bot[0]);
        if (ya1 == ya0)
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                top[1][i] = top[0][i];
                bot[1][i] = bot[0][i];
            }
        }
        else
        {
            if (ya1 == yb0)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    top[1][i] = bot[0][i];
                }
            }
            else
            {
                unpack(w2, top[1]);
            }
            unpack(w3, bot[1]);
        }
    }
    else
    {
        auto fetch = [&](int y, uint32_t (&t)[4])
        {
            if (y == p.srcH - 1)
            {
                fetchLast(y, t);
            }
            else
            {
                unpack(window(y), t);
            }
        };
        fetch(ya0, top[0]);
        fetch(yb0, bot[0]);
        fetch(ya1, top[1]);
        fetch(yb1, bot[1]);
    }
    pxA[0] = BilinearU8<C>(top[0][0], top[0][1], bot[0][0], bot[0][1], colA.w[0], row0.w[0]);
    pxB[0] = BilinearU8<C>(top[0][2], top[0][3], bot[0][2], bot[0][3], colB.w[0], row0.w[0]);
    pxA[1] = BilinearU8<C>(top[1][0], top[1][1], bot[1][0], bot[1][1], colA.w[0], row1.w[0]);
    pxB[1] = BilinearU8<C>(top[1][2], top[1][3], bot[1][2], bot[1][3], colB.w[0], row1.w[0]);
    // even lanes keep their first-row pair and take the neighbour's, odd lanes the same for the second row
    const uint32_t got0 = FromLaneXor1(odd ? pxA[0] : pxA[1]), got1 = FromLaneXor1(odd ? pxB[0] : pxB[1]);
    const uint32_t q[1][4] = {{odd ? got0 : pxA[0], odd ? got1 : pxB[0], odd ? pxA[1] : got0, odd ? pxB[1] : got1}};
    const int      dy = y0 + (lane & 1), dx0 = x0 + 2 * (lane & ~1);
    if (dy >= p.dstH || dx0 >= p.dstW)
    {
        return;
    }
    uint8_t *to = p.dst + (int64_t)dy * p.dstRow + (int64_t)dx0 * C;
    if (dx0 + 4 <= p.dstW)
    {
        uint32_t w[C];
        PackQuad<C>(q, w);
        StoreDwordsNT<C>(to, w);
    }
    else
    {
#pragma unroll
        for (int k = 0; k < 3; ++k)
        {
            if (dx0 + k < p.dstW)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    to[C * k + c] = (uint8_t)(q[0][k] >> (8 * c));
                }
            }
        }
    }
}

// Enlargements by 1.5 or more (3 * srcW <= 2 * dstW): the taps of FOUR neighbouring output columns lie within 4
// source pixels, so a lane owns 4 columns x 2 rows on the same window loads as the two-column form: half the loads,
// column-independent work (row terms, addresses, funnel shifts) spread over twice the pixels, and a lane's 4 pixels
// of a row are consecutive, so nothing changes lanes before the store. A wave covers 256 columns x 2 rows. The
// distance between the first and the last of a lane's four source columns is at most 2 by the scale; should
// float32 rounding ever make it 3, or the image's last row be involved, the wave takes the two-column form.
template<int C>
__device__ __forceinline__ void ResizeLinearQuadsU8(const Plane &p, int x0, int y0)
{
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    const int            lane = threadIdx.x & 63;
    const int            dx0  = x0 + 4 * lane;
    AxisTerms<1>         col[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        col[j] = Axis<NVCV_INTERP_LINEAR>(p.scaleX, min(dx0 + j, p.dstW - 1), p.srcW);
    }
    const auto rows = Axis<NVCV_INTERP_LINEAR>(p.scaleY, min(y0 + (lane & 1), p.dstH - 1), p.srcH);
    const auto row0 = FromLane(rows, 0), row1 = FromLane(rows, 1);
    const int  ya0 = row0.s, yb0 = min(row0.s + 1, p.srcH - 1), ya1 = row1.s, yb1 = min(row1.s + 1, p.srcH - 1);
    const bool narrow = col[3].s - col[0].s <= 2;
    if (max(yb0, yb1) >= p.srcH - 1 || __builtin_amdgcn_ballot_w64(!narrow) != 0) // wave-uniform
    {
        ResizeLinearPairsU8<C, false>(p, x0, y0);
        ResizeLinearPairsU8<C, false>(p, x0 + 128, y0);
        return;
    }
    // pixels (s, s + 1) of column j out of the window's four
    auto taps = [&](const TapWindow<C> &win, uint32_t (&first)[4], uint32_t (&second)[4])
    {
        const uint32_t k0 = WindowPixel<C>(win, 0), k1 = WindowPixel<C>(win, 1), k2 = WindowPixel<C>(win, 2),
                       k3 = WindowPixel<C>(win, 3);
        first[0]  = k0;
        second[0] = k1;
#pragma unroll
        for (int j = 1; j < 4; ++j)
        {
            const int d = col[j].s - col[0].s;
            first[j]    = d == 0 ? k0 : (d == 1 ? k1 : k2);
            second[j]   = d == 0 ? k1 : (d == 1 ? k2 : k3);
        }
    };
    uint32_t topA[2][4], topB[2][4], botA[2][4], botB[2][4]; // [output row][column]: first and second tap, upper and lower source row
    taps(LoadTapWindow<C>(p, ya0, col[0].s), topA[0], topB[0]);
    taps(LoadTapWindow<C>(p, yb0, col[0].s), botA[0], botB[0]);
    if (ya1 == ya0)
    {
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            topA[1][j] = topA[0][j];
            topB[1][j] = topB[0][j];
            botA[1][j] = botA[0][j];
            botB[1][j] = botB[0][j];
        }
    }
    else if (ya1 == yb0)
    {
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            topA[1][j] = botA[0][j];
            topB[1][j] = botB[0][j];
        }
        taps(LoadTapWindow<C>(p, yb1, col[0].s), botA[1], botB[1]);
    }
    else
    {
        taps(LoadTapWindow<C>(p, ya1, col[0].s), topA[1], topB[1]);
        taps(LoadTapWindow<C>(p, yb1, col[0].s), botA[1], botB[1]);
    }
    if (dx0 >= p.dstW)
    {
        return;
    }
#pragma unroll
    for (int r = 0; r < 2; ++r)
    {
        const int dy = y0 + r;
        if (dy >= p.dstH)
        {
            break;
        }
        const float    wy = r == 0 ? row0.w[0] : row1.w[0];
        uint32_t       q[1][4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            q[0][j] = BilinearU8<C>(topA[r][j], topB[r][j], botA[r][j], botB[r][j], col[j].w[0], wy);
        }
        uint8_t *to = p.dst + (int64_t)dy * p.dstRow + (int64_t)dx0 * C;
        if (dx0 + 4 <= p.dstW)
        {
            uint32_t w[C];
            PackQuad<C>(q, w);
            StoreDwordsNT<C>(to, w);
        }
        else
        {
#pragma unroll
            for (int k = 0; k < 3; ++k)
            {
                if (dx0 + k < p.dstW)
                {
#pragma unroll
                    for (int c = 0; c < C; ++c)
                    {
                        to[C * k + c] = (uint8_t)(q[0][k] >> (8 * c));
                    }
                }
            }
        }
    }
}

// The windows of rows 0 .. last (wave-uniform, under 9) from `at` on, a lane's own column offset included, all of them
// requested before the first is touched: taken into place inside a test on `last`, each load would be waited for
// before the next goes out (nine round trips one after the other: 62 us instead of 51 for the two-column strips).
// The empty statement uses every raw window, so the loads can neither sink below it nor the funnel shifts rise
// above it. That all windows are in before a strip's row loop starts also keeps waits for them out of the loop:
// stores and loads share one counter of outstanding operations here, and such a wait, after rows have been stored,
// would be a wait for those stores to reach memory as well.
// 1 and 3 channels request only the windows that are needed. With 4-byte pixels the compiler joins a window that exists
// on one side of the test only to the statement through a register move, which waits for its load, so those request
// all nine (rows past `last` repeat it: an L1 hit, but a load instruction; 16 x 720p -> 900p u8x3 36.8 us against
// 31.3). Two whole variants, 5 windows or 9, were slower for every pixel size (65 us for the two-column strips).
template<int C>
__device__ __forceinline__ void RequestStripWindows(const uint8_t *at, int rowStride, int last, TapWindow<C> (&win)[9])
{
    RawTapWindow<C> raw[9];
#pragma unroll
    for (int k = 0; k < 9; ++k)
    {
        if constexpr (C == 4)
        {
            raw[k] = RequestTapWindow<C>(at + (int64_t)min(k, last) * rowStride);
        }
        else
        {
            if (k <= last)
            {
                raw[k] = RequestTapWindow<C>(at + (int64_t)k * rowStride);
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::"v"(raw[0].d[0]), "v"(raw[1].d[0]), "v"(raw[2].d[0]), "v"(raw[3].d[0]), "v"(raw[4].d[0]), "v"(raw[5].d[0]),
                 "v"(raw[6].d[0]), "v"(raw[7].d[0]), "v"(raw[8].d[0]));
#pragma unroll
    for (int k = 0; k < 9; ++k)
    {
        win[k] = FinishTapWindow<C>(raw[k]);
    }
}

// The four-column form over a strip of kStripRows output rows per wave. When not reducing vertically those rows
// lie between at most kStripRows + 1 consecutive source rows. All their windows are requested up front, a source
// row's tap pairs are formed once for every output row that uses it as
// its upper or its lower row, and the column terms are paid once per 8 rows instead of once per 2. The blend per
// output pixel is BilinearQ15 as everywhere. A wave that reaches the image's last source row, reduces vertically
// (more source rows than fit) or has a lane whose columns do not fit its window runs as four two-row steps.
constexpr int kStripRows = 8, kStripWindows = kStripRows + 1;
static_assert(kStripWindows == 9);

template<int C>
__device__ __forceinline__ void ResizeLinearQuadStripU8(const Plane &p, int x0, int y0)
{
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    const int    lane = threadIdx.x & 63;
    const int    dx0  = x0 + 4 * lane;
    AxisTerms<1> col[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        col[j] = Axis<NVCV_INTERP_LINEAR>(p.scaleX, min(dx0 + j, p.dstW - 1), p.srcW);
    }
    // lane r holds the terms of output row y0 + r
    const auto     rows   = Axis<NVCV_INTERP_LINEAR>(p.scaleY, min(y0 + (lane & (kStripRows - 1)), p.dstH - 1), p.srcH);
    const uint32_t ayLane = FractionQ15(rows.w[0]);
    const int      yFirst = __builtin_amdgcn_readlane(rows.s, 0), yLast = __builtin_amdgcn_readlane(rows.s, kStripRows - 1) + 1;
    const bool     narrow = col[3].s - col[0].s <= 2;
    if (yLast >= p.srcH - 1 || yLast - yFirst >= kStripWindows || __builtin_amdgcn_ballot_w64(!narrow) != 0) // wave-uniform
    {
#pragma unroll 1
        for (int k = 0; k < kStripRows; k += 2)
        {
            ResizeLinearQuadsU8<C>(p, x0, y0 + k);
        }
        return;
    }
    TapWindow<C>   win[kStripWindows];
    const uint8_t *at = p.src + (int64_t)yFirst * p.srcRow + col[0].s * C;
    RequestStripWindows<C>(at, p.srcRow, yLast - yFirst, win);
    // lanes past the last column stay (the row terms are read from lanes 0 .. 7 below); they store nothing
    uint32_t ax[4];
    int      d[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        ax[j] = FractionQ15(col[j].w[0]);
        d[j]  = col[j].s - col[0].s;
    }
    // (first tap | second tap << 16) of every column and channel of a source row.
    // 1 and 3 channels: the window's four values of a channel are gathered into one dword first (two byte permutes
    // with constant selectors; for one channel the window is that dword), and a column's pair is then ONE permute
    // whose selector the lane holds (bytes d and d + 1): 18 instructions per source row where choosing the column's
    // two pixels with selects and then the channel took 27.
    uint32_t pick[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        pick[j] = 0x0c010c00u + (uint32_t)d[j] * 0x00010001u;
    }
    auto pairs = [&](const TapWindow<C> &w, uint32_t (&t)[4][C])
    {
        if constexpr (C == 4)
        {
            const uint32_t k0 = WindowPixel<C>(w, 0), k1 = WindowPixel<C>(w, 1), k2 = WindowPixel<C>(w, 2), k3 = WindowPixel<C>(w, 3);
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const uint32_t first  = j == 0 ? k0 : (d[j] == 0 ? k0 : (d[j] == 1 ? k1 : k2));
                const uint32_t second = j == 0 ? k1 : (d[j] == 0 ? k1 : (d[j] == 1 ? k2 : k3));
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    t[j][c] = ChannelPair(first, second, c);
                }
            }
        }
        else
        {
            uint32_t x[C]; // byte k: channel c of the window's pixel k
            if constexpr (C == 1)
            {
                x[0] = w.w[0];
            }
            else
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    // bytes c, c + 3, c + 6, c + 9 of the window's 12: the first two (three) lie in its first 8
                    const uint32_t third = c + 6 < 8 ? (uint32_t)(c + 6) : 0x0cu;
                    const uint32_t head  = __builtin_amdgcn_perm(w.w[1], w.w[0], (uint32_t)c | (uint32_t)(c + 3) << 8 | third << 16 | 0x0c000000u);
                    x[c] = __builtin_amdgcn_perm(w.w[2], head, 0x0100u | (c + 6 < 8 ? 2u : (uint32_t)(c + 6 - 8 + 4)) << 16 | (uint32_t)(c + 9 - 8 + 4) << 24);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    t[j][c] = __builtin_amdgcn_perm(x[c], x[c], j == 0 ? 0x0c010c00u : pick[j]);
                }
            }
        }
    };
    const int nRows = min(kStripRows, p.dstH - y0);
    int       r     = 0;
    uint8_t  *to    = p.dst + (int64_t)y0 * p.dstRow + (int64_t)dx0 * C;
    uint32_t  top[4][C], bot[4][C];
    pairs(win[0], bot);
#pragma unroll
    for (int k = 0; k + 1 < kStripWindows; ++k)
    {
        if (r < nRows) // wave-uniform
        {
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    top[j][c] = bot[j][c];
                }
            }
            pairs(win[k + 1], bot);
            // the output rows between source rows yFirst + k and the next one
            while (r < nRows && __builtin_amdgcn_readlane(rows.s, r) == yFirst + k)
            {
                const uint32_t ay = __builtin_amdgcn_readlane(ayLane, r);
                uint32_t       w[C] = {}; // the row's 4 pixels as stored: every channel is rounded into its byte
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    uint32_t wt, wb;
                    WeightPairsQ15(ax[j], ay, wt, wb);
#pragma unroll
                    for (int c = 0; c < C; ++c)
                    {
                        const int at     = j * C + c;
                        w[at >> 2] = BlendQ15(top[j][c], bot[j][c], wt, wb, at & 3, w[at >> 2]);
                    }
                }
                if (dx0 + 4 <= p.dstW)
                {
                    StoreDwordsNT<C>(to, w);
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < 3 * C; ++i)
                    {
                        if (dx0 + i / C < p.dstW)
                        {
                            to[i] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
                        }
                    }
                }
                to += p.dstRow;
                ++r;
            }
        }
    }
}

// Nearest neighbour when enlarging by 1.5 or more (3 * srcW <= 2 * dstW), in the shape of the four-column strips:
// the source pixels of four neighbouring output columns lie within 3 source pixels, so a lane owns 4 columns x 8
// rows, takes them from one window per source row and stores every output row that maps to that source row from
// the same registers. The wave patches spend one 3-byte load per output pixel there (8 x 720p -> 1080p u8x3: 19.0 us,
// the bilinear strips 22.9; as strips 16.7). Indices are those of Axis<NEAREST>; waves that reach the image's last row,
// reduce vertically or have a lane whose columns do not fit its window run as wave patches.
template<int C>
__device__ __forceinline__ void ResizeNearestQuadStripU8(const Plane &p, int x0, int y0)
{
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    const int lane = threadIdx.x & 63;
    const int dx0  = x0 + 4 * lane;
    int       s[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        s[j] = Axis<NVCV_INTERP_NEAREST>(p.scaleX, min(dx0 + j, p.dstW - 1), p.srcW).s;
    }
    // lane r holds the source row of output row y0 + r
    const int  rowLane = Axis<NVCV_INTERP_NEAREST>(p.scaleY, min(y0 + (lane & (kStripRows - 1)), p.dstH - 1), p.srcH).s;
    const int  yFirst = __builtin_amdgcn_readlane(rowLane, 0), yLast = __builtin_amdgcn_readlane(rowLane, kStripRows - 1);
    const bool narrow = s[3] - s[0] <= 3;
    if (yLast >= p.srcH - 1 || yLast - yFirst >= kStripWindows || __builtin_amdgcn_ballot_w64(!narrow) != 0) // wave-uniform
    {
#pragma unroll 1
        for (int i = 0; i < 8; ++i)
        {
            ResizeWavePatch<uint8_t, C, NVCV_INTERP_NEAREST, false>(p, x0 + 64 * (i & 3), y0 + 4 * (i >> 2));
        }
        return;
    }
    TapWindow<C>   win[kStripWindows];
    const uint8_t *at = p.src + (int64_t)yFirst * p.srcRow + s[0] * C;
    RequestStripWindows<C>(at, p.srcRow, yLast - yFirst, win);
    const int nRows = min(kStripRows, p.dstH - y0);
    int       r     = 0;
    uint8_t  *to    = p.dst + (int64_t)y0 * p.dstRow + (int64_t)dx0 * C;
#pragma unroll
    for (int k = 0; k < kStripWindows; ++k)
    {
        if (r < nRows) // wave-uniform
        {
            // the lane's 4 pixels of source row yFirst + k, packed as they are stored
            const uint32_t mask  = C == 4 ? 0xffffffffu : (1u << (8 * C)) - 1u;
            const uint32_t k0 = WindowPixel<C>(win[k], 0) & mask, k1 = WindowPixel<C>(win[k], 1) & mask,
                           k2 = WindowPixel<C>(win[k], 2) & mask, k3 = WindowPixel<C>(win[k], 3) & mask;
            uint32_t       q[1][4];
            q[0][0] = k0;
#pragma unroll
            for (int j = 1; j < 4; ++j)
            {
                const int d = s[j] - s[0];
                q[0][j]     = d == 0 ? k0 : (d == 1 ? k1 : (d == 2 ? k2 : k3));
            }
            uint32_t w[C];
            PackQuad<C>(q, w);
            while (r < nRows && __builtin_amdgcn_readlane(rowLane, r) == yFirst + k)
            {
                if (dx0 + 4 <= p.dstW)
                {
                    StoreDwordsNT<C>(to, w);
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < 3 * C; ++i)
                    {
                        if (dx0 + i / C < p.dstW)
                        {
                            to[i] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
                        }
                    }
                }
                to += p.dstRow;
                ++r;
            }
        }
    }
}

// The two-column form over strips of kPairStripRows output rows per wave (128 columns x 4 rows). At vertical scales
// up to 2 those rows lie between at most 9 consecutive source rows: the windows are requested up front, a source row
// is taken apart into its (first tap | second tap) pairs once for every output row that uses it as its upper or its
// lower row, and the column terms are paid once per 4 rows instead of once per 2. Every output row is finished on its
// own: a lane rounds the channels of its 2 pixels straight into the bytes they have in the row, the lanes of a pair
// swap them, and the even lane stores the 4 pixels as whole dwords. The blend per output pixel is BilinearQ15 as
// everywhere. A wave that reaches the image's last source row or reduces vertically by more than 2 runs as two
// two-row steps.
constexpr int kPairStripRows = 4, kPairStripWindows = 2 * kPairStripRows + 1;
static_assert(kPairStripWindows == 9);

template<int C>
__device__ __forceinline__ void ResizeLinearPairStripU8(const Plane &p, int x0, int y0)
{
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    constexpr int R    = kPairStripRows;
    const int     lane = threadIdx.x & 63;
    const int     dx0  = x0 + 2 * lane;
    // columns and rows past the output compute a duplicate of the last one: every lane takes part in the swap
    const auto colA  = Axis<NVCV_INTERP_LINEAR>(p.scaleX, min(dx0, p.dstW - 1), p.srcW);
    const auto colB  = Axis<NVCV_INTERP_LINEAR>(p.scaleX, min(dx0 + 1, p.dstW - 1), p.srcW);
    const int  delta = colB.s - colA.s; // 0 .. 2 at scales up to 2
    // lane r holds the terms of output row y0 + r
    const auto     rows   = Axis<NVCV_INTERP_LINEAR>(p.scaleY, min(y0 + (lane & (R - 1)), p.dstH - 1), p.srcH);
    const uint32_t ayLane = FractionQ15(rows.w[0]);
    const int      yFirst = __builtin_amdgcn_readlane(rows.s, 0), yLast = __builtin_amdgcn_readlane(rows.s, R - 1) + 1;
    if (yLast >= p.srcH - 1 || yLast - yFirst >= kPairStripWindows) // wave-uniform
    {
        ResizeLinearPairsU8<C, false>(p, x0, y0);
        ResizeLinearPairsU8<C, false>(p, x0, y0 + 2);
        return;
    }
    TapWindow<C>   win[kPairStripWindows];
    const uint8_t *at = p.src + (int64_t)yFirst * p.srcRow + colA.s * C;
    RequestStripWindows<C>(at, p.srcRow, yLast - yFirst, win);
    const uint32_t axA = FractionQ15(colA.w[0]), axB = FractionQ15(colB.w[0]);
    // (first tap | second tap << 16) of both columns and every channel of a source row
    auto pairs = [&](const TapWindow<C> &w, uint32_t (&t)[2][C])
    {
        const uint32_t k0 = WindowPixel<C>(w, 0), k1 = WindowPixel<C>(w, 1), k2 = WindowPixel<C>(w, 2), k3 = WindowPixel<C>(w, 3);
        const uint32_t first = delta == 0 ? k0 : (delta == 1 ? k1 : k2), second = delta == 0 ? k1 : (delta == 1 ? k2 : k3);
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            t[0][c] = ChannelPair(k0, k1, c);
            t[1][c] = ChannelPair(first, second, c);
        }
    };
    const int  nRows = min(R, p.dstH - y0);
    const bool even  = (lane & 1) == 0;
    int        r     = 0;
    uint8_t   *to    = p.dst + (int64_t)y0 * p.dstRow + (int64_t)dx0 * C; // (used by even lanes: 4 pixels from their first)
    uint32_t   top[2][C], bot[2][C];
    pairs(win[0], bot);
#pragma unroll
    for (int k = 0; k + 1 < kPairStripWindows; ++k)
    {
        if (r < nRows) // wave-uniform
        {
#pragma unroll
            for (int j = 0; j < 2; ++j)
            {
#pragma unroll
                for (int c = 0; c < C; ++c)
                {
                    top[j][c] = bot[j][c];
                }
            }
            pairs(win[k + 1], bot);
            // the output rows between source rows yFirst + k and the next one
            while (r < nRows && __builtin_amdgcn_readlane(rows.s, r) == yFirst + k)
            {
                const uint32_t ay = __builtin_amdgcn_readlane(ayLane, r);
                // the lane's 2 pixels as the 2 C bytes they are in the row
                uint32_t mine[2] = {0, 0};
#pragma unroll
                for (int j = 0; j < 2; ++j)
                {
                    uint32_t wt, wb;
                    WeightPairsQ15(j == 0 ? axA : axB, ay, wt, wb);
#pragma unroll
                    for (int c = 0; c < C; ++c)
                    {
                        const int at8 = j * C + c;
                        mine[at8 >> 2] = BlendQ15(top[j][c], bot[j][c], wt, wb, at8 & 3, mine[at8 >> 2]);
                    }
                }
                // the even lane takes its neighbour's and stores 4 pixels
                uint32_t w[C];
                if constexpr (C == 4)
                {
                    w[0] = mine[0];
                    w[1] = mine[1];
                    w[2] = FromLaneXor1(mine[0]);
                    w[3] = FromLaneXor1(mine[1]);
                }
                else if constexpr (C == 3)
                {
                    const uint32_t lo = FromLaneXor1(mine[0]), hi = FromLaneXor1(mine[1]);
                    w[0] = mine[0];
                    w[1] = mine[1] | (lo << 16);
                    w[2] = __builtin_amdgcn_alignbit(hi, lo, 16);
                }
                else
                {
                    static_assert(C == 1);
                    w[0] = mine[0] | (FromLaneXor1(mine[0]) << 16);
                }
                if (even && dx0 < p.dstW)
                {
                    if (dx0 + 4 <= p.dstW)
                    {
                        StoreDwordsNT<C>(to, w);
                    }
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 3 * C; ++i)
                        {
                            if (dx0 + i / C < p.dstW)
                            {
                                to[i] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
                            }
                        }
                    }
                }
                to += p.dstRow;
                ++r;
            }
        }
    }
}

// Which (type, channels, interpolation) take the two-columns-per-lane form. The code is written for 1, 3
// and 4 channels; with 1 and 4 it measured slower than the wave patches (u8x1 43 -> 58 us, u8x4 91 -> 104 us
// on 1080p -> 720p: the column terms of two columns are amortised over 2 rows only), so 3 it is.
template<class T, int C, int INTERP>
constexpr bool kPairsForm = std::is_same_v<T, uint8_t> && INTERP == NVCV_INTERP_LINEAR && (C == 1 || C == 3 || C == 4);

// The scales at which the two-column form is the faster one (per image): horizontal scales up to 2; 4-byte pixels
// only when not reducing (16 x 1080p -> 720p: 34.4 us against the wave patches' 29.9; 720p -> 900p: 37.9 against 42.0).
template<int C>
__host__ __device__ __forceinline__ bool PairsFormScale(int srcW, int dstW)
{
    return srcW >= 4 && srcW <= 2 * dstW && (C != 4 || srcW <= dstW);
}

constexpr int kPairsTileW = 128, kPairsTileH = 8; // image batches: block = 4 waves of 128 columns x 2 rows, stacked

// The tile (in units of a wave's tile) of this wave in a launch of the tensor kernels below: a block's waves lie side by
// side (flat) or are stacked. Flat, a block writes few long row pieces instead of many short ones, which the memory
// likes better when the launch is bound by it (32 x u8x3, the two shapes alternating on one machine: 720p -> 1080p
// bilinear 67.3 -> 65.1 us, nearest 58.0 -> 55.4 us; 1080p -> 720p box filter 61.5 -> 59.6 us, bicubic 79.0 -> 77.3 us,
// bilinear 51.4 -> 51.2 us; bicubic enlarging 120.9 -> 125.8 us, which stays stacked). Rows much shorter than a flat
// block's span leave most of its waves without columns, and on small images the rows of a stacked block share source
// rows in the L1 (256 x 448 x 448 -> 300 x 300 u8x3 bicubic: 72.6 us stacked, 91.8 us flat), so the host chooses flat
// blocks for rows of 1024 pixels and more that fill their blocks to 80 % (FlatBlocks).
struct WaveTile
{
    int x, y;
};

__device__ __forceinline__ WaveTile WaveTileOf(int flat)
{
    // (arithmetic, not a branch: behind a branch on `flat` the compiler loads the kernel's other arguments only after
    // that test, one more round trip to memory before a wave's first pixel load, 0.3 us on the 4 - 6 us launches of small
    // batches)
    // (the wave's number as a scalar: tile origins, row terms and loop counters then stay on the scalar unit)
    const int waves = blockDim.x >> 6, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), f = flat != 0;
    const int across = f * (waves - 1) + 1, down = waves + 1 - across; // flat: waves, 1; stacked: 1, waves
    return WaveTile{(int)blockIdx.x * across + wave * f, (int)blockIdx.y * down + wave * (1 - f)};
}

static inline bool FlatBlocks(int dstW, int waveW)
{
    const int64_t span = 4 * (int64_t)waveW;
    return dstW >= 1024 && DivUp(dstW, (int)span) * span * 4 <= (int64_t)dstW * 5;
}

// Grid of a launch of four-wave blocks whose waves own tiles of waveW x waveH.
static inline dim3 WaveTileGrid(int dstW, int dstH, int N, int waveW, int waveH, bool flat, int waves = 4)
{
    return flat ? dim3(DivUp(dstW, waves * waveW), DivUp(dstH, waveH), N) : dim3(DivUp(dstW, waveW), DivUp(dstH, waves * waveH), N);
}

// Tensors: strips of 4 rows per wave.
template<int C>
__global__ __launch_bounds__(256) void ResizeLinearPairsU8Kernel(const ResizeArgs a, const int flat)
{
    const Plane p = GetPlanes<false>(a, blockIdx.z);
    const WaveTile t = WaveTileOf(flat);
    ResizeLinearPairStripU8<C>(p, t.x * kPairsTileW, t.y * kPairStripRows);
}

constexpr int kQuadsTileW = 256; // a wave's columns; tensors: block = 4 waves side by side (1024 columns x kQuadsRows rows)

// Rows per wave of the four-column form (strips for every pixel size; with 16-byte stores that the compiler had
// split into 12 + 4 bytes, 4-byte pixels were faster in two-row steps: 16 x 720p -> 1080p 43.7 us, now 37.7 as strips).
template<int C>
constexpr int kQuadsRows = kStripRows;

template<int C>
__global__ __launch_bounds__(256) void ResizeLinearQuadsU8Kernel(const ResizeArgs a, const int flat)
{
    const Plane p = GetPlanes<false>(a, blockIdx.z);
    const WaveTile t = WaveTileOf(flat);
    ResizeLinearQuadStripU8<C>(p, t.x * kQuadsTileW, t.y * kStripRows);
}

template<int C>
__global__ __launch_bounds__(256) void ResizeNearestQuadsU8Kernel(const ResizeArgs a, const int flat)
{
    const Plane p = GetPlanes<false>(a, blockIdx.z);
    const WaveTile t = WaveTileOf(flat);
    ResizeNearestQuadStripU8<C>(p, t.x * kQuadsTileW, t.y * kStripRows);
}

// Image batches: the same 128 x 8 tile per block for every image; an image whose horizontal scale is
// above 2 (or whose source is narrower than 4 pixels) is resized as four 64 x 4 wave patches instead.
template<int C>
__global__ __launch_bounds__(256) void ResizeLinearPairsU8VarShapeKernel(const ResizeArgs a, const VarTiles tiles)
{
    const TileCoord tc   = LocateTile(tiles, blockIdx.x);
    const Plane     p    = GetPlanes<true>(a, tc.image);
    const int       wave = threadIdx.x >> 6;
    if (PairsFormScale<C>(p.srcW, p.dstW))
    {
        ResizeLinearPairsU8<C, true>(p, tc.tx * kPairsTileW, tc.ty * kPairsTileH + wave * 2);
    }
    else
    {
        ResizeWavePatch<uint8_t, C, NVCV_INTERP_LINEAR, true>(p, tc.tx * kPairsTileW + (wave & 1) * 64,
                                                             tc.ty * kPairsTileH + (wave >> 1) * 4);
    }
}

// Large image-batch launches resize each image in the tensor kernels' strips; a wave owns a tile of 256 x 8 (WIDE: most of
// the launch is enlarged by 1.5 or more) or 128 x 4 output pixels, a block four of them, side by side or stacked as
// in the tensor kernels (WaveTileOf; the host chooses by the images' widths). WIDE: four columns per lane where the
// image is enlarged so, else two columns per lane at horizontal scales up to 2 (4 strips of 128 x 4), else 8 wave
// patches. Otherwise a two-column strip, or two wave patches.
template<bool WIDE>
constexpr int kStripsWaveW = WIDE ? kQuadsTileW : kPairsTileW;
template<bool WIDE>
constexpr int kStripsWaveH = WIDE ? kStripRows : kPairStripRows;

// The tile (in units of a wave's tile) of this wave in an image-batch block whose tile is 4 wave tiles wide (flat) or high.
__device__ __forceinline__ WaveTile VarWaveTileOf(const TileCoord &tc, int flat)
{
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), f = flat != 0;
    return WaveTile{tc.tx * (3 * f + 1) + wave * f, tc.ty * (4 - 3 * f) + wave * (1 - f)};
}

template<int C>
__host__ __device__ __forceinline__ bool QuadStripScale(int srcW, int dstW)
{
    return kQuadsRows<C> == kStripRows && srcW >= 4 && 3 * (int64_t)srcW <= 2 * (int64_t)dstW;
}

template<int C, bool WIDE>
__global__ __launch_bounds__(256) void ResizeLinearStripsU8VarShapeKernel(const ResizeArgs a, const VarTiles tiles, const int flat)
{
    const TileCoord tc = LocateTile(tiles, blockIdx.x);
    const Plane     p  = GetPlanes<true>(a, tc.image);
    const WaveTile  t  = VarWaveTileOf(tc, flat);
    const int       x0 = t.x * kStripsWaveW<WIDE>, y0 = t.y * kStripsWaveH<WIDE>;
    if constexpr (WIDE)
    {
        if (QuadStripScale<C>(p.srcW, p.dstW))
        {
            ResizeLinearQuadStripU8<C>(p, x0, y0);
        }
        else if (PairsFormScale<C>(p.srcW, p.dstW))
        {
#pragma unroll 1
            for (int i = 0; i < 4; ++i)
            {
                ResizeLinearPairStripU8<C>(p, x0 + (i & 1) * kPairsTileW, y0 + (i >> 1) * kPairStripRows);
            }
        }
        else
        {
#pragma unroll 1
            for (int i = 0; i < 8; ++i)
            {
                ResizeWavePatch<uint8_t, C, NVCV_INTERP_LINEAR, true>(p, x0 + (i & 3) * 64, y0 + (i >> 2) * 4);
            }
        }
    }
    else
    {
        if (PairsFormScale<C>(p.srcW, p.dstW))
        {
            ResizeLinearPairStripU8<C>(p, x0, y0);
        }
        else
        {
            ResizeWavePatch<uint8_t, C, NVCV_INTERP_LINEAR, true>(p, x0, y0);
            ResizeWavePatch<uint8_t, C, NVCV_INTERP_LINEAR, true>(p, x0 + 64, y0);
        }
    }
}

// Nearest neighbour: whether an image takes the four-column strips (enlarged by 1.5 or more across, not reduced down;
// a window may start at a row's last pixel and, with the bytes a load takes along, runs up to 13
// bytes into the next row: sources of 8 columns and more).
template<int C>
__host__ __device__ __forceinline__ bool NearestStripScale(int srcW, int srcH, int dstW, int dstH)
{
    return srcW >= 8 && 3 * (int64_t)srcW <= 2 * (int64_t)dstW && srcH <= dstH;
}

// Large image batches that are mostly such images: a 256 x 8 tile per wave, a strip or eight patches.
template<int C>
__global__ __launch_bounds__(256) void ResizeNearestStripsU8VarShapeKernel(const ResizeArgs a, const VarTiles tiles, const int flat)
{
    const TileCoord tc = LocateTile(tiles, blockIdx.x);
    const Plane     p  = GetPlanes<true>(a, tc.image);
    const WaveTile  t  = VarWaveTileOf(tc, flat);
    const int       x0 = t.x * kStripsWaveW<true>, y0 = t.y * kStripsWaveH<true>;
    if (NearestStripScale<C>(p.srcW, p.srcH, p.dstW, p.dstH))
    {
        ResizeNearestQuadStripU8<C>(p, x0, y0);
    }
    else
    {
#pragma unroll 1
        for (int i = 0; i < 8; ++i)
        {
            ResizeWavePatch<uint8_t, C, NVCV_INTERP_NEAREST, true>(p, x0 + (i & 3) * 64, y0 + (i >> 2) * 4);
        }
    }
}

constexpr int kPatchTileW = 64, kPatchTileH = 16; // block = 4 waves stacked vertically

template<class T, int C, int INTERP>
__global__ __launch_bounds__(256) void ResizePatchTensorKernel(const ResizeArgs a, const int flat)
{
    const Plane p = GetPlanes<false>(a, blockIdx.z);
    // blocks are 4 waves, or single waves when the whole launch is small
    const WaveTile t = WaveTileOf(flat);
    ResizeWavePatch<T, C, INTERP, false>(p, t.x * kPatchTileW, t.y * 4);
}

// Which of the bicubic strip forms an image takes by its vertical scale and row length: 4 (reducing by up to 2), 8
// (enlarging by up to 2) or 0 (none: wave patches).
template<int C>
__host__ __device__ __forceinline__ int CubicStripForm(int srcW, int srcH, int dstH)
{
    if (!(C == 3 || C == 4) || srcW < 4 || srcW * C < 16)
    {
        return 0;
    }
    return (srcH >= dstH && srcH <= 2 * (int64_t)dstH) ? 4 : ((srcH < dstH && 2 * (int64_t)srcH >= dstH) ? 8 : 0);
}

// Large image batches: a 64 x 64 tile per block, a strip per wave where the image's scale allows, else four patches.
template<int C>
__global__ __launch_bounds__(256) void ResizeCubicStripU8VarShapeKernel(const ResizeArgs a, const VarTiles tiles)
{
    const TileCoord tc   = LocateTile(tiles, blockIdx.x);
    const Plane     p    = GetPlanes<true>(a, tc.image);
    const int       x0 = tc.tx * kPatchTileW, y0 = tc.ty * 4 * kCubicStripRows + (threadIdx.x >> 6) * kCubicStripRows;
    const int       form = CubicStripForm<C>(p.srcW, p.srcH, p.dstH);
    if (form == 4)
    {
        ResizeCubicStripU8<C, 4>(p, x0, y0);
    }
    else if (form == 8)
    {
        ResizeCubicStripU8<C, 8>(p, x0, y0);
    }
    else
    {
#pragma unroll 1
        for (int g = 0; g < kCubicStripRows; g += 4)
        {
            ResizeWavePatch<uint8_t, C, NVCV_INTERP_CUBIC, true>(p, x0, y0 + g);
        }
    }
}

// 8-bit bicubic strips: block = 4 waves stacked vertically (64 columns x 64 rows) or, reducing wide images, side by side.
template<int C, int S>
__global__ __launch_bounds__(256) void ResizeCubicStripU8Kernel(const ResizeArgs a, const int flat)
{
    const Plane p = GetPlanes<false>(a, blockIdx.z);
    const WaveTile t = WaveTileOf(flat);
    ResizeCubicStripU8<C, S>(p, t.x * kPatchTileW, t.y * kCubicStripRows);
}

template<class T, int C, int INTERP>
__global__ __launch_bounds__(256) void ResizePatchVarShapeKernel(const ResizeArgs a, const VarTiles tiles, const int flat)
{
    const TileCoord tc = LocateTile(tiles, blockIdx.x);
    const Plane     p  = GetPlanes<true>(a, tc.image);
    const WaveTile  t  = VarWaveTileOf(tc, flat);
    ResizeWavePatch<T, C, INTERP, true>(p, t.x * kPatchTileW, t.y * 4);
}

// ---------------------------------------------------------------------------------------------
// Box filter (AREA) of 8-bit pixels at reductions of up to 3 along both axes, in fixed point.
//
// The weight of a source pixel is the length of its overlap with the box the output pixel covers,
// [d * scale, d * scale + scale): for scales of 1 and more exactly the reference's left-partial, whole and
// right-partial weights (cuda_tools/InterpolationWrap.hpp:668-760; each is one float32 subtraction of the
// same operands), pixels outside the image weigh nothing, and the sum is divided by the length of the box
// inside the image along each axis. A box of up to 3 touches at most 4 pixels per axis; the window of 4
// starts at the box's first pixel or, at the image's far edge, 4 before its end (pixels in front of the box
// then get the weight 0 from the same expression), so a window never leaves its row. Per source row the 4
// pixels are one load of the dwords that hold them; the horizontal weights, already divided, are rounded to
// 15 bits and a row's sum is two v_dot2_u32_u16 per channel on bytes (exact, below 2^24); the rows' sums are
// added in float32 with the rows' weights (wave-uniform), and the result is rounded once.
//
// One wave produces 64 columns x 16 rows: lane l owns column l (its terms are computed once), the 16 rows'
// terms are computed side by side in lanes 0-15 and read back as wave-uniform values, and every 4 rows leave
// through the 4x4 lane transposes as whole dwords.
template<class T, int C, int INTERP>
constexpr bool kAreaFixed = std::is_same_v<T, uint8_t> && INTERP == NVCV_INTERP_AREA && (C == 1 || C == 3 || C == 4);

constexpr int kAreaRowsPerWave = 16;
constexpr int kAreaTileW = 64, kAreaTileH = 4 * kAreaRowsPerWave; // image batches: block = 4 waves stacked vertically; tensors: side by side

// Per image: both scales within 1 .. 3 and a source of at least 4 rows of at least 32 bytes.
__host__ __device__ __forceinline__ bool AreaFixedDomain(float scaleX, float scaleY, int srcRowBytes, int srcH)
{
    return scaleX >= 1.f && scaleX <= 3.f && scaleY >= 1.f && scaleY <= 3.f && srcRowBytes >= 32 && srcH >= 4;
}

// Weights of the 4 source indices from `start` on (a whole number) for output index d: each one's overlap with
// the box, divided by the box's length inside the image, times `unit`. The overlap of index x is written
// clamp(f2 - x, 0, 1) - clamp(f1 - x, 0, 1) (a clamp is one v_med3_f32): for an index the box
// covers partly, wholly or not at all that is f2 - x or (x + 1) - f1 (both exact), 1, or 0. With `bounded`,
// indices behind the image weigh nothing (callers that pass a start of at most srcSize - 4 need no test).
__device__ __forceinline__ void AreaWeights(float scale, int d, int srcSize, float unit, float start, bool bounded, float (&w)[4])
{
    const float f1 = d * scale, end = f1 + scale;
    const float f2 = bounded ? fminf(end, (float)srcSize) : end;
    const float norm = (1.f / fminf(scale, srcSize - f1)) * unit;
    float       x = start;
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        w[k] = (__builtin_amdgcn_fmed3f(f2 - x, 0.f, 1.f) - __builtin_amdgcn_fmed3f(f1 - x, 0.f, 1.f)) * norm;
        x += 1.f;
    }
}

__device__ __forceinline__ uint32_t Dot2U16(uint32_t taps, uint32_t weights, uint32_t acc)
{
    typedef unsigned short U16x2 __attribute__((ext_vector_type(2)));
    U16x2 t, w;
    __builtin_memcpy(&t, &taps, 4);
    __builtin_memcpy(&w, &weights, 4);
    return __builtin_amdgcn_udot2(t, w, acc, false);
}

// A source row's sums per channel from its window and the packed horizontal weights, each plus 2^23: the integer sum
// (below 2^23) is accumulated on the bit pattern of 8388608.0f, whose unit in the last place is 1, so the register
// read as a float IS 2^23 + sum and no conversion is needed. The caller's accumulator starts at minus 2^23 times
// the sum of the rows' weights.
template<int C>
__device__ __forceinline__ void AreaRowSums(const uint32_t (&r)[C], uint32_t w01, uint32_t w23, float (&s)[C])
{
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        s[c] = __uint_as_float(Dot2U16(QuadTapPair<C>(r, 2, c), w23, Dot2U16(QuadTapPair<C>(r, 0, c), w01, 0x4b000000u)));
    }
}

// K output pixels per lane (vertically adjacent) from N source rows, the first at `row`; wy[k][j] is the weight of
// source row j in output pixel k. All N windows are requested before the first sum; every row's sums are formed once.
// Rows are added in ascending order, the first as a product, the others with fused multiply-adds: a row of weight 0
// changes nothing, so the result does not depend on which rows are passed beside those of the pixel's box.
template<int C, int N, int K>
__device__ __forceinline__ void AreaSumRows(const uint32_t (&r)[N][C], uint32_t w01, uint32_t w23, const float (&wy)[K][4],
                                            const float (&start)[K], uint32_t *out)
{
    float acc[K][C];
#pragma unroll
    for (int j = 0; j < N; ++j)
    {
        float s[C];
        AreaRowSums<C>(r[j], w01, w23, s);
#pragma unroll
        for (int k = 0; k < K; ++k)
        {
#pragma unroll
            for (int c = 0; c < C; ++c)
            {
                acc[k][c] = fmaf(s[c], wy[k][j], j == 0 ? start[k] : acc[k][c]);
            }
        }
    }
#pragma unroll
    for (int k = 0; k < K; ++k)
    {
        out[k] = 0;
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out[k] = __builtin_amdgcn_cvt_pk_u8_f32(acc[k][c], c, out[k]);
        }
    }
}

template<int C, int N, int K, bool GUARDED>
__device__ __forceinline__ void AreaFixedPixels(const uint8_t *row, int srcRow, int lastRowIn, uint32_t at, uint32_t shift,
                                                uint32_t rowBytes, uint32_t w01, uint32_t w23, const float (&wy)[K][4],
                                                const float (&start)[K], uint32_t (&out)[K])
{
    uint32_t r[N][C];
#pragma unroll
    for (int j = 0; j < N; ++j)
    {
        LoadQuadWindow<C, GUARDED>(row + (int64_t)j * srcRow, at, shift, j == lastRowIn, rowBytes, r[j]);
    }
    AreaSumRows<C, N, K>(r, w01, w23, wy, start, out);
}

// Two such pairs of output pixels (4 vertically adjacent ones) from 3 source rows each, none of them the image's last:
// the six windows are requested together. A pair that needs only 2 rows passes a third of weight 0.
template<int C>
__device__ __forceinline__ void AreaFixedTwoPairs(const uint8_t *rowA, const uint8_t *rowB, int srcRow, uint32_t at, uint32_t shift,
                                                  uint32_t rowBytes, uint32_t w01, uint32_t w23, const float (&wyA)[2][4],
                                                  const float (&wyB)[2][4], const float (&startA)[2], const float (&startB)[2],
                                                  uint32_t (&out)[4])
{
    uint32_t ra[3][C], rb[3][C];
#pragma unroll
    for (int j = 0; j < 3; ++j)
    {
        LoadQuadWindow<C, false>(rowA + (int64_t)j * srcRow, at, shift, false, rowBytes, ra[j]);
    }
#pragma unroll
    for (int j = 0; j < 3; ++j)
    {
        LoadQuadWindow<C, false>(rowB + (int64_t)j * srcRow, at, shift, false, rowBytes, rb[j]);
    }
    AreaSumRows<C, 3, 2>(ra, w01, w23, wyA, startA, &out[0]);
    AreaSumRows<C, 3, 2>(rb, w01, w23, wyB, startB, &out[2]);
}

template<int C, int K, bool GUARDED>
__device__ __forceinline__ void AreaFixedRowsOf(int n, const uint8_t *row, int srcRow, int lastRowIn, uint32_t at, uint32_t shift,
                                                uint32_t rowBytes, uint32_t w01, uint32_t w23, const float (&wy)[K][4],
                                                const float (&start)[K], uint32_t (&out)[K])
{
    // (wave-uniform)
    if (n == 3)
    {
        AreaFixedPixels<C, 3, K, GUARDED>(row, srcRow, lastRowIn, at, shift, rowBytes, w01, w23, wy, start, out);
    }
    else if (n == 2)
    {
        AreaFixedPixels<C, 2, K, GUARDED>(row, srcRow, lastRowIn, at, shift, rowBytes, w01, w23, wy, start, out);
    }
    else if (n == 4)
    {
        AreaFixedPixels<C, 4, K, GUARDED>(row, srcRow, lastRowIn, at, shift, rowBytes, w01, w23, wy, start, out);
    }
    else
    {
        AreaFixedPixels<C, 1, K, GUARDED>(row, srcRow, lastRowIn, at, shift, rowBytes, w01, w23, wy, start, out);
    }
}

// n source rows from `row` on; lastRowIn: which of them is the image's last row (n or more: none).
template<int C, int K>
__device__ __forceinline__ void AreaFixedRows(int n, const uint8_t *row, int srcRow, int lastRowIn, uint32_t at, uint32_t shift,
                                              uint32_t rowBytes, uint32_t w01, uint32_t w23, const float (&wy)[K][4],
                                              const float (&start)[K], uint32_t (&out)[K])
{
    if (C != 4 && lastRowIn < n) // wave-uniform, once per image and column tile
    {
        AreaFixedRowsOf<C, K, true>(n, row, srcRow, lastRowIn, at, shift, rowBytes, w01, w23, wy, start, out);
    }
    else
    {
        AreaFixedRowsOf<C, K, false>(n, row, srcRow, lastRowIn, at, shift, rowBytes, w01, w23, wy, start, out);
    }
}

// The tile of 64 columns x 16 rows whose top left pixel is (x0, y0), both wave-uniform (y0 even).
template<int C>
__device__ __forceinline__ void ResizeAreaFixedWaveTile(const Plane &p, int x0, int y0)
{
    if (x0 >= p.dstW || y0 >= p.dstH)
    {
        return;
    }
    const int lane = threadIdx.x & 63;
    // columns and rows past the output compute a duplicate of the last one: every lane takes part in the transposes
    const int   dx = min(x0 + lane, p.dstW - 1);
    const float colStart = fminf(floorf(dx * p.scaleX), (float)(p.srcW - 4)); // the window never leaves its row
    float       cw[4];
    AreaWeights(p.scaleX, dx, p.srcW, 32768.f, colStart, false, cw);
    // rounding to an integer by adding 1.5 * 2^23: the low 16 bits of the sum's pattern are the integer
    uint32_t wq[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        wq[k] = __float_as_uint(cw[k] + 12582912.f);
    }
    const uint32_t w01 = __builtin_amdgcn_perm(wq[1], wq[0], 0x05040100u), w23 = __builtin_amdgcn_perm(wq[3], wq[2], 0x05040100u);
    const uint32_t off = (uint32_t)(int)colStart * C, at = C == 4 ? off : off & ~3u, shift = off & 3u;
    const uint32_t rowBytes = (uint32_t)p.srcW * C;

    // Row terms, lane l: output row y0 + (l & 15). Two vertically adjacent output rows (2i, 2i + 1) share the source
    // row between their boxes wherever the scale is not a whole number, so they are produced together from the
    // source rows first(2i) .. first(2i) + n - 1 when those are at most 4 (`pairRows`, else 0): `pw` are this row's
    // weights counted from first(2i). Otherwise each row on its own from its box's first row: `ow`, `ownRows`.
    const int   dy = min(y0 + (lane & (kAreaRowsPerWave - 1)), p.dstH - 1);
    const float ownStart = floorf(dy * p.scaleY), pairStart = floorf((dy & ~1) * p.scaleY);
    float       ow[4], pw[4];
    AreaWeights(p.scaleY, dy, p.srcH, 1.f / 32768.f, ownStart, true, ow);
    AreaWeights(p.scaleY, dy, p.srcH, 1.f / 32768.f, pairStart, true, pw);
    const int  ownRows = 1 + (ow[1] != 0.f) + (ow[2] != 0.f) + (ow[3] != 0.f);
    const bool fits    = fminf(dy * p.scaleY + p.scaleY, (float)p.srcH) <= pairStart + 4.f;
    const int  pairRows = !fits ? 0 : pw[3] != 0.f ? 4 : pw[2] != 0.f ? 3 : pw[1] != 0.f ? 2 : 1;
    const int  ownFirst = (int)ownStart, pairFirst = (int)pairStart;
    // the accumulator's start: minus 2^23 times the sum of the row's weights (see AreaRowSums), added in ascending order;
    // weights of 0 in front or behind change nothing, so the pair form and the single form start alike
    const float rowStart = -8388608.f * (((ow[0] + ow[1]) + ow[2]) + ow[3]);

    const int rowsHere = min(kAreaRowsPerWave, p.dstH - y0);
    // output rows i, i + 1 -> out[0], out[1]
    auto rowPair = [&](int i, uint32_t *out)
    {
        const int n = __builtin_amdgcn_readlane(pairRows, i + 1);
        if (n != 0)
        {
            const int first = __builtin_amdgcn_readlane(pairFirst, i);
            float     wy[2][4];
            uint32_t  two[2];
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                wy[0][j] = ReadLane(pw[j], i);
                wy[1][j] = ReadLane(pw[j], i + 1);
            }
            const float start[2] = {ReadLane(rowStart, i), ReadLane(rowStart, i + 1)};
            AreaFixedRows<C, 2>(n, p.src + (int64_t)first * p.srcRow, p.srcRow, p.srcH - 1 - first, at, shift, rowBytes, w01,
                                w23, wy, start, two);
            out[0] = two[0];
            out[1] = two[1];
        }
        else
        {
#pragma unroll
            for (int k = 0; k < 2; ++k)
            {
                const int first = __builtin_amdgcn_readlane(ownFirst, i + k);
                float     wy[1][4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    wy[0][j] = ReadLane(ow[j], i + k);
                }
                uint32_t    one[1];
                const float start[1] = {ReadLane(rowStart, i + k)};
                AreaFixedRows<C, 1>(__builtin_amdgcn_readlane(ownRows, i + k), p.src + (int64_t)first * p.srcRow, p.srcRow,
                                    p.srcH - 1 - first, at, shift, rowBytes, w01, w23, wy, start, one);
                out[k] = one[0];
            }
        }
    };
    // 4 output rows per step (rows past the output are duplicates of its last one and are not stored)
#pragma unroll 1
    for (int i = 0; i < rowsHere; i += 4)
    {
        uint32_t  q[1][4];
        const int nA = __builtin_amdgcn_readlane(pairRows, i + 1), nB = __builtin_amdgcn_readlane(pairRows, i + 3);
        const int firstA = __builtin_amdgcn_readlane(pairFirst, i), firstB = __builtin_amdgcn_readlane(pairFirst, i + 2);
        // the usual case at scales up to 1.5: both pairs from at most 3 rows each, clear of the image's last row
        // (wave-uniform)
        if (nA != 0 && nB != 0 && max(nA, nB) <= 3 && max(firstA, firstB) + 2 < p.srcH - 1)
        {
            float wyA[2][4], wyB[2][4];
#pragma unroll
            for (int j = 0; j < 3; ++j)
            {
                wyA[0][j] = ReadLane(pw[j], i);
                wyA[1][j] = ReadLane(pw[j], i + 1);
                wyB[0][j] = ReadLane(pw[j], i + 2);
                wyB[1][j] = ReadLane(pw[j], i + 3);
            }
            const float startA[2] = {ReadLane(rowStart, i), ReadLane(rowStart, i + 1)};
            const float startB[2] = {ReadLane(rowStart, i + 2), ReadLane(rowStart, i + 3)};
            AreaFixedTwoPairs<C>(p.src + (int64_t)firstA * p.srcRow, p.src + (int64_t)firstB * p.srcRow, p.srcRow, at, shift,
                                 rowBytes, w01, w23, wyA, wyB, startA, startB, q[0]);
        }
        else
        {
            rowPair(i, &q[0][0]);
            rowPair(i + 2, &q[0][2]);
        }
        StoreWavePatch<uint8_t, C>(p, x0, y0 + i, lane, q);
    }
}

// The same tile outside the fixed-point form's scales (image batches decide per image): one pixel at a time.
template<int C, bool VARSHAPE>
__device__ __forceinline__ void ResizeAreaPlainWaveTile(const Plane &p, int x0, int y0)
{
    const int dx = x0 + (int)(threadIdx.x & 63);
    if (dx >= p.dstW)
    {
        return;
    }
#pragma unroll 1
    for (int dy = y0; dy < min(y0 + kAreaRowsPerWave, p.dstH); ++dy)
    {
        ResizePixel<uint8_t, C, NVCV_INTERP_AREA, VARSHAPE>(p, dx, dy);
    }
}

template<int C>
__global__ __launch_bounds__(256) void ResizeAreaFixedTensorKernel(const ResizeArgs a, const int flat)
{
    const Plane p = GetPlanes<false>(a, blockIdx.z);
    const WaveTile t = WaveTileOf(flat);
    ResizeAreaFixedWaveTile<C>(p, t.x * kAreaTileW, t.y * kAreaRowsPerWave);
}

template<int C>
__global__ __launch_bounds__(256) void ResizeAreaVarShapeKernel(const ResizeArgs a, const VarTiles tiles)
{
    const TileCoord tc = LocateTile(tiles, blockIdx.x);
    const Plane     p  = GetPlanes<true>(a, tc.image);
    const int       x0 = tc.tx * kAreaTileW, y0 = tc.ty * kAreaTileH + (threadIdx.x >> 6) * kAreaRowsPerWave;
    if (AreaFixedDomain(p.scaleX, p.scaleY, p.srcW * C, p.srcH))
    {
        ResizeAreaFixedWaveTile<C>(p, x0, y0);
    }
    else
    {
        ResizeAreaPlainWaveTile<C, true>(p, x0, y0);
    }
}

// Bicubic for strong horizontal reductions. With one lane per output pixel the four taps of
// neighbouring lanes lie scale*pixel bytes apart, so each of a wave's tap loads touches 64 separate
// cache lines. Here the same 256 taps of a wave's row are fetched tap-major instead: lane l loads
// tap l%4 of pixel 16k + l/4 (k = 0..3), four lanes covering 4 contiguous pixels, and the wave
// hands the taps to their owners through LDS. Arithmetic and its order are those of ResizePixel.
template<int BYTES>
struct alignas(BYTES % 16 == 0 ? 16 : (BYTES % 8 == 0 ? 8 : 4)) LdsSlot
{
    uint32_t w[BYTES / 4];
};

__device__ __forceinline__ void CubicSourceX(int srcW, float scaleX, int dx, int &sx, float &fx)
{
    const float cx = (dx + .5f) * scaleX - .5f;
    sx             = (int)floorf(cx);
    fx             = cx - sx;
    fx             = (sx < 1 || sx >= srcW - 3) ? 0.f : fx;
    sx             = max(1, min(sx, srcW - 3));
}

template<class T, int C>
__global__ __launch_bounds__(256) void ResizeCubicStagedKernel(const ResizeArgs a)
{
    using Px   = Pixel<T, C>;
    using Slot = LdsSlot<sizeof(Px)>;
    static_assert(sizeof(Px) % 4 == 0, "pixels are staged as whole dwords");
    __shared__ Slot stage[kTileH][kTileW * 4];

    const int   lane = threadIdx.x & 63;
    const int   wave = threadIdx.x >> 6;
    const Plane p    = GetPlanes<false>(a, blockIdx.z);
    const int   dx   = blockIdx.x * kTileW + lane;
    const int   dy   = blockIdx.y * kTileH + wave;

    const float scaleX = p.scaleX, scaleY = p.scaleY;

    // lanes and rows past the output compute a duplicate of the last pixel and skip the store: every
    // lane takes part in its wave's exchange (each wave owns one quarter of the staging array)
    int   sx;
    float fx;
    CubicSourceX(p.srcW, scaleX, min(dx, p.dstW - 1), sx, fx);
    const float cy = (min(dy, p.dstH - 1) + .5f) * scaleY - .5f;
    int         sy = (int)floorf(cy);
    const float fy = cy - sy;
    sy             = max(1, min(sy, p.srcH - 3));
    float wx[4], wy[4];
    CubicCoeffs(fx, wx);
    CubicCoeffs(fy, wy);

    // loader role: column of the tap this lane fetches in each of the four instructions
    int tapX[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        int   qsx;
        float qfx;
        CubicSourceX(p.srcW, scaleX, min(blockIdx.x * kTileW + 16 * k + (lane >> 2), p.dstW - 1), qsx, qfx);
        tapX[k] = max(0, min(qsx - 1 + (lane & 3), p.srcW - 1));
    }

    Px   v[4][4];
    auto loadRow = [&](int j)
    {
        const int      yy  = max(0, min(sy - 1 + j, p.srcH - 1));
        const uint8_t *row = p.src + (int64_t)yy * p.srcRow;
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            v[j][k] = LoadPx<T, C>(row, tapX[k]);
        }
    };

    float sum[C];
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        sum[c] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        loadRow(j);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
            __builtin_memcpy(&stage[wave][64 * k + lane], &v[j][k], sizeof(Px));
        }
        WaveExchangeFence();
        Px t[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            __builtin_memcpy(&t[i], &stage[wave][4 * lane + i], sizeof(Px));
        }
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                sum[c] += (float)t[i].v[c] * (wx[i] * wy[j]);
            }
        }
        WaveExchangeFence();
    }
    if (dx < p.dstW && dy < p.dstH)
    {
        Px out;
#pragma unroll
        for (int c = 0; c < C; ++c)
        {
            out.v[c] = SaturateCast<T>(fabsf(sum[c]));
        }
        StorePx<T, C>(p.dst + (int64_t)dy * p.dstRow, dx, out);
    }
}

// Which (type, channels, interpolation) run as wave patches.
template<class T, int C, int INTERP>
constexpr bool kPatchForm = INTERP != NVCV_INTERP_AREA && sizeof(Pixel<T, C>) <= 8;

template<class T, int C, int INTERP>
void LaunchTensor(const ResizeArgs &a, int N, hipStream_t stream)
{
    dim3 grid(DivUp(a.dstW, kTileW), DivUp(a.dstH, kTileH), N);
    if constexpr (INTERP == NVCV_INTERP_CUBIC && sizeof(Pixel<T, C>) % 4 == 0 && !kPatchForm<T, C, INTERP>)
    {
        if (a.srcW >= 2 * a.dstW)
        {
            hipLaunchKernelGGL((ResizeCubicStagedKernel<T, C>), grid, dim3(256), 0, stream, a);
            CheckLaunch("ResizeCubicStagedKernel");
            return;
        }
    }
    // (8 x 720p -> 1080p: 1 channel 12.4 -> 8.4 us, 3 channels 19.0 -> 16.7 us, 4 channels 21.2 -> 18.7 us)
    if constexpr (std::is_same_v<T, uint8_t> && INTERP == NVCV_INTERP_NEAREST && (C == 1 || C == 3 || C == 4))
    {
        const int64_t strips = (int64_t)DivUp(a.dstW, kQuadsTileW) * DivUp(a.dstH, kStripRows) * N;
        if (NearestStripScale<C>(a.srcW, a.srcH, a.dstW, a.dstH) && strips >= 8 * 256)
        {
            const bool flat = FlatBlocks(a.dstW, kQuadsTileW);
            hipLaunchKernelGGL((ResizeNearestQuadsU8Kernel<C>), WaveTileGrid(a.dstW, a.dstH, N, kQuadsTileW, kStripRows, flat), dim3(256), 0,
                               stream, a, (int)flat);
            CheckLaunch("ResizeNearestQuadsU8Kernel");
            return;
        }
    }
    if constexpr (kPairsForm<T, C, INTERP>)
    {
        if (a.srcW >= 4 && 3 * (int64_t)a.srcW <= 2 * (int64_t)a.dstW)
        {
            const bool flat = FlatBlocks(a.dstW, kQuadsTileW);
            hipLaunchKernelGGL((ResizeLinearQuadsU8Kernel<C>), WaveTileGrid(a.dstW, a.dstH, N, kQuadsTileW, kStripRows, flat), dim3(256), 0,
                               stream, a, (int)flat);
            CheckLaunch("ResizeLinearQuadsU8Kernel");
            return;
        }
        if (PairsFormScale<C>(a.srcW, a.dstW))
        {
            const bool flat = FlatBlocks(a.dstW, kPairsTileW);
            hipLaunchKernelGGL((ResizeLinearPairsU8Kernel<C>), WaveTileGrid(a.dstW, a.dstH, N, kPairsTileW, kPairStripRows, flat), dim3(256),
                               0, stream, a, (int)flat);
            CheckLaunch("ResizeLinearPairsU8Kernel");
            return;
        }
    }
    if constexpr (kAreaFixed<T, C, INTERP>)
    {
        if (AreaFixedDomain(a.scaleX, a.scaleY, a.srcW * C, a.srcH))
        {
            const bool flat = FlatBlocks(a.dstW, kAreaTileW);
            hipLaunchKernelGGL((ResizeAreaFixedTensorKernel<C>), WaveTileGrid(a.dstW, a.dstH, N, kAreaTileW, kAreaRowsPerWave, flat),
                               dim3(256), 0, stream, a, (int)flat);
            CheckLaunch("ResizeAreaFixedTensorKernel");
            return;
        }
    }
    if constexpr (INTERP == NVCV_INTERP_CUBIC && std::is_same_v<T, uint8_t> && (C == 3 || C == 4))
    {
        // strips of 16 rows per wave where consecutive windows overlap (vertical scales of 1/2 to 2) and the launch
        // still has 8 waves and more per CU; one channel is as fast or faster as wave patches (16 x 720p -> 1080p
        // 46.6 us against 50.9 as strips, 1080p -> 720p 27.2 against 28.1)
        const int64_t strips = (int64_t)DivUp(a.dstW, kPatchTileW) * DivUp(a.dstH, kCubicStripRows) * N;
        const int     form   = CubicStripForm<C>(a.srcW, a.srcH, a.dstH);
        if (strips >= 8 * 256 && form != 0)
        {
            const bool flat = form == 4 && FlatBlocks(a.dstW, kPatchTileW); // (enlarging: stacked, see WaveTileOf)
            const dim3 sgrid = WaveTileGrid(a.dstW, a.dstH, N, kPatchTileW, kCubicStripRows, flat);
            if (form == 4)
            {
                hipLaunchKernelGGL((ResizeCubicStripU8Kernel<C, 4>), sgrid, dim3(256), 0, stream, a, (int)flat);
            }
            else
            {
                hipLaunchKernelGGL((ResizeCubicStripU8Kernel<C, 8>), sgrid, dim3(256), 0, stream, a, (int)flat);
            }
            CheckLaunch("ResizeCubicStripU8Kernel");
            return;
        }
    }
    if constexpr (kPatchForm<T, C, INTERP>)
    {
        // a launch of under 8 four-wave blocks per CU is spread as single-wave blocks: it is latency-bound
        // and finishes sooner the more CUs take part
        const int64_t blocks = (int64_t)DivUp(a.dstW, kPatchTileW) * DivUp(a.dstH, kPatchTileH) * N;
        const int     waves  = blocks < 8 * 256 ? 1 : 4;
        const bool    flat   = waves == 4 && FlatBlocks(a.dstW, kPatchTileW);
        hipLaunchKernelGGL((ResizePatchTensorKernel<T, C, INTERP>), WaveTileGrid(a.dstW, a.dstH, N, kPatchTileW, 4, flat, waves),
                           dim3(64 * waves), 0, stream, a, (int)flat);
        CheckLaunch("ResizePatchTensorKernel");
        return;
    }
    // Enlarging, the launch's time is its writes and a block that writes one run of a row is faster (8 x 720p -> 1080p
    // f32x3 bilinear 56.4 -> 45.5 us, f32x4 68.1 -> 56.3 us); reducing, it is the reads, and the four rows of the
    // 64 x 4 block share source rows (1080p -> 720p f32x3 bilinear 41.1 us against 49.3 us flat).
    // (bicubic keeps the 64 x 4 block: its time is the arithmetic's and did not change with the block)
    const int flat = INTERP != NVCV_INTERP_CUBIC && (int64_t)a.dstW * a.dstH > (int64_t)a.srcW * a.srcH && FlatBlocks(a.dstW, kTileW);
    hipLaunchKernelGGL((ResizeTensorKernel<T, C, INTERP>), flat ? dim3(DivUp(a.dstW, kTileW * kTileH), a.dstH, N) : grid, dim3(256), 0, stream,
                       a, flat);
    CheckLaunch("ResizeTensorKernel");
}

template<class T, int C, int INTERP>
void LaunchVarShape(const ResizeArgs &a, const NVCVImageBufferStrided *srcHost, const NVCVImageBufferStrided *dstHost, int N,
                    hipStream_t stream)
{
    for (int first = 0; first < N; first += kMaxTileImages)
    {
        VarTiles  tiles;
        const int count = std::min(kMaxTileImages, N - first);
        // whether most output pixels of this launch lie in images for which a block of four waves side by side pays
        // (FlatBlocks), given a wave's tile; and the block's tile either way
        auto flatFor = [&](int waveW)
        {
            int64_t flatPixels = 0, allPixels = 0;
            for (int i = first; i < first + count; ++i)
            {
                const int64_t px = (int64_t)dstHost[i].planes[0].width * dstHost[i].planes[0].height;
                allPixels += px;
                flatPixels += FlatBlocks(dstHost[i].planes[0].width, waveW) ? px : 0;
            }
            return 2 * flatPixels > allPixels;
        };
        auto buildTiles = [&](int waveW, int waveH, bool flat)
        { return BuildVarTiles(tiles, dstHost, first, count, flat ? 4 * waveW : waveW, flat ? waveH : 4 * waveH); };
        if constexpr (kPairsForm<T, C, INTERP>)
        {
            // strips when that still gives every CU 8 blocks: the wide tile where most output pixels belong to images
            // that take four columns per lane
            int64_t quadPixels = 0, allPixels = 0;
            for (int i = first; i < first + count; ++i)
            {
                const int64_t px = (int64_t)dstHost[i].planes[0].width * dstHost[i].planes[0].height;
                allPixels += px;
                quadPixels += QuadStripScale<C>(srcHost[i].planes[0].width, dstHost[i].planes[0].width) ? px : 0;
            }
            bool flat  = flatFor(kStripsWaveW<true>);
            int  total = 2 * quadPixels > allPixels ? buildTiles(kStripsWaveW<true>, kStripsWaveH<true>, flat) : 0;
            if (total >= 8 * 256)
            {
                hipLaunchKernelGGL((ResizeLinearStripsU8VarShapeKernel<C, true>), dim3(total), dim3(256), 0, stream, a, tiles, (int)flat);
                CheckLaunch("ResizeLinearStripsU8VarShapeKernel");
                continue;
            }
            flat  = flatFor(kStripsWaveW<false>);
            total = buildTiles(kStripsWaveW<false>, kStripsWaveH<false>, flat);
            if (total >= 8 * 256)
            {
                hipLaunchKernelGGL((ResizeLinearStripsU8VarShapeKernel<C, false>), dim3(total), dim3(256), 0, stream, a, tiles, (int)flat);
                CheckLaunch("ResizeLinearStripsU8VarShapeKernel");
                continue;
            }
            total = BuildVarTiles(tiles, dstHost, first, count, kPairsTileW, kPairsTileH);
            if (total > 0)
            {
                hipLaunchKernelGGL((ResizeLinearPairsU8VarShapeKernel<C>), dim3(total), dim3(256), 0, stream, a, tiles);
                CheckLaunch("ResizeLinearPairsU8VarShapeKernel");
            }
            continue;
        }
        if constexpr (kAreaFixed<T, C, INTERP>)
        {
            int total = BuildVarTiles(tiles, dstHost, first, count, kAreaTileW, kAreaTileH);
            if (total > 0)
            {
                hipLaunchKernelGGL((ResizeAreaVarShapeKernel<C>), dim3(total), dim3(256), 0, stream, a, tiles);
                CheckLaunch("ResizeAreaVarShapeKernel");
            }
            continue;
        }
        if constexpr (INTERP == NVCV_INTERP_NEAREST && std::is_same_v<T, uint8_t> && (C == 1 || C == 3 || C == 4))
        {
            int64_t stripPixels = 0, allPixels = 0;
            for (int i = first; i < first + count; ++i)
            {
                const NVCVImagePlaneStrided &sp = srcHost[i].planes[0], &dp = dstHost[i].planes[0];
                const int64_t                px = (int64_t)dp.width * dp.height;
                allPixels += px;
                stripPixels += NearestStripScale<C>(sp.width, sp.height, dp.width, dp.height) ? px : 0;
            }
            const bool flat  = flatFor(kStripsWaveW<true>);
            int        total = 2 * stripPixels > allPixels ? buildTiles(kStripsWaveW<true>, kStripsWaveH<true>, flat) : 0;
            if (total >= 8 * 256)
            {
                hipLaunchKernelGGL((ResizeNearestStripsU8VarShapeKernel<C>), dim3(total), dim3(256), 0, stream, a, tiles, (int)flat);
                CheckLaunch("ResizeNearestStripsU8VarShapeKernel");
                continue;
            }
        }
        if constexpr (INTERP == NVCV_INTERP_CUBIC && std::is_same_v<T, uint8_t> && (C == 3 || C == 4))
        {
            // strips where most output pixels belong to images that can take them and every CU still gets 8 blocks
            int64_t stripPixels = 0, allPixels = 0;
            for (int i = first; i < first + count; ++i)
            {
                const int64_t px = (int64_t)dstHost[i].planes[0].width * dstHost[i].planes[0].height;
                allPixels += px;
                stripPixels += CubicStripForm<C>(srcHost[i].planes[0].width, srcHost[i].planes[0].height, dstHost[i].planes[0].height) != 0 ? px : 0;
            }
            int total = 2 * stripPixels > allPixels ? BuildVarTiles(tiles, dstHost, first, count, kPatchTileW, 4 * kCubicStripRows) : 0;
            if (total >= 8 * 256)
            {
                hipLaunchKernelGGL((ResizeCubicStripU8VarShapeKernel<C>), dim3(total), dim3(256), 0, stream, a, tiles);
                CheckLaunch("ResizeCubicStripU8VarShapeKernel");
                continue;
            }
        }
        if constexpr (kPatchForm<T, C, INTERP>)
        {
            const bool flat  = flatFor(kPatchTileW);
            int        total = buildTiles(kPatchTileW, 4, flat);
            if (total > 0)
            {
                hipLaunchKernelGGL((ResizePatchVarShapeKernel<T, C, INTERP>), dim3(total), dim3(256), 0, stream, a,
                                   tiles, (int)flat);
                CheckLaunch("ResizePatchVarShapeKernel");
            }
            continue;
        }
        int total = BuildVarTiles(tiles, dstHost, first, count, kTileW, kTileH);
        if (total > 0)
        {
            hipLaunchKernelGGL((ResizeVarShapeKernel<T, C, INTERP>), dim3(total), dim3(256), 0, stream, a, tiles);
            CheckLaunch("ResizeVarShapeKernel");
        }
    }
}

template<class T, int C>
void DispatchInterp(bool varshape, const ResizeArgs &a, const NVCVImageBufferStrided *srcHost,
                    const NVCVImageBufferStrided *dstHost, int N, int interp,
                    hipStream_t stream)
{
    switch (interp)
    {
    case NVCV_INTERP_NEAREST:
        varshape ? LaunchVarShape<T, C, NVCV_INTERP_NEAREST>(a, srcHost, dstHost, N, stream)
                 : LaunchTensor<T, C, NVCV_INTERP_NEAREST>(a, N, stream);
        break;
    case NVCV_INTERP_LINEAR:
        varshape ? LaunchVarShape<T, C, NVCV_INTERP_LINEAR>(a, srcHost, dstHost, N, stream)
                 : LaunchTensor<T, C, NVCV_INTERP_LINEAR>(a, N, stream);
        break;
    case NVCV_INTERP_CUBIC:
        varshape ? LaunchVarShape<T, C, NVCV_INTERP_CUBIC>(a, srcHost, dstHost, N, stream)
                 : LaunchTensor<T, C, NVCV_INTERP_CUBIC>(a, N, stream);
        break;
    case NVCV_INTERP_AREA:
        varshape ? LaunchVarShape<T, C, NVCV_INTERP_AREA>(a, srcHost, dstHost, N, stream)
                 : LaunchTensor<T, C, NVCV_INTERP_AREA>(a, N, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid interpolation (supported: NEAREST, LINEAR, CUBIC, AREA)");
    }
}

template<class T>
void DispatchChannels(int channels, bool varshape, const ResizeArgs &a, const NVCVImageBufferStrided *srcHost,
                      const NVCVImageBufferStrided *dstHost, int N,
                      int interp, hipStream_t stream)
{
    switch (channels)
    {
    case 1:
        DispatchInterp<T, 1>(varshape, a, srcHost, dstHost, N, interp, stream);
        break;
    case 3:
        DispatchInterp<T, 3>(varshape, a, srcHost, dstHost, N, interp, stream);
        break;
    case 4:
        DispatchInterp<T, 4>(varshape, a, srcHost, dstHost, N, interp, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input data type");
    }
}

void DispatchType(ElemType elem, int channels, bool varshape, const ResizeArgs &a, const NVCVImageBufferStrided *srcHost,
                  const NVCVImageBufferStrided *dstHost, int N, int interp, hipStream_t stream)
{
    if (N == 0)
    {
        return;
    }
    switch (elem)
    {
    case kU8:
        DispatchChannels<uint8_t>(channels, varshape, a, srcHost, dstHost, N, interp, stream);
        break;
    case kU16:
        DispatchChannels<uint16_t>(channels, varshape, a, srcHost, dstHost, N, interp, stream);
        break;
    case kS16:
        DispatchChannels<int16_t>(channels, varshape, a, srcHost, dstHost, N, interp, stream);
        break;
    case kF32:
        DispatchChannels<float>(channels, varshape, a, srcHost, dstHost, N, interp, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input data type");
    }
}

class Resize final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, NVCVInterpolationType interp) const
    {
        NVCVTensorData din, dout;
        ExportTensor(hin, din, "Input");
        ExportTensor(hout, dout, "Output");
        if (din.dtype != dout.dtype)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input and output data type are different");
        }
        if (nvcvTensorLayoutCompare(din.layout, dout.layout) != 0)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input and output data layout are different");
        }
        if (nvcvTensorLayoutCompare(din.layout, NVCV_TENSOR_HWC) != 0
            && nvcvTensorLayoutCompare(din.layout, NVCV_TENSOR_NHWC) != 0)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input must have (N)HWC layout");
        }
        ImageBatchView in  = RequireImageBatchView(din, "Input", NVCV_ERROR_INVALID_ARGUMENT);
        ImageBatchView out = RequireImageBatchView(dout, "Output", NVCV_ERROR_INVALID_ARGUMENT);
        if (in.N != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input and output samples are different");
        }
        if (in.C != out.C)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input and output channels are different");
        }
        if (in.C > 4 || in.C < 1)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid number of channels");
        }
        if (std::max(in.bytesSpanned(), out.bytesSpanned()) > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output tensors are too large");
        }
        ResizeArgs a      = {};
        a.srcBase         = in.base;
        a.dstBase         = out.base;
        a.srcSampleStride = in.strideN;
        a.dstSampleStride = out.strideN;
        a.srcRowStride    = (int32_t)in.strideH;
        a.dstRowStride    = (int32_t)out.strideH;
        a.srcW            = in.W;
        a.srcH            = in.H;
        a.dstW            = out.W;
        a.dstH            = out.H;
        if (out.W == 0 || out.H == 0)
        {
            return;
        }
        a.scaleX = static_cast<float>(in.W) / out.W; // IEEE float32 division, as the kernels would do it
        a.scaleY = static_cast<float>(in.H) / out.H;
        DispatchType(in.elem, in.C, false, a, nullptr, nullptr, in.N, interp, stream);
    }

    void submit(hipStream_t stream, NVCVImageBatchHandle hin, NVCVImageBatchHandle hout,
                NVCVInterpolationType interp) const
    {
        VarShapeView in  = ExportVarShape(hin, stream, "Input");
        VarShapeView out = ExportVarShape(hout, stream, "Output");
        if (in.N != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input and output batch sizes: %d != %d", in.N, out.N);
        }
        if (in.uniqueFormat == NVCV_IMAGE_FORMAT_NONE || in.uniqueFormat != out.uniqueFormat)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                          "All images in the input and output batches must share one format");
        }
        FormatInfo fi = DecodeFormat(in.uniqueFormat);
        if (fi.planes != 1)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images must have a single interleaved plane");
        }
        ResizeArgs a = {};
        a.srcList    = in.data.buffer.varShapeStrided.imageList;
        a.dstList    = out.data.buffer.varShapeStrided.imageList;
        DispatchType(fi.elem, fi.channels, true, a, in.hostList, out.hostList, in.N, interp, stream);
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaResizeCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<Resize>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaResizeSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                            NVCVTensorHandle out, const NVCVInterpolationType interpolation)
{
    return Protect([&] { ToOperator<Resize>(handle).submit(stream, in, out, interpolation); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaResizeVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                    NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                    const NVCVInterpolationType interpolation)
{
    return Protect([&] { ToOperator<Resize>(handle).submit(stream, in, out, interpolation); });
}
}
