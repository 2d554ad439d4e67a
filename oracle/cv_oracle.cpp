// CPU oracle for the image pre-processing operators. TEST INFRASTRUCTURE ONLY: nothing in the
// product libraries links, loads or calls this file; it exists so that tests, the smoke check and
// the benchmark's CPU-baseline leg can compare the GPU results with an independent restatement of
// the reference's arithmetic.
//
// Each function states which reference text it follows. Where the reference's CPU golden (its
// test-suite) and its GPU kernel evaluate a formula differently, both forms are provided and
// selected by `variant`: 0 = golden (tests/cvcuda/system/...), 1 = device formula (src/cvcuda/priv/...).
//
// Built with -ffp-contract=off: no fused multiply-add, so every float expression rounds exactly as
// written (the goldens are plain host C++ built without FMA).
//
// Parity pinning status (see tests/test_oracle_*.py): every function below is pinned by closed
// forms, brute force or library cross-checks; none is "parity unpinned".
#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

// ---- element type codes (same numbering as the reference's legacy DataType enum,
//      src/cvcuda/priv/legacy/CvCudaLegacy.h:53-63) ------------------------------------------------
enum DType
{
    U8  = 0,
    S8  = 1,
    U16 = 2,
    S16 = 3,
    S32 = 4,
    F32 = 5,
    F64 = 6,
    U32 = 8, // not in the reference's legacy enum; used by CropFlipNormalizeReformat only
};

// ---- saturate cast: round-half-to-even then clamp ------------------------------------------------
// follows src/cvcuda/include/cvcuda/cuda_tools/detail/SaturateCastImpl.hpp:31-157 (host path uses
// RoundEvenImpl, device path cvt.rni.sat) and detail/MathWrappersImpl.hpp:403-428.
template<class T>
inline T SatF(float v)
{
    if constexpr (std::is_same_v<T, float>)
    {
        return v;
    }
    else if constexpr (std::is_same_v<T, double>)
    {
        return (double)v;
    }
    else
    {
        if (std::isnan(v))
        {
            return 0;
        }
        float r = std::nearbyint(v); // default rounding mode: to nearest, ties to even
        float lo = (float)std::numeric_limits<T>::min();
        float hi = (float)std::numeric_limits<T>::max();
        if (r <= lo)
        {
            return std::numeric_limits<T>::min();
        }
        if (r >= hi)
        {
            return std::numeric_limits<T>::max();
        }
        return (T)r;
    }
}

template<class T>
inline T SatD(double v)
{
    if constexpr (std::is_floating_point_v<T>)
    {
        return (T)v;
    }
    else
    {
        if (std::isnan(v))
        {
            return 0;
        }
        double r = std::nearbyint(v);
        if (r <= (double)std::numeric_limits<T>::min())
        {
            return std::numeric_limits<T>::min();
        }
        if (r >= (double)std::numeric_limits<T>::max())
        {
            return std::numeric_limits<T>::max();
        }
        return (T)r;
    }
}

inline uint8_t SatI8(int v)
{
    return (uint8_t)(v < 0 ? 0 : v > 255 ? 255 : v);
}

// ---- border index maps --------------------------------------------------------------------------
// follows tests/common/BorderUtils.cpp:24-77 (golden) which agrees with
// cuda_tools/BorderWrap.hpp:62-121 (device) on every input.
inline int BorderIndex(int mode, int c, int s)
{
    switch (mode)
    {
    case 1: // replicate
        return c < 0 ? 0 : (c >= s ? s - 1 : c);
    case 2: // reflect
        c = c % (s * 2);
        if (c < 0)
        {
            c += s * 2;
        }
        return c >= s ? s - 1 - (c - s) : c;
    case 3: // wrap
        c = c % s;
        return c < 0 ? c + s : c;
    case 4: // reflect101
        if (s == 1)
        {
            return 0;
        }
        c = c % (2 * s - 2);
        if (c < 0)
        {
            c += 2 * s - 2;
        }
        return s - 1 - std::abs(s - 1 - c);
    default:
        return c;
    }
}

// Device form of REFLECT (BorderWrap.hpp:100-108), kept separately so tests can assert equivalence.
inline int BorderIndexReflectDevice(int c, int s)
{
    int s2 = s * 2;
    c      = c % s2;
    if (c < 0)
    {
        c += s2;
    }
    return s - 1 - (std::abs(2 * c + 1 - s2) >> 1);
}

template<class F>
void ParallelFor(int n, int threads, F &&fn)
{
    if (threads <= 1 || n <= 1)
    {
        for (int i = 0; i < n; ++i)
        {
            fn(i);
        }
        return;
    }
    threads = std::min(threads, n);
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; ++t)
    {
        pool.emplace_back(
            [=, &fn]
            {
                for (int i = t; i < n; i += threads)
                {
                    fn(i);
                }
            });
    }
    for (auto &th : pool)
    {
        th.join();
    }
}

// =================================================================================================
// Fused resize + crop + convert + reformat, one image.
// order 0: golden  tests/cvcuda/system/TestOpResizeCropConvertReformat.cpp:76-172
//          (val = p00*wy0*wx0 + p01*wy0*wx1 + p10*wy1*wx0 + p11*wy1*wx1)
// order 1: device  src/cvcuda/priv/OpResizeCropConvertReformat.cu:137-198
//          (val = (1-fy)*((1-fx)*p00 + p01*fx) + fy*((1-fx)*p10 + p11*fx))
// Source: u8, 3 interleaved channels, row stride in bytes. Destination addressed in elements:
// dst[y*dstStrideY + x*dstStrideX + c*dstStrideC].
template<class DstT>
void FusedOne(const uint8_t *src, int64_t srcRowStride, int srcW, int srcH, DstT *dst, int64_t dsx, int64_t dsy,
              int64_t dsc, int dstW, int dstH, int newW, int newH, int cropX, int cropY, int interp, int manip,
              float scale, float offset, int srcCast, int order)
{
    const int C      = 3;
    int       mapC[3] = {0, 1, 2};
    if (manip == 1)
    {
        mapC[0] = 2;
        mapC[2] = 0;
    }
    const float scaleW = static_cast<float>(srcW) / newW;
    const float scaleH = static_cast<float>(srcH) / newH;

    for (int dy = 0; dy < dstH; ++dy)
    {
        for (int dx = 0; dx < dstW; ++dx)
        {
            DstT *out = dst + dy * dsy + dx * dsx;
            if (interp == 0)
            {
                int sx = (int)std::floor(scaleW * (dx + cropX + 0.5f));
                int sy = (int)std::floor(scaleH * (dy + cropY + 0.5f));
                const uint8_t *p = src + sy * srcRowStride + sx * C;
                for (int c = 0; c < C; ++c)
                {
                    out[mapC[c] * dsc] = SatF<DstT>(scale * p[c] + offset);
                }
            }
            else
            {
                float fx = scaleW * (dx + cropX + 0.5f) - 0.5f;
                float fy = scaleH * (dy + cropY + 0.5f) - 0.5f;
                int   sx0 = (int)std::floor(fx);
                int   sy0 = (int)std::floor(fy);
                int   sx1 = std::min(sx0 + 1, srcW - 1);
                int   sy1 = std::min(sy0 + 1, srcH - 1);
                fx -= sx0;
                fy -= sy0;
                sx0 = std::max(0, sx0);
                sy0 = std::max(0, sy0);
                const uint8_t *r0 = src + sy0 * srcRowStride;
                const uint8_t *r1 = src + sy1 * srcRowStride;
                for (int c = 0; c < C; ++c)
                {
                    float p00 = r0[sx0 * C + c], p01 = r0[sx1 * C + c];
                    float p10 = r1[sx0 * C + c], p11 = r1[sx1 * C + c];
                    float val;
                    if (order == 0)
                    {
                        float wx0 = 1 - fx, wx1 = fx, wy0 = 1 - fy, wy1 = fy;
                        val = p00 * wy0 * wx0 + p01 * wy0 * wx1 + p10 * wy1 * wx0 + p11 * wy1 * wx1;
                    }
                    else
                    {
                        val = (1 - fy) * ((1 - fx) * p00 + p01 * fx) + fy * ((1 - fx) * p10 + p11 * fx);
                    }
                    if (srcCast)
                    {
                        val = (float)SatF<uint8_t>(val);
                    }
                    val                = scale * val + offset;
                    out[mapC[c] * dsc] = SatF<DstT>(val);
                }
            }
        }
    }
}

// =================================================================================================
// Resize, one image, interleaved channels.
// variant 0 (golden): tests/cvcuda/system/ResizeUtils.cpp:190-304 -- NN in float, linear/cubic with
//                     double weights, rint(abs(.)) and clamp (applied for every T, also float).
// variant 1 (device): src/cvcuda/priv/OpResize.cu:142-164 (NN), 304-330 + 177-301 (linear),
//                     334-388 (cubic) -- float32 throughout, SaturateCast, abs only for cubic.
//                     The per-pixel coordinate is evaluated as (d+.5f)*scale-.5f for every pixel.
// variant 2 (var-shape device): src/cvcuda/priv/legacy/resize_var_shape.cu:92-231 -- same index and
//                     weight rules, different association: linear (1-fx)*(a0*(1-fy)+b0*fy) +
//                     fx*(a1*(1-fy)+b1*fy); cubic accumulates wy[row]*(row dot wx); abs as built
//                     (the legacy-math switch is on).
// ---- area resize, one output pixel ---------------------------------------------------------------
// variant 0: golden tests/cvcuda/system/ResizeUtils.cpp:44-186 (tensor branch) in float64;
// variant 1: device cuda_tools/InterpolationWrap.hpp:668-760 in float32 (taps outside the image read 0).
template<class T>
void AreaPixel(const T *src, int64_t srcStep, int srcW, int srcH, T *out, int C, int dx, int dy, int dstW, int dstH,
               int variant)
{
    auto at = [&](int x, int y, int c) -> double
    { return (x < 0 || x >= srcW || y < 0 || y >= srcH) ? 0.0 : (double)src[y * srcStep + (int64_t)x * C + c]; };
    if (variant == 0 || variant == 3) // golden; 3 = its image-batch flavour (ResizeUtils.cpp:78, 136-176)
    {
        const double scaleH = static_cast<double>(srcH) / dstH, scaleW = static_cast<double>(srcW) / dstW;
        const double fsx1 = dx * scaleW, fsx2 = fsx1 + scaleW, fsy1 = dy * scaleH, fsy2 = fsy1 + scaleH;
        const int    sx1 = (int)std::ceil(fsx1), sx2 = (int)std::floor(fsx2);
        const int    sy1 = (int)std::ceil(fsy1), sy2 = (int)std::floor(fsy2);
        const double lo = (double)std::numeric_limits<T>::lowest(), hi = (double)std::numeric_limits<T>::max();
        for (int c = 0; c < C; ++c)
        {
            double o = 0.0;
            if (std::ceil(scaleW) == scaleW && std::ceil(scaleH) == scaleH)
            {
                const double inv = 1.f / (scaleW * scaleH);
                for (int y = sy1; y < sy2; ++y)
                    for (int x = sx1; x < sx2; ++x) o = o + at(x, y, c) * inv;
            }
            else if (variant == 3 && !(scaleH >= 1.0f && scaleW >= 1.0f))
            {
                // enlargement of image batches: a bilinear variant in mixed float / double
                const double scaleHInv = 1.0 / scaleH, scaleWInv = 1.0 / scaleW;
                int          y1 = (int)std::floor(fsy1), x1 = (int)std::floor(fsx1);
                float        fy = (float)(float(dy + 1) - float(y1 + 1) * scaleHInv);
                fy              = fy <= 0 ? 0.f : fy - (int)std::floor(fy);
                float fx        = (float)(float(dx + 1) - float(x1 + 1) * scaleWInv);
                fx              = fx <= 0 ? 0.f : fx - (int)std::floor(fx);
                if (x1 < 0) { fx = 0; x1 = 0; }
                if (x1 >= srcW - 1) { fx = 0; x1 = srcW - 2; }
                if (y1 >= srcH - 1) { y1 = srcH - 2; }
                // sources of one row or column: the reference indexes outside the image; taps clamped here
                auto tap = [&](int x, int y) -> float // the golden's products and sums here are float
                { return (float)src[std::max(0, std::min(y, srcH - 1)) * srcStep + (int64_t)std::max(0, std::min(x, srcW - 1)) * C + c]; };
                const float cx0 = 1.f - fx, cx1 = fx, cy0 = 1.f - fy, cy1 = fy;
                o = tap(x1, y1) * cx0 * cy0 + tap(x1, y1 + 1) * cx0 * cy1 + tap(x1 + 1, y1) * cx1 * cy0
                  + tap(x1 + 1, y1 + 1) * cx1 * cy1;
            }
            else
            {
                const double inv = 1.f / (std::min(scaleW, srcW - fsx1) * std::min(scaleH, srcH - fsy1));
                for (int y = sy1; y < sy2; ++y)
                {
                    for (int x = sx1; x < sx2; ++x) o = o + at(x, y, c) * inv;
                    if (sx1 > fsx1) o = o + at(sx1 - 1, y, c) * ((sx1 - fsx1) * inv);
                    if (sx2 < fsx2) o = o + at(sx2, y, c) * ((fsx2 - sx2) * inv);
                }
                if (sy1 > fsy1)
                    for (int x = sx1; x < sx2; ++x) o = o + at(x, sy1 - 1, c) * ((sy1 - fsy1) * inv);
                if (sy2 < fsy2)
                    for (int x = sx1; x < sx2; ++x) o = o + at(x, sy2, c) * ((fsy2 - sy2) * inv);
                if (sy1 > fsy1 && sx1 > fsx1) o = o + at(sx1 - 1, sy1 - 1, c) * ((sy1 - fsy1) * (sx1 - fsx1) * inv);
                if (sy1 > fsy1 && sx2 < fsx2) o = o + at(sx2, sy1 - 1, c) * ((sy1 - fsy1) * (fsx2 - sx2) * inv);
                if (sy2 < fsy2 && sx2 < fsx2) o = o + at(sx2, sy2, c) * ((fsy2 - sy2) * (fsx2 - sx2) * inv);
                if (sy2 < fsy2 && sx1 > fsx1) o = o + at(sx1 - 1, sy2, c) * ((fsy2 - sy2) * (sx1 - fsx1) * inv);
            }
            if (std::numeric_limits<T>::is_integer)
            {
                o = std::rint(std::numeric_limits<T>::is_signed ? o : std::abs(o));
            }
            out[c] = (T)(o < lo ? lo : (o > hi ? hi : o));
        }
        return;
    }
    const float scaleX = static_cast<float>(srcW) / dstW, scaleY = static_cast<float>(srcH) / dstH;
    if (variant == 5 || variant == 6)
    {
        // the product library's 8-bit box filter at reductions of up to 3 (sources of 4 rows of 32 bytes or more):
        // a source pixel's weight along an axis is its overlap with the box [d * scale, d * scale + scale) - for
        // scales of 1 and more the same float32 differences as in variants 1 and 2 -, nothing outside the image,
        // divided by the length of the box inside the image. Horizontal weights rounded to multiples of 2^-15 (to nearest,
        // ties to even), a row's sum exact in integers; the rows' sums added in ascending order with fused
        // multiply-adds; one rounding to nearest-even. Outside those scales:
        // variant 1 (5) or 2 (6).
        if (std::is_same_v<T, uint8_t> && (C == 1 || C == 3 || C == 4) && scaleX >= 1.f && scaleX <= 3.f && scaleY >= 1.f
            && scaleY <= 3.f && srcW * C >= 32 && srcH >= 4)
        {
            struct Axis
            {
                int   first;
                float w[4];
            };
            auto box = [](float scale, int d, int size, float unit, bool window)
            {
                Axis        a;
                auto        clamp01 = [](float v) { return std::fmin(std::fmax(v, 0.f), 1.f); };
                const float f1 = d * scale, end = f1 + scale;
                const float f2 = window ? end : std::fmin(end, (float)size); // rows: nothing behind the image
                const float ff = window ? std::fmin(std::floor(f1), (float)(size - 4)) : std::floor(f1);
                const float norm = (1.f / std::fmin(scale, size - f1)) * unit;
                a.first = (int)ff;
                for (int k = 0; k < 4; ++k)
                {
                    // the overlap of pixel x with the box: f2 - x or (x + 1) - f1 for a partly covered one (both
                    // exact), 1 or 0
                    const float x = ff + (float)k;
                    a.w[k]        = (clamp01(f2 - x) - clamp01(f1 - x)) * norm;
                }
                return a;
            };
            // columns: the 4 pixels from the box's first one on, or the image's last 4 where that is earlier;
            // rows: from the box's first one on, none behind the image
            const Axis col = box(scaleX, dx, srcW, 32768.f, true), row = box(scaleY, dy, srcH, 1.f / 32768.f, false);
            uint32_t   wq[4];
            for (int k = 0; k < 4; ++k)
            {
                wq[k] = (uint32_t)std::nearbyint(col.w[k]);
            }
            // a row's integer sum (below 2^23) enters as the float 2^23 + sum, which the kernel gets for free by
            // summing on that float's bit pattern; the accumulator starts at minus 2^23 times the sum of the weights
            const float start = -8388608.f * (((row.w[0] + row.w[1]) + row.w[2]) + row.w[3]);
            for (int c = 0; c < C; ++c)
            {
                float acc = start;
                for (int j = 0; j < 4; ++j)
                {
                    if (row.w[j] == 0.f)
                    {
                        continue;
                    }
                    uint32_t sum = 0;
                    for (int k = 0; k < 4; ++k)
                    {
                        sum += (uint32_t)src[(row.first + j) * srcStep + (int64_t)(col.first + k) * C + c] * wq[k];
                    }
                    acc = std::fmaf(8388608.f + (float)sum, row.w[j], acc);
                }
                const float v = std::nearbyint(acc);
                out[c]        = (T)(v < 0.f ? 0.f : (v > 255.f ? 255.f : v));
            }
            return;
        }
        variant = variant == 5 ? 1 : 2;
    }
    const float fsx1 = dx * scaleX, fsy1 = dy * scaleY, fsx2 = fsx1 + scaleX, fsy2 = fsy1 + scaleY;
    const int   xmin = (int)std::ceil(fsx1), xmax = (int)std::floor(fsx2);
    const int   ymin = (int)std::ceil(fsy1), ymax = (int)std::floor(fsy2);
    if (variant == 2) // image-batch kernel: src/cvcuda/priv/legacy/resize_var_shape.cu:236-428
    {
        const int  iscaleX = (int)std::rint(scaleX), iscaleY = (int)std::rint(scaleY);
        const bool fast = std::fabs(scaleX - iscaleX) < DBL_EPSILON && std::fabs(scaleY - iscaleY) < DBL_EPSILON;
        for (int c = 0; c < C; ++c)
        {
            auto  v = [&](int x, int y) -> float { return (float)at(x, y, c); };
            float o = 0.f;
            if (scaleX >= 1.0f && scaleY >= 1.0f)
            {
                if (fast)
                {
                    const float scale = 1.f / (scaleX * scaleY);
                    for (int cy = ymin; cy < ymax; ++cy)
                        for (int cx = xmin; cx < xmax; ++cx) o = o + v(cx, cy) * scale;
                }
                else
                {
                    const float scale = 1.f / (std::fmin(scaleX, srcW - fsx1) * std::fmin(scaleY, srcH - fsy1));
                    for (int cy = ymin; cy < ymax; ++cy)
                    {
                        for (int cx = xmin; cx < xmax; ++cx) o = o + v(cx, cy) * scale;
                        if (xmin > fsx1) o = o + v(xmin - 1, cy) * ((xmin - fsx1) * scale);
                        if (xmax < fsx2) o = o + v(xmax, cy) * ((fsx2 - xmax) * scale);
                    }
                    if (ymin > fsy1)
                        for (int cx = xmin; cx < xmax; ++cx) o = o + v(cx, ymin - 1) * ((ymin - fsy1) * scale);
                    if (ymax < fsy2)
                        for (int cx = xmin; cx < xmax; ++cx) o = o + v(cx, ymax) * ((fsy2 - ymax) * scale);
                    if (ymin > fsy1 && xmin > fsx1) o = o + v(xmin - 1, ymin - 1) * ((ymin - fsy1) * (xmin - fsx1) * scale);
                    if (ymin > fsy1 && xmax < fsx2) o = o + v(xmax, ymin - 1) * ((ymin - fsy1) * (fsx2 - xmax) * scale);
                    if (ymax < fsy2 && xmax < fsx2) o = o + v(xmax, ymax) * ((fsy2 - ymax) * (fsx2 - xmax) * scale);
                    if (ymax < fsy2 && xmin > fsx1) o = o + v(xmin - 1, ymax) * ((fsy2 - ymax) * (xmin - fsx1) * scale);
                }
            }
            else
            {
                const double invX = 1. / scaleX, invY = 1. / scaleY;
                int          sy = (int)std::floor(dy * scaleY);
                float        fy = (float)((dy + 1) - (sy + 1) * invY);
                fy              = fy <= 0 ? 0.f : fy - (int)std::floor(fy);
                int   sx = (int)std::floor(dx * scaleX);
                float fx = (float)((dx + 1) - (sx + 1) * invX);
                fx       = fx < 0 ? 0.f : fx - (int)std::floor(fx);
                if (sx < 0) { fx = 0; sx = 0; }
                if (sx >= srcW - 1) { fx = 0; sx = srcW - 2; }
                if (sy >= srcH - 1) { sy = srcH - 2; }
                auto tap = [&](int x, int y) -> float
                { return (float)src[std::max(0, std::min(y, srcH - 1)) * srcStep + (int64_t)std::max(0, std::min(x, srcW - 1)) * C + c]; };
                const float cx0 = 1.f - fx, cx1 = fx, cy0 = 1.f - fy, cy1 = fy;
                o = tap(sx, sy) * cx0 * cy0 + tap(sx, sy + 1) * cx0 * cy1 + tap(sx + 1, sy) * cx1 * cy0
                  + tap(sx + 1, sy + 1) * cx1 * cy1;
            }
            out[c] = SatF<T>(o);
        }
        return;
    }
    const bool  integerArea = std::ceil(scaleX) == scaleX && std::ceil(scaleY) == scaleY;
    for (int c = 0; c < C; ++c)
    {
        auto  v = [&](int x, int y) -> float { return (float)at(x, y, c); };
        float o = 0.f;
        if (integerArea)
        {
            const float scale = 1.f / (scaleX * scaleY);
            for (int cy = ymin; cy < ymax; ++cy)
                for (int cx = xmin; cx < xmax; ++cx) o += v(cx, cy) * scale;
        }
        else
        {
            const float scale = 1.f / (std::min(scaleX, srcW - fsx1) * std::min(scaleY, srcH - fsy1));
            for (int cy = ymin; cy < ymax; ++cy)
            {
                for (int cx = xmin; cx < xmax; ++cx) o += v(cx, cy) * scale;
                if (xmin > fsx1) o += v(xmin - 1, cy) * ((xmin - fsx1) * scale);
                if (xmax < fsx2) o += v(xmax, cy) * ((fsx2 - xmax) * scale);
            }
            if (ymin > fsy1)
            {
                for (int cx = xmin; cx < xmax; ++cx) o += v(cx, ymin - 1) * ((ymin - fsy1) * scale);
                if (xmin > fsx1) o += v(xmin - 1, ymin - 1) * ((ymin - fsy1) * (xmin - fsx1) * scale);
                if (xmax < fsx2) o += v(xmax, ymin - 1) * ((ymin - fsy1) * (fsx2 - xmax) * scale);
            }
            if (ymax < fsy2)
            {
                for (int cx = xmin; cx < xmax; ++cx) o += v(cx, ymax) * ((fsy2 - ymax) * scale);
                if (xmax < fsx2) o += v(xmax, ymax) * ((fsy2 - ymax) * (fsx2 - xmax) * scale);
                if (xmin > fsx1) o += v(xmin - 1, ymax) * ((fsy2 - ymax) * (xmin - fsx1) * scale);
            }
        }
        out[c] = SatF<T>(o);
    }
}

template<class T>
void ResizeOne(const T *src, int64_t srcStep, int srcW, int srcH, T *dst, int64_t dstStep, int dstW, int dstH, int C,
               int interp, int variant)
{
    const float scaleH = static_cast<float>(srcH) / dstH;
    const float scaleW = static_cast<float>(srcW) / dstW;
    const double lo = (double)std::numeric_limits<T>::lowest(), hi = (double)std::numeric_limits<T>::max();
    // Sources narrower or lower than the tap window (2 pixels for linear, 4 for cubic): the reference's
    // golden and kernels index outside the image there (undefined values). This restatement defines
    // those taps as clamped into the image, which changes nothing for larger sources.
    auto tapX = [srcW](int x) { return std::max(0, std::min(x, srcW - 1)); };
    auto tapY = [srcH](int y) { return std::max(0, std::min(y, srcH - 1)); };

    for (int dy = 0; dy < dstH; ++dy)
    {
        for (int dx = 0; dx < dstW; ++dx)
        {
            T *out = dst + dy * dstStep + (int64_t)dx * C;
            if (interp == 0)
            {
                float fy = scaleH * (dy + 0.5f);
                float fx = scaleW * (dx + 0.5f);
                int   sy = std::min((int)std::floor(fy), srcH - 1);
                int   sx = std::min((int)std::floor(fx), srcW - 1);
                for (int c = 0; c < C; ++c)
                {
                    out[c] = src[sy * srcStep + (int64_t)sx * C + c];
                }
            }
            else if (interp == 1 && variant == 0)
            {
                double fy = scaleH * (dy + 0.5) - 0.5;
                double fx = scaleW * (dx + 0.5) - 0.5;
                int    sy = (int)std::floor(fy);
                int    sx = (int)std::floor(fx);
                fy        = (sy < 0) ? 0 : ((sy > srcH - 2) ? 1 : fy - sy);
                fx        = (sx < 0) ? 0 : ((sx > srcW - 2) ? 1 : fx - sx);
                sy        = std::max(0, std::min(sy, srcH - 2));
                sx        = std::max(0, std::min(sx, srcW - 2));
                double wy[2] = {1 - fy, fy}, wx[2] = {1 - fx, fx};
                for (int c = 0; c < C; ++c)
                {
                    const int y0 = tapY(sy), y1 = tapY(sy + 1), x0 = tapX(sx), x1 = tapX(sx + 1);
                    double    res = std::rint(std::abs(src[y0 * srcStep + (int64_t)x0 * C + c] * wy[0] * wx[0]
                                                       + src[y1 * srcStep + (int64_t)x0 * C + c] * wy[1] * wx[0]
                                                       + src[y0 * srcStep + (int64_t)x1 * C + c] * wy[0] * wx[1]
                                                       + src[y1 * srcStep + (int64_t)x1 * C + c] * wy[1] * wx[1]));
                    out[c]     = (T)(res < lo ? lo : (res > hi ? hi : res));
                }
            }
            else if (interp == 1 && variant == 4 && std::is_same_v<T, uint8_t>)
            {
                // the product library's 8-bit bilinear resize: indices and weights of the device formula, the
                // weights cut to multiples of 2^-15, four integer weights that add up to 2^15, an exact integer
                // sum, one rounding to nearest-even
                float fy = (dy + .5f) * scaleH - .5f;
                float fx = (dx + .5f) * scaleW - .5f;
                int   sy = (int)std::floor(fy);
                int   sx = (int)std::floor(fx);
                float wyv = (sy < 0) ? 0.f : ((sy > srcH - 2) ? 1.f : fy - sy);
                float wxv = (sx < 0) ? 0.f : ((sx > srcW - 2) ? 1.f : fx - sx);
                sy        = std::max(0, std::min(sy, srcH - 2));
                sx        = std::max(0, std::min(sx, srcW - 2));
                uint32_t ax = (uint32_t)(wxv * 32768.f), ay = (uint32_t)(wyv * 32768.f);
                uint32_t w11 = (ax * ay + 16384u) >> 15, w01 = ax - w11, w10 = ay - w11, w00 = 32768u - ax - ay + w11;
                for (int c = 0; c < C; ++c)
                {
                    uint32_t p00 = src[tapY(sy) * srcStep + (int64_t)tapX(sx) * C + c];
                    uint32_t p01 = src[tapY(sy) * srcStep + (int64_t)tapX(sx + 1) * C + c];
                    uint32_t p10 = src[tapY(sy + 1) * srcStep + (int64_t)tapX(sx) * C + c];
                    uint32_t p11 = src[tapY(sy + 1) * srcStep + (int64_t)tapX(sx + 1) * C + c];
                    uint32_t s   = p00 * w00 + p01 * w01 + p10 * w10 + p11 * w11;
                    out[c]       = (T)((s + 16383u + ((s >> 15) & 1u)) >> 15);
                }
            }
            else if (interp == 1 && (variant == 1 || variant == 4))
            {
                float fy = (dy + .5f) * scaleH - .5f;
                float fx = (dx + .5f) * scaleW - .5f;
                int   sy = (int)std::floor(fy);
                int   sx = (int)std::floor(fx);
                float wyv = (sy < 0) ? 0.f : ((sy > srcH - 2) ? 1.f : fy - sy);
                float wxv = (sx < 0) ? 0.f : ((sx > srcW - 2) ? 1.f : fx - sx);
                sy        = std::max(0, std::min(sy, srcH - 2));
                sx        = std::max(0, std::min(sx, srcW - 2));
                for (int c = 0; c < C; ++c)
                {
                    float p00 = src[tapY(sy) * srcStep + (int64_t)tapX(sx) * C + c];
                    float p01 = src[tapY(sy) * srcStep + (int64_t)tapX(sx + 1) * C + c];
                    float p10 = src[tapY(sy + 1) * srcStep + (int64_t)tapX(sx) * C + c];
                    float p11 = src[tapY(sy + 1) * srcStep + (int64_t)tapX(sx + 1) * C + c];
                    float v   = p00 * ((1.f - wxv) * (1.f - wyv)) + p01 * (wxv * (1.f - wyv)) + p10 * ((1.f - wxv) * wyv)
                            + p11 * (wxv * wyv);
                    out[c] = SatF<T>(v);
                }
            }
            else if (interp == 1) // variant 2
            {
                float fy = (float)((dy + 0.5f) * scaleH - 0.5f);
                float fx = (float)((dx + 0.5f) * scaleW - 0.5f);
                int   sy = (int)std::floor(fy);
                int   sx = (int)std::floor(fx);
                fy       = (sy < 0) ? 0.f : ((sy > srcH - 2) ? 1.f : fy - sy);
                fx       = (sx < 0) ? 0.f : ((sx > srcW - 2) ? 1.f : fx - sx);
                sy       = std::max(0, std::min(sy, srcH - 2));
                sx       = std::max(0, std::min(sx, srcW - 2));
                for (int c = 0; c < C; ++c)
                {
                    float a0 = src[tapY(sy) * srcStep + (int64_t)tapX(sx) * C + c];
                    float a1 = src[tapY(sy) * srcStep + (int64_t)tapX(sx + 1) * C + c];
                    float b0 = src[tapY(sy + 1) * srcStep + (int64_t)tapX(sx) * C + c];
                    float b1 = src[tapY(sy + 1) * srcStep + (int64_t)tapX(sx + 1) * C + c];
                    float v  = (1.0f - fx) * (a0 * (1.0f - fy) + b0 * fy) + fx * (a1 * (1.0f - fy) + b1 * fy);
                    out[c]   = SatF<T>(v);
                }
            }
            else if (interp == 2 && variant == 0)
            {
                double fy = scaleH * (dy + 0.5) - 0.5;
                double fx = scaleW * (dx + 0.5) - 0.5;
                int    sy = (int)std::floor(fy);
                int    sx = (int)std::floor(fx);
                fy -= sy;
                fx -= sx;
                fx = (sx < 1 || sx >= srcW - 3) ? 0 : fx;
                sy = std::max(1, std::min(sy, srcH - 3));
                sx = std::max(1, std::min(sx, srcW - 3));
                const double A = -0.75;
                double       wy[4], wx[4];
                wy[0] = ((A * (fy + 1) - 5 * A) * (fy + 1) + 8 * A) * (fy + 1) - 4 * A;
                wy[1] = ((A + 2) * fy - (A + 3)) * fy * fy + 1;
                wy[2] = ((A + 2) * (1 - fy) - (A + 3)) * (1 - fy) * (1 - fy) + 1;
                wy[3] = 1 - wy[0] - wy[1] - wy[2];
                wx[0] = ((A * (fx + 1) - 5 * A) * (fx + 1) + 8 * A) * (fx + 1) - 4 * A;
                wx[1] = ((A + 2) * fx - (A + 3)) * fx * fx + 1;
                wx[2] = ((A + 2) * (1 - fx) - (A + 3)) * (1 - fx) * (1 - fx) + 1;
                wx[3] = 1 - wx[0] - wx[1] - wx[2];
                for (int c = 0; c < C; ++c)
                {
                    double sum = 0; // golden sums column by column (x outer, y inner)
                    for (int ix = 0; ix < 4; ++ix)
                    {
                        for (int iy = 0; iy < 4; ++iy)
                        {
                            sum += src[tapY(sy - 1 + iy) * srcStep + (int64_t)tapX(sx - 1 + ix) * C + c] * wx[ix] * wy[iy];
                        }
                    }
                    double res = std::rint(std::abs(sum));
                    out[c]     = (T)(res < lo ? lo : (res > hi ? hi : res));
                }
            }
            else if (interp == 2)
            {
                float fy = (dy + .5f) * scaleH - .5f;
                float fx = (dx + .5f) * scaleW - .5f;
                int   sy = (int)std::floor(fy);
                int   sx = (int)std::floor(fx);
                fx       = fx - sx;
                fy       = fy - sy;
                fx       = (sx < 1 || sx >= srcW - 3) ? 0.f : fx;
                sy       = std::max(1, std::min(sy, srcH - 3));
                sx       = std::max(1, std::min(sx, srcW - 3));
                const float A = -0.75f;
                float       wx[4], wy[4];
                auto        coeffs = [A](float d, float *w)
                {
                    w[0] = ((A * (d + 1) - 5 * A) * (d + 1) + 8 * A) * (d + 1) - 4 * A;
                    w[1] = ((A + 2) * d - (A + 3)) * d * d + 1;
                    w[2] = ((A + 2) * (1 - d) - (A + 3)) * (1 - d) * (1 - d) + 1;
                    w[3] = 1.f - w[0] - w[1] - w[2];
                };
                coeffs(fx, wx);
                coeffs(fy, wy);
                if (variant == 7 && std::is_same_v<T, uint8_t>)
                {
                    // the product library's 8-bit bicubic resize: indices and weights of the device formula, the
                    // horizontal weights rounded to multiples of 2^-14 (to nearest, ties to even) with the last one
                    // taking the remainder, a row's sum exact in integers, the four row sums added in float32,
                    // ascending, the first as a product and the others by fused multiply-adds, the magnitude
                    // rounded to nearest-even
                    int wq[4];
                    for (int i = 0; i < 3; ++i)
                    {
                        wq[i] = (int)std::nearbyint(wx[i] * 16384.f);
                    }
                    wq[3] = 16384 - wq[0] - wq[1] - wq[2];
                    for (int c = 0; c < C; ++c)
                    {
                        float acc = 0.f;
                        for (int row = 0; row < 4; ++row)
                        {
                            int h = 0;
                            for (int i = 0; i < 4; ++i)
                            {
                                h += (int)src[tapY(sy + row - 1) * srcStep + (int64_t)tapX(sx + i - 1) * C + c] * wq[i];
                            }
                            const float w = wy[row] * (1.f / 16384.f);
                            acc           = row == 0 ? (float)h * w : std::fmaf((float)h, w, acc);
                        }
                        out[c] = SatF<T>(std::abs(acc));
                    }
                    continue;
                }
                for (int c = 0; c < C; ++c)
                {
                    float sum = 0.f;
                    if (variant == 1 || variant == 7) // tensor kernel: sum += p * (wx*wy), y outer, x inner
                    {
                        for (int cy = -1; cy <= 2; ++cy)
                        {
                            for (int cx = -1; cx <= 2; ++cx)
                            {
                                sum += (float)src[tapY(sy + cy) * srcStep + (int64_t)tapX(sx + cx) * C + c]
                                     * (wx[cx + 1] * wy[cy + 1]);
                            }
                        }
                    }
                    else // var-shape kernel: accum += wy[row] * (wx0*a0 + wx1*a1 + wx2*a2 + wx3*a3)
                    {
                        for (int row = 0; row < 4; ++row)
                        {
                            const T *a = src + tapY(sy + row - 1) * srcStep + c;
                            sum += wy[row]
                                 * (wx[0] * (float)a[(int64_t)tapX(sx - 1) * C] + wx[1] * (float)a[(int64_t)tapX(sx) * C]
                                    + wx[2] * (float)a[(int64_t)tapX(sx + 1) * C]
                                    + wx[3] * (float)a[(int64_t)tapX(sx + 2) * C]);
                        }
                    }
                    out[c] = SatF<T>(std::abs(sum));
                }
            }
            else if (interp == 3)
            {
                AreaPixel<T>(src, srcStep, srcW, srcH, out, C, dx, dy, dstW, dstH, variant);
            }
        }
    }
}

// =================================================================================================
// YUV 4:2:0 -> RGB family, one image. src is the single-channel tensor image of (H*3/2) rows.
// variant 0: integer BT.601 formula of the device, src/cvcuda/priv/legacy/cvt_color.cu:64-69, 618-638
//            with the loads of :514-565 (semi-planar NV12/NV21 and planar I420/YV12).
// variant 1: double-precision golden, tests/cvcuda/system/CvtColorUtils.cpp:93-108, 841-892
//            (semi-planar only).
void Yuv420ToRgbOne(const uint8_t *src, int64_t srcStride, int W, int H, uint8_t *dst, int64_t dstStride, int dcn,
                    int bidx, int uidx, int semiPlanar, int variant)
{
    for (int y = 0; y < H; ++y)
    {
        for (int x = 0; x < W; ++x)
        {
            int Y = src[y * srcStride + x];
            int U, V;
            if (semiPlanar)
            {
                const uint8_t *uv = src + (int64_t)(H + y / 2) * srcStride + (x & ~1);
                U                 = uv[uidx];
                V                 = uv[uidx ^ 1];
            }
            else
            {
                int by  = H + y / 4;
                int h4  = H / 4;
                int uvx = (x / 2) + ((W / 2) & -((y / 2) & 1));
                U       = src[(int64_t)(by + h4 * uidx) * srcStride + uvx];
                V       = src[(int64_t)(by + h4 * (uidx ^ 1)) * srcStride + uvx];
            }
            uint8_t r, g, b;
            if (variant == 0)
            {
                int yy = std::max(0, Y - 16) * 1220542;
                int uu = U - 128;
                int vv = V - 128;
                r      = SatI8((yy + 1673527 * vv + (1 << 19)) >> 20);
                g      = SatI8((yy + -852492 * vv + -409993 * uu + (1 << 19)) >> 20);
                b      = SatI8((yy + 2116026 * uu + (1 << 19)) >> 20);
            }
            else
            {
                double Yd = Y - 16.0, Ud = U - 128.0, Vd = V - 128.0;
                if (Yd < 0.0)
                {
                    Yd = 0.0;
                }
                r = SatD<uint8_t>(1.16895 * Yd + 0.0 * Ud + 1.60229 * Vd);
                g = SatD<uint8_t>(1.16895 * Yd + -0.3933 * Ud + -0.81616 * Vd);
                b = SatD<uint8_t>(1.16895 * Yd + 2.02514 * Ud + 0.0 * Vd);
            }
            uint8_t *o  = dst + y * dstStride + (int64_t)x * dcn;
            o[bidx]     = b;
            o[1]        = g;
            o[bidx ^ 2] = r;
            if (dcn == 4)
            {
                o[3] = 255;
            }
        }
    }
}

// =================================================================================================
// Normalize, one image; follows the golden tests/cvcuda/system/TestOpNormalize.cpp:34-79 generalised
// to any element type through SaturateCast (device: src/cvcuda/priv/legacy/normalize.cu:35-93).
// base/scale are float images with their own width/height/channels, each either 1 or the input's.
template<class T>
void NormalizeOne(const T *src, int64_t srcStep, T *dst, int64_t dstStep, int W, int H, int C, const float *base,
                  int64_t baseStep, int bW, int bH, int bC, const float *scl, int64_t sclStep, int sW, int sH, int sC,
                  float gscale, float gshift, float eps, int stddev)
{
    for (int i = 0; i < H; ++i)
    {
        int bi = bH == 1 ? 0 : i, si = sH == 1 ? 0 : i;
        for (int j = 0; j < W; ++j)
        {
            int bj = bW == 1 ? 0 : j, sj = sW == 1 ? 0 : j;
            for (int k = 0; k < C; ++k)
            {
                int   bk = bC == 1 ? 0 : k, sk = sC == 1 ? 0 : k;
                float mul;
                float s = scl[si * sclStep + (int64_t)sj * sC + sk];
                if (stddev)
                {
                    float x = s * s + eps;
                    mul     = 1.0f / std::sqrt(x);
                }
                else
                {
                    mul = s;
                }
                float v = ((float)src[i * srcStep + (int64_t)j * C + k] - base[bi * baseStep + (int64_t)bj * bC + bk]) * mul
                            * gscale
                        + gshift;
                dst[i * dstStep + (int64_t)j * C + k] = SatF<T>(v);
            }
        }
    }
}

// =================================================================================================
// Warp (affine or perspective), one image.
// golden: tests/cvcuda/system/TestOpWarpAffine.cpp:39-223 (getPixel, calcBicubicCoeff, WarpAffineGold)
// device: src/cvcuda/priv/legacy/warp.cu:28-49, CvCudaLegacy.h:143-183 (coordinate),
//         cuda_tools/InterpolationWrap.hpp:83-104, 332-339, 429-447, 535-565 (sampling).
// `m` is the dst->src matrix (already inverted): 6 coefficients for affine, 9 for perspective.
inline float BicubicGolden(float x_)
{
    float x = std::abs(x_);
    if (x <= 1.0f)
    {
        return x * x * (1.5f * x - 2.5f) + 1.0f;
    }
    else if (x < 2.0f)
    {
        return x * (x * (-0.5f * x + 2.5f) - 4.0f) + 2.0f;
    }
    return 0.0f;
}

inline void CubicCoeffsDevice(float d, float *w)
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

// Catmull-Rom weights times `scale` (a power of two), polynomials by fused multiply-adds: what the product
// library's 8-bit bicubic warp evaluates before it quantises the horizontal weights.
inline void CubicCoeffsFused(float d, float scale, float *w)
{
    w[0] = std::fmaf(-.5f * scale, d, scale);
    w[0] = std::fmaf(w[0], d, -.5f * scale);
    w[0] = w[0] * d;
    w[1] = std::fmaf(1.5f * scale, d, -2.5f * scale);
    w[1] = w[1] * d;
    w[1] = std::fmaf(w[1], d, scale);
    w[2] = std::fmaf(-1.5f * scale, d, 2.f * scale);
    w[2] = std::fmaf(w[2], d, .5f * scale);
    w[2] = w[2] * d;
    w[3] = scale - w[0] - w[1] - w[2];
}

template<class T>
void WarpOne(const T *src, int64_t srcStep, int srcW, int srcH, T *dst, int64_t dstStep, int dstW, int dstH, int C,
             const float *m, int perspective, int interp, int border, const float *bval, int variant)
{
    auto pix = [&](int y, int x, int k) -> T
    {
        if (border == 0)
        {
            return (x >= 0 && x < srcW && y >= 0 && y < srcH) ? src[y * srcStep + (int64_t)x * C + k]
                                                              : static_cast<T>(bval[k]);
        }
        int cx = BorderIndex(border, x, srcW);
        int cy = BorderIndex(border, y, srcH);
        return src[cy * srcStep + (int64_t)cx * C + k];
    };

    for (int dy = 0; dy < dstH; ++dy)
    {
        for (int dx = 0; dx < dstW; ++dx)
        {
            float sx, sy;
            if (!perspective)
            {
                if (variant == 0)
                {
                    sx = (float)(dx * m[0] + dy * m[1] + m[2]);
                    sy = (float)(dx * m[3] + dy * m[4] + m[5]);
                }
                else
                {
                    sx = m[0] * dx + m[1] * dy + m[2];
                    sy = m[3] * dx + m[4] * dy + m[5];
                }
            }
            else
            {
                float coeff = 1.0f / (m[6] * dx + m[7] * dy + m[8]);
                sx          = coeff * (m[0] * dx + m[1] * dy + m[2]);
                sy          = coeff * (m[3] * dx + m[4] * dy + m[5]);
            }
            T *out = dst + dy * dstStep + (int64_t)dx * C;
            if (interp == 0)
            {
                int x1 = (int)std::floor(sx + .5f);
                int y1 = (int)std::floor(sy + .5f);
                for (int k = 0; k < C; ++k)
                {
                    out[k] = pix(y1, x1, k);
                }
            }
            else if (interp == 1)
            {
                int x1 = (int)std::floor(sx), y1 = (int)std::floor(sy);
                int x2 = x1 + 1, y2 = y1 + 1;
                if (variant == 2 && std::is_same_v<T, uint8_t>)
                {
                    // the product library's 8-bit arithmetic: 15-bit fractions, four integer weights that
                    // add up to 2^15, an exact integer sum, one rounding to nearest-even
                    auto frac = [](float v) -> uint32_t
                    {
                        float f = v - std::floor(v);
                        return f >= 0.f ? (uint32_t)(int)(f * 32768.f) : 0u;
                    };
                    uint32_t ax = frac(sx), ay = frac(sy);
                    uint32_t w11 = (ax * ay + 16384u) >> 15, w01 = ax - w11, w10 = ay - w11,
                             w00 = 32768u - ax - ay + w11;
                    for (int k = 0; k < C; ++k)
                    {
                        uint32_t s = (uint32_t)pix(y1, x1, k) * w00 + (uint32_t)pix(y1, x2, k) * w01
                                   + (uint32_t)pix(y2, x1, k) * w10 + (uint32_t)pix(y2, x2, k) * w11;
                        out[k] = (T)((s + 16383u + ((s >> 15) & 1u)) >> 15);
                    }
                    continue;
                }
                for (int k = 0; k < C; ++k)
                {
                    float o = 0;
                    if (variant == 0 || variant == 2)
                    {
                        o += pix(y1, x1, k) * ((x2 - sx) * (y2 - sy));
                        o = o + pix(y1, x2, k) * ((sx - x1) * (y2 - sy));
                        o = o + pix(y2, x1, k) * ((x2 - sx) * (sy - y1));
                        o = o + pix(y2, x2, k) * ((sx - x1) * (sy - y1));
                        if constexpr (std::is_floating_point_v<T>)
                        {
                            out[k] = (T)o;
                        }
                        else
                        {
                            o      = std::rint(o);
                            float lo = (float)std::numeric_limits<T>::min(), hi = (float)std::numeric_limits<T>::max();
                            out[k] = (T)(o < lo ? lo : (o > hi ? hi : o));
                        }
                    }
                    else
                    {
                        // the reference's device expression, tap * wx * wy (InterpolationWrap.hpp:429-447);
                        // kept for comparison: the product library follows the golden's association above
                        o += (float)pix(y1, x1, k) * (x2 - sx) * (y2 - sy);
                        o += (float)pix(y1, x2, k) * (sx - x1) * (y2 - sy);
                        o += (float)pix(y2, x1, k) * (x2 - sx) * (sy - y1);
                        o += (float)pix(y2, x2, k) * (sx - x1) * (sy - y1);
                        out[k] = SatF<T>(o);
                    }
                }
            }
            else if (variant == 2 && std::is_same_v<T, uint8_t>)
            {
                // the product library's 8-bit bicubic: horizontal weights rounded to multiples of 2^-14 (the
                // last takes the remainder), exact integer row sums, float32 vertical sum with fused
                // multiply-adds, one rounding to nearest-even
                int   ix = (int)std::floor(sx), iy = (int)std::floor(sy);
                float wx[4], wy[4];
                CubicCoeffsFused(sx - std::floor(sx), 16384.f, wx);
                CubicCoeffsFused(sy - std::floor(sy), 1.f / 16384.f, wy);
                int wq[4];
                for (int i = 0; i < 3; ++i)
                {
                    wq[i] = wx[i] == wx[i] ? (int)std::nearbyint(wx[i]) : 0;
                }
                wq[3] = 16384 - wq[0] - wq[1] - wq[2];
                for (int k = 0; k < C; ++k)
                {
                    float acc = 0;
                    for (int cy = 0; cy < 4; ++cy)
                    {
                        int h = 0;
                        for (int cx = 0; cx < 4; ++cx)
                        {
                            h += (int)pix(iy + cy - 1, ix + cx - 1, k) * wq[cx];
                        }
                        acc = cy == 0 ? (float)h * wy[0] : std::fmaf((float)h, wy[cy], acc);
                    }
                    out[k] = SatF<T>(acc);
                }
            }
            else if (variant == 0)
            {
                int xmin = (int)std::ceil(sx - 2.0f), xmax = (int)std::floor(sx + 2.0f);
                int ymin = (int)std::ceil(sy - 2.0f), ymax = (int)std::floor(sy + 2.0f);
                for (int k = 0; k < C; ++k)
                {
                    float sum = 0, wsum = 0;
                    for (int cy = ymin; cy <= ymax; ++cy)
                    {
                        for (int cx = xmin; cx <= xmax; ++cx)
                        {
                            float w = BicubicGolden(sx - cx) * BicubicGolden(sy - cy);
                            sum += w * pix(cy, cx, k);
                            wsum += w;
                        }
                    }
                    float res = (!wsum) ? 0 : sum / wsum;
                    if constexpr (std::is_floating_point_v<T>)
                    {
                        out[k] = (T)res;
                    }
                    else
                    {
                        res      = std::rint(res);
                        float lo = (float)std::numeric_limits<T>::min(), hi = (float)std::numeric_limits<T>::max();
                        out[k]   = (T)(res < lo ? lo : (res > hi ? hi : res));
                    }
                }
            }
            else
            {
                int   ix = (int)std::floor(sx), iy = (int)std::floor(sy);
                float wx[4], wy[4];
                CubicCoeffsDevice(sx - ix, wx);
                CubicCoeffsDevice(sy - iy, wy);
                for (int k = 0; k < C; ++k)
                {
                    float sum = 0;
                    for (int cy = -1; cy <= 2; ++cy)
                    {
                        for (int cx = -1; cx <= 2; ++cx)
                        {
                            sum += (float)pix(iy + cy, ix + cx, k) * (wx[cx + 1] * wy[cy + 1]);
                        }
                    }
                    out[k] = SatF<T>(sum);
                }
            }
        }
    }
}

template<class F>
int DispatchType(int dtype, F &&f)
{
    switch (dtype)
    {
    case U8:
        f(uint8_t{});
        return 0;
    case S8:
        f(int8_t{});
        return 0;
    case U16:
        f(uint16_t{});
        return 0;
    case S16:
        f(int16_t{});
        return 0;
    case S32:
        f(int32_t{});
        return 0;
    case F32:
        f(float{});
        return 0;
    case U32:
        f(uint32_t{});
        return 0;
    default:
        return -1;
    }
}

} // namespace

// =================================================================================================
// C entry points (ctypes-friendly). Strides named *Step are in elements, *Stride in bytes.

ORC_API int orc_fused_rccr(const uint8_t *src, int64_t srcRowStride, int64_t srcImgStride, int N, int srcW, int srcH,
                           void *dst, int dstIsF32, int64_t dstStrideN, int64_t dstStrideX, int64_t dstStrideY,
                           int64_t dstStrideC, int dstW, int dstH, int newW, int newH, int cropX, int cropY,
                           int interp, int manip, float scale, float offset, int srcCast, int order, int threads)
{
    if (interp != 0 && interp != 1)
    {
        return -1;
    }
    ParallelFor(N, threads,
                [&](int n)
                {
                    const uint8_t *s = src + n * srcImgStride;
                    if (dstIsF32)
                    {
                        FusedOne<float>(s, srcRowStride, srcW, srcH, (float *)dst + n * dstStrideN, dstStrideX,
                                        dstStrideY, dstStrideC, dstW, dstH, newW, newH, cropX, cropY, interp, manip,
                                        scale, offset, srcCast, order);
                    }
                    else
                    {
                        FusedOne<uint8_t>(s, srcRowStride, srcW, srcH, (uint8_t *)dst + n * dstStrideN, dstStrideX,
                                          dstStrideY, dstStrideC, dstW, dstH, newW, newH, cropX, cropY, interp, manip,
                                          scale, offset, srcCast, order);
                    }
                });
    return 0;
}

ORC_API int orc_resize(const void *src, int64_t srcStep, int64_t srcImgStep, int N, int srcW, int srcH, void *dst,
                       int64_t dstStep, int64_t dstImgStep, int dstW, int dstH, int C, int dtype, int interp,
                       int variant, int threads)
{
    if (interp < 0 || interp > 3)
    {
        return -1;
    }
    return DispatchType(dtype,
                        [&](auto tag)
                        {
                            using T = decltype(tag);
                            ParallelFor(N, threads,
                                        [&](int n)
                                        {
                                            ResizeOne<T>((const T *)src + n * srcImgStep, srcStep, srcW, srcH,
                                                         (T *)dst + n * dstImgStep, dstStep, dstW, dstH, C, interp,
                                                         variant);
                                        });
                        });
}

ORC_API int orc_yuv420_to_rgb(const uint8_t *src, int64_t srcStride, int64_t srcImgStride, int N, int W, int H,
                              uint8_t *dst, int64_t dstStride, int64_t dstImgStride, int dcn, int bidx, int uidx,
                              int semiPlanar, int variant, int threads)
{
    if ((dcn != 3 && dcn != 4) || (bidx != 0 && bidx != 2) || (W & 1) || (H & 1) || (variant == 1 && !semiPlanar))
    {
        return -1;
    }
    ParallelFor(N, threads,
                [&](int n)
                {
                    Yuv420ToRgbOne(src + n * srcImgStride, srcStride, W, H, dst + n * dstImgStride, dstStride, dcn, bidx,
                                   uidx, semiPlanar, variant);
                });
    return 0;
}

// One (Y,U,V) triple through the integer device formula; out = {r,g,b}. For exhaustive checks.
ORC_API void orc_yuv_to_rgb_int(int Y, int U, int V, uint8_t *out)
{
    uint8_t px[6]  = {(uint8_t)Y, (uint8_t)Y, (uint8_t)Y, (uint8_t)Y, (uint8_t)U, (uint8_t)V};
    uint8_t rgb[12];
    Yuv420ToRgbOne(px, 2, 2, 2, rgb, 6, 3, 2, 0, 1, 0);
    out[0] = rgb[0];
    out[1] = rgb[1];
    out[2] = rgb[2];
}

ORC_API int orc_normalize(const void *src, int64_t srcStep, int64_t srcImgStep, void *dst, int64_t dstStep,
                          int64_t dstImgStep, int N, int W, int H, int C, int dtype, const float *base,
                          int64_t baseStep, int64_t baseImgStep, int bN, int bW, int bH, int bC, const float *scale,
                          int64_t scaleStep, int64_t scaleImgStep, int sN, int sW, int sH, int sC, float gscale,
                          float gshift, float eps, int stddev, int threads)
{
    return DispatchType(dtype,
                        [&](auto tag)
                        {
                            using T = decltype(tag);
                            ParallelFor(N, threads,
                                        [&](int n)
                                        {
                                            NormalizeOne<T>((const T *)src + n * srcImgStep, srcStep,
                                                            (T *)dst + n * dstImgStep, dstStep, W, H, C,
                                                            base + (bN == 1 ? 0 : n) * baseImgStep, baseStep, bW, bH, bC,
                                                            scale + (sN == 1 ? 0 : n) * scaleImgStep, scaleStep, sW, sH,
                                                            sC, gscale, gshift, eps, stddev);
                                        });
                        });
}

// Inverse of a 2x3 affine map; follows src/cvcuda/priv/legacy/warp.cu:139-150 (float arithmetic,
// reciprocal of the determinant taken in double then narrowed, singular -> all-zero linear part).
ORC_API void orc_invert_affine(const float *M, float *out)
{
    float den = M[0] * M[4] - M[1] * M[3];
    den       = std::abs(den) > 1e-5 ? 1. / den : .0;
    out[0]    = (float)M[4] * den;
    out[1]    = (float)-M[1] * den;
    out[2]    = (float)(M[1] * M[5] - M[4] * M[2]) * den;
    out[3]    = (float)-M[3] * den;
    out[4]    = (float)M[0] * den;
    out[5]    = (float)(M[3] * M[2] - M[0] * M[5]) * den;
}

// `xform` holds N matrices of `perspective ? 9 : 6` floats, already dst->src.
ORC_API int orc_warp(const void *src, int64_t srcStep, int64_t srcImgStep, int N, int srcW, int srcH, void *dst,
                     int64_t dstStep, int64_t dstImgStep, int dstW, int dstH, int C, int dtype, const float *xform,
                     int perspective, int interp, int border, const float *borderValue, int variant, int threads)
{
    if (interp < 0 || interp > 2 || border < 0 || border > 4)
    {
        return -1;
    }
    int mlen = perspective ? 9 : 6;
    return DispatchType(dtype,
                        [&](auto tag)
                        {
                            using T = decltype(tag);
                            ParallelFor(N, threads,
                                        [&](int n)
                                        {
                                            WarpOne<T>((const T *)src + n * srcImgStep, srcStep, srcW, srcH,
                                                       (T *)dst + n * dstImgStep, dstStep, dstW, dstH, C,
                                                       xform + n * mlen, perspective, interp, border, borderValue,
                                                       variant);
                                        });
                        });
}

// ---- ConvertTo ---------------------------------------------------------------------------------------
// variant 1 (device): src/cvcuda/priv/legacy/convert_to.cu:36-47, 77-83: alpha*src+beta evaluated in
// float32, or float64 when either element type is float64, alpha/beta first converted to that type.
// variant 0 (golden): tests/cvcuda/system/TestOpConvertTo.cpp:132 evaluates it in float64 always.
template<class TS, class TD>
void ConvertRows(const TS *src, TD *dst, int64_t count, double alpha, double beta, int variant)
{
    constexpr bool dbl = std::is_same_v<TS, double> || std::is_same_v<TD, double>;
    for (int64_t i = 0; i < count; ++i)
    {
        if (dbl || variant == 0)
        {
            dst[i] = SatD<TD>(alpha * (double)src[i] + beta);
        }
        else
        {
            const float v = (float)alpha * (float)src[i] + (float)beta;
            dst[i]        = SatF<TD>(v);
        }
    }
}

template<class TS>
int ConvertDst(const TS *src, void *dst, int dstType, int64_t count, double alpha, double beta, int variant)
{
    switch (dstType)
    {
    case U8:
        ConvertRows(src, (uint8_t *)dst, count, alpha, beta, variant);
        return 0;
    case S8:
        ConvertRows(src, (int8_t *)dst, count, alpha, beta, variant);
        return 0;
    case U16:
        ConvertRows(src, (uint16_t *)dst, count, alpha, beta, variant);
        return 0;
    case S16:
        ConvertRows(src, (int16_t *)dst, count, alpha, beta, variant);
        return 0;
    case S32:
        ConvertRows(src, (int32_t *)dst, count, alpha, beta, variant);
        return 0;
    case F32:
        ConvertRows(src, (float *)dst, count, alpha, beta, variant);
        return 0;
    case F64:
        ConvertRows(src, (double *)dst, count, alpha, beta, variant);
        return 0;
    default:
        return 1;
    }
}

// Packed arrays of `count` scalars.
ORC_API int orc_convert_to(const void *src, int srcType, void *dst, int dstType, int64_t count, double alpha,
                           double beta, int variant)
{
    switch (srcType)
    {
    case U8:
        return ConvertDst((const uint8_t *)src, dst, dstType, count, alpha, beta, variant);
    case S8:
        return ConvertDst((const int8_t *)src, dst, dstType, count, alpha, beta, variant);
    case U16:
        return ConvertDst((const uint16_t *)src, dst, dstType, count, alpha, beta, variant);
    case S16:
        return ConvertDst((const int16_t *)src, dst, dstType, count, alpha, beta, variant);
    case S32:
        return ConvertDst((const int32_t *)src, dst, dstType, count, alpha, beta, variant);
    case F32:
        return ConvertDst((const float *)src, dst, dstType, count, alpha, beta, variant);
    case F64:
        return ConvertDst((const double *)src, dst, dstType, count, alpha, beta, variant);
    default:
        return 1;
    }
}

// ---- CropFlipNormalizeReformat ------------------------------------------------------------------------
// follows the golden tests/cvcuda/system/TestOpCropFlipNormalizeReformat.cpp:44-170 (identical to the
// device expression src/cvcuda/priv/OpCropFlipNormalizeReformat.cu:73-74, 165-187): one image, source
// and destination as packed HWC arrays.
template<class TS, class TD>
void CropFlipNormOne(const TS *src, int W, int H, int C, TD *dst, int dw, int dh, const int *crop, int flip, int border,
                     float borderValue, const float *base, const float *scale, float gscale, float shift, float eps,
                     int stddev)
{
    for (int i = 0; i < dh; ++i)
    {
        for (int j = 0; j < dw; ++j)
        {
            TD *o = dst + ((int64_t)i * dw + j) * C;
            if (i >= crop[3] || j >= crop[2])
            {
                for (int k = 0; k < C; ++k)
                {
                    o[k] = 0;
                }
                continue;
            }
            int x = j + crop[0], y = i + crop[1];
            if (flip == 1 || flip == -1)
            {
                x = crop[2] - 1 - j + crop[0];
            }
            if (flip == 0 || flip == -1)
            {
                y = crop[3] - 1 - i + crop[1];
            }
            const bool outside = x < 0 || x >= W || y < 0 || y >= H;
            if (outside && border != 0)
            {
                x = BorderIndex(border, x, W);
                y = BorderIndex(border, y, H);
            }
            for (int k = 0; k < C; ++k)
            {
                float mul = scale[k];
                if (stddev)
                {
                    float t = scale[k] * scale[k] + eps;
                    mul     = 1.0f / std::sqrt(t);
                }
                TS v;
                if (outside && border == 0)
                {
                    if constexpr (std::is_same_v<TS, float>)
                    {
                        v = borderValue;
                    }
                    else
                    {
                        float t = std::trunc(borderValue);
                        t       = std::min(std::max(t, (float)std::numeric_limits<TS>::min()),
                                           (float)std::numeric_limits<TS>::max());
                        v       = (TS)(int64_t)t;
                    }
                }
                else
                {
                    v = src[((int64_t)y * W + x) * C + k];
                }
                o[k] = SatF<TD>(((float)v - base[k]) * mul * gscale + shift);
            }
        }
    }
}

ORC_API int orc_crop_flip_normalize(const void *src, int W, int H, int C, int srcType, void *dst, int dw, int dh,
                                    int dstType, const int *crop, int flip, int border, float borderValue,
                                    const float *base, const float *scale, float gscale, float shift, float eps,
                                    int stddev)
{
    int rc = 1;
    DispatchType(srcType,
                 [&](auto ts)
                 {
                     using TS = decltype(ts);
                     rc       = DispatchType(dstType,
                                             [&](auto td)
                                             {
                                           using TD = decltype(td);
                                           CropFlipNormOne<TS, TD>((const TS *)src, W, H, C, (TD *)dst, dw, dh, crop, flip,
                                                                   border, borderValue, base, scale, gscale, shift, eps,
                                                                   stddev);
                                       });
                 });
    return rc;
}

// ---- primitives exposed for known-answer tests ----------------------------------------------------
ORC_API int orc_saturate_f32(float v, int dtype)
{
    switch (dtype)
    {
    case U8:
        return SatF<uint8_t>(v);
    case S8:
        return SatF<int8_t>(v);
    case U16:
        return SatF<uint16_t>(v);
    case S16:
        return SatF<int16_t>(v);
    case S32:
        return SatF<int32_t>(v);
    default:
        return 0;
    }
}

ORC_API int orc_border_index(int mode, int c, int s)
{
    return BorderIndex(mode, c, s);
}

ORC_API int orc_border_index_reflect_device(int c, int s)
{
    return BorderIndexReflectDevice(c, s);
}

// ---- seeded input generator: splitmix64, consumed byte-wise for u8 and as 24-bit fractions for f32.
static inline uint64_t SplitMix64(uint64_t &state)
{
    uint64_t z = (state += 0x9E3779B97F4A7C15ULL);
    z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z          = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

ORC_API void orc_fill_u8(uint8_t *buf, int64_t n, uint64_t seed, int lo, int hi)
{
    uint64_t st   = seed;
    int      span = hi - lo + 1;
    for (int64_t i = 0; i < n; i += 8)
    {
        uint64_t r = SplitMix64(st);
        for (int k = 0; k < 8 && i + k < n; ++k)
        {
            int b      = (int)((r >> (8 * k)) & 0xFF);
            buf[i + k] = (uint8_t)(span == 256 ? b : lo + (b * span >> 8));
        }
    }
}

ORC_API void orc_fill_f32(float *buf, int64_t n, uint64_t seed)
{
    uint64_t st = seed;
    for (int64_t i = 0; i < n; ++i)
    {
        buf[i] = (float)(SplitMix64(st) >> 40) * (1.0f / 16777216.0f);
    }
}
