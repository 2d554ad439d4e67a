// Colour conversion: channel swizzles (BGR<->RGB, add/drop alpha) and YUV 4:2:0 -> RGB family; every other
// supported code is forwarded to the per-pixel families of OpCvtColorPixel.hip.
//
// Arithmetic follows the reference: integer BT.601 limited-range conversion in 20-bit fixed point
// (src/cvcuda/priv/legacy/cvt_color.cu:64-69, 618-638) with the 4:2:0 addressing of :514-565; swizzle
// and alpha rules of :181-230, 775-854. Validation follows :1387-1451 and :1768-1790 (every failure
// is reported as INVALID_ARGUMENT, as the reference's error translation does).
//
// NV12/NV21 kernel shape: a lane converts a block of 4x2 pixels -- two 4-byte luma loads, one 4-byte
// chroma load (U0 V0 U1 V1 serves all eight pixels), two 12- or 16-byte streaming stores. Consecutive
// lanes touch consecutive addresses in all three streams, so every cache line is fetched and written
// exactly once: 1.5 bytes in, 3 (4) bytes out per pixel.
#include "CvtColorFamilies.hpp"
#include "DeviceUtils.hpp"
#include "OpCommon.hpp"
#include "LaneExchange.hpp"
#include "RunIO.hpp"
#include "VarShapeTiles.hpp"

#include <cvcuda/OpCvtColor.h>

#include <algorithm>

namespace cvamd {

namespace {

// ---------------------------------------------------------------------------------------------------
// YUV 4:2:0 -> RGB
constexpr int kYuvBlockW = 8;               // pixels per lane and row (a lane converts a kYuvBlockW x 2 block)
constexpr int kYuvTileW  = 64 * kYuvBlockW; // pixels per wave and row
constexpr int kYuvTileH  = 8;               // image batches: rows per block, 4 waves x 2 rows (tensors: 4 waves side by side)

struct YuvArgs
{
    const uint8_t *srcBase;
    uint8_t       *dstBase;
    int64_t        srcSampleStride, dstSampleStride;
    int32_t        srcRowStride, dstRowStride;
    int32_t        W, H; // RGB size
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
    int32_t bidx, uidx;
};

__device__ __forceinline__ void YuvToRgb(int Y, int uu, int vv, uint32_t &r, uint32_t &g, uint32_t &b)
{
    const int yy = max(0, Y - 16) * 1220542;
    r            = (uint32_t)min(max((yy + 1673527 * vv + (1 << 19)) >> 20, 0), 255);
    g            = (uint32_t)min(max((yy - 852492 * vv - 409993 * uu + (1 << 19)) >> 20, 0), 255);
    b            = (uint32_t)min(max((yy + 2116026 * uu + (1 << 19)) >> 20, 0), 255);
}

template<int DCN>
struct __attribute__((packed, aligned(1))) RgbQuad
{
    uint32_t w[DCN]; // 4 pixels of DCN bytes
};

template<int DCN, bool SEMIPLANAR>
__device__ __forceinline__ void ConvertBlock(const uint8_t *src, int srcRow, uint8_t *dst, int dstRow, int W, int H,
                                             int x, int y, int bidx, int uidx)
{
    // chroma for pixel pairs (x, x+1) and (x+2, x+3)
    int U[2], V[2];
    if constexpr (SEMIPLANAR)
    {
        const uint8_t *uv = src + (int64_t)(H + (y >> 1)) * srcRow + x;
        if (x + 3 < W)
        {
            const uint32_t c = LoadU32Unaligned(uv);
            U[0]             = (c >> (8 * uidx)) & 0xFF;
            V[0]             = (c >> (8 * (uidx ^ 1))) & 0xFF;
            U[1]             = (c >> (16 + 8 * uidx)) & 0xFF;
            V[1]             = (c >> (16 + 8 * (uidx ^ 1))) & 0xFF;
        }
        else
        {
            U[0] = U[1] = uv[uidx];
            V[0] = V[1] = uv[uidx ^ 1];
        }
    }
    else
    {
        // planar: each chroma plane is (H/2) x (W/2), stored as H/4 rows of W bytes after the luma rows
        const int      h4  = H >> 2;
        const int      uvx = (x >> 1) + ((W >> 1) & -((y >> 1) & 1));
        const uint8_t *pu  = src + (int64_t)(H + (y >> 2) + h4 * uidx) * srcRow + uvx;
        const uint8_t *pv  = src + (int64_t)(H + (y >> 2) + h4 * (uidx ^ 1)) * srcRow + uvx;
        const int      i1  = (x + 3 < W) ? 1 : 0;
        U[0]               = pu[0];
        U[1]               = pu[i1];
        V[0]               = pv[0];
        V[1]               = pv[i1];
    }
    const int uu[2] = {U[0] - 128, U[1] - 128};
    const int vv[2] = {V[0] - 128, V[1] - 128};

#pragma unroll
    for (int ry = 0; ry < 2; ++ry)
    {
        const int yy = y + ry;
        if (yy >= H)
        {
            break;
        }
        const uint8_t *py  = src + (int64_t)yy * srcRow + x;
        uint8_t       *out = dst + (int64_t)yy * dstRow + (int64_t)x * DCN;
        if (x + 3 < W)
        {
            const uint32_t luma = LoadU32Unaligned(py);
            uint32_t       px[4][3]; // [pixel][byte position in the output pixel]
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                uint32_t r, g, b;
                YuvToRgb((luma >> (8 * i)) & 0xFF, uu[i >> 1], vv[i >> 1], r, g, b);
                px[i][0] = bidx == 0 ? b : r;
                px[i][1] = g;
                px[i][2] = bidx == 0 ? r : b;
            }
            RgbQuad<DCN> q;
            if constexpr (DCN == 3)
            {
                q.w[0] = px[0][0] | (px[0][1] << 8) | (px[0][2] << 16) | (px[1][0] << 24);
                q.w[1] = px[1][1] | (px[1][2] << 8) | (px[2][0] << 16) | (px[2][1] << 24);
                q.w[2] = px[2][2] | (px[3][0] << 8) | (px[3][1] << 16) | (px[3][2] << 24);
            }
            else
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    q.w[i] = px[i][0] | (px[i][1] << 8) | (px[i][2] << 16) | 0xFF000000u;
                }
            }
            RgbQuad<DCN> *o = reinterpret_cast<RgbQuad<DCN> *>(out);
#pragma unroll
            for (int i = 0; i < DCN; ++i)
            {
                __builtin_nontemporal_store(q.w[i], &o->w[i]);
            }
        }
        else
        {
            for (int i = 0; i < 4 && x + i < W; ++i) // ragged right edge (width not a multiple of 4)
            {
                uint32_t r, g, b;
                YuvToRgb(py[i], uu[i >> 1], vv[i >> 1], r, g, b);
                out[i * DCN + bidx]       = (uint8_t)b;
                out[i * DCN + 1]          = (uint8_t)g;
                out[i * DCN + (bidx ^ 2)] = (uint8_t)r;
                if constexpr (DCN == 4)
                {
                    out[i * DCN + 3] = 255;
                }
            }
        }
    }
}

// A kYuvBlockW x 2 block that lies wholly inside the row (x + kYuvBlockW <= W): every access is a vector
// of whole dwords (luma 8 bytes per row, chroma 8 or 4 + 4 bytes, 24 or 32 output bytes per row).
template<int DCN, bool SEMIPLANAR>
__device__ __forceinline__ void ConvertWideBlock(const uint8_t *src, int srcRow, uint8_t *dst, int dstRow, int W, int H,
                                                 int x, int y, int bidx, int uidx)
{
    constexpr int BW = kYuvBlockW, NC = BW / 2;
    // lanes 0 .. lanes-1 of this wave take this path (the wave covers consecutive blocks of one row)
    const int lane = threadIdx.x & 63, lanes = min(64, (W - (x - lane * BW)) / BW);
    int       uu[NC], vv[NC];
    if constexpr (SEMIPLANAR)
    {
        uint8_t  c[BW];
        uint32_t w[BW / 4];
        LoadRun<uint8_t, BW>(src + (int64_t)(H + (y >> 1)) * srcRow + x, c);
        __builtin_memcpy(w, c, sizeof(w));
#pragma unroll
        for (int k = 0; k < NC; ++k)
        {
            const int sh = 16 * (k & 1);
            uu[k]        = (int)((w[k >> 1] >> (sh + 8 * uidx)) & 0xFF) - 128;
            vv[k]        = (int)((w[k >> 1] >> (sh + 8 * (uidx ^ 1))) & 0xFF) - 128;
        }
    }
    else
    {
        const int h4  = H >> 2;
        const int uvx = (x >> 1) + ((W >> 1) & -((y >> 1) & 1));
        uint8_t   pu[NC], pv[NC];
        LoadRun<uint8_t, NC>(src + (int64_t)(H + (y >> 2) + h4 * uidx) * srcRow + uvx, pu);
        LoadRun<uint8_t, NC>(src + (int64_t)(H + (y >> 2) + h4 * (uidx ^ 1)) * srcRow + uvx, pv);
#pragma unroll
        for (int k = 0; k < NC; ++k)
        {
            uu[k] = (int)pu[k] - 128;
            vv[k] = (int)pv[k] - 128;
        }
    }
    // The chroma terms and the rounding constant of YuvToRgb's three sums, once per chroma sample (4
    // pixels share them), already in output channel order; integer addition is associative, so the
    // results are the same.
    int c0[NC], c1[NC], c2[NC];
#pragma unroll
    for (int k = 0; k < NC; ++k)
    {
        const int rC = 1673527 * vv[k] + (1 << 19);
        const int bC = 2116026 * uu[k] + (1 << 19);
        c0[k]        = bidx == 0 ? bC : rC;
        c1[k]        = -852492 * vv[k] - 409993 * uu[k] + (1 << 19);
        c2[k]        = bidx == 0 ? rC : bC;
    }
#pragma unroll
    for (int ry = 0; ry < 2; ++ry)
    {
        const int yy = y + ry;
        if (yy >= H)
        {
            break;
        }
        uint8_t luma[BW], out[BW * DCN];
        LoadRun<uint8_t, BW>(src + (int64_t)yy * srcRow + x, luma);
#pragma unroll
        for (int i = 0; i < BW; ++i)
        {
            const int t      = max(0, (int)luma[i] - 16) * 1220542;
            out[i * DCN + 0] = (uint8_t)min(max((t + c0[i >> 1]) >> 20, 0), 255);
            out[i * DCN + 1] = (uint8_t)min(max((t + c1[i >> 1]) >> 20, 0), 255);
            out[i * DCN + 2] = (uint8_t)min(max((t + c2[i >> 1]) >> 20, 0), 255);
            if constexpr (DCN == 4)
            {
                out[i * DCN + 3] = 255;
            }
        }
        StoreRowRunNT<uint8_t, BW * DCN>(dst + (int64_t)yy * dstRow + (int64_t)(x - lane * BW) * DCN, out, lane, lanes);
    }
}

// The lane's kYuvBlockW x 2 block at (x, y): the wide form inside the row, 4 x 2 blocks at its ragged end.
template<int DCN, bool SEMIPLANAR>
__device__ __forceinline__ void ConvertLaneBlock(const uint8_t *src, int srcRow, uint8_t *dst, int dstRow, int W, int H,
                                                 int x, int y, int bidx, int uidx)
{
    if (x + kYuvBlockW <= W)
    {
        ConvertWideBlock<DCN, SEMIPLANAR>(src, srcRow, dst, dstRow, W, H, x, y, bidx, uidx);
        return;
    }
    for (int xx = x; xx < W; xx += 4)
    {
        ConvertBlock<DCN, SEMIPLANAR>(src, srcRow, dst, dstRow, W, H, xx, y, bidx, uidx);
    }
}

template<int DCN, bool SEMIPLANAR>
__global__ __launch_bounds__(256) void Yuv420ToRgbTensor(const YuvArgs a, const int flat)
{
    // flat: a block's four waves side by side on one pair of rows (2048 columns) instead of 512 columns x 8 rows: 32 x
    // 1080p 51.5 -> 50.8 us, the two alternating on one machine. The host asks for it where rows fill such blocks to 80 %.
    // (arithmetic rather than a branch on `flat`, so that the other arguments are loaded at once)
    const int f = flat != 0;
    const int x = (int)(blockIdx.x * (64u << (2 * f)) + (threadIdx.x & (63u | (192u * f)))) * kYuvBlockW;
    const int y = (int)(blockIdx.y * (4 - 3 * f) + (threadIdx.x >> 6) * (1 - f)) * 2;
    if (x >= a.W || y >= a.H)
    {
        return;
    }
    const int n = blockIdx.z;
    ConvertLaneBlock<DCN, SEMIPLANAR>(a.srcBase + n * a.srcSampleStride, a.srcRowStride, a.dstBase + n * a.dstSampleStride,
                                      a.dstRowStride, a.W, a.H, x, y, a.bidx, a.uidx);
}

template<int DCN, bool SEMIPLANAR>
__global__ __launch_bounds__(256) void Yuv420ToRgbVarShape(const YuvArgs a, const VarTiles tiles)
{
    const TileCoord              tc = LocateTile(tiles, blockIdx.x);
    const NVCVImagePlaneStrided &s  = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided &d  = a.dstList[tc.image].planes[0];
    const int                    W = d.width, H = d.height;
    const int                    x = (tc.tx * 64 + (threadIdx.x & 63)) * kYuvBlockW;
    const int                    y = (tc.ty * 4 + (threadIdx.x >> 6)) * 2;
    if (x >= W || y >= H)
    {
        return;
    }
    ConvertLaneBlock<DCN, SEMIPLANAR>(AsGlobal(s.basePtr), s.rowStride, AsGlobal(d.basePtr), d.rowStride, W, H, x, y, a.bidx,
                                      a.uidx);
}

template<class T, int C>
using Px = Packed<T, C>;

struct SwizzleArgs
{
    const uint8_t *srcBase;
    uint8_t       *dstBase;
    int64_t        srcSampleStride, dstSampleStride;
    int32_t        srcRowStride, dstRowStride;
    int32_t        W, H;
    const NVCVImageBufferStrided *srcList;
    const NVCVImageBufferStrided *dstList;
    int32_t  bidx;  // 2: swap channels 0 and 2, 0: keep order
    uint64_t alpha; // bit pattern of the alpha value written when the source has none
};

template<class T, int SCH, int DCH>
__device__ __forceinline__ void SwizzlePixel(const uint8_t *srcRow, uint8_t *dstRow, int x, int bidx, uint64_t alpha)
{
    const Px<T, SCH> s = reinterpret_cast<const Px<T, SCH> *>(srcRow)[x];
    Px<T, DCH>       d;
    d.v[0] = bidx ? s.v[2] : s.v[0];
    d.v[1] = s.v[1];
    d.v[2] = bidx ? s.v[0] : s.v[2];
    if constexpr (DCH == 4)
    {
        if constexpr (SCH == 4)
        {
            d.v[3] = s.v[3];
        }
        else
        {
            d.v[3] = (T)alpha;
        }
    }
    Px<T, DCH> *o = reinterpret_cast<Px<T, DCH> *>(dstRow) + x;
#pragma unroll
    for (int c = 0; c < DCH; ++c)
    {
        __builtin_nontemporal_store(d.v[c], &o->v[c]);
    }
}

// A run of pixels of a row from x0 on (one run per lane); the ragged end of a row goes pixel by pixel.
template<class T, int SCH, int DCH>
__device__ __forceinline__ void SwizzleRun(const uint8_t *srcRow, uint8_t *dstRow, int W, int x0, int bidx,
                                           uint64_t alpha)
{
    constexpr int P = kRunPixelsFor<T, T>;
    if (x0 + P > W)
    {
        for (int x = x0; x < W; ++x)
        {
            SwizzlePixel<T, SCH, DCH>(srcRow, dstRow, x, bidx, alpha);
        }
        return;
    }
    T in[P * SCH], out[P * DCH];
    LoadRun<T, P * SCH>(srcRow + (int64_t)x0 * SCH * sizeof(T), in);
    const bool swap = bidx != 0;
#pragma unroll
    for (int k = 0; k < P; ++k)
    {
        out[k * DCH + 0] = swap ? in[k * SCH + 2] : in[k * SCH + 0];
        out[k * DCH + 1] = in[k * SCH + 1];
        out[k * DCH + 2] = swap ? in[k * SCH + 0] : in[k * SCH + 2];
        if constexpr (DCH == 4)
        {
            if constexpr (SCH == 4)
            {
                out[k * DCH + 3] = in[k * SCH + 3];
            }
            else
            {
                out[k * DCH + 3] = (T)alpha;
            }
        }
    }
    const int lane = threadIdx.x & 63, lanes = min(64, (W - (x0 - lane * P)) / P);
    StoreRowRunNT<T, P * DCH>(dstRow + (int64_t)(x0 - lane * P) * DCH * sizeof(T), out, lane, lanes);
}

template<class T, int SCH, int DCH>
__global__ __launch_bounds__(256) void SwizzleTensor(const SwizzleArgs a)
{
    const int x0 = (blockIdx.x * 64 + (threadIdx.x & 63)) * kRunPixelsFor<T, T>;
    const int y  = blockIdx.y * kRunTileH + (threadIdx.x >> 6);
    if (x0 >= a.W || y >= a.H)
    {
        return;
    }
    const int n = blockIdx.z;
    SwizzleRun<T, SCH, DCH>(a.srcBase + n * a.srcSampleStride + (int64_t)y * a.srcRowStride,
                            a.dstBase + n * a.dstSampleStride + (int64_t)y * a.dstRowStride, a.W, x0, a.bidx, a.alpha);
}

template<class T, int DCH>
constexpr int kSwizzleVarRows = kVarShapeRows<kRunPixelsFor<T, T> * DCH * (int)sizeof(T)>;

template<class T, int SCH, int DCH>
__global__ __launch_bounds__(256) void SwizzleVarShape(const SwizzleArgs a, const VarTiles tiles)
{
    const TileCoord              tc = LocateTile(tiles, blockIdx.x);
    const NVCVImagePlaneStrided &s  = a.srcList[tc.image].planes[0];
    const NVCVImagePlaneStrided &d  = a.dstList[tc.image].planes[0];
    const int                    x0 = (tc.tx * 64 + (threadIdx.x & 63)) * kRunPixelsFor<T, T>;
    const uint8_t *src = AsGlobal(s.basePtr);
    uint8_t       *dst = AsGlobal(d.basePtr);
    const int      W = d.width, H = d.height, srcRow = s.rowStride, dstRow = d.rowStride;
    if (x0 >= W)
    {
        return;
    }
    constexpr int R = kSwizzleVarRows<T, DCH>;
    for (int r = 0; r < R; ++r)
    {
        const int y = (tc.ty * R + r) * kRunTileH + (threadIdx.x >> 6);
        if (y >= H)
        {
            return;
        }
        SwizzleRun<T, SCH, DCH>(src + (int64_t)y * srcRow, dst + (int64_t)y * dstRow, W, x0, a.bidx, a.alpha);
    }
}

// ---------------------------------------------------------------------------------------------------
enum class Family
{
    Swizzle,
    Yuv420ToRgb,
    Unsupported
};

Family FamilyOf(ColorCode code)
{
    const int c = (int)code;
    if (c >= NVCV_COLOR_BGR2BGRA && c <= NVCV_COLOR_BGRA2RGBA)
    {
        return Family::Swizzle;
    }
    if (c >= NVCV_COLOR_YUV2RGB_NV12 && c <= NVCV_COLOR_YUV2BGRA_IYUV)
    {
        return Family::Yuv420ToRgb;
    }
    return Family::Unsupported;
}

struct YuvCode
{
    int  bidx, uidx;
    bool planar;
};

YuvCode DecodeYuvCode(ColorCode code)
{
    YuvCode y;
    switch (code)
    {
    case NVCV_COLOR_YUV2BGR_NV12:
    case NVCV_COLOR_YUV2BGRA_NV12:
    case NVCV_COLOR_YUV2BGR_NV21:
    case NVCV_COLOR_YUV2BGRA_NV21:
    case NVCV_COLOR_YUV2BGR_YV12:
    case NVCV_COLOR_YUV2BGRA_YV12:
    case NVCV_COLOR_YUV2BGR_IYUV:
    case NVCV_COLOR_YUV2BGRA_IYUV:
        y.bidx = 0;
        break;
    default:
        y.bidx = 2;
        break;
    }
    switch (code)
    {
    case NVCV_COLOR_YUV2BGR_NV12:
    case NVCV_COLOR_YUV2BGRA_NV12:
    case NVCV_COLOR_YUV2RGB_NV12:
    case NVCV_COLOR_YUV2RGBA_NV12:
    case NVCV_COLOR_YUV2BGR_IYUV:
    case NVCV_COLOR_YUV2BGRA_IYUV:
    case NVCV_COLOR_YUV2RGB_IYUV:
    case NVCV_COLOR_YUV2RGBA_IYUV:
        y.uidx = 0;
        break;
    default:
        y.uidx = 1;
        break;
    }
    y.planar = (int)code >= NVCV_COLOR_YUV2RGB_YV12;
    return y;
}

uint64_t AlphaBits(ElemType e)
{
    switch (e)
    {
    case kU8:
    case kS8:
        return 0xFF;
    case kU16:
    case kS16:
    case kF16:
        return 0xFFFF;
    case kS32:
        return 0x7FFFFFFF;
    case kF32:
        return 0x3F800000ull; // 1.0f
    case kF64:
        return 0x3FF0000000000000ull; // 1.0
    default:
        return 0;
    }
}

template<class T, int SCH, int DCH>
void LaunchSwizzle(const SwizzleArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    if (dstHost == nullptr)
    {
        dim3 grid(DivUp(a.W, 64 * kRunPixelsFor<T, T>), DivUp(a.H, kRunTileH), N);
        hipLaunchKernelGGL((SwizzleTensor<T, SCH, DCH>), grid, dim3(256), 0, stream, a);
        CheckLaunch("SwizzleTensor");
        return;
    }
    for (int first = 0; first < N; first += kMaxTileImages)
    {
        VarTiles tiles;
        int total = BuildVarTiles(tiles, dstHost, first, std::min(kMaxTileImages, N - first), 64 * kRunPixelsFor<T, T>,
                                  kRunTileH * kSwizzleVarRows<T, DCH>);
        if (total > 0)
        {
            hipLaunchKernelGGL((SwizzleVarShape<T, SCH, DCH>), dim3(total), dim3(256), 0, stream, a, tiles);
            CheckLaunch("SwizzleVarShape");
        }
    }
}

template<class T>
void DispatchSwizzle(int sch, int dch, const SwizzleArgs &a, int N, const NVCVImageBufferStrided *dstHost,
                     hipStream_t stream)
{
    if (sch == 3 && dch == 3)
    {
        LaunchSwizzle<T, 3, 3>(a, N, dstHost, stream);
    }
    else if (sch == 3 && dch == 4)
    {
        LaunchSwizzle<T, 3, 4>(a, N, dstHost, stream);
    }
    else if (sch == 4 && dch == 3)
    {
        LaunchSwizzle<T, 4, 3>(a, N, dstHost, stream);
    }
    else
    {
        LaunchSwizzle<T, 4, 4>(a, N, dstHost, stream);
    }
}

// The swizzle only moves bits: element types of equal size share a kernel. Alpha is passed as bits.
void RunSwizzle(ColorCode code, ElemType elem, int inC, int outC, SwizzleArgs &a, int N,
                const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    const int sch = (code == NVCV_COLOR_BGRA2BGR || code == NVCV_COLOR_RGBA2BGR || code == NVCV_COLOR_BGRA2RGBA) ? 4 : 3;
    const int dch = (code == NVCV_COLOR_BGR2BGRA || code == NVCV_COLOR_BGR2RGBA || code == NVCV_COLOR_BGRA2RGBA) ? 4 : 3;
    a.bidx        = (code != NVCV_COLOR_BGRA2BGR && code != NVCV_COLOR_BGR2BGRA) ? 2 : 0;
    if (inC != sch)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input channel number %d -- expecting %d", inC, sch);
    }
    if (outC != dch)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid output channel number %d -- expecting %d", outC, dch);
    }
    if (elem == kF16 && sch < 4 && dch == 4)
    {
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Adding alpha to the output is not supported for 16-bit floats");
    }
    a.alpha = AlphaBits(elem);
    if (N == 0)
    {
        return;
    }
    switch (ElemSize(elem))
    {
    case 1:
        DispatchSwizzle<uint8_t>(sch, dch, a, N, dstHost, stream);
        break;
    case 2:
        DispatchSwizzle<uint16_t>(sch, dch, a, N, dstHost, stream);
        break;
    case 4:
        DispatchSwizzle<uint32_t>(sch, dch, a, N, dstHost, stream);
        break;
    case 8:
        DispatchSwizzle<uint64_t>(sch, dch, a, N, dstHost, stream);
        break;
    default:
        throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Unsupported DataType");
    }
}

template<int DCN, bool SEMIPLANAR>
void LaunchYuv(const YuvArgs &a, int N, const NVCVImageBufferStrided *dstHost, hipStream_t stream)
{
    if (dstHost == nullptr)
    {
        const int64_t span = 4 * kYuvTileW;
        const bool    flat = DivUp(a.W, (int)span) * span * 4 <= (int64_t)a.W * 5;
        dim3          grid(DivUp(a.W, flat ? 4 * kYuvTileW : kYuvTileW), DivUp(a.H, flat ? 2 : kYuvTileH), N);
        hipLaunchKernelGGL((Yuv420ToRgbTensor<DCN, SEMIPLANAR>), grid, dim3(256), 0, stream, a, (int)flat);
        CheckLaunch("Yuv420ToRgbTensor");
        return;
    }
    for (int first = 0; first < N; first += kMaxTileImages)
    {
        VarTiles tiles;
        int total = BuildVarTiles(tiles, dstHost, first, std::min(kMaxTileImages, N - first), kYuvTileW, kYuvTileH);
        if (total > 0)
        {
            hipLaunchKernelGGL((Yuv420ToRgbVarShape<DCN, SEMIPLANAR>), dim3(total), dim3(256), 0, stream, a, tiles);
            CheckLaunch("Yuv420ToRgbVarShape");
        }
    }
}

void RunYuv(const YuvCode &yc, int dcn, const YuvArgs &a, int N, const NVCVImageBufferStrided *dstHost,
            hipStream_t stream)
{
    if (N == 0)
    {
        return;
    }
    if (yc.planar)
    {
        dcn == 3 ? LaunchYuv<3, false>(a, N, dstHost, stream) : LaunchYuv<4, false>(a, N, dstHost, stream);
    }
    else
    {
        dcn == 3 ? LaunchYuv<3, true>(a, N, dstHost, stream) : LaunchYuv<4, true>(a, N, dstHost, stream);
    }
}

class CvtColor final : public IOperator
{
public:
    void submit(hipStream_t stream, NVCVTensorHandle hin, NVCVTensorHandle hout, ColorCode code) const
    {
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
        if (std::max(in.bytesSpanned(), out.bytesSpanned()) > INT64_MAX / 2 || in.strideH > INT32_MAX
            || out.strideH > INT32_MAX)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Input or output tensors are too large");
        }
        switch (FamilyOf(code))
        {
        case Family::Swizzle:
        {
            if (out.elem != in.elem)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Mismatched input / output DataTypes");
            }
            if (out.H != in.H || out.W != in.W || out.N != in.N)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Shape mismatch -- output tensor shape doesn't match input");
            }
            SwizzleArgs a     = {};
            a.srcBase         = in.base;
            a.dstBase         = out.base;
            a.srcSampleStride = in.strideN;
            a.dstSampleStride = out.strideN;
            a.srcRowStride    = (int32_t)in.strideH;
            a.dstRowStride    = (int32_t)out.strideH;
            a.W               = in.W;
            a.H               = in.H;
            RunSwizzle(code, in.elem, in.C, out.C, a, in.N, nullptr, stream);
            break;
        }
        case Family::Yuv420ToRgb:
        {
            const YuvCode yc = DecodeYuvCode(code);
            if (out.C != 3 && out.C != 4)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid output channel number %d", out.C);
            }
            if (in.C != 1)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input channel number %d", in.C);
            }
            if (in.H % 3 != 0 || in.W % 2 != 0)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input shape: height %d must be a multiple of 3 and "
                                                           "width %d a multiple of 2",
                              in.H, in.W);
            }
            if (in.elem != kU8 || out.elem != kU8)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Unsupported input/output DataType, must be 8-bit unsigned");
            }
            const int rgbH = in.H * 2 / 3;
            if (out.H != rgbH || out.W != in.W || out.N != in.N)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid output shape, expected %d x %d x %d", in.N, rgbH, in.W);
            }
            if (yc.planar && rgbH % 4 != 0)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                              "Invalid input shape: to convert from YUV 420 planar formats, the output tensor height "
                              "must be a multiple of 4; height = %d",
                              rgbH);
            }
            YuvArgs a         = {};
            a.srcBase         = in.base;
            a.dstBase         = out.base;
            a.srcSampleStride = in.strideN;
            a.dstSampleStride = out.strideN;
            a.srcRowStride    = (int32_t)in.strideH;
            a.dstRowStride    = (int32_t)out.strideH;
            a.W               = in.W;
            a.H               = rgbH;
            a.bidx            = yc.bidx;
            a.uidx            = yc.uidx;
            RunYuv(yc, out.C, a, in.N, nullptr, stream);
            break;
        }
        default:
        {
            if (out.N != in.N)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Shape mismatch -- input and output batch sizes differ");
            }
            ColorIO io = {};
            io.src     = in.base;
            io.dst     = out.base;
            io.srcN    = in.strideN;
            io.dstN    = out.strideN;
            io.srcRow  = (int32_t)in.strideH;
            io.dstRow  = (int32_t)out.strideH;
            io.N       = in.N;
            io.srcW    = in.W;
            io.srcH    = in.H;
            io.srcC    = in.C;
            io.dstW    = out.W;
            io.dstH    = out.H;
            io.dstC    = out.C;
            io.srcElem = in.elem;
            io.dstElem = out.elem;
            if (!RunPixelColorFamily(code, io, stream))
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Unsupported conversion code %d", (int)code);
            }
        }
        }
    }

    void submit(hipStream_t stream, NVCVImageBatchHandle hin, NVCVImageBatchHandle hout,
                ColorCode code) const
    {
        VarShapeView in  = ExportVarShape(hin, stream, "Input");
        VarShapeView out = ExportVarShape(hout, stream, "Output");
        if (in.N != out.N)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Invalid input and output batch sizes: %d != %d", in.N, out.N);
        }
        if (in.uniqueFormat == NVCV_IMAGE_FORMAT_NONE || out.uniqueFormat == NVCV_IMAGE_FORMAT_NONE)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images in the input (output) batch must all share one format");
        }
        FormatInfo fi = DecodeFormat(in.uniqueFormat), fo = DecodeFormat(out.uniqueFormat);
        if (fi.planes != 1 || fo.planes != 1)
        {
            throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Images must have a single plane");
        }
        switch (FamilyOf(code))
        {
        case Family::Swizzle:
        {
            if (fi.elem != fo.elem)
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Mismatched input / output DataTypes");
            }
            for (int i = 0; i < in.N; ++i)
            {
                if (in.hostList[i].planes[0].width != out.hostList[i].planes[0].width
                    || in.hostList[i].planes[0].height != out.hostList[i].planes[0].height)
                {
                    throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Image %d: input and output sizes differ", i);
                }
            }
            SwizzleArgs a = {};
            a.srcList     = in.data.buffer.varShapeStrided.imageList;
            a.dstList     = out.data.buffer.varShapeStrided.imageList;
            RunSwizzle(code, fi.elem, fi.channels, fo.channels, a, in.N, out.hostList, stream);
            break;
        }
        case Family::Yuv420ToRgb:
        {
            const YuvCode yc = DecodeYuvCode(code);
            if (fi.channels != 1 || fi.elem != kU8 || fo.elem != kU8 || (fo.channels != 3 && fo.channels != 4))
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT,
                              "YUV 4:2:0 conversion needs single-channel u8 input images and 3/4-channel u8 output");
            }
            for (int i = 0; i < in.N; ++i)
            {
                const NVCVImagePlaneStrided &s = in.hostList[i].planes[0], &d = out.hostList[i].planes[0];
                if (s.height % 3 != 0 || s.width % 2 != 0 || d.width != s.width || d.height != s.height * 2 / 3
                    || (yc.planar && d.height % 4 != 0))
                {
                    throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Image %d: invalid input/output shape", i);
                }
            }
            YuvArgs a = {};
            a.srcList = in.data.buffer.varShapeStrided.imageList;
            a.dstList = out.data.buffer.varShapeStrided.imageList;
            a.bidx    = yc.bidx;
            a.uidx    = yc.uidx;
            RunYuv(yc, fo.channels, a, in.N, out.hostList, stream);
            break;
        }
        default:
        {
            ColorIO io = {};
            io.N       = in.N;
            io.srcC    = fi.channels;
            io.dstC    = fo.channels;
            io.srcElem = fi.elem;
            io.dstElem = fo.elem;
            io.srcList = in.data.buffer.varShapeStrided.imageList;
            io.dstList = out.data.buffer.varShapeStrided.imageList;
            io.srcHost = in.hostList;
            io.dstHost = out.hostList;
            if (!RunPixelColorFamily(code, io, stream))
            {
                throw OpError(NVCV_ERROR_INVALID_ARGUMENT, "Unsupported conversion code %d", (int)code);
            }
        }
        }
    }
};

} // namespace
} // namespace cvamd

using namespace cvamd;

extern "C"
{
CVCUDA_PUBLIC NVCVStatus cvcudaCvtColorCreate(NVCVOperatorHandle *handle)
{
    return CreateOperator<CvtColor>(handle);
}

CVCUDA_PUBLIC NVCVStatus cvcudaCvtColorSubmit(NVCVOperatorHandle handle, hipStream_t stream, NVCVTensorHandle in,
                                              NVCVTensorHandle out, NVCVColorConversionCode code)
{
    const ColorCode value = EnumBits(code);
    return Protect([&] { ToOperator<CvtColor>(handle).submit(stream, in, out, value); });
}

CVCUDA_PUBLIC NVCVStatus cvcudaCvtColorVarShapeSubmit(NVCVOperatorHandle handle, hipStream_t stream,
                                                      NVCVImageBatchHandle in, NVCVImageBatchHandle out,
                                                      NVCVColorConversionCode code)
{
    const ColorCode value = EnumBits(code);
    return Protect([&] { ToOperator<CvtColor>(handle).submit(stream, in, out, value); });
}
}
