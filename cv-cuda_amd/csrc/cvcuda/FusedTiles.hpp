// Launch geometry and source addressing of the fused resize-crop-convert-reformat kernels: the argument
// block, the workgroup -> tile map and the tap loads. Shared by the operator
// (OpResizeCropConvertReformat.hip) and by the benchmark's copy-bound twin of its bilinear kernel
// (csrc/bench/BenchKernels.hip), which must read the same bytes through the same grid.
#ifndef CVCUDA_AMD_FUSEDTILES_HPP
#define CVCUDA_AMD_FUSEDTILES_HPP

#include "DeviceUtils.hpp"

#include <nvcv/ImageBatchData.h>

namespace cvamd {

// Output rows per wave. One: the launch is bound by HBM and by the time its last waves take to drain,
// and short waves drain fastest (batch-64 1080p -> 224x224 f32 planar: 22.6 us with 1 row, 23.5 with 2,
// 24.9 with 4; full occupancy is needed at every setting: capping the resident workgroups per CU at
// 7 / 6 / 4 of 8 gave 23.7 / 25.9 / 28.8 us).
constexpr int kRowsPerWave  = 1;
constexpr int kWavesPerBlk  = 4;
// Waves of a workgroup side by side on an output row (the others stacked): 1 or 4, chosen per launch
// (FusedArgs::wavesAcross). With all four on ONE row a workgroup reads two contiguous source spans of 2.8 KB and
// writes 896 contiguous bytes per plane; against 64 columns x 4 rows, alternating on one machine, three times each:
// 22.58 -> 22.48 us for the batch of 64 tensor images, 22.21 -> 22.03 us for the image batch (two waves across: no
// change). Other row lengths keep 64 x 4 (FusedWavesAcross).
__host__ __device__ __forceinline__ int FusedColsPerBlock(int wavesAcross)
{
    return 64 * wavesAcross;
}

__host__ __device__ __forceinline__ int FusedRowsPerBlock(int wavesAcross)
{
    return kRowsPerWave * kWavesPerBlk / wavesAcross;
}

inline int FusedWavesAcross(int dstW)
{
    // one workgroup per output row where the row fills it to 80 % (205 .. 256 columns: the 224 of the usual network
    // input). Wider rows measured no gain for planar outputs and a loss for interleaved 8-bit ones (64 x 1280 x 720 ->
    // 640 x 360: 47.9 -> 51.6 us), narrower ones leave waves without columns.
    const int span = FusedColsPerBlock(kWavesPerBlk);
    return dstW <= span && (int64_t)dstW * 5 >= (int64_t)span * 4 ? kWavesPerBlk : 1;
}

// Output column of this lane and first output row of its wave within tile (tx, ty).
__device__ __forceinline__ int FusedColumnOf(int tx, int wavesAcross)
{
    const int cols = FusedColsPerBlock(wavesAcross);
    return tx * cols + (int)(threadIdx.x & (cols - 1));
}

__device__ __forceinline__ int FusedFirstRowOf(int ty, int wavesAcross)
{
    // (1 wave across: the workgroup's waves are its rows; 4 across: one row)
    return wavesAcross == 1 ? ty * (kRowsPerWave * kWavesPerBlk) + (int)(threadIdx.x >> 6) * kRowsPerWave : ty * kRowsPerWave;
}

struct FusedArgs
{
    // source: tensor (base + n*sampleStride) or var-shape descriptor list
    const uint8_t                *srcBase;
    int64_t                       srcSampleStride;
    int32_t                       srcRowStride;
    int32_t                       srcW, srcH;
    const NVCVImageBufferStrided *srcList;
    // destination, strides in elements
    void   *dstBase;
    int64_t dstStrideN;
    int32_t dstStrideY, dstStrideX;
    int64_t dstOffC[3]; // element offset of source channel c in the destination (mapping applied)
    int32_t interleaved; // 0: any strides; 1 / 2: pixels are 3 adjacent elements in source / reversed channel order
    int32_t dstW, dstH;
    // geometry
    int32_t newW, newH;
    int32_t cropX, cropY;
    float   scaleX, scaleY; // tensor path: srcW/newW, srcH/newH
    float   scale, offset;
    int32_t srcCast;
    // launch shape: column tiles and row tiles per image, first image of this launch
    uint32_t tilesX, tilesY;
    int32_t  wavesAcross; // 1 or 4: the workgroup is 64 columns x 4 rows or 256 columns x 1 row (set by SetFusedGrid)
    uint32_t firstImage;
    // per-channel normalisation of the extension entry points, indexed by source channel:
    // ((scale*v + offset) - normBase) * normMul * normGlobal + normShift
    float normBase[3], normMul[3];
    float normGlobal, normShift;
};

struct TilePos
{
    int n, tx, ty;
};

// Hardware workgroup id -> (image, row tile, column tile).
// The column tiles of one row tile read overlapping cache lines (a 128-byte line straddles each
// tile boundary). MI355X deals workgroups to its 8 XCDs round-robin in the order of their linear id
// (x fastest) and each XCD has its own L2, so with the natural order both neighbours would fetch the
// shared line from memory. The grid is (8 * column tiles, row tiles / 8, images): x % 8 is the XCD and
// selects one of 8 consecutive row tiles, x / 8 the column tile, so the column tiles of a row tile go
// to ONE XCD on consecutive turns (the second hits in L2) while consecutive row tiles go to
// consecutive XCDs and all XCDs stream through the same region of an image at the same time. The
// decode is shifts and masks only (no division: it sits in front of every wave's first load). Row
// tiles are padded to a multiple of 8 per image; padding workgroups get an out-of-range column and
// leave at once.
__device__ __forceinline__ TilePos LocateFusedTile(const FusedArgs &a)
{
    const uint32_t xcd = blockIdx.x % kXcdCount;
    TilePos        p;
    p.n  = (int)(blockIdx.z + a.firstImage);
    p.ty = (int)(blockIdx.y * kXcdCount + xcd);
    p.tx = (uint32_t)p.ty < a.tilesY ? (int)(blockIdx.x / kXcdCount) : (1 << 24);
    return p;
}

// Largest number of images one launch covers (the grid's z extent).
constexpr int kFusedImagesPerLaunch = 65535;

// Fills the launch-shape fields of `a` and returns the grid of 256-thread workgroups for `images`
// images (at most kFusedImagesPerLaunch) starting at a.firstImage.
inline dim3 SetFusedGrid(FusedArgs &a, int images)
{
    a.wavesAcross = FusedWavesAcross(a.dstW);
    a.tilesX      = (uint32_t)((a.dstW + FusedColsPerBlock(a.wavesAcross) - 1) / FusedColsPerBlock(a.wavesAcross));
    a.tilesY      = (uint32_t)((a.dstH + FusedRowsPerBlock(a.wavesAcross) - 1) / FusedRowsPerBlock(a.wavesAcross));
    return dim3(a.tilesX * kXcdCount, (a.tilesY + kXcdCount - 1) / kXcdCount, (uint32_t)images);
}

struct SrcImage
{
    const uint8_t *base;
    int32_t        rowStride, w, h;
    float          scaleX, scaleY;
};

template<bool VARSHAPE>
__device__ __forceinline__ SrcImage GetSource(const FusedArgs &a, int n)
{
    SrcImage s;
    if constexpr (VARSHAPE)
    {
        const NVCVImagePlaneStrided &pl = a.srcList[n].planes[0];
        s.base                          = AsGlobal(pl.basePtr);
        s.rowStride                     = pl.rowStride;
        s.w                             = pl.width;
        s.h                             = pl.height;
        s.scaleX                        = static_cast<float>(s.w) / a.newW;
        s.scaleY                        = static_cast<float>(s.h) / a.newH;
    }
    else
    {
        s.base      = a.srcBase + n * a.srcSampleStride;
        s.rowStride = a.srcRowStride;
        s.w         = a.srcW;
        s.h         = a.srcH;
        s.scaleX    = a.scaleX;
        s.scaleY    = a.scaleY;
    }
    return s;
}


// Terms of the bilinear map that depend on the output column only: byte offset of the first tap in a
// source row, the weight of the second tap, and whether the second tap is the next pixel (otherwise
// the same pixel: the map is clamped at the image's right edge).
struct FusedColumn
{
    int   xoff;
    float fx;
    bool  twoTap;
};

__device__ __forceinline__ FusedColumn ColumnTerms(const FusedArgs &a, const SrcImage &s, int dx)
{
    float fx  = (dx + a.cropX + 0.5f) * s.scaleX - 0.5f;
    int   sx0 = (int)floorf(fx);
    int   sx1 = min(sx0 + 1, s.w - 1);
    fx -= sx0;
    sx0 = max(0, sx0);
    FusedColumn c;
    c.twoTap = sx1 > sx0;
    c.xoff   = sx0 * 3;
    c.fx     = fx;
    return c;
}

// Terms that depend on the output row: byte offsets (within the image) of the lane's first tap in the
// upper and lower source row, and the lower row's weight.
struct FusedRow
{
    int64_t off0, off1;
    float   fy;
};

__device__ __forceinline__ FusedRow RowTerms(const FusedArgs &a, const SrcImage &s, int dy, int xoff)
{
    float fy  = (dy + a.cropY + 0.5f) * s.scaleY - 0.5f;
    int   sy0 = (int)floorf(fy);
    int   sy1 = min(sy0 + 1, s.h - 1);
    fy -= sy0;
    sy0 = max(0, sy0);
    FusedRow r;
    r.off0 = (int64_t)sy0 * s.rowStride + xoff;
    r.off1 = (int64_t)sy1 * s.rowStride + xoff;
    r.fy   = fy;
    return r;
}

// Last byte offset at which an 8-byte load still ends inside the image.
__device__ __forceinline__ int64_t LastTapLoad(const SrcImage &s)
{
    return (int64_t)(s.h - 1) * s.rowStride + (int64_t)s.w * 3 - 8;
}

// The two horizontal taps of a source row are 6 contiguous bytes: ONE unaligned 8-byte load per row.
// The load may extend up to 5 bytes past the taps; inside the image that is harmless, at the very end
// of the image buffer the load is moved back so that it ends with the buffer and the value is
// shifted into place (no divergent branch). Needs an image of >= 8 bytes. Bytes 0..2 of a0 / b0:
// first tap of the upper / lower row; a1 / b1: second tap.
__device__ __forceinline__ void LoadTapPairs(const SrcImage &s, const FusedRow &row, int64_t lastLoad, bool twoTap,
                                             uint32_t &a0, uint32_t &a1, uint32_t &b0, uint32_t &b1)
{
    const int      back0 = (int)max((int64_t)0, row.off0 - lastLoad);
    const int      back1 = (int)max((int64_t)0, row.off1 - lastLoad);
    const uint64_t q0    = LoadU64Unaligned(s.base + row.off0 - back0) >> (8 * back0);
    const uint64_t q1    = LoadU64Unaligned(s.base + row.off1 - back1) >> (8 * back1);
    a0                   = (uint32_t)q0;
    b0                   = (uint32_t)q1;
    a1                   = twoTap ? __builtin_amdgcn_alignbyte((uint32_t)(q0 >> 32), a0, 3) : a0;
    b1                   = twoTap ? __builtin_amdgcn_alignbyte((uint32_t)(q1 >> 32), b0, 3) : b0;
}

// A streaming store that is also written through the L2 (sc0 sc1 nt): the planes of an f32 NCHW output
// are written once, in 256-byte runs per wave, and nothing of them is left dirty in the XCD's L2 for
// the end-of-kernel write-back (batch-64 1080p -> 224x224: 22.56 -> 22.26 us against plain streaming
// stores). The compiler offers no spelling for this cache policy, hence the instruction itself.
__device__ __forceinline__ void StoreStreamThrough(float v, float *p)
{
    asm volatile("global_store_dword %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(v) : "memory");
}

__device__ __forceinline__ void StoreStreamThrough(uint8_t v, uint8_t *p)
{
    __builtin_nontemporal_store(v, p);
}


} // namespace cvamd

#endif // CVCUDA_AMD_FUSEDTILES_HPP
