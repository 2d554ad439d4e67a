// Packed launch grid for batches of differently sized images.
//
// Instead of launching a (maxWidth, maxHeight, N) grid in which blocks beyond their image's size
// exit immediately, the host walks the batch's host-side descriptor list, counts the tiles each
// image needs and passes the running totals to the kernel BY VALUE in the kernel-argument segment.
// Block b finds its image by a binary search over those totals (uniform per block, so it runs on
// the scalar unit) and derives its tile coordinates. No device round trip, no host sync, no
// operator-owned scratch; batches larger than kMaxTileImages are processed in several launches.
#ifndef CVCUDA_AMD_VARSHAPETILES_HPP
#define CVCUDA_AMD_VARSHAPETILES_HPP

#include <nvcv/ImageData.h>

#include <hip/hip_runtime.h>

#include <cstdint>

namespace cvamd {

constexpr int kMaxTileImages = 384;

struct VarTiles
{
    int32_t firstImage;                     // index of entry 0 in the batch
    int32_t numImages;                      // entries used
    int32_t tileStart[kMaxTileImages + 1];  // tileStart[i] = tiles of images [0, i)
    int32_t tilesX[kMaxTileImages];         // tiles per row of image i
};

struct TileCoord
{
    int image; // index into the batch
    int tx, ty;
};

__device__ __forceinline__ TileCoord LocateTile(const VarTiles &t, int tile)
{
    int lo = 0, hi = t.numImages; // invariant: tileStart[lo] <= tile < tileStart[hi]
    while (hi - lo > 1)
    {
        int mid = (lo + hi) >> 1;
        if (t.tileStart[mid] <= tile)
        {
            lo = mid;
        }
        else
        {
            hi = mid;
        }
    }
    int       local = tile - t.tileStart[lo];
    int       tx    = local % t.tilesX[lo];
    TileCoord c     = {t.firstImage + lo, tx, local / t.tilesX[lo]};
    return c;
}

// Fills `out` for images [first, first+count) of `list` (host descriptors; plane 0 gives the size,
// `heightNum/heightDen` rescales it for formats whose plane holds more rows than the image, e.g.
// 4:2:0 data stored as one plane of H*3/2 rows). Returns the total number of tiles.
inline int BuildVarTiles(VarTiles &out, const NVCVImageBufferStrided *list, int first, int count, int tileW, int tileH,
                         int heightNum = 1, int heightDen = 1)
{
    out.firstImage = first;
    out.numImages  = count;
    int total      = 0;
    for (int i = 0; i < count; ++i)
    {
        const NVCVImagePlaneStrided &pl = list[first + i].planes[0];
        int                          h  = pl.height * heightNum / heightDen;
        int                          nx = (pl.width + tileW - 1) / tileW;
        int                          ny = (h + tileH - 1) / tileH;
        out.tileStart[i]                = total;
        out.tilesX[i]                   = nx > 0 ? nx : 1;
        total += nx * ny;
    }
    out.tileStart[count] = total;
    return total;
}

} // namespace cvamd

#endif // CVCUDA_AMD_VARSHAPETILES_HPP
