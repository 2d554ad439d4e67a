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

#include <algorithm>
#include <cstdint>

namespace cvamd {

constexpr int kMaxTileImages = 384;
constexpr int kTileChunks    = 128; // entries of the chunk table

// One entry per image: tiles before it and tiles per row of it, side by side so that one 8-byte load
// fetches both.
struct TileSpan
{
    int32_t start;  // tiles of images [0, i)
    int32_t tilesX; // tiles per row of image i
};

struct VarTiles
{
    int32_t  firstImage;                   // index of entry 0 in the batch
    int32_t  numImages;                    // entries used
    int32_t  chunkShift;                   // a chunk is 2^chunkShift consecutive tiles
    int32_t  total;                        // tiles of the launch
    TileSpan span[kMaxTileImages + 1];     // span[numImages].start = total
    // per chunk c: the image that holds its first tile, and in the upper half the image that holds the first tile
    // of the next chunk (or the launch's last tile). Whole dwords: the scalar unit loads nothing narrower.
    uint32_t chunkImages[kTileChunks];
};

// kernels take a VarTiles and their own arguments by value: together they must fit the 4 KB argument segment
static_assert(sizeof(VarTiles) <= 3712, "VarTiles leaves too little of the kernel-argument segment");

struct TileCoord
{
    int image; // index into the batch
    int tx, ty;
};

// Block `tile` of the launch -> image and tile coordinates. The images that a chunk of tiles touches come
// from the chunk table (one load from the kernel-argument segment); with images of more than a chunk's
// tiles that leaves at most two candidates, so the search over the running totals that follows takes one
// step or none where a plain binary search over the batch takes log2(images) dependent loads in front of
// every wave's first pixel load.
__device__ __forceinline__ TileCoord LocateTile(const VarTiles &t, int tile)
{
    const uint32_t pair = t.chunkImages[tile >> t.chunkShift];
    int            lo = (int)(pair & 0xFFFFu), hi = (int)(pair >> 16) + 1; // invariant: span[lo].start <= tile < span[hi].start
    while (hi - lo > 1)
    {
        int mid = (lo + hi) >> 1;
        if (t.span[mid].start <= tile)
        {
            lo = mid;
        }
        else
        {
            hi = mid;
        }
    }
    const TileSpan sp    = t.span[lo];
    const int      local = tile - sp.start;
    const int      ty    = local / sp.tilesX;
    TileCoord      r     = {t.firstImage + lo, local - ty * sp.tilesX, ty};
    return r;
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
        out.span[i].start               = total;
        out.span[i].tilesX              = nx > 0 ? nx : 1;
        total += nx * ny;
    }
    out.span[count].start  = total;
    out.span[count].tilesX = 1;
    out.total              = total;
    // chunk table: the smallest power-of-two chunk that covers the launch with kTileChunks chunks
    out.chunkShift = 0;
    while (((int64_t)total + (1 << out.chunkShift) - 1) >> out.chunkShift > kTileChunks)
    {
        ++out.chunkShift;
    }
    const int chunks = (int)(((int64_t)total + (1 << out.chunkShift) - 1) >> out.chunkShift);
    int       image  = 0;
    uint32_t  startImage = 0;
    for (int c = 0; c <= chunks; ++c)
    {
        // the image that holds tile c << shift (images without tiles are stepped over; past the launch's end:
        // its last tile)
        const int64_t tile = std::min<int64_t>((int64_t)c << out.chunkShift, total > 0 ? total - 1 : 0);
        while (image + 1 < count && out.span[image + 1].start <= tile)
        {
            ++image;
        }
        if (c > 0)
        {
            out.chunkImages[c - 1] = startImage | ((uint32_t)image << 16);
        }
        startImage = (uint32_t)image;
    }
    return total;
}

} // namespace cvamd

#endif // CVCUDA_AMD_VARSHAPETILES_HPP
