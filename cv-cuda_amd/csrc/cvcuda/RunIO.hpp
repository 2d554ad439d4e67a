// Streaming operators (element-wise maps, channel swizzles, layout changes, mirroring) move a run of
// 4 consecutive pixels per lane: with 1-3 byte pixels a lane that moves one pixel issues one memory
// instruction per channel and the kernel is bound by the number of memory instructions at a quarter
// to a third of the HBM rate. A run is read with one vector load and written as whole dwords with
// streaming stores; neighbouring lanes cover neighbouring runs, so a wave touches one dense span.
#ifndef CVCUDA_AMD_RUNIO_HPP
#define CVCUDA_AMD_RUNIO_HPP

#include "DeviceUtils.hpp"
#include "LaneExchange.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>

namespace cvamd {

constexpr int kRunPixels = 4;               // pixels per lane ...
constexpr int kRunTileW  = 64 * kRunPixels; // ... columns per wave
constexpr int kRunTileH  = 4;               // rows per 256-thread block (one per wave)

// Pixels of 4-byte elements on both sides are whole dwords already: one pixel per lane keeps a
// wave's accesses dense (4-pixel runs of 12-16 byte pixels would stride each load by 48-64 bytes).
template<class TS, class TD>
constexpr int kRunPixelsFor = (sizeof(TS) >= 4 && sizeof(TD) >= 4) ? 1 : kRunPixels;

template<class T, int N>
using Run = Packed<T, N>;

// N dwords starting at p, which need not be dword aligned. Bytes that are taken apart with shifts afterwards
// are read through this: as a run of bytes the compiler may split such a load into 1- and 2-byte pieces (the 16
// source bytes of a 4:2:2 group came in as eight loads, and the kernel ran at 0.57 instead of 0.71 of the memory
// rate).
template<int N>
__device__ __forceinline__ void LoadDwords(const uint8_t *p, uint32_t (&w)[N])
{
    struct __attribute__((packed, aligned(1))) Words
    {
        uint32_t v[N];
    };
    const Words r = *reinterpret_cast<const Words *>(p);
#pragma unroll
    for (int i = 0; i < N; ++i)
    {
        w[i] = r.v[i];
        // every bit counts as used: where a caller drops some bytes (the alpha of 4-byte pixels), the load would
        // otherwise be narrowed to the bytes it keeps, one small load each
        asm("" : "+v"(w[i]));
    }
}

// N elements starting at p (aligned to one element). Runs of 1- and 2-byte elements that fill whole dwords
// come in as dwords (see LoadDwords).
template<class T, int N>
__device__ __forceinline__ void LoadRun(const uint8_t *p, T (&v)[N])
{
    if constexpr (sizeof(T) < 4 && (N * sizeof(T)) % 4 == 0)
    {
        uint32_t w[N * sizeof(T) / 4];
        LoadDwords<(int)(N * sizeof(T) / 4)>(p, w);
        __builtin_memcpy(v, w, sizeof(w));
    }
    else
    {
        const Run<T, N> r = *reinterpret_cast<const Run<T, N> *>(p);
#pragma unroll
        for (int i = 0; i < N; ++i)
        {
            v[i] = r.v[i];
        }
    }
}

// N elements to p as whole dwords (N * sizeof(T) is a multiple of 4; p need not be dword aligned),
// streaming: the data is not read back by the kernel.
template<class T, int N>
__device__ __forceinline__ void StoreRunNT(uint8_t *p, const T (&v)[N])
{
    static_assert((N * sizeof(T)) % 4 == 0, "runs are whole dwords");
    constexpr int D = N * sizeof(T) / 4;
    uint32_t      w[D];
    __builtin_memcpy(w, v, sizeof(w));
    StoreDwordsNT<D>(p, w);
}

// A wave whose lanes 0 .. lanes-1 hold consecutive RB-byte pieces of one output row (RB = 24 or 32, more
// than one store instruction per lane) writes the row through `stage` (64 * RB bytes of LDS private to
// the wave, 16-byte aligned): stored as they are, every 32-byte sector would be completed by two store
// instructions, and with streaming stores part of those sectors goes to memory twice (7.6 % more bytes
// written, a quarter more time on NV12 -> RGB when the input comes from memory as well). Handed round
// as 16-byte chunks (chunk c to lane c % lanes), every instruction writes one dense span. All of the
// wave's lanes that take part must call it together; rowOut is where lane 0's piece goes.
template<int RB>
__device__ __forceinline__ void StoreRowPiecesNT(uint8_t *stage, uint8_t *rowOut, const uint8_t (&piece)[RB], int lane,
                                                 int lanes)
{
    static_assert(RB % 8 == 0 && RB > 16, "pieces of whole 8-byte halves, longer than one store");
    const int chunks = lanes * RB / 16;
    __builtin_memcpy(stage + lane * RB, piece, RB);
    WaveExchangeFence();
#pragma unroll
    for (int j = 0; j < (RB + 15) / 16; ++j)
    {
        const int c = j * lanes + lane;
        if (c < chunks)
        {
            uint32_t w[4];
            __builtin_memcpy(w, stage + c * 16, 16);
            StoreDwordsNT<4>(rowOut + c * 16, w);
        }
    }
    if constexpr (RB % 16 != 0)
    {
        if (lane == 0 && (lanes & 1)) // an odd number of pieces ends with half a chunk
        {
            uint32_t w[2];
            __builtin_memcpy(w, stage + chunks * 16, 8);
            StoreDwordsNT<2>(rowOut + chunks * 16, w);
        }
    }
    WaveExchangeFence(); // the next row may overwrite the staging area
}

// N elements per lane as one piece of an output row: lanes 0 .. lanes-1 of the wave hold consecutive
// pieces, lane 0's at row0. Pieces of up to 16 bytes are one dense store instruction already; longer
// ones go through StoreRowPiecesNT (blocks of 4 waves; the staging area is this function's own).
template<class T, int N>
__device__ __forceinline__ void StoreRowRunNT(uint8_t *row0, const T (&v)[N], int lane, int lanes)
{
    constexpr int RB = N * (int)sizeof(T);
    if constexpr (RB > 16 && RB % 8 == 0)
    {
        __shared__ __attribute__((aligned(16))) uint8_t stage[4][64 * RB];
        uint8_t                                         piece[RB];
        __builtin_memcpy(piece, v, RB);
        StoreRowPiecesNT<RB>(stage[threadIdx.x >> 6], row0, piece, lane, lanes);
    }
    else
    {
        StoreRunNT<T, N>(row0 + (int64_t)lane * RB, v);
    }
}

// Rows a wave of an image-batch run kernel works through. The tile search and the descriptor loads are a
// dependent chain of memory round trips before the first pixel load, a quarter of a one-row wave's life
// (Normalize, 32 x 1080p u8x3: 94 -> 71 us with 4 rows). Outputs that go through the row-regrouped stores
// keep 1 (Normalize u8x3 -> f32x3: 171 us with 1 row, 190 us with 4).
template<int PIECE_BYTES>
constexpr int kVarShapeRows = PIECE_BYTES > 16 ? 1 : 4;

} // namespace cvamd

#endif // CVCUDA_AMD_RUNIO_HPP
