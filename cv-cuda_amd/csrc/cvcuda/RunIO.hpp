// Streaming operators (element-wise maps, channel swizzles, layout changes, mirroring) move a run of
// 4 consecutive pixels per lane: with 1-3 byte pixels a lane that moves one pixel issues one memory
// instruction per channel and the kernel is bound by the number of memory instructions at a quarter
// to a third of the HBM rate. A run is read with one vector load and written as whole dwords with
// streaming stores; neighbouring lanes cover neighbouring runs, so a wave touches one dense span.
#ifndef CVCUDA_AMD_RUNIO_HPP
#define CVCUDA_AMD_RUNIO_HPP

#include "DeviceUtils.hpp"

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

// N elements starting at p (aligned to one element).
template<class T, int N>
__device__ __forceinline__ void LoadRun(const uint8_t *p, T (&v)[N])
{
    const Run<T, N> r = *reinterpret_cast<const Run<T, N> *>(p);
#pragma unroll
    for (int i = 0; i < N; ++i)
    {
        v[i] = r.v[i];
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

} // namespace cvamd

#endif // CVCUDA_AMD_RUNIO_HPP
