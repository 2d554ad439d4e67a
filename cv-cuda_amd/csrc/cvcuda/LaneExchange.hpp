// Exchange of results between neighbouring lanes so that every lane ends up with 4 consecutive
// pixels of one row, which it can store as whole dwords.
#ifndef CVCUDA_AMD_LANEEXCHANGE_HPP
#define CVCUDA_AMD_LANEEXCHANGE_HPP

#include <hip/hip_runtime.h>

#include <cstdint>

namespace cvamd {

// Within every group of 4 adjacent lanes: r[k] of lane i <-> r[i] of lane k (i = lane & 3), as two
// butterfly stages of cross-lane moves inside the group (no LDS).
__device__ __forceinline__ uint32_t FromLaneXor1(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1 /* quad_perm 1,0,3,2 */, 0xF, 0xF, false);
}

__device__ __forceinline__ uint32_t FromLaneXor2(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E /* quad_perm 2,3,0,1 */, 0xF, 0xF, false);
}

__device__ __forceinline__ void QuadTranspose(uint32_t (&r)[4], int i)
{
    const bool odd = (i & 1) != 0, upper = (i & 2) != 0;
#pragma unroll
    for (int b = 0; b < 4; b += 2) // 2x2 blocks (r0,r1) and (r2,r3) between lanes i and i^1
    {
        const uint32_t got = FromLaneXor1(odd ? r[b] : r[b + 1]);
        r[b]               = odd ? got : r[b];
        r[b + 1]           = odd ? r[b + 1] : got;
    }
#pragma unroll
    for (int b = 0; b < 2; ++b) // (r0,r2) and (r1,r3) between lanes i and i^2
    {
        const uint32_t got = FromLaneXor2(upper ? r[b] : r[b + 2]);
        r[b]               = upper ? got : r[b];
        r[b + 2]           = upper ? r[b + 2] : got;
    }
}

// 4 pixels of PB bytes, each held zero-extended in ceil(PB/4) dwords (q[d][k] = dword d of pixel k),
// packed back to back into PB dwords.
template<int PB>
__device__ __forceinline__ void PackQuad(const uint32_t (&q)[(PB + 3) / 4][4], uint32_t (&w)[PB])
{
    if constexpr (PB % 4 == 0)
    {
#pragma unroll
        for (int k = 0; k < 4; ++k)
        {
#pragma unroll
            for (int d = 0; d < PB / 4; ++d)
            {
                w[k * (PB / 4) + d] = q[d][k];
            }
        }
    }
    else if constexpr (PB == 1)
    {
        w[0] = q[0][0] | (q[0][1] << 8) | (q[0][2] << 16) | (q[0][3] << 24);
    }
    else if constexpr (PB == 2)
    {
        w[0] = q[0][0] | (q[0][1] << 16);
        w[1] = q[0][2] | (q[0][3] << 16);
    }
    else if constexpr (PB == 3)
    {
        w[0] = q[0][0] | (q[0][1] << 24);
        w[1] = (q[0][1] >> 8) | (q[0][2] << 16);
        w[2] = (q[0][2] >> 16) | (q[0][3] << 8);
    }
    else
    {
        static_assert(PB == 6, "pixel sizes: 1, 2, 3, 4, 6, 8, 12, 16 bytes");
        w[0] = q[0][0];
        w[1] = q[1][0] | (q[0][1] << 16);
        w[2] = (q[0][1] >> 16) | (q[1][1] << 16);
        w[3] = q[0][2];
        w[4] = q[1][2] | (q[0][3] << 16);
        w[5] = (q[0][3] >> 16) | (q[1][3] << 16);
    }
}

// Orders a wave's LDS writes before its later LDS reads (and the reverse) where lanes of the same
// wave exchange data: LDS instructions of one wave execute in order, so only the compiler has to
// be kept from moving them.
__device__ __forceinline__ void WaveExchangeFence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

} // namespace cvamd

#endif // CVCUDA_AMD_LANEEXCHANGE_HPP
