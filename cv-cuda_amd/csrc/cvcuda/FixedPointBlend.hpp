// Blends of 8-bit taps in fixed point, shared by the warp and resize kernels. Bilinear, 15 bits:
//
// The two fractions of a sample are cut to 15 bits (ax, ay in 0 .. 2^15), the four weights are integers
// that add up to exactly 2^15,
//     w11 = (ax * ay + 2^14) >> 15,  w01 = ax - w11,  w10 = ay - w11,  w00 = 2^15 - ax - ay + w11,
// the weighted sum of the four taps is exact in 24 bits and is rounded to nearest, ties to even, once.
// Each weight is within 2^-15 of the product the float32 expressions of the reference form, so the
// unrounded sum is within 4 * 255 * 2^-15 < 0.032 of theirs: results differ from the reference's goldens
// by at most 1 and agree wherever the fractions are multiples of 2^-7, because then nothing is rounded
// before the final rounding. What it buys: the taps stay bytes (two taps and two weights per
// v_dot2_u32_u16 instead of a conversion, a multiply and an add per tap and channel in float32).
#ifndef CVCUDA_AMD_FIXEDPOINTBLEND_HPP
#define CVCUDA_AMD_FIXEDPOINTBLEND_HPP

#include <hip/hip_runtime.h>

#include <cstdint>

namespace cvamd {

constexpr uint32_t kQ15 = 32768u;

// (w00 | w01 << 16) and (w10 | w11 << 16) from the two 15-bit fractions (each 0 .. 2^15).
__device__ __forceinline__ void WeightPairsQ15(uint32_t ax, uint32_t ay, uint32_t &top, uint32_t &bottom)
{
    const uint32_t w11 = (__umul24(ax, ay) + (kQ15 >> 1)) >> 15;
    bottom             = __umul24(w11, 65535u) + ay;          // (ay - w11) | w11 << 16
    top                = (__umul24(ax, 65535u) + kQ15) - bottom; // (2^15 - ax | ax << 16) - bottom: no borrow
}

// Weighted sum of one channel: tap pairs as (left | right << 16), result in units of 2^-15, rounded to
// nearest-even, saturated (never needed) and placed into byte `c` of q. The sum is accumulated on top
// of the bit pattern of 256.0f, whose unit in the last place is 2^-15: read as a float the register
// then holds 256 + sum / 2^15 exactly.
__device__ __forceinline__ uint32_t BlendQ15(uint32_t topTaps, uint32_t bottomTaps, uint32_t top, uint32_t bottom, int c,
                                             uint32_t q)
{
    typedef unsigned short U16x2 __attribute__((ext_vector_type(2)));
    U16x2 t0, t1, w0, w1;
    __builtin_memcpy(&t0, &topTaps, 4);
    __builtin_memcpy(&t1, &bottomTaps, 4);
    __builtin_memcpy(&w0, &top, 4);
    __builtin_memcpy(&w1, &bottom, 4);
    uint32_t acc = __builtin_amdgcn_udot2(t0, w0, 0x43800000u, false);
    acc          = __builtin_amdgcn_udot2(t1, w1, acc, false);
    return __builtin_amdgcn_cvt_pk_u8_f32(__uint_as_float(acc) - 256.f, c, q);
}

// A sum accumulated in plain integer arithmetic (one tap at a time), rounded the same way.
__device__ __forceinline__ uint8_t RoundQ15(uint32_t sum)
{
    return (uint8_t)((sum + (kQ15 / 2 - 1) + ((sum >> 15) & 1u)) >> 15);
}

// Bytes c (of lo) and c (of hi) as (lo byte | hi byte << 16): the two taps of channel c from two pixels
// held one per dword; selector 0x0c gives a zero byte.
__device__ __forceinline__ uint32_t ChannelPair(uint32_t lo, uint32_t hi, int c)
{
    return __builtin_amdgcn_perm(hi, lo, 0x0c000c00u | (uint32_t)c | ((uint32_t)(4 + c) << 16));
}

// One pixel of C channels from its four taps, each a dword with channel c in byte c; returns the same.
template<int C>
__device__ __forceinline__ uint32_t BilinearQ15(uint32_t p00, uint32_t p01, uint32_t p10, uint32_t p11, uint32_t ax,
                                                uint32_t ay)
{
    uint32_t top, bottom, q = 0;
    WeightPairsQ15(ax, ay, top, bottom);
#pragma unroll
    for (int c = 0; c < C; ++c)
    {
        q = BlendQ15(ChannelPair(p00, p01, c), ChannelPair(p10, p11, c), top, bottom, c, q);
    }
    return q;
}

// The same sum for one channel in plain integer arithmetic.
__device__ __forceinline__ uint8_t BilinearQ15Scalar(uint32_t t00, uint32_t t01, uint32_t t10, uint32_t t11, uint32_t ax,
                                                     uint32_t ay)
{
    const uint32_t w11 = (ax * ay + (kQ15 >> 1)) >> 15;
    return RoundQ15(t00 * (kQ15 - ax - ay + w11) + t01 * (ax - w11) + t10 * (ay - w11) + t11 * w11);
}

// ---- bicubic: the four taps of a row times weights in units of 2^-14 (signed), shared by the warp and resize kernels

// Horizontal bicubic weights, given times 2^14, as signed 16-bit integers: (w0 | w1 << 16), (w2 | w3 << 16).
// Adding 1.5 * 2^23 rounds a weight to the nearest integer, ties to even, and leaves it in the low bits of
// the sum's bit pattern (two's complement for negative values); w3 = 2^14 - w0 - w1 - w2 on those integers.
__device__ __forceinline__ void CubicWeightPairsQ14(const float (&w)[4], uint32_t &p01, uint32_t &p23)
{
    constexpr float    kMagic = 12582912.f;
    constexpr uint32_t kBits  = 0x4B400000u;
    const uint32_t     b0 = __float_as_uint(w[0] + kMagic);
    const uint32_t     b1 = __float_as_uint(w[1] + kMagic);
    const uint32_t     b2 = __float_as_uint(w[2] + kMagic);
    const uint32_t     w3 = (16384u + 3u * kBits) - (b0 + b1 + b2);
    p01                   = __builtin_amdgcn_perm(b1, b0, 0x05040100u);
    p23                   = __builtin_amdgcn_perm(w3, b2, 0x05040100u);
}

// The same four integers one by one (border path), also from weights times 2^14. NaN weights give 0.
__device__ __forceinline__ void CubicWeightsQ14(const float (&w)[4], int (&q)[4])
{
    q[0] = (int)rintf(w[0]);
    q[1] = (int)rintf(w[1]);
    q[2] = (int)rintf(w[2]);
    q[3] = 16384 - q[0] - q[1] - q[2];
}

// Bytes lo and hi of a row held in dwords r[] -> (byte lo | byte hi << 16), one byte permute.
template<int N>
__device__ __forceinline__ uint32_t BytePair(const uint32_t (&r)[N], int lo, int hi)
{
    const uint32_t sel = 0x0c000c00u | (uint32_t)(lo & 3) | ((uint32_t)(4 + (hi & 3)) << 16);
    return __builtin_amdgcn_perm(r[hi >> 2], r[lo >> 2], sel);
}

__device__ __forceinline__ int Dot2I16(uint32_t a, uint32_t b, int c)
{
    typedef short I16x2 __attribute__((ext_vector_type(2)));
    I16x2 x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    return __builtin_amdgcn_sdot2(x, y, c, false);
}

// a.lo * b.lo + a.hi * b.hi with nothing added: the three-operand form with the constant 0 (for a sum
// that starts here the compiler picks the accumulate-in-place form and spends a move on clearing it).
__device__ __forceinline__ int Dot2I16(uint32_t a, uint32_t b)
{
    int d;
    asm("v_dot2_i32_i16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
}

} // namespace cvamd

#endif // CVCUDA_AMD_FIXEDPOINTBLEND_HPP
