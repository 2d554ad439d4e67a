// Device-side numeric helpers shared by the kernels (gfx950, wave64).
#ifndef CVCUDA_AMD_DEVICEUTILS_HPP
#define CVCUDA_AMD_DEVICEUTILS_HPP

#include <hip/hip_runtime.h>
#include <nvcv/BorderType.h>

#include <cstdint>
#include <limits>
#include <type_traits>

namespace cvamd {

// N interleaved elements of type T, naturally aligned to one element only: the compiler may merge the
// accesses into wider instructions (unaligned vector access is legal on gfx950). Pixels, runs of pixels
// and groups of adjacent taps are all moved through this type.
template<class T, int N>
struct __attribute__((packed, aligned(sizeof(T)))) Packed
{
    using Elem              = T;
    static constexpr int kC = N;
    T v[N];
};

// float -> T with round-half-to-even and saturation; NaN -> 0 for integer targets
// (semantics of the reference's SaturateCast, cuda_tools/detail/SaturateCastImpl.hpp:41-50, 125).
template<class T>
__device__ __forceinline__ T SaturateCast(float v)
{
    if constexpr (std::is_same_v<T, float>)
    {
        return v;
    }
    else if constexpr (std::is_same_v<T, uint8_t>)
    {
        // one instruction: round half to even, saturate to [0, 255], NaN -> 0
        return (uint8_t)__builtin_amdgcn_cvt_pk_u8_f32(v, 0, 0);
    }
    else if constexpr (std::is_same_v<T, int8_t>)
    {
        float r = rintf(v);
        r       = fminf(fmaxf(r, -128.f), 127.f);
        return (int8_t)(int)(v != v ? 0.f : r);
    }
    else if constexpr (std::is_same_v<T, uint16_t>)
    {
        float r = rintf(v);
        r       = fminf(fmaxf(r, 0.f), 65535.f);
        return (uint16_t)(int)r;
    }
    else if constexpr (std::is_same_v<T, int16_t>)
    {
        float r = rintf(v);
        r       = fminf(fmaxf(r, -32768.f), 32767.f);
        return (int16_t)(int)(v != v ? 0.f : r);
    }
    else if constexpr (std::is_same_v<T, uint32_t>)
    {
        const float r = rintf(v);
        if (!(r > 0.f)) // also NaN
        {
            return 0u;
        }
        return r >= 4294967296.f ? 0xFFFFFFFFu : (uint32_t)r;
    }
    else if constexpr (std::is_same_v<T, int32_t>)
    {
        if (v != v)
        {
            return 0;
        }
        float r = rintf(v);
        if (r >= 2147483648.f)
        {
            return 2147483647;
        }
        if (r <= -2147483648.f)
        {
            return (int32_t)(-2147483647 - 1);
        }
        return (int32_t)r;
    }
    else
    {
        return (T)v;
    }
}

__device__ __forceinline__ uint8_t SaturateU8(int v)
{
    return (uint8_t)min(max(v, 0), 255);
}

// A pointer read from memory (an image descriptor's base address) is generic to the compiler, and
// every access through it becomes a flat instruction that also waits on the LDS counter. Image data
// always lives in global memory: saying so turns those accesses into global loads and stores.
template<class T>
__device__ __forceinline__ T *AsGlobal(T *p)
{
    // through an integer: a plain pointer cast to the global address space and back is folded away
    return (T *)(__attribute__((address_space(1))) T *)reinterpret_cast<uintptr_t>(p);
}

// Loads of 4 / 8 bytes from an address of arbitrary alignment. gfx950 global memory instructions
// accept unaligned addresses, so these compile to a single global_load_dword / _dwordx2.
struct __attribute__((packed, aligned(1))) UnalignedU32
{
    uint32_t v;
};

struct __attribute__((packed, aligned(1))) UnalignedU64
{
    uint64_t v;
};

__device__ __forceinline__ uint32_t LoadU32Unaligned(const uint8_t *p)
{
    return reinterpret_cast<const UnalignedU32 *>(p)->v;
}

__device__ __forceinline__ uint64_t LoadU64Unaligned(const uint8_t *p)
{
    return reinterpret_cast<const UnalignedU64 *>(p)->v;
}

// N dwords to an address of arbitrary alignment, as streaming stores (for output that the kernel does
// not read back).
template<int N>
__device__ __forceinline__ void StoreDwordsNT(uint8_t *p, const uint32_t (&w)[N])
{
    if constexpr (N == 4)
    {
        // as one 16-byte value: left to merge four dword stores the compiler sometimes settles for 12 + 4 or
        // 4 + 8 + 4 bytes, i.e. two or three partial writes of every 16 bytes
        typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
        typedef U32x4    UnalignedU32x4 __attribute__((aligned(1)));
        const U32x4      v = {w[0], w[1], w[2], w[3]};
        __builtin_nontemporal_store(v, reinterpret_cast<UnalignedU32x4 *>(p));
        return;
    }
    UnalignedU32 *o = reinterpret_cast<UnalignedU32 *>(p);
#pragma unroll
    for (int i = 0; i < N; ++i)
    {
        __builtin_nontemporal_store(w[i], &o[i].v);
    }
}

// 8 bytes starting at the arbitrary byte address base + off, fetched as 3 ALIGNED dwords and funnel-
// shifted into place. The texture path serves a misaligned multi-dword load at a fraction of the
// rate of an aligned one (measured on a gather of u8x3 pixel pairs: 31 vs 22 cycles per wave-load),
// which costs more than the two extra shifts. Reads the aligned window [p & ~3, (p & ~3) + 12) for
// p = base + off: up to 3 bytes before p (same dword as p, so never another page) and up to 6 bytes
// after the data; the caller keeps that tail inside its allocation. base must be uniform over the
// wave: its misalignment is folded into the 32-bit offset, so the per-lane address arithmetic is one
// mask (the load takes the aligned base from scalar registers plus a 32-bit lane offset) instead of
// 64-bit adds per lane.
__device__ __forceinline__ uint64_t LoadU64Window(const uint8_t *base, uint32_t off)
{
    struct alignas(4) W3
    {
        uint32_t d[3];
    };
    const uint32_t mis = (uint32_t)reinterpret_cast<uintptr_t>(base) & 3u;
    const uint32_t o   = off + mis;
    const W3       w   = *reinterpret_cast<const W3 *>((base - mis) + (o & ~3u));
    const uint32_t lo  = __builtin_amdgcn_alignbyte(w.d[1], w.d[0], o); // shifts by the bytes in bits 1:0
    const uint32_t hi  = __builtin_amdgcn_alignbyte(w.d[2], w.d[1], o);
    return ((uint64_t)hi << 32) | lo;
}

// 4 bytes starting at the arbitrary byte address base + off, the same way: 2 aligned dwords and one
// funnel shift. Reads up to 3 bytes before and up to 4 bytes after the data.
__device__ __forceinline__ uint32_t LoadU32Window(const uint8_t *base, uint32_t off)
{
    struct alignas(4) W2
    {
        uint32_t d[2];
    };
    const uint32_t mis = (uint32_t)reinterpret_cast<uintptr_t>(base) & 3u;
    const uint32_t o   = off + mis;
    const W2       w   = *reinterpret_cast<const W2 *>((base - mis) + (o & ~3u));
    return __builtin_amdgcn_alignbyte(w.d[1], w.d[0], o);
}

// The constant a caller gives for pixels outside the image, as an element of type T: truncated toward
// zero and saturated to T's range (floats pass through).
template<class T>
__device__ __forceinline__ T BorderValueAs(float v)
{
    if constexpr (std::is_same_v<T, float>)
    {
        return v;
    }
    else
    {
        const float lo = (float)std::numeric_limits<T>::min(), hi = (float)std::numeric_limits<T>::max();
        return (T)(long long)fminf(fmaxf(truncf(v), lo), hi);
    }
}

// Coordinate c outside [0, s) -> the coordinate inside that the border mode stands for (every mode
// but NVCV_BORDER_CONSTANT); index maps of the reference's border wrappers
// (cuda_tools/BorderWrap.hpp:62-121, BorderVarShapeWrap.hpp:290-368).
__device__ __forceinline__ int BorderIndex(int border, int c, int s)
{
    switch (border)
    {
    case NVCV_BORDER_REPLICATE:
        return c < 0 ? 0 : (c >= s ? s - 1 : c);
    case NVCV_BORDER_WRAP:
        c = c % s;
        return c < 0 ? c + s : c;
    case NVCV_BORDER_REFLECT:
    {
        const int s2 = s * 2;
        c            = c % s2;
        if (c < 0)
        {
            c += s2;
        }
        return s - 1 - (abs(2 * c + 1 - s2) >> 1);
    }
    default: // REFLECT101
        if (s == 1)
        {
            return 0;
        }
        c = c % (2 * s - 2);
        if (c < 0)
        {
            c += 2 * s - 2;
        }
        return s - 1 - abs(s - 1 - c);
    }
}

// MI355X hands the workgroups of a launch to its 8 XCDs round-robin (hardware id % 8) and every
// XCD has an L2 of its own.
constexpr uint32_t kXcdCount = 8;

} // namespace cvamd

#endif // CVCUDA_AMD_DEVICEUTILS_HPP
