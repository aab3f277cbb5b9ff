// Shared host/device helpers of libmiq (gfx950 only).
#ifndef MIQ_COMMON_H
#define MIQ_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/miq.h"

namespace miq
{
// ---- error plumbing --------------------------------------------------------------------------------------------
void set_error(const char* fmt, ...);

#define MIQ_CHECK_ARG(cond, ...)                                                                                       \
    do                                                                                                                 \
    {                                                                                                                  \
        if (!(cond))                                                                                                   \
        {                                                                                                              \
            ::miq::set_error(__VA_ARGS__);                                                                             \
            return MIQ_ERR_INVALID_ARG;                                                                                \
        }                                                                                                              \
    } while (0)

#define MIQ_CHECK_HIP(expr)                                                                                            \
    do                                                                                                                 \
    {                                                                                                                  \
        hipError_t e_ = (expr);                                                                                        \
        if (e_ != hipSuccess)                                                                                          \
        {                                                                                                              \
            ::miq::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__);               \
            return MIQ_ERR_HIP;                                                                                        \
        }                                                                                                              \
    } while (0)

#define MIQ_CHECK_LAUNCH() MIQ_CHECK_HIP(hipGetLastError())

inline bool aligned16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

constexpr int kBlock  = 256;   // 4 wavefronts of 64 lanes
constexpr int kUnroll = 2;     // 16-byte vectors in flight per lane (measured: 2 beats 4 and 8 for streaming)

// ---- unsigned division of a 31-bit value by a launch-invariant divisor --------------------------------------
// For n < 2^31 and 1 <= d < 2^31:  n / d == (n * magic) >> (31 + s)  with s = ceil(log2 d),
// magic = floor(2^(31+s) / d) + 1 < 2^32  (round-up method; exact because the dividend has at most 31 bits).
struct FastDiv
{
    uint32_t d;
    uint32_t magic;
    uint32_t shift;   // 31 + s - 32 when d > 1 (applied to the high word of the product)
};

inline FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.d = d;
    if (d <= 1)
    {
        f.magic = 0;
        f.shift = 0;
        return f;
    }
    uint32_t s = 0;
    while ((1ull << s) < d)
        ++s;
    unsigned __int128 num = ((unsigned __int128) 1) << (31 + s);
    f.magic              = (uint32_t) (num / d) + 1u;
    f.shift              = s - 1;
    return f;
}

__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv& f)
{
    return (f.d <= 1) ? n : (__umulhi(n, f.magic) >> f.shift);
}

// ---- bf16 storage <-> float (round to nearest even; NaN -> 0x7FC0 as torch's conversion does) -----------------
__device__ __forceinline__ float bf16_to_f32(uint32_t h)
{
    return __uint_as_float(h << 16);
}

__device__ __forceinline__ uint32_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return ((u & 0x7fffffffu) > 0x7f800000u) ? 0x7fc0u : r;
}

// two floats -> packed bf16 pair with the hardware's round-to-nearest-even conversion (v_cvt_pk_bf16_f32); NaN is
// canonicalised to 0x7FC0 as above
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi)
{
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2));
    if (lo != lo)
        w = (w & 0xffff0000u) | 0x7fc0u;
    if (hi != hi)
        w = (w & 0x0000ffffu) | 0x7fc00000u;
    return w;
}

// the same conversion for values known not to be NaN (nothing to canonicalise)
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_no_nan(float lo, float hi)
{
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2));
}

}   // namespace miq
#endif