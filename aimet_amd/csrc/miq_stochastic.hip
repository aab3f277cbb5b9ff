// Stochastic rounding for the v1 quantize / quantize-dequantize entry points:  q = floor(t + u),  u uniform in [0, 1),
// t = clamp(x, min, max) / delta - offset  (DlQuantization/src/trim_functions.cpp:141-166).
//
// The reference draws u from libc rand() on the CPU (trim_functions.cpp:56-59) and from a clock-seeded generator per
// element on the GPU (trim_functions.cuh:49-66): neither sequence can be reproduced by a parallel kernel, and neither
// is part of the interface.  Here u is a pure function of (seed, call number, element index), so a seeded run is
// repeatable and any element can be recomputed on its own:
//
//     key       = splitmix64(seed + 0x9E3779B97F4A7C15 * (call + 1));   k0 = low word, k1 = high word
//     r(i)      = mix32((uint32) i + k0) ^ k1 ^ (uint32)(i >> 32)
//     u(i)      = (r(i) >> 8) * 2^-24
//     mix32(x)  : x ^= x >> 16; x *= 0x7feb352d; x ^= x >> 15; x *= 0x846ca68b; x ^= x >> 16
//
// (one round of a low-bias integer hash over the element counter, keyed before and after: the integer multiplies run
// at a quarter of the float rate on this part and a second round would make the kernel compute-bound.)
// `seed` is set with miq_set_stochastic_seed (the counterpart of srand) and `call` counts the stochastic launches since
// then.  The sum t + u is formed as the reference forms it (float t widened to double, then floor).
#include <atomic>
#include <cmath>

#include "miq_common.h"
#include "miq_fastmath.h"
#include "miq_io.h"
#include "miq_stochastic.h"

namespace miq
{
namespace
{
std::atomic<uint64_t> g_seed{0};
std::atomic<uint64_t> g_calls{0};

uint64_t splitmix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ uint32_t mix32(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

struct StochArgs
{
    const float* mn;   // per-channel parameter vectors (null for per-tensor)
    const float* mx;
    const float* delta;
    const float* offset;
    float4 scalar;     // per-tensor (min, max, delta, offset)
    float scalar_rcp;  // correctly rounded 1 / delta when the exact fast division applies, else 0
    float shift;       // subtracted from the grid index when DEQUANT is false
    uint32_t num_channel;
    FastDiv fd;        // elements per channel
    uint32_t k0, k1;
};

// floor(t + u) with u = r24 * 2^-24.  For 0 <= t < 2^23 the double sum of the reference is exact (t >= 0.5) or cannot
// be rounded across an integer (t < 0.5), so the decision equals frac(t) >= 1 - u, every term of which float32 holds
// exactly; everything else takes the reference's double arithmetic.
__device__ __forceinline__ float stochastic_round(float t, uint32_t r24)
{
    if (t >= 0.0f && t < 8388608.0f)
    {
        const float f    = floorf(t);
        const float frac = t - f;
        const float thr  = (float) (16777216u - r24) * 0x1p-24f;
        return f + (frac >= thr ? 1.0f : 0.0f);
    }
    return (float) floor((double) t + (double) r24 * 0x1p-24);
}

struct Params
{
    float4 p;    // min, max, delta, offset
    float rcp;   // RN(1 / delta), or 0 when x / delta has to be an IEEE division
};

__host__ __device__ __forceinline__ float exact_rcp(const float4& p)
{
    const float bound = fmaxf(fabsf(p.x), fabsf(p.y));
    return (fastdiv_divisor_ok(p.z) && bound <= kFastDivMaxDividend) ? 1.0f / p.z : 0.0f;
}

template <bool DEQUANT>
__device__ __forceinline__ float stoch_elem(float x, const Params& c, float shift, uint32_t k0, uint32_t k1, uint64_t i)
{
    const float4& p = c.p;
    float t         = fmaxf(fminf(x, p.y), p.x);
    t               = (c.rcp != 0.0f) ? div_by_invariant(t, p.z, c.rcp) : t / p.z;
    t               = t - p.w;
    const uint32_t r = mix32((uint32_t) i + k0) ^ k1 ^ (uint32_t) (i >> 32);
    const float q    = stochastic_round(t, r >> 8);
    return DEQUANT ? p.z * (q + p.w) : q - shift;
}

__device__ __forceinline__ Params channel_params(const StochArgs& a, uint32_t ch)
{
    Params c;
    c.p   = make_float4(a.mn[ch], a.mx[ch], a.delta[ch], a.offset[ch]);
    c.rcp = exact_rcp(c.p);
    return c;
}

__device__ __forceinline__ Params tensor_params(const StochArgs& a)
{
    return Params{a.scalar, a.scalar_rcp};
}

// One 16-byte vector per lane and iteration, grid-stride.  Per-channel: n < 2^31 (checked by the launcher).
template <typename IO, bool PER_CHANNEL, bool DEQUANT>
__global__ __launch_bounds__(kBlock) void stoch_vec_kernel(const IO* __restrict__ x, IO* __restrict__ y, int64_t n,
                                                           StochArgs a)
{
    using T              = IOTraits<IO>;
    using Vec            = typename T::Vec;
    constexpr int VEC    = T::VEC;
    const int64_t nvec   = n / VEC;
    const int64_t stride = (int64_t) gridDim.x * kBlock;
    const Params pt      = tensor_params(a);
    for (int64_t v = (int64_t) blockIdx.x * kBlock + threadIdx.x; v < nvec; v += stride)
    {
        float fx[VEC], fy[VEC];
        T::unpack(stream_load(reinterpret_cast<const Vec*>(x) + v), fx);
        const uint64_t e0 = (uint64_t) v * VEC;
        if constexpr (PER_CHANNEL)
        {
            const uint32_t row = fastdiv((uint32_t) e0, a.fd);
            const uint32_t rem = (uint32_t) e0 - row * a.fd.d;
            uint32_t ch        = row;
            if (ch >= a.num_channel)   // only tensors with an outer dimension pay for the modulo
                ch %= a.num_channel;
            const Params p0    = channel_params(a, ch);
            if (rem + VEC <= a.fd.d)
            {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    fy[j] = stoch_elem<DEQUANT>(fx[j], p0, a.shift, a.k0, a.k1, e0 + j);
            }
            else
            {
                // the vector crosses channel boundaries (possibly several: rows may be shorter than a vector)
                uint32_t r = rem;
                Params p   = p0;
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                {
                    if (r == a.fd.d)
                    {
                        r  = 0;
                        ch = (ch + 1 == a.num_channel) ? 0 : ch + 1;
                        p  = channel_params(a, ch);
                    }
                    fy[j] = stoch_elem<DEQUANT>(fx[j], p, a.shift, a.k0, a.k1, e0 + j);
                    ++r;
                }
            }
        }
        else
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                fy[j] = stoch_elem<DEQUANT>(fx[j], pt, a.shift, a.k0, a.k1, e0 + j);
        }
        stream_store(reinterpret_cast<Vec*>(y) + v, T::pack(fy));
    }
    // tail (fewer than VEC elements): first lanes of the first block
    const int64_t tail = nvec * VEC;
    if (blockIdx.x == 0 && tail + threadIdx.x < n)
    {
        const int64_t e = tail + threadIdx.x;
        Params p        = pt;
        if constexpr (PER_CHANNEL)
            p = channel_params(a, (uint32_t) ((e / a.fd.d) % a.num_channel));
        T::store1(y + e, stoch_elem<DEQUANT>(T::load1(x + e), p, a.shift, a.k0, a.k1, (uint64_t) e));
    }
}

// Any alignment, any size.
template <typename IO, bool PER_CHANNEL, bool DEQUANT>
__global__ __launch_bounds__(kBlock) void stoch_scalar_kernel(const IO* __restrict__ x, IO* __restrict__ y, int64_t n,
                                                              StochArgs a, int64_t n_per_channel)
{
    using T = IOTraits<IO>;
    for (int64_t e = (int64_t) blockIdx.x * kBlock + threadIdx.x; e < n; e += (int64_t) gridDim.x * kBlock)
    {
        Params p = tensor_params(a);
        if constexpr (PER_CHANNEL)
            p = channel_params(a, (uint32_t) ((e / n_per_channel) % a.num_channel));
        T::store1(y + e, stoch_elem<DEQUANT>(T::load1(x + e), p, a.shift, a.k0, a.k1, (uint64_t) e));
    }
}

template <typename IO, bool PER_CHANNEL, bool DEQUANT>
int launch(const IO* x, IO* y, int64_t n, StochArgs a, int64_t n_per_channel, hipStream_t stream)
{
    if (n == 0)
        return MIQ_OK;
    const uint64_t call = g_calls.fetch_add(1);
    const uint64_t key  = splitmix64(g_seed.load() + 0x9E3779B97F4A7C15ull * (call + 1));
    a.k0                = (uint32_t) key;
    a.k1                = (uint32_t) (key >> 32);
    a.fd                = make_fastdiv(PER_CHANNEL && n_per_channel < (1ll << 31) ? (uint32_t) n_per_channel : 1u);
    constexpr int VEC   = IOTraits<IO>::VEC;
    const bool vec_ok   = aligned16(x) && aligned16(y) && (!PER_CHANNEL || (n < (1ll << 31) && n_per_channel < (1ll << 31)));
    if (vec_ok)
    {
        int64_t blocks = (n / VEC + kBlock - 1) / kBlock;
        blocks         = blocks < 1 ? 1 : (blocks > 8192 ? 8192 : blocks);
        hipLaunchKernelGGL((stoch_vec_kernel<IO, PER_CHANNEL, DEQUANT>), dim3((unsigned) blocks), dim3(kBlock), 0,
                           stream, x, y, n, a);
    }
    else
    {
        int64_t blocks = (n + kBlock - 1) / kBlock;
        blocks         = blocks > 65536 ? 65536 : blocks;
        hipLaunchKernelGGL((stoch_scalar_kernel<IO, PER_CHANNEL, DEQUANT>), dim3((unsigned) blocks), dim3(kBlock), 0,
                           stream, x, y, n, a, n_per_channel);
    }
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}
}   // namespace

template <typename IO>
int stochastic_qdq_per_tensor(const IO* in, IO* out, int64_t n, const miq_encoding& e, hipStream_t stream)
{
    StochArgs a{};
    a.scalar     = make_float4((float) e.min, (float) e.max, (float) e.delta, (float) e.offset);
    a.scalar_rcp = exact_rcp(a.scalar);
    return launch<IO, false, true>(in, out, n, a, 1, stream);
}

int stochastic_quantize_per_tensor(const float* in, float* out, int64_t n, const miq_encoding& e, float shift,
                                   hipStream_t stream)
{
    StochArgs a{};
    a.scalar     = make_float4((float) e.min, (float) e.max, (float) e.delta, (float) e.offset);
    a.scalar_rcp = exact_rcp(a.scalar);
    a.shift      = shift;
    return launch<float, false, false>(in, out, n, a, 1, stream);
}

template <typename IO>
int stochastic_qdq_per_channel(const IO* in, IO* out, int64_t num_channel, int64_t n, int64_t n_per_channel,
                               const float* mn, const float* mx, const float* delta, const float* offset,
                               hipStream_t stream)
{
    StochArgs a{};
    a.mn          = mn;
    a.mx          = mx;
    a.delta       = delta;
    a.offset      = offset;
    a.num_channel = (uint32_t) num_channel;
    return launch<IO, true, true>(in, out, n, a, n_per_channel, stream);
}

template int stochastic_qdq_per_tensor<float>(const float*, float*, int64_t, const miq_encoding&, hipStream_t);
template int stochastic_qdq_per_tensor<uint16_t>(const uint16_t*, uint16_t*, int64_t, const miq_encoding&,
                                                 hipStream_t);
template int stochastic_qdq_per_channel<float>(const float*, float*, int64_t, int64_t, int64_t, const float*,
                                               const float*, const float*, const float*, hipStream_t);
template int stochastic_qdq_per_channel<uint16_t>(const uint16_t*, uint16_t*, int64_t, int64_t, int64_t, const float*,
                                                  const float*, const float*, const float*, hipStream_t);
}   // namespace miq

extern "C" {

int miq_set_stochastic_seed(uint64_t seed)
{
    miq::g_seed.store(seed);
    miq::g_calls.store(0);
    return MIQ_OK;
}

int miq_get_stochastic_state(uint64_t* seed, uint64_t* calls)
{
    MIQ_CHECK_ARG(seed && calls, "null pointer");
    *seed  = miq::g_seed.load();
    *calls = miq::g_calls.load();
    return MIQ_OK;
}

}   // extern "C"
