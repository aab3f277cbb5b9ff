// Quantize-dequantize (fake-quant) forward and straight-through backward kernels for gfx950.
//
// One streaming kernel template serves every variant.  Each lane moves 16-byte vectors (4 x f32 or 8 x bf16),
// kUnroll of them in flight, so a 256-lane workgroup covers a contiguous tile of 4096 (f32) or 8192 (bf16)
// elements.  Per-tensor parameters travel as kernel arguments (scalar registers).  Per-channel parameters are
// staged once per workgroup into an LDS window that holds just the channel rows the tile touches
// (tile / elements-per-channel + 2 rows), and the row of a vector is found with one multiply-high (the divisor is
// launch-invariant), so no per-element integer division or dependent global loads remain.
//
// Arithmetic is the reference's, operation for operation, in float32 with IEEE division and no contraction:
//   v1  (DlQuantization): t = fmax(fmin(x, max), min); q = roundf(t / delta - offset); y = delta * (q + offset)
//       ModelOptimizations/DlQuantization/src/trim_functions.cpp:141-182, 698-709
//   v2  (aimet_torch.v2): r = rint(x / scale) - offset; y = (clamp(r, qmin, qmax) + offset) * scale
//       TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/backends/torch_builtins.py:303-344
#include <hip/hip_fp16.h>

#include "miq_common.h"
#include "miq_encoding_math.h"
#include "miq_fastmath.h"
#include "miq_io.h"
#include "miq_stochastic.h"

#include <cmath>

namespace miq
{
namespace
{
// -------------------------------------------------------------------------------------------------- the operations
// Channel parameter sources (device pointers) and per-tensor values; which fields an op reads is up to the op.
struct ParamSrc
{
    const float* a;   // v1: min      v2: scale
    const float* b;   // v1: max      v2: offset
    const float* c;   // v1: delta
    const float* d;   // v1: offset
    const float* e;   // v1 with a saved mask: the stored encoding's min (the straight-through bounds)
    const float* f;   // v1 with a saved mask: the stored encoding's max
    float2 raw;       // per-tensor: the same two values
    float4 scalar;    // per-tensor: the same four values
    float scalar_rcp; // per-tensor: RN(1/delta), or 0 when delta is outside the fast-division contract
    int qmin, qmax;   // v2 grid
    float shift;      // v1 quantize-only: 2^(bw-1) or 0
    int ishift;       // the same as an integer, for byte codes
};

// v1 channel parameters.  rcp = RN(1/delta) when delta lies inside the contract of div_by_invariant, else 0, in
// which case the quotient is formed with the ordinary division (both give the same bits; see miq_fastmath.h).
struct V1P
{
    float mn, mx, delta, offset, rcp;
};

// RN(1/d) if every quotient this channel can form stays inside the contract of div_by_invariant, else 0
__device__ __forceinline__ float safe_rcp(float d, float bound)
{
    return (fastdiv_divisor_ok(d) && bound <= kFastDivMaxDividend) ? 1.0f / d : 0.0f;
}

struct OpV1
{
    using P = V1P;
    __device__ static P load(const ParamSrc& s, uint32_t ch)
    {
        const float mn = s.a[ch], mx = s.b[ch], d = s.c[ch];
        // the dividend is clamped to [mn, mx] first, so max(|mn|, |mx|) bounds it
        return P{mn, mx, d, s.d[ch], safe_rcp(d, fmaxf(fabsf(mn), fabsf(mx)))};
    }
    // one decision per vector, not per element: whether the fast exact quotient may be used
    __device__ static bool fast_ok(const P& p, const float*, int)
    {
        return p.rcp != 0.0f;
    }
    template <bool FAST>
    __device__ static float quant(const P& p, float x)
    {
        float t = fmaxf(fminf(x, p.mx), p.mn);
        t       = FAST ? div_by_invariant(t, p.delta, p.rcp) : t / p.delta;
        t       = t - p.offset;
        return round_half_away(t);   // == roundf(t), three operations instead of six
    }
};

// y = QDQ(x); optional byte codes
struct OpV1Qdq : OpV1
{
    static constexpr int NIN = 1;
    using Code               = uint8_t;
    template <bool FAST>
    __device__ static float apply(const ParamSrc& s, const P& p, float x, float, int& code)
    {
        float q = quant<FAST>(p, x);
        code    = (int) q - s.ishift;
        return p.delta * (q + p.offset);
    }
};

// y = QDQ(x) and, as the "code", whether x lies inside the stored encoding's [min, max]: the factor the straight-through
// backward multiplies the gradient with (TORCH/v1/quantsim_straight_through_grad.py:100-118).  The kernel packs these
// flags into the saved mask (one bit per element) instead of integer codes.
struct V1PM
{
    float mn, mx, delta, offset, rcp, raw_min, raw_max;
};
struct OpV1QdqMask
{
    static constexpr bool kMask = true;
    using P                  = V1PM;
    static constexpr int NIN = 1;
    using Code               = uint8_t;
    __device__ static P load(const ParamSrc& s, uint32_t ch)
    {
        const V1P q = OpV1::load(s, ch);
        return P{q.mn, q.mx, q.delta, q.offset, q.rcp, s.e[ch], s.f[ch]};
    }
    __device__ static bool fast_ok(const P& p, const float*, int)
    {
        return p.rcp != 0.0f;
    }
    template <bool FAST>
    __device__ static float apply(const ParamSrc&, const P& p, float x, float, int& code)
    {
        const float q = OpV1::quant<FAST>(V1P{p.mn, p.mx, p.delta, p.offset, p.rcp}, x);
        code          = (p.raw_min <= x) && (x <= p.raw_max);
        return p.delta * (q + p.offset);
    }
};

// y = grid index - shift (float valued), reference quantizeToFxp
struct OpV1Quantize : OpV1
{
    static constexpr int NIN = 1;
    using Code               = uint8_t;
    template <bool FAST>
    __device__ static float apply(const ParamSrc& s, const P& p, float x, float, int& code)
    {
        float q = quant<FAST>(p, x);
        code    = 0;
        return q - s.shift;
    }
};

// y = float(half(x)): the simulation of a float16 tensor (TORCH/v1/tensor_quantizer.py:1104-1107, tensor.half().float()),
// round to nearest even, overflow to infinity, as the conversion instruction does
struct OpFp16
{
    using P                  = int;   // no parameters
    static constexpr int NIN = 1;
    using Code               = uint8_t;
    __device__ static P load(const ParamSrc&, uint32_t)
    {
        return 0;
    }
    __device__ static bool fast_ok(const P&, const float*, int)
    {
        return true;
    }
    template <bool FAST>
    __device__ static float apply(const ParamSrc&, const P&, float x, float, int& code)
    {
        code = 0;
        return __half2float(__float2half_rn(x));
    }
};

// y = float(bfloat16(x)): the v2 float quantizer's bfloat16 case (TORCH/v2/quantization/float/quantizer.py:309-314,
// input.to(torch.bfloat16).to(input.dtype)), round to nearest even
struct OpBf16
{
    using P                  = int;   // no parameters
    static constexpr int NIN = 1;
    using Code               = uint8_t;
    __device__ static P load(const ParamSrc&, uint32_t)
    {
        return 0;
    }
    __device__ static bool fast_ok(const P&, const float*, int)
    {
        return true;
    }
    template <bool FAST>
    __device__ static float apply(const ParamSrc&, const P&, float x, float, int& code)
    {
        code = 0;
        return bf16_to_f32(f32_to_bf16(x));
    }
};

// gin = g * (min <= x <= max)
struct OpV1Ste
{
    using P                  = float2;   // min, max
    static constexpr int NIN = 2;
    using Code               = uint8_t;
    __device__ static P load(const ParamSrc& s, uint32_t ch)
    {
        return make_float2(s.a[ch], s.b[ch]);
    }
    __device__ static bool fast_ok(const P&, const float*, int)
    {
        return true;   // no division in this op
    }
    template <bool FAST>
    __device__ static float apply(const ParamSrc&, const P& p, float x, float g, int& code)
    {
        code = 0;
        return g * (float) ((p.x <= x) && (x <= p.y));
    }
};

struct V2P
{
    float scale, offset, rcp;
};

struct OpV2
{
    using P = V2P;
    __device__ static P load(const ParamSrc& s, uint32_t ch)
    {
        const float sc = s.a[ch];
        return P{sc, s.b[ch], safe_rcp(sc, 0.0f)};
    }
    // x is not clamped before the division here, so the dividend bound is checked on the vector's largest |x|
    __device__ static bool fast_ok(const P& p, const float* x, int n)
    {
        float m = 0.0f;
        for (int j = 0; j < n; ++j)
            m = fmaxf(m, fabsf(x[j]));   // NaN elements are skipped: they give NaN on either path
        return p.rcp != 0.0f && m <= kFastDivMaxDividend;
    }
    // round-half-even(x / scale) - offset
    template <bool FAST>
    __device__ static float grid(const P& p, float x)
    {
        const float q = FAST ? div_by_invariant(x, p.scale, p.rcp) : x / p.scale;
        return rintf(q) - p.offset;
    }
};

struct OpV2Qdq : OpV2
{
    static constexpr int NIN = 1;
    using Code               = int32_t;
    template <bool FAST>
    __device__ static float apply(const ParamSrc& s, const P& p, float x, float, int& code)
    {
        float r = grid<FAST>(p, x);
        // torch.clamp semantics: NaN stays NaN
        float q = r;
        q       = (q < (float) s.qmin) ? (float) s.qmin : q;
        q       = (q > (float) s.qmax) ? (float) s.qmax : q;
        code    = (int) q;
        return (q + p.offset) * p.scale;
    }
};

// The v2 forward with the mask its backward multiplies the gradient with (torch_builtins.py:303-327 saves exactly
// this mask) as the "code"
struct OpV2QdqMask : OpV2
{
    static constexpr bool kMask = true;
    static constexpr int NIN = 1;
    using Code               = int32_t;
    template <bool FAST>
    __device__ static float apply(const ParamSrc& s, const P& p, float x, float, int& code)
    {
        const float r = grid<FAST>(p, x);
        code          = ((float) s.qmin <= r) && (r <= (float) s.qmax);
        float q       = r;
        q             = (q < (float) s.qmin) ? (float) s.qmin : q;
        q             = (q > (float) s.qmax) ? (float) s.qmax : q;
        return (q + p.offset) * p.scale;
    }
};

struct OpV2Bwd : OpV2
{
    static constexpr int NIN = 2;
    using Code               = int32_t;
    template <bool FAST>
    __device__ static float apply(const ParamSrc& s, const P& p, float x, float g, int& code)
    {
        float r = grid<FAST>(p, x);
        code    = 0;
        return g * (float) (((float) s.qmin <= r) && (r <= (float) s.qmax));
    }
};

// Whether a vector's results are known not to be NaN from its parameters alone.  The v1 forward clamps its input with
// fminf / fmaxf (a NaN input comes out as a bound) and then only rounds, adds the offset and multiplies by delta: with
// finite min, max, delta (what a non-zero rcp says) and offset every result is finite.
template <typename OP>
struct NoNanOut
{
    __device__ static bool get(const typename OP::P&)
    {
        return false;
    }
};
template <>
struct NoNanOut<OpV1Qdq>
{
    __device__ static bool get(const V1P& p)
    {
        return p.rcp != 0.0f && fabsf(p.offset) < INFINITY;
    }
};

template <>
struct NoNanOut<OpV1QdqMask>
{
    __device__ static bool get(const V1PM& p)
    {
        return p.rcp != 0.0f && fabsf(p.offset) < INFINITY;
    }
};

template <typename OP>
__device__ typename OP::P scalar_params(const ParamSrc& s);
template <>
__device__ V1PM scalar_params<OpV1QdqMask>(const ParamSrc& s)
{
    return V1PM{s.scalar.x, s.scalar.y, s.scalar.z, s.scalar.w, s.scalar_rcp, s.raw.x, s.raw.y};
}
template <>
__device__ V2P scalar_params<OpV2QdqMask>(const ParamSrc& s)
{
    return OpV2::load(s, 0);
}
template <>
__device__ V1P scalar_params<OpV1Qdq>(const ParamSrc& s)
{
    return V1P{s.scalar.x, s.scalar.y, s.scalar.z, s.scalar.w, s.scalar_rcp};
}
template <>
__device__ V1P scalar_params<OpV1Quantize>(const ParamSrc& s)
{
    return V1P{s.scalar.x, s.scalar.y, s.scalar.z, s.scalar.w, s.scalar_rcp};
}
template <>
__device__ int scalar_params<OpFp16>(const ParamSrc&)
{
    return 0;
}
template <>
__device__ int scalar_params<OpBf16>(const ParamSrc&)
{
    return 0;
}
template <>
__device__ float2 scalar_params<OpV1Ste>(const ParamSrc& s)
{
    return make_float2(s.scalar.x, s.scalar.y);
}
// v2 per-tensor: scale/offset are one-element device tensors; the load is wave-uniform (scalar load)
template <>
__device__ V2P scalar_params<OpV2Qdq>(const ParamSrc& s)
{
    return OpV2::load(s, 0);
}
template <>
__device__ V2P scalar_params<OpV2Bwd>(const ParamSrc& s)
{
    return OpV2::load(s, 0);
}

// Applies OP to N elements that share one parameter set; the fast/plain quotient decision is taken once.
template <typename OP, int N, bool TWO_IN>
__device__ __forceinline__ void apply_n(const ParamSrc& s, const typename OP::P& p, const float* fx, const float* fg,
                                        float* fy, int* code)
{
    if (OP::fast_ok(p, fx, N))
    {
#pragma unroll
        for (int j = 0; j < N; ++j)
            fy[j] = OP::template apply<true>(s, p, fx[j], TWO_IN ? fg[j] : 0.f, code[j]);
    }
    else
    {
#pragma unroll
        for (int j = 0; j < N; ++j)
            fy[j] = OP::template apply<false>(s, p, fx[j], TWO_IN ? fg[j] : 0.f, code[j]);
    }
}

// ----------------------------------------------------------------------------------------------------- the kernels
template <typename IO, typename CodeT>
struct EwPtrs
{
    const IO* x;
    const IO* g;    // second input (backward), else unused
    IO* y;          // may be null when only codes are wanted
    CodeT* codes;   // may be null
    uint64_t* mask; // saved straight-through mask (mask ops only), else null
};

// ---- the saved straight-through mask ---------------------------------------------------------------------------
// One bit per element, laid out for wavefront-wide compares: with V = the elements of a 16-byte vector (4 for
// float32, 8 for bfloat16 storage) the elements are taken in groups of 64 V; group g owns the V consecutive 64-bit
// words g V .. g V + V - 1, and bit t of word j is the flag of element 64 V g + V t + j -- element j of the vector
// lane t of a wavefront holds, i.e. exactly what a compare over the wavefront leaves in a scalar register pair.  The
// n % V elements after the last whole vector have their flags in bits 0 .. of one more word after the last group.
template <int VEC>
__host__ __device__ inline int64_t mask_groups(int64_t n)
{
    return (n / VEC + 63) / 64;
}
template <int VEC>
__host__ __device__ inline int64_t mask_words(int64_t n)
{
    return mask_groups<VEC>(n) * VEC + 1;
}

// One group's V words from V wavefront-wide compares: lane j < V keeps word j and stores it.  (Written without an
// array of words: the compiler moved such an array to LDS.)
template <int VEC, typename FLAG>
__device__ __forceinline__ void store_mask_group(uint64_t* dst, int lane, bool store, FLAG flag)
{
    uint64_t mine = 0;
#pragma unroll
    for (int j = 0; j < VEC; ++j)
    {
        const uint64_t w = __builtin_amdgcn_ballot_w64(flag(j));
        mine             = (lane == j) ? w : mine;
    }
    if (store && lane < VEC)
        __builtin_nontemporal_store(mine, dst + lane);
}

constexpr int kWin = 264;   // LDS window rows; host guarantees tile / elements-per-channel + 2 <= kWin

template <typename CodeT, int VEC>
__device__ __forceinline__ void store_codes(CodeT* dst, const int* c);

template <>
__device__ __forceinline__ void store_codes<uint8_t, 4>(uint8_t* dst, const int* c)
{
    uint32_t w = (uint32_t) (c[0] & 0xff) | ((uint32_t) (c[1] & 0xff) << 8) | ((uint32_t) (c[2] & 0xff) << 16) |
                 ((uint32_t) (c[3] & 0xff) << 24);
    *reinterpret_cast<uint32_t*>(dst) = w;
}
template <>
__device__ __forceinline__ void store_codes<uint8_t, 8>(uint8_t* dst, const int* c)
{
    store_codes<uint8_t, 4>(dst, c);
    store_codes<uint8_t, 4>(dst + 4, c + 4);
}
template <>
__device__ __forceinline__ void store_codes<int32_t, 4>(int32_t* dst, const int* c)
{
    *reinterpret_cast<int4*>(dst) = make_int4(c[0], c[1], c[2], c[3]);
}
template <>
__device__ __forceinline__ void store_codes<int32_t, 8>(int32_t* dst, const int* c)
{
    store_codes<int32_t, 4>(dst, c);
    store_codes<int32_t, 4>(dst + 4, c + 4);
}

// Vectorised tile kernel.  Requires 16-byte aligned pointers; n < 2^31 when PER_CHANNEL.  CODES: the integer codes are
// stored too (ptr.codes is not null); without it their arithmetic (two operations per element) is not compiled in.
// MASK: the ops' "codes" are in-range flags, packed into ptr.mask (see above) instead of being stored as integers.
// `tile`: which tile of the tensor this workgroup takes (the workgroup's index for a launch over one tensor).
template <typename IO, typename OP, bool PER_CHANNEL, int kUnroll, bool CODES, bool MASK = false>
__device__ __forceinline__ void ew_vec_tile(const EwPtrs<IO, typename OP::Code>& ptr, const ParamSrc& src, int64_t n,
                                            uint32_t num_channel, const FastDiv& fd, uint32_t tile)
{
    using T                 = IOTraits<IO>;
    using Vec               = typename T::Vec;
    using P                 = typename OP::P;
    constexpr int VEC       = T::VEC;
    constexpr uint32_t TILE = kBlock * kUnroll * VEC;
    const int64_t e_base    = (int64_t) tile * TILE;
    const int64_t nvec      = n / VEC;

    // 1. the tile's loads go out first; everything below overlaps their latency.  A workgroup whose whole tile exists
    //    (all but the last) requests them without a condition per lane: under a per-lane condition the compiler moves
    //    the first arithmetic on a vector into the conditional block, waits for that vector there, and only then
    //    requests the next one.
    Vec vx[kUnroll], vg[kUnroll];
    bool live[kUnroll];
    const bool whole_tile = e_base / VEC + (int64_t) kUnroll * kBlock <= nvec;   // workgroup-uniform
    if (whole_tile)
    {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            const int64_t v = e_base / VEC + (int64_t) u * kBlock + threadIdx.x;
            live[u]         = true;
            vx[u]           = stream_load(reinterpret_cast<const Vec*>(ptr.x) + v);
            if constexpr (OP::NIN == 2)
                vg[u] = stream_load(reinterpret_cast<const Vec*>(ptr.g) + v);
        }
    }
    else
    {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            const int64_t v = e_base / VEC + (int64_t) u * kBlock + threadIdx.x;
            live[u]         = v < nvec;
            if (live[u])
            {
                vx[u] = stream_load(reinterpret_cast<const Vec*>(ptr.x) + v);
                if constexpr (OP::NIN == 2)
                    vg[u] = stream_load(reinterpret_cast<const Vec*>(ptr.g) + v);
            }
        }
    }

    // 2. parameters: kernel arguments (per-tensor), scalar loads when the whole tile lies in one channel row (the
    //    usual case for weights: a row is at least a tile long), else the LDS window of the rows the tile touches
    __shared__ P win[PER_CHANNEL ? kWin : 1];
    uint32_t rem0   = 0;
    bool one_row    = true;
    P pt;
    if constexpr (PER_CHANNEL)
    {
        const uint32_t eb   = (uint32_t) e_base;
        const uint32_t row0 = fastdiv(eb, fd);
        rem0                = eb - row0 * fd.d;
        const uint32_t ee   = (uint32_t) (((int64_t) eb + TILE < n) ? eb + TILE : n);
        const uint32_t row1 = fastdiv(ee - 1, fd);
        one_row             = (row0 == row1);   // workgroup-uniform
        if (one_row)
        {
            pt = OP::load(src, row0 % num_channel);
        }
        else
        {
            for (uint32_t r = threadIdx.x; r <= row1 - row0; r += kBlock)
                win[r] = OP::load(src, (row0 + r) % num_channel);
            __syncthreads();
        }
    }
    else
    {
        pt = scalar_params<OP>(src);
    }

    // 3. compute every vector, then store them: with a store between two vectors' arithmetic the wait for the second
    //    vector would also wait for that store (loads and stores complete in one order, and the store is conditional)
    float fy[kUnroll][VEC];
    int code[kUnroll][VEC];
    bool no_nan[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
    {
        no_nan[u] = false;
        if (!live[u])
            continue;
        const uint32_t le = ((uint32_t) u * kBlock + threadIdx.x) * VEC;
        float fx[VEC], fg[VEC];
        T::unpack(vx[u], fx);
        if constexpr (OP::NIN == 2)
            T::unpack(vg[u], fg);
        if (one_row)
        {
            apply_n<OP, VEC, OP::NIN == 2>(src, pt, fx, fg, fy[u], code[u]);
            no_nan[u] = NoNanOut<OP>::get(pt);
        }
        else
        {
            const uint32_t t   = rem0 + le;
            const uint32_t lr  = fastdiv(t, fd);
            const uint32_t rem = t - lr * fd.d;
            if (rem + VEC <= fd.d)
            {
                const P p = win[lr];
                apply_n<OP, VEC, OP::NIN == 2>(src, p, fx, fg, fy[u], code[u]);
                no_nan[u] = NoNanOut<OP>::get(p);
            }
            else
            {
                // the vector straddles one channel boundary (elements-per-channel is not a multiple of VEC)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                {
                    const P p = win[lr + ((rem + j >= fd.d) ? 1u : 0u)];
                    fy[u][j]  = OP::template apply<false>(src, p, fx[j], OP::NIN == 2 ? fg[j] : 0.f, code[u][j]);
                }
            }
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
    {
        if (!live[u])
            continue;
        const int64_t v = e_base / VEC + (int64_t) u * kBlock + threadIdx.x;
        if (ptr.y)
            stream_store(reinterpret_cast<Vec*>(ptr.y) + v, no_nan[u] ? T::pack_no_nan(fy[u]) : T::pack(fy[u]));
        if constexpr (CODES)
            store_codes<typename OP::Code, VEC>(ptr.codes + v * VEC, code[u]);
    }
    if constexpr (MASK)
    {
        // every lane of the wavefront takes part in the compares; a wavefront whose first lane has no vector has none
        const int wave = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            const int64_t v0 = e_base / VEC + (int64_t) u * kBlock + wave * 64;   // wavefront-uniform
            store_mask_group<VEC>(ptr.mask + (v0 / 64) * VEC, lane, v0 < nvec,
                                  [&](int j) { return live[u] && code[u][j] != 0; });
        }
    }
    // the n % VEC trailing elements
    if (tile == 0 && threadIdx.x < (uint32_t) (n - nvec * VEC))
    {
        const int64_t e = nvec * VEC + threadIdx.x;
        P p;
        if constexpr (PER_CHANNEL)
            p = OP::load(src, (uint32_t) ((e / fd.d) % num_channel));
        else
            p = pt;
        int code;
        const float y =
            OP::template apply<false>(src, p, T::load1(ptr.x + e), OP::NIN == 2 ? T::load1(ptr.g + e) : 0.f, code);
        if (ptr.y)
            T::store1(ptr.y + e, y);
        if constexpr (MASK)
        {
            const uint64_t w = __builtin_amdgcn_ballot_w64(code != 0);   // the active lanes are 0 .. n % VEC - 1
            if (threadIdx.x == 0)
                ptr.mask[mask_words<VEC>(n) - 1] = w;
        }
        else if (ptr.codes)
            ptr.codes[e] = (typename OP::Code) code;
    }
    if constexpr (MASK)
        if (tile == 0 && threadIdx.x == 0 && n == nvec * VEC)
            ptr.mask[mask_words<VEC>(n) - 1] = 0;   // no trailing elements: the word is still defined
}

template <typename IO, typename OP, bool PER_CHANNEL, int kUnroll, bool CODES, bool MASK = false>
__global__ __launch_bounds__(kBlock) void ew_vec_kernel(EwPtrs<IO, typename OP::Code> ptr, ParamSrc src, int64_t n,
                                                        uint32_t num_channel, FastDiv fd)
{
    ew_vec_tile<IO, OP, PER_CHANNEL, kUnroll, CODES, MASK>(ptr, src, n, num_channel, fd, blockIdx.x);
}

// ---- several tensors in one launch --------------------------------------------------------------------------------
// The workgroups of one launch are dealt out over the tiles of all segments (miq_qdq_segment, a table in device
// memory): a workgroup finds its segment by counting the segments that start at or before its tile -- every lane reads
// one segment's first tile, one round trip -- reads that segment's record and runs the per-channel tile code on it.
// For the dozens of small weight tensors of a convolutional network, each a few microseconds of traffic, this removes
// the launches' fixed cost and lets the tensors' ramps overlap.
constexpr int kMaxSegments = kBlock;
template <typename IO>
__global__ __launch_bounds__(kBlock) void ew_multi_kernel(const miq_qdq_segment* __restrict__ segs, int num_segments)
{
    __shared__ int s_count[kBlock / 64];
    const uint32_t tile = blockIdx.x;
    const bool before   = (int) threadIdx.x < num_segments && (uint32_t) segs[threadIdx.x].first_tile <= tile;
    const int in_wave   = __popcll(__builtin_amdgcn_ballot_w64(before));
    if ((threadIdx.x & 63) == 0)
        s_count[threadIdx.x >> 6] = in_wave;
    __syncthreads();
    int count = 0;
#pragma unroll
    for (int k = 0; k < kBlock / 64; ++k)
        count += s_count[k];
    const int seg             = __builtin_amdgcn_readfirstlane(count - 1);   // first_tile of segment 0 is 0
    const miq_qdq_segment sg  = segs[seg];
    EwPtrs<IO, uint8_t> ptr{static_cast<const IO*>(sg.in), nullptr, static_cast<IO*>(sg.out), nullptr, nullptr};
    ParamSrc src{};
    src.a = sg.enc_min;
    src.b = sg.enc_max;
    src.c = sg.enc_delta;
    src.d = sg.enc_offset;
    FastDiv fd;
    fd.d     = (uint32_t) sg.num_element_per_channel;
    fd.magic = sg.fd_magic;
    fd.shift = sg.fd_shift;
    ew_vec_tile<IO, OpV1Qdq, true, kUnroll, false, false>(ptr, src, sg.num_element, (uint32_t) sg.num_channel, fd,
                                                         tile - (uint32_t) sg.first_tile);
}

// Fallback for unaligned pointers, tiny channels (elements-per-channel < 16) and n >= 2^31: one element per lane,
// grid-stride, 64-bit indexing, parameters read through the cache.
template <typename IO, typename OP, bool PER_CHANNEL>
__global__ __launch_bounds__(kBlock) void ew_scalar_kernel(EwPtrs<IO, typename OP::Code> ptr, ParamSrc src, int64_t n,
                                                           int64_t num_channel, int64_t n_per_channel)
{
    using T = IOTraits<IO>;
    using P = typename OP::P;
    for (int64_t e = (int64_t) blockIdx.x * kBlock + threadIdx.x; e < n; e += (int64_t) gridDim.x * kBlock)
    {
        P p;
        if constexpr (PER_CHANNEL)
            p = OP::load(src, (uint32_t) ((e / n_per_channel) % num_channel));
        else
            p = scalar_params<OP>(src);
        int code;
        const float y =
            OP::template apply<false>(src, p, T::load1(ptr.x + e), OP::NIN == 2 ? T::load1(ptr.g + e) : 0.f, code);
        if (ptr.y)
            T::store1(ptr.y + e, y);
        if (ptr.codes)
            ptr.codes[e] = (typename OP::Code) code;
    }
}

// Mask-writing forward for what the tile kernel does not take (unaligned pointers, tiny channels, n >= 2^31): a
// wavefront per mask group, lane t handling elements V t .. V t + V - 1 of the group one at a time, 64-bit indexing,
// parameters read through the cache.  Same mask layout as the tile kernel.
template <typename IO, typename OP, bool PER_CHANNEL>
__global__ __launch_bounds__(kBlock) void ew_mask_group_kernel(EwPtrs<IO, typename OP::Code> ptr, ParamSrc src,
                                                               int64_t n, int64_t num_channel, int64_t n_per_channel)
{
    using T           = IOTraits<IO>;
    using P           = typename OP::P;
    constexpr int VEC = T::VEC;
    const int lane    = threadIdx.x & 63;
    const int64_t nvec = n / VEC, groups = mask_groups<VEC>(n);
    const int64_t wave0 = (int64_t) blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    for (int64_t grp = wave0; grp < groups; grp += (int64_t) gridDim.x * (kBlock / 64))
    {
        const int64_t v = grp * 64 + lane;
        store_mask_group<VEC>(ptr.mask + grp * VEC, lane, true, [&](int j) {
            int code = 0;
            if (v < nvec)
            {
                const int64_t e = v * VEC + j;
                P p;
                if constexpr (PER_CHANNEL)
                    p = OP::load(src, (uint32_t) ((e / n_per_channel) % num_channel));
                else
                    p = scalar_params<OP>(src);
                T::store1(ptr.y + e, OP::template apply<false>(src, p, T::load1(ptr.x + e), 0.f, code));
            }
            return code != 0;
        });
    }
    if (blockIdx.x == 0 && threadIdx.x < (uint32_t) (n - nvec * VEC))
    {
        const int64_t e = nvec * VEC + threadIdx.x;
        P p;
        if constexpr (PER_CHANNEL)
            p = OP::load(src, (uint32_t) ((e / n_per_channel) % num_channel));
        else
            p = scalar_params<OP>(src);
        int code;
        T::store1(ptr.y + e, OP::template apply<false>(src, p, T::load1(ptr.x + e), 0.f, code));
        const uint64_t w = __builtin_amdgcn_ballot_w64(code != 0);
        if (threadIdx.x == 0)
            ptr.mask[mask_words<VEC>(n) - 1] = w;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0 && n == nvec * VEC)
        ptr.mask[mask_words<VEC>(n) - 1] = 0;
}

// ---- straight-through backward from the saved mask: grad_in = grad_out * bit -------------------------------------
// No parameters and no x: 4 bytes read + 1/8 byte of mask + 4 bytes written per float32 element (8.125 instead of the
// 12 of the backward that recomputes the mask from x).  A wavefront's V mask words are one scalar load, and each word
// is used as the lane mask of a select as it stands.
template <typename IO, int kUnroll>
__global__ __launch_bounds__(kBlock) void ste_mask_bwd_kernel(const uint64_t* __restrict__ mask,
                                                              const IO* __restrict__ g, IO* __restrict__ gin, int64_t n)
{
    using T                 = IOTraits<IO>;
    using Vec               = typename T::Vec;
    constexpr int VEC       = T::VEC;
    constexpr uint32_t TILE = kBlock * kUnroll * VEC;
    const int64_t e_base    = (int64_t) blockIdx.x * TILE;
    const int64_t nvec      = n / VEC;
    const int wave          = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    Vec vg[kUnroll];
    bool live[kUnroll];
    const bool whole_tile = e_base / VEC + (int64_t) kUnroll * kBlock <= nvec;   // workgroup-uniform
    if (whole_tile)
    {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            live[u] = true;
            vg[u]   = stream_load(reinterpret_cast<const Vec*>(g) + e_base / VEC + (int64_t) u * kBlock + threadIdx.x);
        }
    }
    else
    {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            const int64_t v = e_base / VEC + (int64_t) u * kBlock + threadIdx.x;
            live[u]         = v < nvec;
            if (live[u])
                vg[u] = stream_load(reinterpret_cast<const Vec*>(g) + v);
        }
    }
    uint64_t w[kUnroll][VEC];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
    {
        const int64_t v0 = e_base / VEC + (int64_t) u * kBlock + wave * 64;   // wavefront-uniform
        const uint64_t* mw = mask + (v0 / 64) * VEC;
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            w[u][j] = (v0 < nvec) ? mw[j] : 0;
    }
    Vec out[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
    {
        float fg[VEC], fy[VEC];
        T::unpack(vg[u], fg);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            fy[j] = fg[j] * (__builtin_amdgcn_inverse_ballot_w64(w[u][j]) ? 1.0f : 0.0f);
        out[u] = T::pack(fy);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
        if (live[u])
            stream_store(reinterpret_cast<Vec*>(gin) + e_base / VEC + (int64_t) u * kBlock + threadIdx.x, out[u]);
    if (blockIdx.x == 0 && threadIdx.x < (uint32_t) (n - nvec * VEC))
    {
        const int64_t e  = nvec * VEC + threadIdx.x;
        const uint64_t t = mask[mask_words<VEC>(n) - 1];
        T::store1(gin + e, T::load1(g + e) * (float) ((t >> threadIdx.x) & 1));
    }
}

// the same for unaligned pointers: a wavefront per mask group, one element at a time
template <typename IO>
__global__ __launch_bounds__(kBlock) void ste_mask_bwd_group_kernel(const uint64_t* __restrict__ mask,
                                                                    const IO* __restrict__ g, IO* __restrict__ gin,
                                                                    int64_t n)
{
    using T           = IOTraits<IO>;
    constexpr int VEC = T::VEC;
    const int lane    = threadIdx.x & 63;
    const int64_t nvec = n / VEC, groups = mask_groups<VEC>(n);
    const int64_t wave0 = (int64_t) blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    for (int64_t grp = wave0; grp < groups; grp += (int64_t) gridDim.x * (kBlock / 64))
    {
        const int64_t v = grp * 64 + lane;
        if (v < nvec)
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                const int64_t e = v * VEC + j;
                T::store1(gin + e, T::load1(g + e) * (float) ((mask[grp * VEC + j] >> lane) & 1));
            }
    }
    if (blockIdx.x == 0 && threadIdx.x < (uint32_t) (n - nvec * VEC))
    {
        const int64_t e  = nvec * VEC + threadIdx.x;
        const uint64_t t = mask[mask_words<VEC>(n) - 1];
        T::store1(gin + e, T::load1(g + e) * (float) ((t >> threadIdx.x) & 1));
    }
}

template <typename IO>
int launch_ste_mask_bwd(const uint64_t* mask, const IO* g, IO* gin, int64_t n, hipStream_t stream)
{
    if (n == 0)
        return MIQ_OK;
    using T                = IOTraits<IO>;
    constexpr int64_t TILE = (int64_t) kBlock * kUnroll * T::VEC;
    if (aligned16(g) && aligned16(gin))
    {
        hipLaunchKernelGGL((ste_mask_bwd_kernel<IO, kUnroll>), dim3((unsigned) ((n + TILE - 1) / TILE)), dim3(kBlock), 0,
                           stream, mask, g, gin, n);
    }
    else
    {
        int64_t blocks = (mask_groups<T::VEC>(n) + kBlock / 64 - 1) / (kBlock / 64);
        blocks         = blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks);
        hipLaunchKernelGGL((ste_mask_bwd_group_kernel<IO>), dim3((unsigned) blocks), dim3(kBlock), 0, stream, mask, g, gin,
                           n);
    }
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

// whether OP's codes are straight-through flags (the mask-writing kernels are compiled for these only)
template <typename OP, typename = void>
struct WritesMask
{
    static constexpr bool value = false;
};
template <typename OP>
struct WritesMask<OP, decltype((void) OP::kMask)>
{
    static constexpr bool value = true;
};

template <typename IO, typename OP, bool PER_CHANNEL>
int launch_ew(EwPtrs<IO, typename OP::Code> ptr, const ParamSrc& src, int64_t n, int64_t num_channel,
              int64_t n_per_channel, hipStream_t stream)
{
    if (n == 0)
        return MIQ_OK;
    using T                = IOTraits<IO>;
    // 16-byte vectors in flight per lane.  Measured on [32,64,56,56], [4096,4096] and [11008,4096], one and two
    // inputs, float32 and bfloat16: 1, 4 and 8 are never faster than 2 by more than the run-to-run spread and are
    // slower on the bfloat16 forward (+7 %) and on two-input kernels (+5 %)
    constexpr int U        = kUnroll;
    constexpr int64_t TILE = (int64_t) kBlock * U * T::VEC;
    bool vec_ok = aligned16(ptr.x) && (OP::NIN == 1 || aligned16(ptr.g)) && (!ptr.y || aligned16(ptr.y)) &&
                  (!ptr.codes || aligned16(ptr.codes));
    if (PER_CHANNEL)
        vec_ok = vec_ok && n < (1ll << 31) && n_per_channel < (1ll << 31) &&
                 (TILE / n_per_channel + 2 <= kWin);
    if (vec_ok)
    {
        const int64_t blocks = (n + TILE - 1) / TILE;
        FastDiv fd           = make_fastdiv(PER_CHANNEL ? (uint32_t) n_per_channel : 1u);
        if constexpr (WritesMask<OP>::value)
            hipLaunchKernelGGL((ew_vec_kernel<IO, OP, PER_CHANNEL, U, false, true>), dim3((unsigned) blocks),
                               dim3(kBlock), 0, stream, ptr, src, n, (uint32_t) num_channel, fd);
        else if (ptr.codes)
            hipLaunchKernelGGL((ew_vec_kernel<IO, OP, PER_CHANNEL, U, true>), dim3((unsigned) blocks), dim3(kBlock), 0,
                               stream, ptr, src, n, (uint32_t) num_channel, fd);
        else
            hipLaunchKernelGGL((ew_vec_kernel<IO, OP, PER_CHANNEL, U, false>), dim3((unsigned) blocks), dim3(kBlock), 0,
                               stream, ptr, src, n, (uint32_t) num_channel, fd);
    }
    else if constexpr (WritesMask<OP>::value)
    {
        int64_t blocks = (mask_groups<T::VEC>(n) + kBlock / 64 - 1) / (kBlock / 64);
        blocks         = blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks);
        hipLaunchKernelGGL((ew_mask_group_kernel<IO, OP, PER_CHANNEL>), dim3((unsigned) blocks), dim3(kBlock), 0, stream,
                           ptr, src, n, num_channel, n_per_channel);
    }
    else
    {
        int64_t blocks = (n + kBlock - 1) / kBlock;
        if (blocks > 65536)
            blocks = 65536;
        hipLaunchKernelGGL((ew_scalar_kernel<IO, OP, PER_CHANNEL>), dim3((unsigned) blocks), dim3(kBlock), 0, stream,
                           ptr, src, n, num_channel, n_per_channel);
    }
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int check_round(int rounding_mode)
{
    if (rounding_mode == MIQ_ROUND_NEAREST)
        return MIQ_OK;
    if (rounding_mode == MIQ_ROUND_STOCHASTIC)
        return MIQ_OK;
    set_error("unknown rounding mode %d", rounding_mode);
    return MIQ_ERR_INVALID_ARG;
}

int check_channels(int64_t num_channel, int64_t num_element, int64_t n_per_channel)
{
    MIQ_CHECK_ARG(num_channel > 0 && num_channel < (1ll << 31), "num_channel must be in [1, 2^31)");
    MIQ_CHECK_ARG(n_per_channel > 0, "num_element_per_channel must be positive");
    MIQ_CHECK_ARG(num_element >= 0, "num_element must be non-negative");
    return MIQ_OK;
}

ParamSrc per_tensor_src(const miq_encoding& e)
{
    ParamSrc s{};
    s.scalar = make_float4((float) e.min, (float) e.max, (float) e.delta, (float) e.offset);
    // IEEE single division on the host gives the same correctly rounded reciprocal the device would compute
    const float bound = std::fmax(std::fabs(s.scalar.x), std::fabs(s.scalar.y));
    s.scalar_rcp      = (fastdiv_divisor_ok(s.scalar.z) && bound <= kFastDivMaxDividend) ? 1.0f / s.scalar.z : 0.0f;
    return s;
}

// per-channel parameter recipe, float32, operation for operation as the ATen sequence of the reference
__global__ void per_channel_params_kernel(const float* enc_min, const float* enc_max, int64_t c, float num_steps,
                                          float* omin, float* omax, float* odelta, float* ooffset)
{
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= c)
        return;
    float lo = enc_min[i], hi = enc_max[i];
    // torch.minimum / torch.maximum propagate NaN
    lo        = (lo != lo) ? lo : fminf(lo, 0.f);
    hi        = (hi != hi) ? hi : fmaxf(hi, 0.f);
    float eps = lo + 1e-5f;
    hi        = (hi != hi || eps != eps) ? (hi + eps) : fmaxf(hi, eps);
    float d   = (hi - lo) / num_steps;
    omin[i]   = lo;
    omax[i]   = hi;
    odelta[i] = d;
    ooffset[i] = rintf(lo / d);
}

// TF (min / max) encodings of every channel of a tensor and the kernel parameters that follow from them, without a
// visit to the host: channel c's running (min, max) -> TfEncodingAnalyzer::computeEncoding
// (DlQuantization/src/TfEncodingAnalyzer.cpp:80-101: zero inside the range, at least 0.01 wide) -> getComputedEncodings in
// double -> the float32 recipe of per_channel_params_kernel on float32(min), float32(max).  The number of steps of that
// recipe depends on channel 0's encoding (one step less iff its min == -max), which every thread derives for itself.
__device__ __forceinline__ EncodingD tf_channel_encoding(float lo_f, float hi_f, int bw, bool sym, bool strict, bool uns)
{
    double lo = enc_min2(0.0, (double) lo_f);
    double hi = enc_max2(0.0, (double) hi_f);
    hi        = enc_max2(hi, lo + 0.01);
    return computed_encodings(bw, lo, hi, sym, strict, uns);
}

__global__ void tf_channel_encodings_kernel(const float* ch_min, const float* ch_max, int64_t c, int bw, int sym, int strict,
                                            int uns, double* enc, float* omin, float* omax, float* odelta, float* ooffset,
                                            float* raw_min, float* raw_max)
{
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= c)
        return;
    const EncodingD first = tf_channel_encoding(ch_min[0], ch_max[0], bw, sym, strict, uns);
    const EncodingD e     = tf_channel_encoding(ch_min[i], ch_max[i], bw, sym, strict, uns);
    enc[4 * i + 0]        = e.min;
    enc[4 * i + 1]        = e.max;
    enc[4 * i + 2]        = e.delta;
    enc[4 * i + 3]        = e.offset;
    const ChannelKernelParams p = channel_kernel_params(e.min, e.max, first.min == -first.max, bw);
    omin[i]    = p.min;
    omax[i]    = p.max;
    odelta[i]  = p.delta;
    ooffset[i] = p.offset;
    raw_min[i] = p.raw_min;
    raw_max[i] = p.raw_max;
}

struct BcastArgs
{
    int64_t istride[8];
    int64_t estride[8];
    int ndims;
};

// numpy-style broadcast of the encoding (DlQuantization/src/trim_functions.cpp:634-660); the reference keeps the
// running remainder and the indices in `int`, so this path is defined for fewer than 2^31 elements.
__global__ __launch_bounds__(kBlock) void qdq_broadcast_kernel(const float* in, float* out, int64_t n, BcastArgs b,
                                                               const float* mn, const float* mx, const float* delta,
                                                               const float* offset)
{
    for (int64_t e = (int64_t) blockIdx.x * kBlock + threadIdx.x; e < n; e += (int64_t) gridDim.x * kBlock)
    {
        int enc = 0;
        int rem = (int) e;
        for (int d = 0; d < b.ndims; ++d)
        {
            int idx = (int) (rem / b.istride[d]);
            rem     = (int) (rem - idx * b.istride[d]);
            enc += (int) (b.estride[d] * idx);
        }
        const V1P p   = V1P{mn[enc], mx[enc], delta[enc], offset[enc], 0.0f};
        const float q = OpV1::quant<false>(p, in[e]);
        out[e]        = p.delta * (q + p.offset);
    }
}
// True when the broadcast is "encoding (e / run) % channels for element e" of a dense row-major tensor; see the caller.
static bool broadcast_as_channels(const BcastArgs& b, int64_t n, int64_t& channels, int64_t& run)
{
    int64_t size[8];
    for (int d = 0; d < b.ndims; ++d)
    {
        const int64_t outer = d == 0 ? n : b.istride[d - 1];
        if (outer % b.istride[d] != 0)
            return false;
        size[d] = outer / b.istride[d];
    }
    if (b.istride[b.ndims - 1] != 1)
        return false;   // not densely laid out
    int first = -1, last = -1;
    for (int d = 0; d < b.ndims; ++d)
        if (b.estride[d] != 0 && size[d] != 1)
        {
            if (first < 0)
                first = d;
            last = d;
        }
    if (first < 0)
    {
        channels = 1;
        run      = n;
        return true;
    }
    int64_t expect = 1;
    for (int d = last; d >= first; --d)
    {
        if (size[d] != 1 && b.estride[d] != expect)
            return false;   // a broadcast axis inside the run, or an encoding that is not dense over it
        expect *= size[d];
    }
    channels = expect;
    run      = b.istride[last];
    return true;
}

static ParamSrc v1_channel_src(const float* mn, const float* mx, const float* d, const float* o)
{
    ParamSrc s{};
    s.a = mn;
    s.b = mx;
    s.c = d;
    s.d = o;
    return s;
}

static int check_v2(int64_t num_channel, int64_t num_element, int64_t npc, const float* scale, const float* offset,
                    int qmin, int qmax)
{
    if (int rc = check_channels(num_channel, num_element, npc))
        return rc;
    MIQ_CHECK_ARG(scale && offset, "null scale/offset pointer");
    MIQ_CHECK_ARG(qmin <= qmax, "qmin (%d) must be smaller than or equal to qmax (%d)", qmin, qmax);
    // float32 must represent the grid exactly (torch_builtins.py:52-69)
    MIQ_CHECK_ARG(qmin > -(1 << 24) && qmax < (1 << 24), "float32 is unable to represent the grid [%d, %d]", qmin,
                  qmax);
    return MIQ_OK;
}

template <typename IO, typename OP>
static int launch_v2(EwPtrs<IO, int32_t> p, const ParamSrc& s, int64_t n, int64_t num_channel, int64_t npc,
                     hipStream_t stream)
{
    if (num_channel == 1)
        return launch_ew<IO, OP, false>(p, s, n, 1, 1, stream);
    return launch_ew<IO, OP, true>(p, s, n, num_channel, npc, stream);
}

static ParamSrc v2_src(const float* scale, const float* offset, int qmin, int qmax)
{
    ParamSrc s{};
    s.a    = scale;
    s.b    = offset;
    s.qmin = qmin;
    s.qmax = qmax;
    return s;
}
}   // namespace
}   // namespace miq

using namespace miq;

template <typename IO>
static int qdq_mask_per_tensor(const IO* in, IO* out, uint64_t* mask, int64_t n, double enc_min, double enc_max, int bw,
                               float mask_min, float mask_max, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && out && mask)), "null tensor pointer or negative count");
    MIQ_CHECK_ARG((reinterpret_cast<uintptr_t>(mask) & 7u) == 0, "the mask must be 8-byte aligned");
    miq_encoding e;
    if (int rc = miq_fill_encoding_info(bw, enc_min, enc_max, &e))
        return rc;
    ParamSrc s = per_tensor_src(e);
    s.raw      = make_float2(mask_min, mask_max);
    EwPtrs<IO, uint8_t> p{in, nullptr, out, nullptr, mask};
    return launch_ew<IO, OpV1QdqMask, false>(p, s, n, 1, 1, (hipStream_t) stream);
}

template <typename IO>
static int qdq_mask_per_channel(const IO* in, IO* out, uint64_t* mask, int64_t num_channel, int64_t num_element,
                                int64_t npc, const float* enc_min, const float* enc_max, const float* enc_delta,
                                const float* enc_offset, const float* raw_min, const float* raw_max, void* stream)
{
    if (int rc = check_channels(num_channel, num_element, npc))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (in && out && mask && enc_min && enc_max && enc_delta && enc_offset && raw_min &&
                                       raw_max),
                  "null pointer");
    MIQ_CHECK_ARG((reinterpret_cast<uintptr_t>(mask) & 7u) == 0, "the mask must be 8-byte aligned");
    ParamSrc s = v1_channel_src(enc_min, enc_max, enc_delta, enc_offset);
    s.e        = raw_min;
    s.f        = raw_max;
    EwPtrs<IO, uint8_t> p{in, nullptr, out, nullptr, mask};
    return launch_ew<IO, OpV1QdqMask, true>(p, s, num_element, num_channel, npc, (hipStream_t) stream);
}

template <typename IO>
static int v2_qdq_mask(const IO* in, IO* out, uint64_t* mask, int64_t num_channel, int64_t num_element, int64_t npc,
                       const float* scale, const float* offset, int qmin, int qmax, void* stream)
{
    if (int rc = check_v2(num_channel, num_element, npc, scale, offset, qmin, qmax))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (in && out && mask), "null pointer");
    MIQ_CHECK_ARG((reinterpret_cast<uintptr_t>(mask) & 7u) == 0, "the mask must be 8-byte aligned");
    EwPtrs<IO, int32_t> p{in, nullptr, out, nullptr, mask};
    return launch_v2<IO, OpV2QdqMask>(p, v2_src(scale, offset, qmin, qmax), num_element, num_channel, npc,
                                      (hipStream_t) stream);
}

template <typename IO>
static int qdq_multi(const miq_qdq_segment* segments, int num_segments, int64_t total_tiles, void* stream)
{
    MIQ_CHECK_ARG(segments && num_segments >= 1 && num_segments <= kMaxSegments, "1..%d segments per launch",
                  kMaxSegments);
    MIQ_CHECK_ARG(total_tiles >= 1 && total_tiles < (1ll << 31), "total_tiles must be what miq_qdq_multi_plan returned");
    hipLaunchKernelGGL((ew_multi_kernel<IO>), dim3((unsigned) total_tiles), dim3(kBlock), 0, (hipStream_t) stream,
                       segments, num_segments);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

extern "C" {

int miq_qdq_per_tensor_f32(const float* in, float* out, int64_t n, double enc_min, double enc_max, int bw,
                           int rounding_mode, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && out)), "null tensor pointer or negative count");
    if (int rc = check_round(rounding_mode))
        return rc;
    miq_encoding e;
    if (int rc = miq_fill_encoding_info(bw, enc_min, enc_max, &e))
        return rc;
    if (rounding_mode == MIQ_ROUND_STOCHASTIC)
        return stochastic_qdq_per_tensor<float>(in, out, n, e, (hipStream_t) stream);
    EwPtrs<float, uint8_t> p{in, nullptr, out, nullptr};
    return launch_ew<float, OpV1Qdq, false>(p, per_tensor_src(e), n, 1, 1, (hipStream_t) stream);
}

int miq_qdq_per_tensor_bf16(const uint16_t* in, uint16_t* out, int64_t n, double enc_min, double enc_max, int bw,
                            int rounding_mode, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && out)), "null tensor pointer or negative count");
    if (int rc = check_round(rounding_mode))
        return rc;
    miq_encoding e;
    if (int rc = miq_fill_encoding_info(bw, enc_min, enc_max, &e))
        return rc;
    if (rounding_mode == MIQ_ROUND_STOCHASTIC)
        return stochastic_qdq_per_tensor<uint16_t>(in, out, n, e, (hipStream_t) stream);
    EwPtrs<uint16_t, uint8_t> p{in, nullptr, out, nullptr};
    return launch_ew<uint16_t, OpV1Qdq, false>(p, per_tensor_src(e), n, 1, 1, (hipStream_t) stream);
}

int miq_fp16_round_trip_f32(const float* in, float* out, int64_t n, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && out)), "null tensor pointer or negative count");
    EwPtrs<float, uint8_t> p{in, nullptr, out, nullptr};
    return launch_ew<float, OpFp16, false>(p, ParamSrc{}, n, 1, 1, (hipStream_t) stream);
}

int miq_bf16_round_trip_f32(const float* in, float* out, int64_t n, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && out)), "null tensor pointer or negative count");
    EwPtrs<float, uint8_t> p{in, nullptr, out, nullptr};
    return launch_ew<float, OpBf16, false>(p, ParamSrc{}, n, 1, 1, (hipStream_t) stream);
}

int miq_quantize_per_tensor_f32(const float* in, float* out, int64_t n, double enc_min, double enc_max, int bw,
                                int rounding_mode, int shift_to_signed, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && out)), "null tensor pointer or negative count");
    if (int rc = check_round(rounding_mode))
        return rc;
    miq_encoding e;
    if (int rc = miq_fill_encoding_info(bw, enc_min, enc_max, &e))
        return rc;
    ParamSrc s = per_tensor_src(e);
    // DlQuantization/src/trim_functions.cpp:207-216: shift = 2^(bw-1) held in an unsigned int, subtracted in float
    unsigned int shift = shift_to_signed ? (unsigned int) std::pow(2, bw - 1) : 0u;
    s.shift            = (float) shift;
    if (rounding_mode == MIQ_ROUND_STOCHASTIC)
        return stochastic_quantize_per_tensor(in, out, n, e, s.shift, (hipStream_t) stream);
    EwPtrs<float, uint8_t> p{in, nullptr, out, nullptr};
    return launch_ew<float, OpV1Quantize, false>(p, s, n, 1, 1, (hipStream_t) stream);
}

int miq_qdq_codes_per_tensor_f32(const float* in, float* out, uint8_t* codes, int64_t n, double enc_min,
                                 double enc_max, int bw, int shift_to_signed, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && codes)), "null tensor pointer or negative count");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 8, "byte codes need 1 <= bw <= 8 (got %d)", bw);
    miq_encoding e;
    if (int rc = miq_fill_encoding_info(bw, enc_min, enc_max, &e))
        return rc;
    ParamSrc s = per_tensor_src(e);
    s.ishift   = shift_to_signed ? (1 << (bw - 1)) : 0;
    EwPtrs<float, uint8_t> p{in, nullptr, out, codes};
    return launch_ew<float, OpV1Qdq, false>(p, s, n, 1, 1, (hipStream_t) stream);
}

int miq_per_channel_params_f32(const float* enc_min, const float* enc_max, int64_t num_channel, double num_steps,
                               float* out_min, float* out_max, float* out_delta, float* out_offset, void* stream)
{
    MIQ_CHECK_ARG(num_channel > 0 && enc_min && enc_max && out_min && out_max && out_delta && out_offset,
                  "null pointer or non-positive channel count");
    MIQ_CHECK_ARG(num_steps > 0, "num_steps must be positive");
    const int64_t blocks = (num_channel + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(per_channel_params_kernel, dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream,
                       enc_min, enc_max, num_channel, (float) num_steps, out_min, out_max, out_delta, out_offset);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}


int miq_tf_encodings_per_channel_f32(const float* ch_min, const float* ch_max, int64_t num_channel, int bw,
                                     int use_symmetric, int use_strict_symmetric, int use_unsigned_symmetric, double* enc,
                                     float* out_min, float* out_max, float* out_delta, float* out_offset, float* raw_min,
                                     float* raw_max, void* stream)
{
    MIQ_CHECK_ARG(ch_min && ch_max && enc && out_min && out_max && out_delta && out_offset && raw_min && raw_max &&
                      num_channel > 0,
                  "null pointer or non-positive channel count");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 31, "bitwidth must be in [1, 31] (got %d)", bw);
    const int64_t blocks = (num_channel + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(tf_channel_encodings_kernel, dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream, ch_min,
                       ch_max, num_channel, bw, use_symmetric, use_strict_symmetric, use_unsigned_symmetric, enc, out_min,
                       out_max, out_delta, out_offset, raw_min, raw_max);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_qdq_per_channel_f32(const float* in, float* out, int64_t num_channel, int64_t num_element,
                            int64_t num_element_per_channel, const float* enc_min, const float* enc_max,
                            const float* enc_delta, const float* enc_offset, int rounding_mode, void* stream)
{
    if (int rc = check_channels(num_channel, num_element, num_element_per_channel))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (in && out && enc_min && enc_max && enc_delta && enc_offset), "null pointer");
    if (int rc = check_round(rounding_mode))
        return rc;
    if (rounding_mode == MIQ_ROUND_STOCHASTIC)
        return stochastic_qdq_per_channel<float>(in, out, num_channel, num_element, num_element_per_channel, enc_min,
                                                 enc_max, enc_delta, enc_offset, (hipStream_t) stream);
    EwPtrs<float, uint8_t> p{in, nullptr, out, nullptr};
    return launch_ew<float, OpV1Qdq, true>(p, v1_channel_src(enc_min, enc_max, enc_delta, enc_offset), num_element,
                                           num_channel, num_element_per_channel, (hipStream_t) stream);
}

int miq_qdq_per_channel_bf16(const uint16_t* in, uint16_t* out, int64_t num_channel, int64_t num_element,
                             int64_t num_element_per_channel, const float* enc_min, const float* enc_max,
                             const float* enc_delta, const float* enc_offset, int rounding_mode, void* stream)
{
    if (int rc = check_channels(num_channel, num_element, num_element_per_channel))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (in && out && enc_min && enc_max && enc_delta && enc_offset), "null pointer");
    if (int rc = check_round(rounding_mode))
        return rc;
    if (rounding_mode == MIQ_ROUND_STOCHASTIC)
        return stochastic_qdq_per_channel<uint16_t>(in, out, num_channel, num_element, num_element_per_channel,
                                                    enc_min, enc_max, enc_delta, enc_offset, (hipStream_t) stream);
    EwPtrs<uint16_t, uint8_t> p{in, nullptr, out, nullptr};
    return launch_ew<uint16_t, OpV1Qdq, true>(p, v1_channel_src(enc_min, enc_max, enc_delta, enc_offset), num_element,
                                              num_channel, num_element_per_channel, (hipStream_t) stream);
}

int miq_qdq_codes_per_channel_f32(const float* in, float* out, uint8_t* codes, int64_t num_channel,
                                  int64_t num_element, int64_t num_element_per_channel, const float* enc_min,
                                  const float* enc_max, const float* enc_delta, const float* enc_offset,
                                  int shift_to_signed, int bw, void* stream)
{
    if (int rc = check_channels(num_channel, num_element, num_element_per_channel))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (in && codes && enc_min && enc_max && enc_delta && enc_offset), "null pointer");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 8, "byte codes need 1 <= bw <= 8 (got %d)", bw);
    ParamSrc s = v1_channel_src(enc_min, enc_max, enc_delta, enc_offset);
    s.ishift   = shift_to_signed ? (1 << (bw - 1)) : 0;
    EwPtrs<float, uint8_t> p{in, nullptr, out, codes};
    return launch_ew<float, OpV1Qdq, true>(p, s, num_element, num_channel, num_element_per_channel,
                                           (hipStream_t) stream);
}

int miq_qdq_broadcast_f32(const float* in, float* out, int64_t num_element, int64_t num_dims,
                          const int64_t* input_strides, const int64_t* encoding_strides, const float* enc_min,
                          const float* enc_max, const float* enc_delta, const float* enc_offset, void* stream)
{
    MIQ_CHECK_ARG(num_element >= 0 && num_element < (1ll << 31), "num_element must be in [0, 2^31)");
    MIQ_CHECK_ARG(num_dims >= 1 && num_dims <= 8, "num_dims must be in [1, 8]");
    MIQ_CHECK_ARG(input_strides && encoding_strides, "null stride array");
    MIQ_CHECK_ARG(num_element == 0 || (in && out && enc_min && enc_max && enc_delta && enc_offset), "null pointer");
    if (num_element == 0)
        return MIQ_OK;
    BcastArgs b{};
    b.ndims = (int) num_dims;
    for (int d = 0; d < b.ndims; ++d)
    {
        MIQ_CHECK_ARG(input_strides[d] > 0, "input strides must be positive");
        b.istride[d] = input_strides[d];
        b.estride[d] = encoding_strides[d];
    }
    // The usual broadcasts -- one encoding for the tensor, or encodings that vary along one run of adjacent axes of a
    // densely laid out tensor, themselves densely laid out (per channel on any axis, blocks that cut the last varying
    // axis) -- are the [outer, channel, run] layout of the vector kernel: element e uses encoding (e / run) % channels.
    int64_t channels = 0, run = 0;
    if (broadcast_as_channels(b, num_element, channels, run))
    {
        EwPtrs<float, uint8_t> p{in, nullptr, out, nullptr};
        if (channels == 1)
            return launch_ew<float, OpV1Qdq, true>(p, v1_channel_src(enc_min, enc_max, enc_delta, enc_offset), num_element, 1,
                                                   num_element, (hipStream_t) stream);
        return launch_ew<float, OpV1Qdq, true>(p, v1_channel_src(enc_min, enc_max, enc_delta, enc_offset), num_element,
                                               channels, run, (hipStream_t) stream);
    }
    int64_t blocks = (num_element + kBlock - 1) / kBlock;
    if (blocks > 65536)
        blocks = 65536;
    hipLaunchKernelGGL(qdq_broadcast_kernel, dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream, in, out,
                       num_element, b, enc_min, enc_max, enc_delta, enc_offset);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_ste_bwd_per_tensor_f32(const float* x, const float* grad_out, float* grad_in, int64_t n, float enc_min,
                               float enc_max, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (x && grad_out && grad_in)), "null tensor pointer or negative count");
    ParamSrc s{};
    s.scalar = make_float4(enc_min, enc_max, 0.f, 0.f);
    EwPtrs<float, uint8_t> p{x, grad_out, grad_in, nullptr};
    return launch_ew<float, OpV1Ste, false>(p, s, n, 1, 1, (hipStream_t) stream);
}

int miq_ste_bwd_per_tensor_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t n,
                                float enc_min, float enc_max, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (x && grad_out && grad_in)), "null tensor pointer or negative count");
    ParamSrc s{};
    s.scalar = make_float4(enc_min, enc_max, 0.f, 0.f);
    EwPtrs<uint16_t, uint8_t> p{x, grad_out, grad_in, nullptr};
    return launch_ew<uint16_t, OpV1Ste, false>(p, s, n, 1, 1, (hipStream_t) stream);
}

int miq_ste_bwd_per_channel_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                                int64_t num_element, int64_t num_element_per_channel, const float* enc_min,
                                const float* enc_max, void* stream)
{
    if (int rc = check_channels(num_channel, num_element, num_element_per_channel))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (x && grad_out && grad_in && enc_min && enc_max), "null pointer");
    ParamSrc s{};
    s.a = enc_min;
    s.b = enc_max;
    EwPtrs<float, uint8_t> p{x, grad_out, grad_in, nullptr};
    return launch_ew<float, OpV1Ste, true>(p, s, num_element, num_channel, num_element_per_channel,
                                           (hipStream_t) stream);
}

int miq_ste_bwd_per_channel_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in,
                                 int64_t num_channel, int64_t num_element, int64_t num_element_per_channel,
                                 const float* enc_min, const float* enc_max, void* stream)
{
    if (int rc = check_channels(num_channel, num_element, num_element_per_channel))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (x && grad_out && grad_in && enc_min && enc_max), "null pointer");
    ParamSrc s{};
    s.a = enc_min;
    s.b = enc_max;
    EwPtrs<uint16_t, uint8_t> p{x, grad_out, grad_in, nullptr};
    return launch_ew<uint16_t, OpV1Ste, true>(p, s, num_element, num_channel, num_element_per_channel,
                                              (hipStream_t) stream);
}




int miq_v2_qdq_f32(const float* in, float* out, int32_t* codes, int64_t num_channel, int64_t num_element,
                   int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                   void* stream)
{
    if (int rc = check_v2(num_channel, num_element, num_element_per_channel, scale, offset, qmin, qmax))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (in && (out || codes)), "null pointer");
    EwPtrs<float, int32_t> p{in, nullptr, out, codes};
    return launch_v2<float, OpV2Qdq>(p, v2_src(scale, offset, qmin, qmax), num_element, num_channel,
                                     num_element_per_channel, (hipStream_t) stream);
}

int miq_v2_qdq_bf16(const uint16_t* in, uint16_t* out, int64_t num_channel, int64_t num_element,
                    int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                    void* stream)
{
    if (int rc = check_v2(num_channel, num_element, num_element_per_channel, scale, offset, qmin, qmax))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (in && out), "null pointer");
    EwPtrs<uint16_t, int32_t> p{in, nullptr, out, nullptr};
    return launch_v2<uint16_t, OpV2Qdq>(p, v2_src(scale, offset, qmin, qmax), num_element, num_channel,
                                        num_element_per_channel, (hipStream_t) stream);
}

int miq_v2_qdq_bwd_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                       int64_t num_element, int64_t num_element_per_channel, const float* scale,
                       const float* offset, int qmin, int qmax, void* stream)
{
    if (int rc = check_v2(num_channel, num_element, num_element_per_channel, scale, offset, qmin, qmax))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (x && grad_out && grad_in), "null pointer");
    EwPtrs<float, int32_t> p{x, grad_out, grad_in, nullptr};
    return launch_v2<float, OpV2Bwd>(p, v2_src(scale, offset, qmin, qmax), num_element, num_channel,
                                     num_element_per_channel, (hipStream_t) stream);
}

int miq_v2_qdq_bwd_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t num_channel,
                        int64_t num_element, int64_t num_element_per_channel, const float* scale,
                        const float* offset, int qmin, int qmax, void* stream)
{
    if (int rc = check_v2(num_channel, num_element, num_element_per_channel, scale, offset, qmin, qmax))
        return rc;
    MIQ_CHECK_ARG(num_element == 0 || (x && grad_out && grad_in), "null pointer");
    EwPtrs<uint16_t, int32_t> p{x, grad_out, grad_in, nullptr};
    return launch_v2<uint16_t, OpV2Bwd>(p, v2_src(scale, offset, qmin, qmax), num_element, num_channel,
                                        num_element_per_channel, (hipStream_t) stream);
}

/* ---- several tensors in one launch ------------------------------------------------------------------------- */

int64_t miq_qdq_multi_plan(miq_qdq_segment* segments, int num_segments, int elem_bytes)
{
    if (!segments || num_segments < 1 || num_segments > kMaxSegments || (elem_bytes != 4 && elem_bytes != 2))
    {
        set_error("miq_qdq_multi_plan takes 1..%d segments of float32 (4) or bfloat16 (2) elements", kMaxSegments);
        return -1;
    }
    const int64_t tile = (int64_t) kBlock * kUnroll * (elem_bytes == 4 ? 4 : 8);
    int64_t tiles      = 0;
    for (int i = 0; i < num_segments; ++i)
    {
        miq_qdq_segment& g = segments[i];
        const bool ok = g.in && g.out && g.enc_min && g.enc_max && g.enc_delta && g.enc_offset && g.num_element > 0 &&
                        g.num_channel > 0 && g.num_element_per_channel > 0 && g.num_element < (1ll << 31) &&
                        g.num_channel < (1ll << 31) && aligned16(g.in) && aligned16(g.out) &&
                        tile / g.num_element_per_channel + 2 <= kWin;
        if (!ok)
        {
            set_error("segment %d cannot go into a multi-tensor launch (null or unaligned pointer, empty, 2^31 elements "
                      "or more, or fewer than %lld elements per channel): quantize it on its own", i,
                      (long long) (tile / (kWin - 2) + 1));
            return -1;
        }
        const FastDiv fd = make_fastdiv((uint32_t) g.num_element_per_channel);
        g.fd_magic       = fd.magic;
        g.fd_shift       = fd.shift;
        if (tiles >= (1ll << 31) - (g.num_element + tile - 1) / tile)
        {
            set_error("too many tiles for one launch");
            return -1;
        }
        g.first_tile = (int32_t) tiles;
        tiles += (g.num_element + tile - 1) / tile;
    }
    return tiles;
}

int miq_qdq_per_channel_multi_f32(const miq_qdq_segment* segments, int num_segments, int64_t total_tiles, void* stream)
{
    return qdq_multi<float>(segments, num_segments, total_tiles, stream);
}

int miq_qdq_per_channel_multi_bf16(const miq_qdq_segment* segments, int num_segments, int64_t total_tiles, void* stream)
{
    return qdq_multi<uint16_t>(segments, num_segments, total_tiles, stream);
}

/* ---- forward with the saved straight-through mask, backward from the mask ----------------------------------- */

int64_t miq_ste_mask_bytes(int64_t num_element, int elem_bytes)
{
    if (num_element < 0 || (elem_bytes != 4 && elem_bytes != 2))
        return -1;
    return 8 * (elem_bytes == 4 ? mask_words<4>(num_element) : mask_words<8>(num_element));
}

int miq_qdq_mask_per_tensor_f32(const float* in, float* out, uint64_t* mask, int64_t n, double enc_min, double enc_max,
                                int bw, float mask_min, float mask_max, void* stream)
{
    return qdq_mask_per_tensor<float>(in, out, mask, n, enc_min, enc_max, bw, mask_min, mask_max, stream);
}

int miq_qdq_mask_per_tensor_bf16(const uint16_t* in, uint16_t* out, uint64_t* mask, int64_t n, double enc_min,
                                 double enc_max, int bw, float mask_min, float mask_max, void* stream)
{
    return qdq_mask_per_tensor<uint16_t>(in, out, mask, n, enc_min, enc_max, bw, mask_min, mask_max, stream);
}

int miq_qdq_mask_per_channel_f32(const float* in, float* out, uint64_t* mask, int64_t num_channel, int64_t num_element,
                                 int64_t num_element_per_channel, const float* enc_min, const float* enc_max,
                                 const float* enc_delta, const float* enc_offset, const float* raw_min,
                                 const float* raw_max, void* stream)
{
    return qdq_mask_per_channel<float>(in, out, mask, num_channel, num_element, num_element_per_channel, enc_min,
                                       enc_max, enc_delta, enc_offset, raw_min, raw_max, stream);
}

int miq_qdq_mask_per_channel_bf16(const uint16_t* in, uint16_t* out, uint64_t* mask, int64_t num_channel,
                                  int64_t num_element, int64_t num_element_per_channel, const float* enc_min,
                                  const float* enc_max, const float* enc_delta, const float* enc_offset,
                                  const float* raw_min, const float* raw_max, void* stream)
{
    return qdq_mask_per_channel<uint16_t>(in, out, mask, num_channel, num_element, num_element_per_channel, enc_min,
                                          enc_max, enc_delta, enc_offset, raw_min, raw_max, stream);
}

int miq_v2_qdq_mask_f32(const float* in, float* out, uint64_t* mask, int64_t num_channel, int64_t num_element,
                        int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                        void* stream)
{
    return v2_qdq_mask<float>(in, out, mask, num_channel, num_element, num_element_per_channel, scale, offset, qmin,
                              qmax, stream);
}

int miq_v2_qdq_mask_bf16(const uint16_t* in, uint16_t* out, uint64_t* mask, int64_t num_channel, int64_t num_element,
                         int64_t num_element_per_channel, const float* scale, const float* offset, int qmin, int qmax,
                         void* stream)
{
    return v2_qdq_mask<uint16_t>(in, out, mask, num_channel, num_element, num_element_per_channel, scale, offset, qmin,
                                 qmax, stream);
}

int miq_ste_bwd_mask_f32(const uint64_t* mask, const float* grad_out, float* grad_in, int64_t n, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (mask && grad_out && grad_in)), "null tensor pointer or negative count");
    MIQ_CHECK_ARG((reinterpret_cast<uintptr_t>(mask) & 7u) == 0, "the mask must be 8-byte aligned");
    return launch_ste_mask_bwd<float>(mask, grad_out, grad_in, n, (hipStream_t) stream);
}

int miq_ste_bwd_mask_bf16(const uint64_t* mask, const uint16_t* grad_out, uint16_t* grad_in, int64_t n, void* stream)
{
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (mask && grad_out && grad_in)), "null tensor pointer or negative count");
    MIQ_CHECK_ARG((reinterpret_cast<uintptr_t>(mask) & 7u) == 0, "the mask must be 8-byte aligned");
    return launch_ste_mask_bwd<uint16_t>(mask, grad_out, grad_in, n, (hipStream_t) stream);
}

}   // extern "C"
