// Backward of the v2 quantize-dequantize with learnable scale and offset, in one pass over x and grad.
//
// The reference forms three full-size intermediates and lets autograd reduce two of them to the parameter shape
// (TrainingExtensions/torch/src/python/aimet_torch/v2/quantization/affine/backends/torch_builtins.py:329-344):
//     q = x / scale;  r = round(q);  mask = qmin <= r - offset <= qmax
//     tensor_grad = grad * mask
//     scale_grad  = sum( grad * (clamp(r, offset + qmin, offset + qmax) - q * mask) )
//     offset_grad = sum( grad * (~mask * scale) )
// Here every element is read once: the workgroup streams a span of one channel row, writes tensor_grad, keeps the
// two sums in registers, and stores one (scale, offset) partial per workgroup.  A second small kernel adds the
// partials of each channel in double precision in a fixed order, so results do not depend on scheduling.
//
// Rows of at most kShortRow elements (blockwise scales, small convolution kernels) are given to groups of 1..64 lanes
// instead of whole workgroups: a group streams its row, the sums are combined with lane shuffles inside the group, and
// the group's first lane stores the row's pair.
//
// Layout: the tensor is [outer][channel][elements-per-channel] in memory (outer = 1 for weights quantized along
// axis 0, channel = 1 for per-tensor), so a "row" is one contiguous run that shares its parameters.
#include "miq_common.h"
#include "miq_fastmath.h"
#include "miq_io.h"

#include <algorithm>
#include <cmath>

namespace miq
{
namespace
{
struct LearnGeom
{
    uint32_t num_channel;
    uint32_t chunks;        // workgroups per row
    FastDiv chunks_div;
    int64_t npc;            // elements per row
    int64_t span;           // elements per workgroup (multiple of the vector width)
    int64_t rows;           // outer * num_channel
    uint32_t outer;
    bool direct;            // one workgroup per channel in total: its sums are the result, no second kernel
    // short rows: lane groups instead of workgroups
    bool short_rows;
    uint32_t lanes;             // lanes per row, a power of two in 1..64
    uint32_t lanes_log2;
    uint32_t rows_per_block;
};

constexpr int64_t kShortRow = 2048;

// What becomes of a channel's two sums.  mode < 0: they are the results (scale_grad, offset_grad).  Otherwise they
// are turned into the gradients of the encoding min / max the grid was made from, and those are stored in their place
// (the formulas are stated with the modes in miq.h).
struct RangeGrads
{
    int mode;
    const float* enc_min;
    const float* enc_max;
    float steps;        // qmax - qmin
    float steps_rcp;    // float32(1 / steps)
    float half_steps;   // steps div 2
};

__device__ __forceinline__ void store_sums(const RangeGrads& r, const float* __restrict__ scale, uint32_t ch,
                                           uint32_t at, float sum_s, float sum_o, float* __restrict__ out_a,
                                           float* __restrict__ out_b)
{
    if (r.mode < 0)
    {
        if (out_a)
            out_a[at] = sum_s;
        if (out_b)
            out_b[at] = sum_o;
        return;
    }
    const float mn = r.enc_min[ch], mx = r.enc_max[ch];
    float gmin, gmax;
    switch (r.mode)
    {
    case MIQ_RANGE_V2_ASYMMETRIC:
    {
        const float sc = scale[ch];
        const float s  = sum_s + -sum_o * ((mn / sc) / sc);
        gmax           = s * r.steps_rcp;
        gmin           = sum_o / sc + -gmax;
        break;
    }
    case MIQ_RANGE_V2_SYMMETRIC:
        gmax = sum_s * r.steps_rcp;
        gmin = -gmax;
        break;
    case MIQ_RANGE_V1_ASYMMETRIC:
    {
        const float t1 = sum_s / r.steps;
        const float d  = mx - mn;
        const float t2 = r.steps / (d * d) * sum_o;
        gmin           = -t1 + mx * t2;
        gmax           = t1 - mn * t2;
        break;
    }
    default:   // the two v1 symmetric modes
        gmax = sum_s / r.half_steps;
        gmin = -gmax;
        break;
    }
    out_a[at] = gmin;
    out_b[at] = gmax;
}

struct LearnParams
{
    float scale, offset, rcp, lo, hi, qmin, qmax;
};

__device__ __forceinline__ LearnParams load_params(const float* scale, const float* offset, uint32_t ch, int qmin,
                                                   int qmax)
{
    LearnParams p;
    p.scale  = scale[ch];
    p.offset = offset[ch];
    p.rcp    = fastdiv_divisor_ok(p.scale) ? 1.0f / p.scale : 0.0f;
    p.qmin   = (float) qmin;
    p.qmax   = (float) qmax;
    p.lo     = p.offset + p.qmin;
    p.hi     = p.offset + p.qmax;
    return p;
}

// one element: returns tensor_grad, adds this element's terms to the two sums
template <bool FAST>
__device__ __forceinline__ float learn_elem(const LearnParams& p, float x, float g, float& sg, float& og)
{
    const float q   = FAST ? div_by_invariant(x, p.scale, p.rcp) : x / p.scale;
    const float r   = rintf(q);
    const float rm  = r - p.offset;
    const bool in   = (p.qmin <= rm) && (rm <= p.qmax);
    const float m   = in ? 1.0f : 0.0f;
    float c         = r;   // torch.clamp: NaN stays NaN
    c               = (c < p.lo) ? p.lo : c;
    c               = (c > p.hi) ? p.hi : c;
    sg += g * (c - q * m);
    og += g * ((1.0f - m) * p.scale);
    return g * m;
}

// one vector already in registers: the exact-division fast path is decided once for the vector
template <int V>
__device__ __forceinline__ void learn_vec_regs(const LearnParams& p, const float* xf, const float* gf, float* of,
                                               float& sg, float& og)
{
    float m = 0.0f;
#pragma unroll
    for (int j = 0; j < V; ++j)
        m = fmaxf(m, fabsf(xf[j]));
    if (p.rcp != 0.0f && m <= kFastDivMaxDividend)
    {
#pragma unroll
        for (int j = 0; j < V; ++j)
            of[j] = learn_elem<true>(p, xf[j], gf[j], sg, og);
    }
    else
    {
#pragma unroll
        for (int j = 0; j < V; ++j)
            of[j] = learn_elem<false>(p, xf[j], gf[j], sg, og);
    }
}

template <typename IO, bool WRITE_GX>
__device__ __forceinline__ void learn_vec(const LearnParams& p, const IO* x, const IO* g, IO* gx, int64_t at,
                                          float& sg, float& og)
{
    using T = IOTraits<IO>;
    float xf[T::VEC], gf[T::VEC], of[T::VEC];
    T::unpack(stream_load(reinterpret_cast<const typename T::Vec*>(x + at)), xf);
    T::unpack(stream_load(reinterpret_cast<const typename T::Vec*>(g + at)), gf);
    learn_vec_regs<T::VEC>(p, xf, gf, of, sg, og);
    if (WRITE_GX)
        stream_store(reinterpret_cast<typename T::Vec*>(gx + at), T::pack(of));
}

template <typename IO, bool VECTOR, bool WRITE_GX>
__global__ __launch_bounds__(kBlock) void learn_bwd_kernel(const IO* __restrict__ x, const IO* __restrict__ g,
                                                           IO* __restrict__ gx, const float* __restrict__ scale,
                                                           const float* __restrict__ offset, int qmin, int qmax,
                                                           LearnGeom geo, float2* __restrict__ partial,
                                                           float* __restrict__ scale_grad,
                                                           float* __restrict__ offset_grad, RangeGrads range)
{
    using T              = IOTraits<IO>;
    const uint32_t row   = fastdiv(blockIdx.x, geo.chunks_div);
    const uint32_t chunk = blockIdx.x - row * geo.chunks;
    const LearnParams p  = load_params(scale, offset, row % geo.num_channel, qmin, qmax);
    const int64_t first  = (int64_t) chunk * geo.span;
    const int64_t len    = min(geo.span, geo.npc - first);
    const int64_t base   = (int64_t) row * geo.npc + first;
    float sg = 0.0f, og = 0.0f;
    if (VECTOR)
    {
        // len and base are multiples of the vector width on this path (checked by the host)
        constexpr int64_t kStep = (int64_t) kBlock * T::VEC;
        int64_t i               = (int64_t) threadIdx.x * T::VEC;
        // two vectors per array in flight before the arithmetic starts, and the next pair of each array requested
        // before this pair's results are stored: loads and stores complete in one order, so a load requested after a
        // store cannot be used before that store has finished its trip to memory
        typedef typename T::Vec Vec;
        Vec nxa, nxb, nga, ngb;
        auto request = [&](int64_t at) {
            nxa = stream_load(reinterpret_cast<const Vec*>(x + base + at));
            nxb = stream_load(reinterpret_cast<const Vec*>(x + base + at + kStep));
            nga = stream_load(reinterpret_cast<const Vec*>(g + base + at));
            ngb = stream_load(reinterpret_cast<const Vec*>(g + base + at + kStep));
        };
        // The wait for a requested pair is placed by hand, where the number of younger stores is known (none before
        // the loop, this iteration's two at its end): left to the first use at the top of the loop, it would have to
        // cover both ways into the loop and would wait for the stores as well.
        auto arrived = [&]() {
            asm volatile("" : "+v"(nxa.x), "+v"(nxa.y), "+v"(nxa.z), "+v"(nxa.w), "+v"(nxb.x), "+v"(nxb.y), "+v"(nxb.z),
                         "+v"(nxb.w));
            asm volatile("" : "+v"(nga.x), "+v"(nga.y), "+v"(nga.z), "+v"(nga.w), "+v"(ngb.x), "+v"(ngb.y), "+v"(ngb.z),
                         "+v"(ngb.w));
        };
        bool have = i + kStep < len;
        if (have)
        {
            request(i);
            arrived();
        }
        while (have)
        {
            float xa[T::VEC], ga[T::VEC], xb[T::VEC], gb[T::VEC], oa[T::VEC], ob[T::VEC];
            T::unpack(nxa, xa);
            T::unpack(nxb, xb);
            T::unpack(nga, ga);
            T::unpack(ngb, gb);
            const int64_t i_next = i + 2 * kStep;
            have                 = i_next + kStep < len;
            if (have)
                request(i_next);
            float m = 0.0f;
#pragma unroll
            for (int j = 0; j < T::VEC; ++j)
                m = fmaxf(m, fmaxf(fabsf(xa[j]), fabsf(xb[j])));
            if (p.rcp != 0.0f && m <= kFastDivMaxDividend)
            {
#pragma unroll
                for (int j = 0; j < T::VEC; ++j)
                {
                    oa[j] = learn_elem<true>(p, xa[j], ga[j], sg, og);
                    ob[j] = learn_elem<true>(p, xb[j], gb[j], sg, og);
                }
            }
            else
            {
#pragma unroll
                for (int j = 0; j < T::VEC; ++j)
                {
                    oa[j] = learn_elem<false>(p, xa[j], ga[j], sg, og);
                    ob[j] = learn_elem<false>(p, xb[j], gb[j], sg, og);
                }
            }
            if (WRITE_GX)
            {
                stream_store(reinterpret_cast<Vec*>(gx + base + i), T::pack(oa));
                stream_store(reinterpret_cast<Vec*>(gx + base + i + kStep), T::pack(ob));
            }
            if (have)
                arrived();
            i = i_next;
        }
        if (i < len)
            learn_vec<IO, WRITE_GX>(p, x, g, gx, base + i, sg, og);
    }
    else
    {
        for (int64_t i = threadIdx.x; i < len; i += kBlock)
        {
            const float o = learn_elem<false>(p, T::load1(x + base + i), T::load1(g + base + i), sg, og);
            if (WRITE_GX)
                T::store1(gx + base + i, o);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        sg += __shfl_xor(sg, o);
        og += __shfl_xor(og, o);
    }
    __shared__ float2 wave_sum[kBlock / 64];
    if ((threadIdx.x & 63) == 0)
        wave_sum[threadIdx.x >> 6] = make_float2(sg, og);
    __syncthreads();
    if (threadIdx.x == 0)
    {
        float a = 0.0f, b = 0.0f;
#pragma unroll
        for (int w = 0; w < kBlock / 64; ++w)
        {
            a += wave_sum[w].x;
            b += wave_sum[w].y;
        }
        if (geo.direct)   // one workgroup per channel, outer == 1: the block number is the channel
            store_sums(range, scale, blockIdx.x, blockIdx.x, a, b, scale_grad, offset_grad);
        else
            partial[blockIdx.x] = make_float2(a, b);
    }
}

// Adds the partial pairs of each channel (outer x chunks of them) in double: LANES lanes per channel (a wavefront,
// or the whole workgroup when a channel has many pairs), each lane a strided share in index order, then a fixed
// tree over the lanes -- the result does not depend on scheduling.
template <int LANES>
__global__ __launch_bounds__(kBlock) void learn_reduce_kernel(const float2* __restrict__ partial, LearnGeom geo,
                                                              const float* __restrict__ scale,
                                                              float* __restrict__ scale_grad,
                                                              float* __restrict__ offset_grad, RangeGrads range)
{
    constexpr int kPerBlock = kBlock / LANES;
    const uint32_t ch       = blockIdx.x * kPerBlock + threadIdx.x / LANES;
    const uint32_t lane     = threadIdx.x % LANES;
    double a = 0.0, b = 0.0;
    if (ch < geo.num_channel)
    {
        const uint32_t items = geo.outer * geo.chunks;
        for (uint32_t j = lane; j < items; j += LANES)
        {
            const uint32_t o = fastdiv(j, geo.chunks_div);
            const uint32_t k = j - o * geo.chunks;
            const float2 v   = partial[((int64_t) o * geo.num_channel + ch) * geo.chunks + k];
            a += (double) v.x;
            b += (double) v.y;
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        a += __shfl_xor(a, o);
        b += __shfl_xor(b, o);
    }
    if (LANES > 64)
    {
        __shared__ double wave_sum[2][kBlock / 64];
        if ((threadIdx.x & 63) == 0)
        {
            wave_sum[0][threadIdx.x >> 6] = a;
            wave_sum[1][threadIdx.x >> 6] = b;
        }
        __syncthreads();
        a = b = 0.0;
#pragma unroll
        for (int w = 0; w < kBlock / 64; ++w)
        {
            a += wave_sum[0][w];
            b += wave_sum[1][w];
        }
    }
    if (lane == 0 && ch < geo.num_channel)
        store_sums(range, scale, ch, ch, (float) a, (float) b, scale_grad, offset_grad);
}

// Short rows.  A group of geo.lanes lanes owns a row at a time; a workgroup owns rows_per_block consecutive rows, so
// what it reads and writes is one contiguous stretch.  Two rows are in flight per group.  partial has one pair per
// row (chunks == 1), or, when outer == 1, the sums go straight to scale_grad / offset_grad.
template <typename IO, bool VECTOR, bool WRITE_GX>
__global__ __launch_bounds__(kBlock) void learn_rows_kernel(const IO* __restrict__ x, const IO* __restrict__ g,
                                                            IO* __restrict__ gx, const float* __restrict__ scale,
                                                            const float* __restrict__ offset, int qmin, int qmax,
                                                            LearnGeom geo, float2* __restrict__ partial,
                                                            float* __restrict__ scale_grad,
                                                            float* __restrict__ offset_grad, RangeGrads range)
{
    using T                 = IOTraits<IO>;
    constexpr int V         = VECTOR ? T::VEC : 1;
    const uint32_t lane     = threadIdx.x & (geo.lanes - 1);
    const uint32_t group    = threadIdx.x >> geo.lanes_log2;
    const uint32_t groups   = kBlock >> geo.lanes_log2;
    const int64_t row_begin = (int64_t) blockIdx.x * geo.rows_per_block;
    const int64_t row_end   = min(row_begin + (int64_t) geo.rows_per_block, geo.rows);
    const int64_t stride    = (int64_t) geo.lanes * V;
    for (int64_t row0 = row_begin + group; row0 < row_end; row0 += 2 * groups)
    {
        float sg[2] = {0.0f, 0.0f}, og[2] = {0.0f, 0.0f};
        const int64_t row1 = row0 + groups;
        const bool two     = row1 < row_end;   // uniform over the group
        const LearnParams p0 = load_params(scale, offset, (uint32_t) (row0 % geo.num_channel), qmin, qmax);
        const LearnParams p1 =
            load_params(scale, offset, (uint32_t) ((two ? row1 : row0) % geo.num_channel), qmin, qmax);
        for (int64_t i = (int64_t) lane * V; i < geo.npc; i += stride)
        {
            if (VECTOR)
            {
                float xa[V], ga[V], xb[V], gb[V], oa[V], ob[V];
                const int64_t at0 = row0 * geo.npc + i, at1 = row1 * geo.npc + i;
                T::unpack(stream_load(reinterpret_cast<const typename T::Vec*>(x + at0)), xa);
                T::unpack(stream_load(reinterpret_cast<const typename T::Vec*>(g + at0)), ga);
                if (two)
                {
                    T::unpack(stream_load(reinterpret_cast<const typename T::Vec*>(x + at1)), xb);
                    T::unpack(stream_load(reinterpret_cast<const typename T::Vec*>(g + at1)), gb);
                }
                learn_vec_regs<V>(p0, xa, ga, oa, sg[0], og[0]);
                if (WRITE_GX)
                    stream_store(reinterpret_cast<typename T::Vec*>(gx + at0), T::pack(oa));
                if (two)
                {
                    learn_vec_regs<V>(p1, xb, gb, ob, sg[1], og[1]);
                    if (WRITE_GX)
                        stream_store(reinterpret_cast<typename T::Vec*>(gx + at1), T::pack(ob));
                }
            }
            else
            {
                const int64_t at0 = row0 * geo.npc + i, at1 = row1 * geo.npc + i;
                const float xa = T::load1(x + at0), ga = T::load1(g + at0);
                const float xb = two ? T::load1(x + at1) : 0.0f, gb = two ? T::load1(g + at1) : 0.0f;
                const float oa = learn_elem<false>(p0, xa, ga, sg[0], og[0]);
                if (WRITE_GX)
                    T::store1(gx + at0, oa);
                if (two)
                {
                    const float ob = learn_elem<false>(p1, xb, gb, sg[1], og[1]);
                    if (WRITE_GX)
                        T::store1(gx + at1, ob);
                }
            }
        }
        // every lane of the group is here (lanes past the end of a short row hold zeros)
        for (uint32_t o = geo.lanes >> 1; o > 0; o >>= 1)
        {
            sg[0] += __shfl_xor(sg[0], o);
            og[0] += __shfl_xor(og[0], o);
            sg[1] += __shfl_xor(sg[1], o);
            og[1] += __shfl_xor(og[1], o);
        }
        if (lane == 0)
        {
#pragma unroll
            for (int k = 0; k < 2; ++k)
            {
                if (k == 1 && !two)
                    break;
                const int64_t row = k ? row1 : row0;
                if (geo.direct)   // outer == 1: the row number is the channel
                    store_sums(range, scale, (uint32_t) row, (uint32_t) row, sg[k], og[k], scale_grad, offset_grad);
                else
                    partial[row] = make_float2(sg[k], og[k]);
            }
        }
    }
}

// rows, chunks and span for a tensor of num_channel x npc rows repeated `outer` times
int make_learn_geom(int64_t num_channel, int64_t n, int64_t npc, int vec, LearnGeom& geo, int64_t& outer)
{
    MIQ_CHECK_ARG(num_channel >= 1 && npc >= 1 && n >= 0, "non-positive channel geometry");
    MIQ_CHECK_ARG(num_channel <= 0x7fffffff, "too many channels");
    MIQ_CHECK_ARG(n % (num_channel * npc) == 0, "num_element is not a multiple of num_channel * elements per channel");
    outer    = n / (num_channel * npc);
    geo.rows = outer * num_channel;
    geo.npc  = npc;
    geo.num_channel = (uint32_t) num_channel;
    geo.outer      = (uint32_t) outer;
    geo.short_rows = npc <= kShortRow;
    if (geo.short_rows)
    {
        // lanes per row: enough to cover the row with one vector (or element) each, at most a wavefront
        const int64_t per_lane = (npc % vec == 0) ? vec : 1;
        uint32_t lanes = 1, log2 = 0;
        while (lanes < 64 && (int64_t) lanes * per_lane < npc)
        {
            lanes <<= 1;
            ++log2;
        }
        geo.lanes      = lanes;
        geo.lanes_log2 = log2;
        // about 8192 elements per workgroup, in whole passes of two rows per group; fewer when the tensor is small
        const int64_t groups = kBlock / lanes;
        int64_t rows_pb      = 2 * groups * std::max<int64_t>(1, 8192 / (2 * groups * npc));
        while (rows_pb > 2 * groups && (geo.rows + rows_pb - 1) / rows_pb < 2048)
            rows_pb -= 2 * groups;
        geo.rows_per_block = (uint32_t) rows_pb;
        geo.span           = npc;
        geo.chunks         = 1;
        geo.chunks_div     = make_fastdiv(1);
        geo.direct         = outer == 1;
        MIQ_CHECK_ARG((geo.rows + rows_pb - 1) / rows_pb < 0x7fffffff, "tensor too large for one launch");
        return MIQ_OK;
    }
    // Spans of 8192 elements keep partials few; shorter ones when that would leave compute units idle.
    int64_t span = 8192;
    while (span > 2048 && geo.rows * ((npc + span - 1) / span) < 2048)
        span /= 2;
    const int64_t chunks = (npc + span - 1) / span;
    MIQ_CHECK_ARG(geo.rows * chunks < 0x7fffffff, "tensor too large for one launch");
    geo.span       = span;
    geo.chunks     = (uint32_t) chunks;
    geo.chunks_div = make_fastdiv((uint32_t) chunks);
    geo.direct     = outer == 1 && chunks == 1;
    return MIQ_OK;
}

template <typename IO>
int launch_learn(const IO* x, const IO* g, IO* gx, int64_t num_channel, int64_t n, int64_t npc, const float* scale,
                 const float* offset, int qmin, int qmax, float* scale_grad, float* offset_grad, void* workspace,
                 hipStream_t stream, const RangeGrads& range)
{
    MIQ_CHECK_ARG(scale && offset, "null parameter pointer");
    MIQ_CHECK_ARG(qmin <= qmax, "qmin must not exceed qmax");
    MIQ_CHECK_ARG(scale_grad || offset_grad, "neither scale_grad nor offset_grad requested");
    const bool vector = npc % IOTraits<IO>::VEC == 0 && aligned16(x) && aligned16(g) && (!gx || aligned16(gx));
    LearnGeom geo{};
    int64_t outer = 0;
    if (int rc = make_learn_geom(num_channel, n, npc, vector ? IOTraits<IO>::VEC : 1, geo, outer))
        return rc;
    MIQ_CHECK_ARG(n == 0 || (x && g && workspace), "null pointer");
    float2* partial = static_cast<float2*>(workspace);
    // an empty tensor launches only the reduction, which then writes the zero sums
    if (n > 0)
    {
#define MIQ_LEARN(KERNEL, V, W)                                                                                        \
    KERNEL<IO, V, W><<<grid, kBlock, 0, stream>>>(x, g, gx, scale, offset, qmin, qmax, geo, partial, scale_grad,       \
                                                  offset_grad, range)
#define MIQ_LEARN_VARIANTS(KERNEL)                                                                                     \
    if (vector && gx)                                                                                                  \
        MIQ_LEARN(KERNEL, true, true);                                                                                 \
    else if (vector)                                                                                                   \
        MIQ_LEARN(KERNEL, true, false);                                                                                \
    else if (gx)                                                                                                       \
        MIQ_LEARN(KERNEL, false, true);                                                                                \
    else                                                                                                               \
        MIQ_LEARN(KERNEL, false, false)
        if (geo.short_rows)
        {
            const dim3 grid((uint32_t) ((geo.rows + geo.rows_per_block - 1) / geo.rows_per_block));
            MIQ_LEARN_VARIANTS(learn_rows_kernel);
        }
        else
        {
            const dim3 grid((uint32_t) (geo.rows * geo.chunks));
            MIQ_LEARN_VARIANTS(learn_bwd_kernel);
        }
#undef MIQ_LEARN_VARIANTS
#undef MIQ_LEARN
        MIQ_CHECK_LAUNCH();
    }
    if (!geo.direct)
    {
        if ((int64_t) geo.outer * geo.chunks >= 1024)
            learn_reduce_kernel<kBlock><<<dim3(geo.num_channel), kBlock, 0, stream>>>(partial, geo, scale, scale_grad,
                                                                                      offset_grad, range);
        else
            learn_reduce_kernel<64><<<dim3((geo.num_channel + 3) / 4), kBlock, 0, stream>>>(
                partial, geo, scale, scale_grad, offset_grad, range);
        MIQ_CHECK_LAUNCH();
    }
    return MIQ_OK;
}
constexpr RangeGrads kNoRange = {-1, nullptr, nullptr, 0.f, 0.f, 0.f};

int make_range(RangeGrads& r, int mode, int qmin, int qmax, const float* grid, int64_t num_channel)
{
    MIQ_CHECK_ARG(mode >= MIQ_RANGE_V2_ASYMMETRIC && mode <= MIQ_RANGE_V1_UNSIGNED_SYMMETRIC, "unknown range mode %d",
                  mode);
    MIQ_CHECK_ARG(qmin < qmax, "qmin must be below qmax");
    MIQ_CHECK_ARG(mode < MIQ_RANGE_V1_ASYMMETRIC || qmin == 0, "the v1 grids start at 0 (qmin = %d)", qmin);
    MIQ_CHECK_ARG((int64_t) qmax - qmin < (1 << 24), "grid too wide for float32 (%d..%d)", qmin, qmax);
    r.mode       = mode;
    r.enc_min    = grid ? grid + 2 * num_channel : nullptr;
    r.enc_max    = grid ? grid + 3 * num_channel : nullptr;
    r.steps      = (float) (qmax - qmin);
    r.steps_rcp  = 1.0f / r.steps;
    r.half_steps = (float) ((qmax - qmin) / 2);
    return MIQ_OK;
}

// torch.clamp / torch.maximum keep NaN
__device__ __forceinline__ float max_keep_nan(float a, float b)
{
    return (a != a || b != b) ? NAN : fmaxf(a, b);
}

// One thread per channel: the range is put in order (gate), copied, and turned into scale and offset.
__global__ __launch_bounds__(kBlock) void range_to_grid_kernel(float* __restrict__ enc_min, float* __restrict__ enc_max,
                                                               int num_channel, float qmin, RangeGrads r, bool gate,
                                                               float* __restrict__ grid)
{
    const int ch = blockIdx.x * kBlock + threadIdx.x;
    if (ch >= num_channel)
        return;
    float mn = enc_min[ch], mx = enc_max[ch];
    if (gate)
    {
        mn = (mn > 0.0f) ? 0.0f : mn;   // clamp_(max=0): a NaN compares false and stays
        mx = (mx < 0.0f) ? 0.0f : mx;
        mx = max_keep_nan(mx, mn + 1e-5f);
        enc_min[ch] = mn;
        enc_max[ch] = mx;
    }
    float scale, offset;
    switch (r.mode)
    {
    case MIQ_RANGE_V2_ASYMMETRIC:
        scale  = (mx - mn) * r.steps_rcp;
        offset = rintf(mn / scale) - qmin;
        break;
    case MIQ_RANGE_V2_SYMMETRIC:
        scale  = (mx - mn) * r.steps_rcp;
        offset = 0.0f;
        break;
    case MIQ_RANGE_V1_ASYMMETRIC:
    {
        scale   = (mx - mn) / r.steps;
        float z = rintf(-mn / scale);                 // torch.min(steps, torch.max(0, z)): NaN stays
        z       = max_keep_nan(0.0f, z);
        z       = (z != z) ? z : fminf(r.steps, z);
        offset  = -z;
        break;
    }
    case MIQ_RANGE_V1_SIGNED_SYMMETRIC:
        scale  = mx / r.half_steps;                   // floor(steps / 2)
        offset = -(r.steps - r.half_steps);           // -ceil(steps / 2)
        break;
    default:   // MIQ_RANGE_V1_UNSIGNED_SYMMETRIC
        scale  = (mx - mn) / r.steps;
        offset = mn / scale;
        break;
    }
    grid[ch]                   = scale;
    grid[num_channel + ch]     = offset;
    grid[2 * num_channel + ch] = mn;
    grid[3 * num_channel + ch] = mx;
}
template <typename IO>
int bwd_range(const IO* x, const IO* grad_out, IO* grad_in, int64_t num_channel, int64_t num_element,
                     int64_t num_element_per_channel, const float* grid, int qmin, int qmax, int mode, float* grad_min,
                     float* grad_max, void* workspace, void* stream)
{
    MIQ_CHECK_ARG(grid && grad_min && grad_max, "null pointer");
    MIQ_CHECK_ARG(num_channel >= 1, "bad channel count");
    RangeGrads r;
    if (int rc = make_range(r, mode, qmin, qmax, grid, num_channel))
        return rc;
    return launch_learn<IO>(x, grad_out, grad_in, num_channel, num_element, num_element_per_channel, grid,
                            grid + num_channel, qmin, qmax, grad_min, grad_max, workspace, (hipStream_t) stream, r);
}

}   // namespace
}   // namespace miq

using namespace miq;

extern "C" {

int64_t miq_v2_qdq_bwd_params_workspace_bytes(int64_t num_channel, int64_t num_element,
                                              int64_t num_element_per_channel)
{
    LearnGeom geo{};
    int64_t outer = 0;
    if (make_learn_geom(num_channel, num_element, num_element_per_channel, 1, geo, outer) != MIQ_OK)
        return 0;
    const int64_t blocks = geo.rows * geo.chunks;
    return (int64_t) sizeof(float2) * (blocks > 0 ? blocks : 1);
}

int miq_v2_qdq_bwd_params_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                              int64_t num_element, int64_t num_element_per_channel, const float* scale,
                              const float* offset, int qmin, int qmax, float* scale_grad, float* offset_grad,
                              void* workspace, void* stream)
{
    return launch_learn<float>(x, grad_out, grad_in, num_channel, num_element, num_element_per_channel, scale, offset,
                               qmin, qmax, scale_grad, offset_grad, workspace, (hipStream_t) stream, kNoRange);
}

int miq_v2_qdq_bwd_params_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t num_channel,
                               int64_t num_element, int64_t num_element_per_channel, const float* scale,
                               const float* offset, int qmin, int qmax, float* scale_grad, float* offset_grad,
                               void* workspace, void* stream)
{
    return launch_learn<uint16_t>(x, grad_out, grad_in, num_channel, num_element, num_element_per_channel, scale,
                                  offset, qmin, qmax, scale_grad, offset_grad, workspace, (hipStream_t) stream,
                                  kNoRange);
}

int miq_range_to_grid_f32(float* enc_min, float* enc_max, int64_t num_channel, int qmin, int qmax, int mode, int gate,
                          float* grid, void* stream)
{
    MIQ_CHECK_ARG(num_channel >= 1 && num_channel <= 0x7fffffff, "bad channel count %lld", (long long) num_channel);
    MIQ_CHECK_ARG(enc_min && enc_max && grid, "null pointer");
    RangeGrads r;
    if (int rc = make_range(r, mode, qmin, qmax, nullptr, num_channel))
        return rc;
    const dim3 blocks((uint32_t) ((num_channel + kBlock - 1) / kBlock));
    range_to_grid_kernel<<<blocks, kBlock, 0, (hipStream_t) stream>>>(enc_min, enc_max, (int) num_channel,
                                                                      (float) qmin, r, gate != 0, grid);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_qdq_bwd_range_f32(const float* x, const float* grad_out, float* grad_in, int64_t num_channel,
                          int64_t num_element, int64_t num_element_per_channel, const float* grid, int qmin, int qmax,
                          int mode, float* grad_min, float* grad_max, void* workspace, void* stream)
{
    return bwd_range<float>(x, grad_out, grad_in, num_channel, num_element, num_element_per_channel, grid, qmin, qmax,
                            mode, grad_min, grad_max, workspace, stream);
}

int miq_qdq_bwd_range_bf16(const uint16_t* x, const uint16_t* grad_out, uint16_t* grad_in, int64_t num_channel,
                           int64_t num_element, int64_t num_element_per_channel, const float* grid, int qmin,
                           int qmax, int mode, float* grad_min, float* grad_max, void* workspace, void* stream)
{
    return bwd_range<uint16_t>(x, grad_out, grad_in, num_channel, num_element, num_element_per_channel, grid, qmin,
                               qmax, mode, grad_min, grad_max, workspace, stream);
}

}   // extern "C"
