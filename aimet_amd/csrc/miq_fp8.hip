// Simulation of a narrow float grid: every element is rounded to the grid of a float format with M mantissa and E
// exponent bits (the 8-bit formats have E = 7 - M) whose largest value is the tensor's (or the channel's) maxval
// (TORCH/fp_quantization.py:133-209, quantize_to_fp8 / fake_cast_to_ieee_float; the v2 float quantizer calls the latter
// with any E and M: TORCH/v2/quantization/float/quantizer.py:302-322).  A float grid is an integer grid whose
// step depends on the element's own exponent:
//   x_c   = clamp(x, -maxval, maxval)
//   e     = max(floor(log2|x_c| + bias), 1)                    bias = 2^E - log2(maxval) + log2(2 - 2^-M) - 1
//   step  = 2^((e - M) - bias)
//   y     = round_half_even(x_c / step) * step
// in float32, one operation at a time and in this order, so that the result follows the reference's torch expression.
// e is an integer in [1, 2^E] (|x_c| <= maxval bounds it), so the steps of a channel form a table of 2^E + 1 floats:
// the caller computes bias and that table once per maxval (with the same float32 operations), and the kernel is left
// with a log2, a floor, one table read that hits the L1, a division and a rounding per element.  With pow() evaluated
// per element instead, the kernel ran at 1.8 TB/s, bound by the vector ALU.
//
// HBM-bound: 4 B read + 4 B written per element.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "miq_common.h"
#include "miq_fastmath.h"

namespace miq
{
namespace
{
__device__ __forceinline__ float fp8_elem(float x, float mx, float bias, const float* __restrict__ steps, int last)
{
    float xc = x != x ? x : fminf(fmaxf(x, -mx), mx);   // clamp that lets NaN through, as torch.clamp does
    float e  = fmaxf(floorf(log2f(fabsf(xc)) + bias), 1.0f);   // -inf (x = 0) and NaN end at 1
    int idx  = (int) fminf(e, (float) last);
    float st = steps[idx];
    return rintf(xc / st) * st;
}

// Rows of `inner4` 16-byte groups, row r belonging to channel r % channels: workgroup b takes piece b % pieces of row
// b / pieces, so the channel is found once per workgroup (the element-indexed kernel below divides twice in 64 bits
// per group of four, which made it ALU-bound at 56 % of HBM peak on [11008, 4096]).  The channel's steps go to LDS next
// to their reciprocals, and the division runs through div_by_invariant() when every step and maxval are inside its
// contract (a quotient below its 2^-36 limit rounds to zero either way).
constexpr int kFp8TableMax = 257;   // 2^8 + 1 steps: eight exponent bits (bfloat16's)
__global__ void __launch_bounds__(256) fp8_rows_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                        int64_t inner4, int64_t channels, int pieces,
                                                        const float* __restrict__ maxval,
                                                        const float* __restrict__ bias,
                                                        const float* __restrict__ steps, int table)
{
    typedef float vec4 __attribute__((ext_vector_type(4)));
    constexpr int kInFlight = 4;   // loads of a lane in flight before the first is used
    __shared__ float2 s_step[kFp8TableMax];
    const int64_t row  = blockIdx.x / (unsigned) pieces;
    const int piece    = (int) (blockIdx.x - row * pieces);
    const int64_t c    = row % channels;
    const vec4* src    = reinterpret_cast<const vec4*>(in) + row * inner4;
    vec4* dst          = reinterpret_cast<vec4*>(out) + row * inner4;
    const int64_t step = (int64_t) pieces * 256;
    int64_t j          = (int64_t) piece * 256 + threadIdx.x;
    vec4 v[kInFlight];
    auto request = [&]() {
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
            if (j + u * step < inner4)
                v[u] = __builtin_nontemporal_load(src + j + u * step);
    };
    request();   // the first loads travel while the channel's table is set up
    const float mx = maxval[c], b = bias[c];
    bool in_contract = true;
    for (int t = threadIdx.x; t < table; t += 256)
    {
        const float st = steps[c * table + t];
        s_step[t]      = make_float2(st, 1.0f / st);
        in_contract    = in_contract && fastdiv_divisor_ok(st);
    }
    const bool short_div = __syncthreads_and(in_contract) && mx <= kFastDivMaxDividend;
    const float last     = (float) (table - 1);
    auto elem = [&](float x) {
        const float xc = x != x ? x : fminf(fmaxf(x, -mx), mx);
        const float e  = fmaxf(floorf(log2f(fabsf(xc)) + b), 1.0f);
        const float2 s = s_step[(int) fminf(e, last)];
        const float q  = short_div ? div_by_invariant(xc, s.x, s.y) : xc / s.x;
        return rintf(q) * s.x;
    };
    while (true)
    {
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
            if (j + u * step < inner4)
            {
                v[u][0] = elem(v[u][0]);
                v[u][1] = elem(v[u][1]);
                v[u][2] = elem(v[u][2]);
                v[u][3] = elem(v[u][3]);
                __builtin_nontemporal_store(v[u], dst + j + u * step);
            }
        j += kInFlight * step;
        if (j >= inner4)
            break;
        request();
    }
}

// Elements are [outer][channels][inner]; a vector of four never straddles a channel when inner % 4 == 0.
template <bool VEC>
__global__ void __launch_bounds__(256) fp8_kernel(const float* __restrict__ in, float* __restrict__ out, int64_t n,
                                                   int64_t channels, int64_t inner, const float* __restrict__ maxval,
                                                   const float* __restrict__ bias,
                                                   const float* __restrict__ steps, int table)
{
    const int64_t stride = (int64_t) gridDim.x * blockDim.x;
    int64_t i            = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (VEC)
    {
        const int64_t nv = n >> 2;
        for (; i < nv; i += stride)
        {
            const int64_t c = channels == 1 ? 0 : ((i << 2) / inner) % channels;
            const float mx = maxval[c], b = bias[c];
            const float* st = steps + c * table;
            float4 v        = reinterpret_cast<const float4*>(in)[i];
            v.x             = fp8_elem(v.x, mx, b, st, table - 1);
            v.y             = fp8_elem(v.y, mx, b, st, table - 1);
            v.z             = fp8_elem(v.z, mx, b, st, table - 1);
            v.w             = fp8_elem(v.w, mx, b, st, table - 1);
            reinterpret_cast<float4*>(out)[i] = v;
        }
    }
    else
    {
        for (; i < n; i += stride)
        {
            const int64_t c = channels == 1 ? 0 : (i / inner) % channels;
            out[i]          = fp8_elem(in[i], maxval[c], bias[c], steps + c * table, table - 1);
        }
    }
}
}   // namespace
}   // namespace miq

extern "C" {

int miq_float_fake_cast_f32(const float* in, float* out, int64_t n, int64_t num_channels, int64_t inner,
                            const float* maxval, const float* bias, const float* steps, int table, void* stream)
{
    using namespace miq;
    MIQ_CHECK_ARG(n >= 0 && (n == 0 || (in && out && maxval && bias && steps)), "null tensor pointer or negative count");
    MIQ_CHECK_ARG(num_channels >= 1 && inner >= 1, "num_channels and inner must be positive");
    MIQ_CHECK_ARG(n % (num_channels * inner) == 0, "element count is not a multiple of num_channels * inner");
    MIQ_CHECK_ARG(table >= 3 && table <= kFp8TableMax, "the step table must hold 2^E + 1 entries, E in [1, 8] (got %d)",
                  table);
    if (n == 0)
        return MIQ_OK;
    const bool vec = (n % 4 == 0) && (num_channels == 1 || inner % 4 == 0) &&
                     ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) % 16 == 0);
    const int64_t work   = vec ? n / 4 : n;
    const int64_t blocks = (work + 255) / 256;
    const unsigned grid  = (unsigned) (blocks < 8192 ? blocks : 8192);
    // rows long enough to give every wavefront of a workgroup its own loads go by rows
    const int64_t row_len = num_channels == 1 ? n : inner;
    const int64_t rows    = n / row_len;
    if (vec && row_len >= 1024)
    {
        // four 16-byte groups per lane, and no more pieces than keep the grid near 16K workgroups
        const int64_t inner4 = row_len / 4;
        int64_t pieces       = (inner4 + 1023) / 1024;
        const int64_t most   = rows >= 16384 ? 1 : 16384 / rows;
        pieces               = pieces < most ? pieces : most;
        MIQ_CHECK_ARG(rows * pieces < (int64_t) 1 << 31, "too many rows");
        hipLaunchKernelGGL(fp8_rows_kernel, dim3((unsigned) (rows * pieces)), dim3(256), 0, (hipStream_t) stream, in, out,
                           inner4, num_channels, (int) pieces, maxval, bias, steps, table);
    }
    else if (vec)
        hipLaunchKernelGGL(fp8_kernel<true>, dim3(grid), dim3(256), 0, (hipStream_t) stream, in, out, n, num_channels,
                           inner, maxval, bias, steps, table);
    else
        hipLaunchKernelGGL(fp8_kernel<false>, dim3(grid), dim3(256), 0, (hipStream_t) stream, in, out, n,
                           num_channels, inner, maxval, bias, steps, table);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_fp8_fake_cast_f32(const float* in, float* out, int64_t n, int64_t num_channels, int64_t inner,
                          const float* maxval, const float* bias, const float* steps, int mantissa_bits, void* stream)
{
    MIQ_CHECK_ARG(mantissa_bits >= 1 && mantissa_bits <= 6, "mantissa_bits must be in [1, 6]");
    return miq_float_fake_cast_f32(in, out, n, num_channels, inner, maxval, bias, steps,
                                   (1 << (7 - mantissa_bits)) + 1, stream);
}

}   // extern "C"
