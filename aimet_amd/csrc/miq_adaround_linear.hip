// AdaRound iteration of a Linear layer with the soft rounding fused into MFMA GEMMs (gfx950).
//
// Reference (ADA = TrainingExtensions/torch/src/python/aimet_torch/v1/adaround), one iteration of
// AdaroundOptimizer._optimize_rounding (ADA/adaround_optimizer.py:182-218) for torch.nn.Linear:
//   W'   = apply_adaround(W)                                   ADA/adaround_wrapper.py:124-149
//   out  = functional.linear(x[batch], W', bias)               ADA/adaround_optimizer.py:276-277
//   loss = recon_loss(act(out), act(y[batch])) + round_loss    ADA/adaround_loss.py:70-111
//   loss.backward(); Adam step on alpha
//
// With 32 rows per iteration the GEMMs are bandwidth-bound on the weight-shaped operands, so the point of fusing is
// that W' and dLoss/dW' never exist in memory:
//   (W enters as F = floor(W / delta), computed once per layer: W and delta do not change during the optimisation)
//   lin_fwd_kernel   reads F and alpha once, forms W' in registers and feeds it to 16x16x4 fp32 MFMAs as the B
//                    operand; the K dimension is split over workgroups, partial [32, O] products go to a workspace
//   lin_loss_kernel  adds the partials in a fixed order (deterministic), bias, activation, and writes
//                    G = dLoss_recon/dout = 2 (act(out) - act(y)) act'(out) / batch
//   lin_bwd_kernel   forms dLoss/dW'[o][k] = sum_b G[b][o] x[b][k] as a rank-32 MFMA product in registers and runs
//                    the alpha-gradient + regulariser + Adam epilogue on it (reads W, alpha, m, v; writes alpha, m, v)
//
// MFMA operand layout used below (v_mfma_f32_16x16x4_f32, one wavefront): lane l supplies A[m = l % 16][k = l / 16]
// and B[k = l / 16][n = l % 16]; it receives D[m = 4 (l / 16) + i][n = l % 16] in element i of the accumulator.
#include "miq_adaround_math.h"

namespace miq
{
namespace
{
using namespace ada;

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kBatch  = 32;    // rows per iteration (BATCH_SIZE of ADA/adaround_optimizer.py:58)
constexpr int kTileO  = 32;    // output channels per workgroup
constexpr int kTileK  = 256;   // K extent per workgroup: one 1 KiB row segment per wavefront-wide 16-byte access

struct LinGeom
{
    int out_features, in_features;
    int chan_stride;      // 1: delta/offset per output channel, 0: one entry for the whole tensor
    const float* delta;
    const float* offset;
    float clip_min, clip_max;
};

__device__ __forceinline__ v4f mfma16(float a, float b, v4f c)
{
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// Row of x / target for batch entry b.  An index outside [0, num_rows) is clamped so that the read stays inside the
// buffer; lin_loss_kernel marks such a row's results NaN.
__device__ __forceinline__ int64_t gather_row(const int* row_index, int b, int num_rows)
{
    const int r = row_index ? row_index[b] : b;
    return (int64_t) min(max(r, 0), num_rows - 1);
}

__device__ __forceinline__ v4f ldg4(const float* p)
{
    return *reinterpret_cast<const v4f*>(p);
}

__device__ __forceinline__ v4f ldg4_stream(const float* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
}

// Four consecutive values of floor(W / delta), stored as float32 or, where every channel's window of useful values fits,
// as int8 or int16 (miq_adaround_floor_i8 / _i16): a quarter or half of the bytes of the operand that never changes
// during the optimisation.
template <typename FT>
__device__ __forceinline__ v4f load_floor4(const FT* p);
template <>
__device__ __forceinline__ v4f load_floor4<float>(const float* p)
{
    return ldg4_stream(p);
}
template <>
__device__ __forceinline__ v4f load_floor4<int8_t>(const int8_t* p)
{
    const int32_t w = __builtin_nontemporal_load(reinterpret_cast<const int32_t*>(p));
    return (v4f) {(float) (int8_t) (w & 0xff), (float) (int8_t) ((w >> 8) & 0xff), (float) (int8_t) ((w >> 16) & 0xff),
                  (float) (w >> 24)};
}

template <>
__device__ __forceinline__ v4f load_floor4<int16_t>(const int16_t* p)
{
    typedef int v2i __attribute__((ext_vector_type(2)));
    const v2i w = __builtin_nontemporal_load(reinterpret_cast<const v2i*>(p));
    return (v4f) {(float) (int16_t) (w[0] & 0xffff), (float) (w[0] >> 16), (float) (int16_t) (w[1] & 0xffff),
                  (float) (w[1] >> 16)};
}

constexpr int kLdsRow = kTileK + 4;   // floats per LDS tile row; the pad spreads the MFMA-layout accesses over banks

// Both kernels work on a [32 o] x [256 k] tile of the weight-shaped tensors per workgroup and move it through LDS, so
// that global memory is always touched in the streaming layout (lane l of a wavefront owns floats 4l..4l+3 of a 1 KiB
// row segment: fully coalesced) while the MFMAs see their own operand / accumulator layout.
// (Measured alternative: wavefront-private [16 o] x [128 k] tiles without workgroup barriers were 10-20 % slower.)

// grid (K / 256, O / 32), 256 threads: consecutive workgroups walk along the rows, so the workgroups that run together
// cover contiguous memory (with the row blocks as the fast index the same tile reads measured 25 % slower).
template <typename FT>
__global__ __launch_bounds__(256) void lin_fwd_kernel(const FT* __restrict__ F, const float* __restrict__ alpha,
                                                      const float* __restrict__ X, const int* __restrict__ row_index,
                                                      int num_rows, int64_t x_row_stride, float* __restrict__ partial,
                                                      LinGeom g)
{
    __shared__ __attribute__((aligned(16))) float tile[kTileO * kLdsRow];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = lane & 15, s = lane >> 4;
    const int o_blk = blockIdx.y * kTileO;
    const int k_blk = blockIdx.x * kTileK;
    const int K     = g.in_features;

    // phase 1: adarounded weight tile, streaming layout: wavefront w forms rows 8w .. 8w+7
    // the rows' delta / offset are requested first: a load issued where it is used makes that row wait for a round trip
    float dl[8], of[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
    {
        const int c = (o_blk + wave * 8 + j) * g.chan_stride;
        dl[j]       = g.delta[c];
        of[j]       = g.offset[c];
    }
    v4f f[8], al[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
    {
        const int64_t e = (int64_t) (o_blk + wave * 8 + j) * K + k_blk + 4 * lane;
        f[j]            = load_floor4<FT>(F + e);
        al[j]           = ldg4_stream(alpha + e);
    }
    // the activations of this wavefront's MFMA k-range [64w, 64w + 64), fetched while the weights are in flight
    const float* xrow[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
    {
        const int b = mt * 16 + n;
        xrow[mt]    = X + gather_row(row_index, b, num_rows) * x_row_stride + k_blk + wave * 64 + 4 * s;
    }
    v4f a[4][2];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
            a[kk][mt] = ldg4(xrow[mt] + kk * 16);
#pragma unroll
    for (int j = 0; j < 8; ++j)
    {
        const int r = wave * 8 + j;
        v4f wq;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            wq[t] = adarounded_f<true>(f[j][t], al[j][t], dl[j], of[j], g.clip_min, g.clip_max);
        *reinterpret_cast<v4f*>(&tile[r * kLdsRow + 4 * lane]) = wq;
    }
    __syncthreads();

    // phase 2: out[b][o] += x[b][k] W'[o][k] over this wavefront's 64 k
    v4f acc[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            acc[mt][nt] = (v4f) {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
    {
        const int col = wave * 64 + kk * 16 + 4 * s;
        v4f wq[2];
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            wq[nt] = *reinterpret_cast<const v4f*>(&tile[(nt * 16 + n) * kLdsRow + col]);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
                    acc[mt][nt] = mfma16(a[kk][mt][t], wq[nt][t], acc[mt][nt]);
    }
    __syncthreads();   // every wavefront is done reading the weight tile: its memory now holds the partial products

    // add the four wavefronts' products in wavefront order, then one partial [32, 32] tile per workgroup
    v4f* red = reinterpret_cast<v4f*>(tile);   // [4 waves][4 tiles][64 lanes]
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            red[(wave * 4 + mt * 2 + nt) * 64 + lane] = acc[mt][nt];
    __syncthreads();
    {
        const int t4 = threadIdx.x >> 6, ln = threadIdx.x & 63;   // tile index, lane within the tile
        const v4f sum = ((red[(0 * 4 + t4) * 64 + ln] + red[(1 * 4 + t4) * 64 + ln]) + red[(2 * 4 + t4) * 64 + ln]) +
                        red[(3 * 4 + t4) * 64 + ln];
        const int mt = t4 >> 1, nt = t4 & 1;
        const int o  = o_blk + nt * 16 + (ln & 15);
        const int b0 = mt * 16 + 4 * (ln >> 4);
        float* dst   = partial + ((int64_t) blockIdx.x * kBatch + b0) * g.out_features + o;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            dst[(int64_t) i * g.out_features] = sum[i];
    }
}

// one thread per (b, o): out = sum_s partial[s][b][o] + bias[o]; G = 2 (act(out) - act(y)) act'(out) / batch
__global__ __launch_bounds__(256) void lin_loss_kernel(const float* __restrict__ partial, int num_split,
                                                       const float* __restrict__ bias, const float* __restrict__ Y,
                                                       const int* __restrict__ row_index, int num_rows,
                                                       int64_t y_row_stride, int out_features, int act, float* __restrict__ out,
                                                       float* __restrict__ G, float* __restrict__ loss_partial)
{
    const int idx = blockIdx.x * 256 + threadIdx.x;
    float sq      = 0.f;
    if (idx < kBatch * out_features)
    {
        const int b = idx / out_features, o = idx - b * out_features;
        float acc = 0.f;
        for (int s = 0; s < num_split; ++s)
            acc += partial[((int64_t) s * kBatch + b) * out_features + o];
        if (bias)
            acc += bias[o];
        const int r = row_index ? row_index[b] : b;
        float y     = Y[gather_row(row_index, b, num_rows) * y_row_stride + o];
        if (r < 0 || r >= num_rows)
            acc = NAN;   // no such row: poison everything derived from it
        if (out)
            out[idx] = acc;
        float pass = 1.f, ao = acc;
        if (act == 1)
        {
            pass = acc > 0.f ? 1.f : 0.f;
            ao   = fmaxf(acc, 0.f);
            y    = fmaxf(y, 0.f);
        }
        const float diff = ao - y;
        sq               = diff * diff;
        G[idx]           = (acc != acc) ? acc : 2.0f * diff * pass * (1.0f / kBatch);
    }
    if (loss_partial)
    {
        const float t = block_sum_256(sq);
        if (threadIdx.x == 0)
            loss_partial[blockIdx.x] = t * (1.0f / kBatch);
    }
}

// grid (K / 256, O / 32), 256 threads.  Phase 1: wavefront w forms dLoss/dW' for k in [64w, 64w + 64) as four 16-wide k
// tiles (the M dimension of the MFMA) by two 16-wide o tiles (N), the batch being the MFMA's K dimension (8 steps of
// 4), and parks it in the LDS tile.  Phase 2: the alpha-gradient + regulariser + Adam epilogue in the streaming layout.
template <int PF, typename FT>
__global__ __launch_bounds__(256) void lin_bwd_kernel(const FT* __restrict__ F, const float* __restrict__ G,
                                                      const float* __restrict__ X, const int* __restrict__ row_index,
                                                      int num_rows, int64_t x_row_stride, float* __restrict__ alpha,
                                                      float* __restrict__ m, float* __restrict__ v,
                                                      float* __restrict__ grad_out, LinGeom g, AdamArgs a,
                                                      float* __restrict__ reg_partial)
{
    __shared__ __attribute__((aligned(16))) float tile[kTileO * kLdsRow];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = lane & 15, s = lane >> 4;
    const int o_blk = blockIdx.y * kTileO;
    const int k_blk = blockIdx.x * kTileK;
    const int K = g.in_features, O = g.out_features;

    // the epilogue's first rows are requested before the MFMA phase so that they arrive while it runs
    v4f fv[PF], av[PF], mv[PF], vv[PF];
#pragma unroll
    for (int j = 0; j < PF; ++j)
    {
        const int64_t e = (int64_t) (o_blk + wave * 8 + j) * K + k_blk + 4 * lane;
        fv[j]           = load_floor4<FT>(F + e);
        av[j]           = ldg4(alpha + e);
        mv[j]           = ldg4(m + e);
        vv[j]           = ldg4(v + e);
    }

    float dl[8], of[8];   // per-row delta / offset, requested here and not where they are used (see lin_fwd_kernel)
#pragma unroll
    for (int j = 0; j < 8; ++j)
    {
        const int c = (o_blk + wave * 8 + j) * g.chan_stride;
        dl[j]       = g.delta[c];
        of[j]       = g.offset[c];
    }

    v4f acc[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            acc[mt][nt] = (v4f) {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int step = 0; step < 8; ++step)
    {
        const int b       = 4 * step + s;
        const float* xrow = X + gather_row(row_index, b, num_rows) * x_row_stride + k_blk + wave * 64 + n;
        const float* grow = G + (int64_t) b * O + o_blk + n;
        float xa[4], gb[2];
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
            xa[mt] = xrow[mt * 16];
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            gb[nt] = grow[nt * 16];
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int nt = 0; nt < 2; ++nt)
                acc[mt][nt] = mfma16(xa[mt], gb[nt], acc[mt][nt]);
    }
    // lane holds dW'[o = 16 nt + n][k = 64 w + 16 mt + 4 s + i], i = 0..3
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
            *reinterpret_cast<v4f*>(&tile[(nt * 16 + n) * kLdsRow + wave * 64 + mt * 16 + 4 * s]) = acc[mt][nt];
    __syncthreads();

    float reg = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j)
    {
        const int r     = wave * 8 + j;
        const int slot  = j % PF;
        const int64_t e = (int64_t) (o_blk + r) * K + k_blk + 4 * lane;
        const v4f f4 = fv[slot], a4 = av[slot], m4 = mv[slot], v4 = vv[slot];
        if (j + PF < 8)
        {
            const int64_t e2 = e + PF * (int64_t) K;
            fv[slot]         = load_floor4<FT>(F + e2);
            av[slot]         = ldg4(alpha + e2);
            mv[slot]         = ldg4(m + e2);
            vv[slot]         = ldg4(v + e2);
        }
        const float d = dl[j], off = of[j];
        const v4f gw  = *reinterpret_cast<const v4f*>(&tile[r * kLdsRow + 4 * lane]);
        float as[4] = {a4[0], a4[1], a4[2], a4[3]}, ms[4] = {m4[0], m4[1], m4[2], m4[3]};
        float vs[4] = {v4[0], v4[1], v4[2], v4[3]};
        v4f gr;
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            float rr;
            const float gi = alpha_grad_f(f4[i], gw[i], as[i], d, off, g.clip_min, g.clip_max, a, rr);
            reg += rr;
            adam_update(gi, as[i], ms[i], vs[i], a);
            gr[i] = gi;
        }
        *reinterpret_cast<v4f*>(alpha + e) = (v4f) {as[0], as[1], as[2], as[3]};
        *reinterpret_cast<v4f*>(m + e)     = (v4f) {ms[0], ms[1], ms[2], ms[3]};
        *reinterpret_cast<v4f*>(v + e)     = (v4f) {vs[0], vs[1], vs[2], vs[3]};
        if (grad_out)
            *reinterpret_cast<v4f*>(grad_out + e) = gr;
    }
    if (reg_partial)
    {
        const float t = block_sum_256(reg);
        if (threadIdx.x == 0)
            reg_partial[blockIdx.y * gridDim.x + blockIdx.x] = t;
    }
}

int make_lin_geom(LinGeom& g, int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                  const float* offset, float clip_min, float clip_max)
{
    MIQ_CHECK_ARG(out_features > 0 && in_features > 0, "bad layer shape");
    MIQ_CHECK_ARG(out_features % kTileO == 0 && in_features % kTileK == 0,
                  "the fused Linear path takes out_features that are a multiple of 32 and in_features that are a "
                  "multiple of 256 (got %lld x %lld)", (long long) out_features, (long long) in_features);
    MIQ_CHECK_ARG(out_features * in_features < (1ll << 31), "layer too large for the fused Linear path");
    MIQ_CHECK_ARG(num_channel == 1 || num_channel == out_features,
                  "delta/offset must have one entry, or one per output channel");
    MIQ_CHECK_ARG(delta && offset, "null delta/offset");
    MIQ_CHECK_ARG(clip_min <= clip_max, "clip_min must not exceed clip_max");
    g.out_features = (int) out_features;
    g.in_features  = (int) in_features;
    g.chan_stride  = num_channel == 1 ? 0 : 1;
    g.delta        = delta;
    g.offset       = offset;
    g.clip_min     = clip_min;
    g.clip_max     = clip_max;
    return MIQ_OK;
}
}   // namespace
}   // namespace miq

using namespace miq;

template <typename FT>
static int linear_fwd(const FT* weight_floor, const float* alpha, const float* x, const int32_t* row_index,
                      int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                      int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                      const float* offset, float clip_min, float clip_max, int activation, float* workspace, float* out,
                      float* grad_out, float* loss_partial, void* stream)
{
    LinGeom g;
    if (int rc = make_lin_geom(g, out_features, in_features, num_channel, delta, offset, clip_min, clip_max))
        return rc;
    MIQ_CHECK_ARG(weight_floor && alpha && x && target && workspace && grad_out, "null tensor pointer");
    MIQ_CHECK_ARG(aligned16(weight_floor) && aligned16(alpha) && aligned16(x) && (x_row_stride % 4) == 0,
                  "weight_floor, alpha and the rows of x must be 16-byte aligned");
    MIQ_CHECK_ARG(x_row_stride >= in_features && target_row_stride >= out_features, "row stride shorter than a row");
    MIQ_CHECK_ARG(activation == 0 || activation == 1, "activation must be 0 (none) or 1 (ReLU)");
    MIQ_CHECK_ARG(num_rows >= 1 && num_rows < (1ll << 31) && (row_index || num_rows >= kBatch),
                  "num_rows (%lld) must be positive, and at least 32 without a row index", (long long) num_rows);
    const int splits = (int) (in_features / kTileK);
    hipLaunchKernelGGL((lin_fwd_kernel<FT>), dim3((unsigned) splits, (unsigned) (out_features / kTileO)), dim3(256), 0,
                       (hipStream_t) stream, weight_floor, alpha, x, row_index, (int) num_rows, x_row_stride, workspace,
                       g);
    MIQ_CHECK_LAUNCH();
    const unsigned blocks = (unsigned) ((kBatch * out_features + 255) / 256);
    hipLaunchKernelGGL(lin_loss_kernel, dim3(blocks), dim3(256), 0, (hipStream_t) stream, workspace, splits, bias, target,
                       row_index, (int) num_rows, target_row_stride, (int) out_features, activation, out, grad_out,
                       loss_partial);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

template <typename FT>
static int linear_bwd_adam(const FT* weight_floor, const float* grad_out, const float* x, const int32_t* row_index,
                           int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg, float* exp_avg_sq, float* grad_alpha,
                           int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                           const float* offset, float clip_min, float clip_max, float reg_param, float beta, float lr,
                           float beta1, float beta2, float eps, int step, float* reg_partial, void* stream)
{
    LinGeom g;
    if (int rc = make_lin_geom(g, out_features, in_features, num_channel, delta, offset, clip_min, clip_max))
        return rc;
    MIQ_CHECK_ARG(weight_floor && grad_out && x && alpha && exp_avg && exp_avg_sq, "null tensor pointer");
    MIQ_CHECK_ARG(aligned16(weight_floor) && aligned16(alpha) && aligned16(exp_avg) && aligned16(exp_avg_sq) &&
                      aligned16(grad_alpha),
                  "tensors must be 16-byte aligned");
    MIQ_CHECK_ARG(x_row_stride >= in_features, "row stride shorter than a row");
    MIQ_CHECK_ARG(num_rows >= 1 && num_rows < (1ll << 31) && (row_index || num_rows >= kBatch),
                  "num_rows (%lld) must be positive, and at least 32 without a row index", (long long) num_rows);
    AdamArgs a;
    if (int rc = make_adam(a, reg_param, beta, lr, beta1, beta2, eps, step))
        return rc;
    // two rows of the epilogue in flight per lane: deeper prefetch (3, 4) costs registers and measured no faster
    hipLaunchKernelGGL((lin_bwd_kernel<2, FT>), dim3((unsigned) (in_features / kTileK), (unsigned) (out_features / kTileO)),
                       dim3(256), 0, (hipStream_t) stream, weight_floor, grad_out, x, row_index, (int) num_rows, x_row_stride, alpha,
                       exp_avg, exp_avg_sq, grad_alpha, g, a, reg_partial);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

extern "C" {

int64_t miq_adaround_linear_workspace_bytes(int64_t out_features, int64_t in_features)
{
    if (out_features <= 0 || in_features <= 0)
        return 0;
    const int64_t splits = (in_features + kTileK - 1) / kTileK;
    return splits * kBatch * out_features * (int64_t) sizeof(float);
}

int miq_adaround_linear_blocks(int64_t out_features, int64_t in_features)
{
    return (int) ((out_features / kTileO) * (in_features / kTileK));
}

int miq_adaround_linear_fwd_f32(const float* weight_floor, const float* alpha, const float* x, const int32_t* row_index,
                                int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride,
                                const float* bias, int64_t out_features, int64_t in_features, int64_t num_channel,
                                const float* delta, const float* offset, float clip_min, float clip_max,
                                int activation, float* workspace, float* out, float* grad_out, float* loss_partial,
                                void* stream)
{
    return linear_fwd<float>(weight_floor, alpha, x, row_index, num_rows, x_row_stride, target, target_row_stride, bias,
                             out_features, in_features, num_channel, delta, offset, clip_min, clip_max, activation,
                             workspace, out, grad_out, loss_partial, stream);
}

int miq_adaround_linear_fwd_i8(const int8_t* weight_floor, const float* alpha, const float* x, const int32_t* row_index,
                               int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                               int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                               const float* offset, float clip_min, float clip_max, int activation, float* workspace,
                               float* out, float* grad_out, float* loss_partial, void* stream)
{
    return linear_fwd<int8_t>(weight_floor, alpha, x, row_index, num_rows, x_row_stride, target, target_row_stride, bias,
                              out_features, in_features, num_channel, delta, offset, clip_min, clip_max, activation,
                              workspace, out, grad_out, loss_partial, stream);
}

int miq_adaround_linear_bwd_adam_f32(const float* weight_floor, const float* grad_out, const float* x,
                                     const int32_t* row_index, int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                     float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                     int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                     float clip_max, float reg_param, float beta, float lr, float beta1, float beta2,
                                     float eps, int step, float* reg_partial, void* stream)
{
    return linear_bwd_adam<float>(weight_floor, grad_out, x, row_index, num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq,
                                  grad_alpha, out_features, in_features, num_channel, delta, offset, clip_min, clip_max,
                                  reg_param, beta, lr, beta1, beta2, eps, step, reg_partial, stream);
}

int miq_adaround_linear_bwd_adam_i8(const int8_t* weight_floor, const float* grad_out, const float* x,
                                    const int32_t* row_index, int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                    float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                    int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                    float clip_max, float reg_param, float beta, float lr, float beta1, float beta2,
                                    float eps, int step, float* reg_partial, void* stream)
{
    return linear_bwd_adam<int8_t>(weight_floor, grad_out, x, row_index, num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq,
                                   grad_alpha, out_features, in_features, num_channel, delta, offset, clip_min,
                                   clip_max, reg_param, beta, lr, beta1, beta2, eps, step, reg_partial, stream);
}

int miq_adaround_linear_fwd_i16(const int16_t* weight_floor, const float* alpha, const float* x, const int32_t* row_index,
                               int64_t num_rows, int64_t x_row_stride, const float* target, int64_t target_row_stride, const float* bias,
                               int64_t out_features, int64_t in_features, int64_t num_channel, const float* delta,
                               const float* offset, float clip_min, float clip_max, int activation, float* workspace,
                               float* out, float* grad_out, float* loss_partial, void* stream)
{
    return linear_fwd<int16_t>(weight_floor, alpha, x, row_index, num_rows, x_row_stride, target, target_row_stride, bias,
                              out_features, in_features, num_channel, delta, offset, clip_min, clip_max, activation,
                              workspace, out, grad_out, loss_partial, stream);
}

int miq_adaround_linear_bwd_adam_i16(const int16_t* weight_floor, const float* grad_out, const float* x,
                                    const int32_t* row_index, int64_t num_rows, int64_t x_row_stride, float* alpha, float* exp_avg,
                                    float* exp_avg_sq, float* grad_alpha, int64_t out_features, int64_t in_features,
                                    int64_t num_channel, const float* delta, const float* offset, float clip_min,
                                    float clip_max, float reg_param, float beta, float lr, float beta1, float beta2,
                                    float eps, int step, float* reg_partial, void* stream)
{
    return linear_bwd_adam<int16_t>(weight_floor, grad_out, x, row_index, num_rows, x_row_stride, alpha, exp_avg, exp_avg_sq,
                                   grad_alpha, out_features, in_features, num_channel, delta, offset, clip_min,
                                   clip_max, reg_param, beta, lr, beta1, beta2, eps, step, reg_partial, stream);
}

}   // extern "C"
