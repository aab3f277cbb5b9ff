// AdaRound kernels for gfx950: soft/hard rounding forward, and the fused backward that turns dL/dW' into the Adam
// update of alpha (rectified-sigmoid chain rule + rounding regulariser gradient + Adam step in one pass).
//
// Reference arithmetic (paths relative to the reference root,
// ADA = TrainingExtensions/torch/src/python/aimet_torch/v1/adaround):
//   apply_adaround              ADA/adaround_wrapper.py:124-149
//   _generate_alpha_parameter   ADA/adaround_wrapper.py:211-224
//   compute_round_loss          ADA/adaround_loss.py:82-111
//   optimiser step              torch.optim.Adam (single-tensor form), ADA/adaround_optimizer.py:157-218
//   constants zeta = 1.1, gamma = -0.1   TrainingExtensions/common/src/python/aimet_common/defs.py:302-306
//
// The reference runs about fifteen elementwise ATen kernels per iteration over weight-shaped tensors plus their
// autograd twins; here the forward is one pass (read W, alpha; write W') and the backward one pass (read dW', W,
// alpha, m, v; write alpha, m, v).
#include "miq_adaround_math.h"

#include <cmath>

namespace miq
{
namespace ada
{
int make_adam(AdamArgs& a, double reg_param, double beta, double lr, double beta1, double beta2, double eps, int step)
{
    a           = {};
    a.reg_param = (float) reg_param;
    a.beta      = (float) beta;
    a.pow_exp   = (double) (float) (beta - 1.0);
    if (step < 1)
        return MIQ_OK;
    MIQ_CHECK_ARG(beta1 >= 0.0 && beta1 < 1.0 && beta2 >= 0.0 && beta2 < 1.0, "Adam betas must lie in [0, 1)");
    MIQ_CHECK_ARG((float) (1.0 - beta1) < 0.5f, "beta1 must exceed 0.5 (the update uses lerp's small-weight form)");
    // Python-float arithmetic of torch/optim/adam.py, then the casts of the kernels that receive the scalars
    const double bc1 = 1.0 - std::pow(beta1, (double) step);
    const double bc2 = 1.0 - std::pow(beta2, (double) step);
    a.w1             = (float) (1.0 - beta1);
    a.beta2          = (float) beta2;
    a.c2             = (float) (1.0 - beta2);
    a.bc2_sqrt_rcp   = 1.0f / (float) std::pow(bc2, 0.5);
    a.eps            = (float) eps;
    a.neg_step       = (float) (-(lr / bc1));
    return MIQ_OK;
}
}   // namespace ada

namespace
{
using namespace ada;

struct AdaGeom
{
    int64_t n;
    uint32_t num_channel;
    FastDiv fd;          // elements per channel
    const float* delta;  // [num_channel]
    const float* offset; // [num_channel]
    float clip_min, clip_max;
};

__device__ __forceinline__ uint32_t channel_of(int64_t e, const AdaGeom& g)
{
    // e < 2^31 on this path (checked by the host)
    return fastdiv((uint32_t) e, g.fd) % g.num_channel;
}

template <bool SOFT>
__global__ __launch_bounds__(kBlock) void soft_round_kernel(const float* __restrict__ w, const float* __restrict__ alpha,
                                                            float* __restrict__ out, AdaGeom g)
{
    const int64_t nvec = g.n / 4;
    const int64_t v    = (int64_t) blockIdx.x * kBlock + threadIdx.x;
    if (v < nvec)
    {
        const float4 wv = reinterpret_cast<const float4*>(w)[v];
        const float4 av = reinterpret_cast<const float4*>(alpha)[v];
        const float ws[4] = {wv.x, wv.y, wv.z, wv.w};
        const float as[4] = {av.x, av.y, av.z, av.w};
        float ys[4];
        const uint32_t c0 = channel_of(v * 4, g), c3 = channel_of(v * 4 + 3, g);
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const uint32_t c = (c0 == c3) ? c0 : channel_of(v * 4 + j, g);
            ys[j] = adarounded<SOFT>(ws[j], as[j], g.delta[c], g.offset[c], g.clip_min, g.clip_max);
        }
        reinterpret_cast<float4*>(out)[v] = make_float4(ys[0], ys[1], ys[2], ys[3]);
    }
    if (blockIdx.x == 0 && threadIdx.x < (uint32_t) (g.n - nvec * 4))
    {
        const int64_t e  = nvec * 4 + threadIdx.x;
        const uint32_t c = channel_of(e, g);
        out[e] = adarounded<SOFT>(w[e], alpha[e], g.delta[c], g.offset[c], g.clip_min, g.clip_max);
    }
}

__global__ __launch_bounds__(kBlock) void floor_kernel(const float* __restrict__ w, float* __restrict__ out, AdaGeom g)
{
    for (int64_t e = (int64_t) blockIdx.x * kBlock + threadIdx.x; e < g.n; e += (int64_t) gridDim.x * kBlock)
        out[e] = floorf(w[e] / g.delta[channel_of(e, g)]);
}

// floor(w / delta) saturated to [offset + clip_min - 2, offset + clip_max + 1] and stored as int8 or int16.  Outside that window
// the value no longer matters: h(alpha) lies in [0, 1], so floor + h - offset stays below clip_min (resp. above
// clip_max) whatever alpha is, the clamp returns the same grid end and its gradient mask stays closed.  A channel whose
// window does not fit the integer type raises *unfit (the caller then takes the next wider form).
template <typename T, int LO, int HI>
__global__ __launch_bounds__(kBlock) void floor_int_kernel(const float* __restrict__ w, T* __restrict__ out, AdaGeom g,
                                                           int* __restrict__ unfit)
{
    for (int64_t e = (int64_t) blockIdx.x * kBlock + threadIdx.x; e < g.n; e += (int64_t) gridDim.x * kBlock)
    {
        const uint32_t c = channel_of(e, g);
        const float lo   = g.offset[c] + g.clip_min - 2.0f;
        const float hi   = g.offset[c] + g.clip_max + 1.0f;
        if (!(lo >= (float) LO && hi <= (float) HI))   // also true for NaN parameters
        {
            *unfit = 1;
            out[e] = 0;
            continue;
        }
        const float f = floorf(w[e] / g.delta[c]);
        out[e]        = (T) (int) fminf(fmaxf(f, lo), hi);   // NaN -> lo, as fmaxf drops it
    }
}

__global__ __launch_bounds__(kBlock) void init_alpha_kernel(const float* __restrict__ w, float* __restrict__ alpha,
                                                            AdaGeom g)
{
    for (int64_t e = (int64_t) blockIdx.x * kBlock + threadIdx.x; e < g.n; e += (int64_t) gridDim.x * kBlock)
    {
        const float d    = g.delta[channel_of(e, g)];
        const float s    = w[e] / d;
        const float frac = s - floorf(s);
        // alpha = -log((zeta - gamma) / (frac - gamma) - 1)
        alpha[e] = -logf(kZetaMinusGamma / (frac - kGamma) - 1.0f);
    }
}

// ADAM = true : alpha, m, v updated in place; grad_out (optional) receives dLoss/dalpha
// ADAM = false: grad_out receives dLoss/dalpha; alpha, m, v untouched (m, v may be null)
template <bool ADAM>
__global__ __launch_bounds__(kBlock) void bwd_kernel(const float* __restrict__ w, const float* __restrict__ gw,
                                                     float* __restrict__ alpha, float* __restrict__ m,
                                                     float* __restrict__ v, float* __restrict__ grad_out, AdaGeom g,
                                                     AdamArgs a, float* __restrict__ reg_partial)
{
    __shared__ PowEntry tab[128];
    PowTableLoad tl;
    tl.request();
    tl.store(tab);
    __syncthreads();
    const int64_t nvec = g.n / 4;
    const int64_t i    = (int64_t) blockIdx.x * kBlock + threadIdx.x;
    float reg          = 0.0f;
    if (i < nvec)
    {
        const float4 wv = reinterpret_cast<const float4*>(w)[i];
        const float4 gv = reinterpret_cast<const float4*>(gw)[i];
        const float4 av = reinterpret_cast<const float4*>(alpha)[i];
        float4 mv = make_float4(0, 0, 0, 0), vv = mv;
        if (ADAM)
        {
            mv = reinterpret_cast<const float4*>(m)[i];
            vv = reinterpret_cast<const float4*>(v)[i];
        }
        const uint32_t c0 = channel_of(i * 4, g), c3 = channel_of(i * 4 + 3, g);
        const float ws[4] = {wv.x, wv.y, wv.z, wv.w};
        const float gs[4] = {gv.x, gv.y, gv.z, gv.w};
        float as[4] = {av.x, av.y, av.z, av.w}, ms[4] = {mv.x, mv.y, mv.z, mv.w}, vs[4] = {vv.x, vv.y, vv.z, vv.w};
        float gr[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const uint32_t c = (c0 == c3) ? c0 : channel_of(i * 4 + j, g);
            float r;
            gr[j] = alpha_grad(ws[j], gs[j], as[j], g.delta[c], g.offset[c], g.clip_min, g.clip_max, a, tab, r);
            reg += r;
            if (ADAM)
                adam_update(gr[j], as[j], ms[j], vs[j], a);
        }
        if (ADAM)
        {
            reinterpret_cast<float4*>(alpha)[i] = make_float4(as[0], as[1], as[2], as[3]);
            reinterpret_cast<float4*>(m)[i]     = make_float4(ms[0], ms[1], ms[2], ms[3]);
            reinterpret_cast<float4*>(v)[i]     = make_float4(vs[0], vs[1], vs[2], vs[3]);
        }
        if (grad_out)
            reinterpret_cast<float4*>(grad_out)[i] = make_float4(gr[0], gr[1], gr[2], gr[3]);
    }
    if (blockIdx.x == 0 && threadIdx.x < (uint32_t) (g.n - nvec * 4))
    {
        const int64_t e  = nvec * 4 + threadIdx.x;
        const uint32_t c = channel_of(e, g);
        float r;
        const float gr = alpha_grad(w[e], gw[e], alpha[e], g.delta[c], g.offset[c], g.clip_min, g.clip_max, a, tab, r);
        reg += r;
        if (ADAM)
            adam_update(gr, alpha[e], m[e], v[e], a);
        if (grad_out)
            grad_out[e] = gr;
    }
    if (reg_partial)
    {
        // per-workgroup partial of the regulariser sum, combined in a fixed order by the caller (deterministic)
        const float t = block_sum_256(reg);
        if (threadIdx.x == 0)
            reg_partial[blockIdx.x] = t;
    }
}

// The kernels' own per-element terms for arrays of alpha (what = 0: sigmoid, h, dh/dalpha) or of h (what = 1:
// 1 - |2h - 1|^beta and its derivative with respect to h), for accuracy measurements against float64.
__global__ __launch_bounds__(kBlock) void eval_terms_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                            int64_t n, int what, AdamArgs a)
{
    __shared__ PowEntry tab[128];
    PowTableLoad tl;
    tl.request();
    tl.store(tab);
    __syncthreads();
    for (int64_t e = (int64_t) blockIdx.x * kBlock + threadIdx.x; e < n; e += (int64_t) gridDim.x * kBlock)
    {
        if (what == 0)
        {
            float sig, inner, ee, dh;
            soft_h(in[e], sig, inner, ee);
            const float h  = soft_h_grad(in[e], dh);
            out[e]         = sig;
            out[n + e]     = h;
            out[2 * n + e] = dh;
        }
        else
        {
            float dreg;
            out[e]     = reg_terms(in[e], a, tab, dreg);
            out[n + e] = dreg;
        }
    }
}

int make_geom(AdaGeom& g, int64_t num_channel, int64_t num_element, int64_t n_per_channel, const float* delta,
              const float* offset, float clip_min, float clip_max)
{
    MIQ_CHECK_ARG(num_channel > 0 && n_per_channel > 0 && num_element >= 0, "bad channel geometry");
    MIQ_CHECK_ARG(num_element < (1ll << 31) && n_per_channel < (1ll << 31) && num_channel < (1ll << 31),
                  "AdaRound kernels take tensors of fewer than 2^31 elements");
    MIQ_CHECK_ARG(delta && offset, "null delta/offset");
    MIQ_CHECK_ARG(clip_min <= clip_max, "clip_min must not exceed clip_max");
    g.n           = num_element;
    g.num_channel = (uint32_t) num_channel;
    g.fd          = make_fastdiv((uint32_t) n_per_channel);
    g.delta       = delta;
    g.offset      = offset;
    g.clip_min    = clip_min;
    g.clip_max    = clip_max;
    return MIQ_OK;
}

// relu as torch evaluates it: NaN stays NaN
__device__ __forceinline__ float relu_keep_nan(float v)
{
    return (v > 0.0f || v != v) ? v : 0.0f;
}

// dLoss/dout of the reconstruction loss for one sample row of `per_sample` elements per workgroup row: the target row
// is gathered from the cached outputs by the sample's number.  The operations, in the order autograd's backward of
// relu / sub / square / sum / mean performs them: (act(out) - act(target)) * scale, then * (act(out) > 0) under relu.
template <bool RELU, bool VEC>
__global__ __launch_bounds__(kBlock) void recon_grad_kernel(const float* __restrict__ out,
                                                            const float* __restrict__ target_all,
                                                            const int64_t* __restrict__ index, int64_t num_cached,
                                                            int64_t per_sample, float scale, float* __restrict__ grad)
{
    const int64_t sample = blockIdx.y;
    int64_t row          = index ? index[sample] : sample;
    row                  = row < 0 ? row + num_cached : row;    // as torch's indexing: negative numbers count from the end
    const bool bad_row   = row < 0 || row >= num_cached;        // no such sample: the row of results becomes NaN
    row                  = bad_row ? 0 : row;
    const float* o       = out + sample * per_sample;
    const float* t       = target_all + row * per_sample;
    float* g             = grad + sample * per_sample;
    constexpr int W      = VEC ? 4 : 1;
    for (int64_t i = ((int64_t) blockIdx.x * kBlock + threadIdx.x) * W; i < per_sample;
         i += (int64_t) gridDim.x * kBlock * W)
    {
        float ov[W], tv[W], gv[W];
        if (VEC)
        {
            const float4 a = *reinterpret_cast<const float4*>(o + i), b = *reinterpret_cast<const float4*>(t + i);
            ov[0] = a.x, ov[W > 1 ? 1 : 0] = a.y, ov[W > 1 ? 2 : 0] = a.z, ov[W > 1 ? 3 : 0] = a.w;
            tv[0] = b.x, tv[W > 1 ? 1 : 0] = b.y, tv[W > 1 ? 2 : 0] = b.z, tv[W > 1 ? 3 : 0] = b.w;
        }
        else
        {
            ov[0] = o[i];
            tv[0] = t[i];
        }
#pragma unroll
        for (int j = 0; j < W; ++j)
        {
            const float qa = RELU ? relu_keep_nan(ov[j]) : ov[j];
            const float ta = RELU ? relu_keep_nan(tv[j]) : tv[j];
            float v        = (qa - ta) * scale;
            if (RELU)
                v = v * (qa > 0.0f ? 1.0f : 0.0f);
            gv[j] = bad_row ? NAN : v;
        }
        if (VEC)
            *reinterpret_cast<float4*>(g + i) = make_float4(gv[0], gv[W > 1 ? 1 : 0], gv[W > 1 ? 2 : 0], gv[W > 1 ? 3 : 0]);
        else
            g[i] = gv[0];
    }
}

inline unsigned vec_blocks(int64_t n)
{
    int64_t nvec = n / 4;
    int64_t b    = (nvec + kBlock - 1) / kBlock;
    return (unsigned) (b < 1 ? 1 : b);
}
}   // namespace
}   // namespace miq

using namespace miq;

extern "C" {

int miq_adaround_blocks(int64_t num_element)
{
    return (int) vec_blocks(num_element);
}

int miq_adaround_soft_round_f32(const float* weight, const float* alpha, float* out, int64_t num_channel,
                                int64_t num_element, int64_t num_element_per_channel, const float* delta,
                                const float* offset, float clip_min, float clip_max, int use_soft_rounding,
                                void* stream)
{
    AdaGeom g;
    if (int rc = make_geom(g, num_channel, num_element, num_element_per_channel, delta, offset, clip_min, clip_max))
        return rc;
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(weight && alpha && out, "null tensor pointer");
    MIQ_CHECK_ARG(aligned16(weight) && aligned16(alpha) && aligned16(out), "tensors must be 16-byte aligned");
    if (use_soft_rounding)
        hipLaunchKernelGGL(soft_round_kernel<true>, dim3(vec_blocks(num_element)), dim3(kBlock), 0,
                           (hipStream_t) stream, weight, alpha, out, g);
    else
        hipLaunchKernelGGL(soft_round_kernel<false>, dim3(vec_blocks(num_element)), dim3(kBlock), 0,
                           (hipStream_t) stream, weight, alpha, out, g);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_floor_f32(const float* weight, float* weight_floor, int64_t num_channel, int64_t num_element,
                           int64_t num_element_per_channel, const float* delta, void* stream)
{
    AdaGeom g;
    if (int rc = make_geom(g, num_channel, num_element, num_element_per_channel, delta, delta, 0.f, 0.f))
        return rc;
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(weight && weight_floor, "null tensor pointer");
    int64_t blocks = (num_element + kBlock - 1) / kBlock;
    if (blocks > 65536)
        blocks = 65536;
    hipLaunchKernelGGL(floor_kernel, dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream, weight, weight_floor,
                       g);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_floor_i8(const float* weight, int8_t* weight_floor, int64_t num_channel, int64_t num_element,
                          int64_t num_element_per_channel, const float* delta, const float* offset, float clip_min,
                          float clip_max, int32_t* unfit, void* stream)
{
    AdaGeom g;
    if (int rc = make_geom(g, num_channel, num_element, num_element_per_channel, delta, offset, clip_min, clip_max))
        return rc;
    MIQ_CHECK_ARG(unfit, "null flag pointer");
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(weight && weight_floor, "null tensor pointer");
    int64_t blocks = (num_element + kBlock - 1) / kBlock;
    if (blocks > 65536)
        blocks = 65536;
    hipLaunchKernelGGL((floor_int_kernel<int8_t, -128, 127>), dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream, weight,
                       weight_floor, g, unfit);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_floor_i16(const float* weight, int16_t* weight_floor, int64_t num_channel, int64_t num_element,
                          int64_t num_element_per_channel, const float* delta, const float* offset, float clip_min,
                          float clip_max, int32_t* unfit, void* stream)
{
    AdaGeom g;
    if (int rc = make_geom(g, num_channel, num_element, num_element_per_channel, delta, offset, clip_min, clip_max))
        return rc;
    MIQ_CHECK_ARG(unfit, "null flag pointer");
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(weight && weight_floor, "null tensor pointer");
    int64_t blocks = (num_element + kBlock - 1) / kBlock;
    if (blocks > 65536)
        blocks = 65536;
    hipLaunchKernelGGL((floor_int_kernel<int16_t, -32768, 32767>), dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream, weight,
                       weight_floor, g, unfit);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_init_alpha_f32(const float* weight, float* alpha, int64_t num_channel, int64_t num_element,
                                int64_t num_element_per_channel, const float* delta, void* stream)
{
    AdaGeom g;
    if (int rc = make_geom(g, num_channel, num_element, num_element_per_channel, delta, delta, 0.f, 0.f))
        return rc;
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(weight && alpha, "null tensor pointer");
    int64_t blocks = (num_element + kBlock - 1) / kBlock;
    if (blocks > 65536)
        blocks = 65536;
    hipLaunchKernelGGL(init_alpha_kernel, dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream, weight, alpha,
                       g);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_bwd_f32(const float* weight, const float* grad_weight, const float* alpha, float* grad_alpha,
                         int64_t num_channel, int64_t num_element, int64_t num_element_per_channel,
                         const float* delta, const float* offset, float clip_min, float clip_max, double reg_param,
                         double beta, float* reg_partial, void* stream)
{
    AdaGeom g;
    if (int rc = make_geom(g, num_channel, num_element, num_element_per_channel, delta, offset, clip_min, clip_max))
        return rc;
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(weight && grad_weight && alpha && grad_alpha, "null tensor pointer");
    MIQ_CHECK_ARG(aligned16(weight) && aligned16(grad_weight) && aligned16(alpha) && aligned16(grad_alpha),
                  "tensors must be 16-byte aligned");
    AdamArgs a;
    if (int rc = make_adam(a, reg_param, beta, 0.0, 0.0, 0.0, 0.0, 0))
        return rc;
    hipLaunchKernelGGL(bwd_kernel<false>, dim3(vec_blocks(num_element)), dim3(kBlock), 0, (hipStream_t) stream, weight,
                       grad_weight, const_cast<float*>(alpha), (float*) nullptr, (float*) nullptr, grad_alpha, g, a,
                       reg_partial);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_bwd_adam_f32(const float* weight, const float* grad_weight, float* alpha, float* exp_avg,
                              float* exp_avg_sq, float* grad_alpha, int64_t num_channel, int64_t num_element,
                              int64_t num_element_per_channel, const float* delta, const float* offset, float clip_min,
                              float clip_max, double reg_param, double beta, double lr, double beta1, double beta2,
                              double eps, int step, float* reg_partial, void* stream)
{
    AdaGeom g;
    if (int rc = make_geom(g, num_channel, num_element, num_element_per_channel, delta, offset, clip_min, clip_max))
        return rc;
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(weight && grad_weight && alpha && exp_avg && exp_avg_sq, "null tensor pointer");
    MIQ_CHECK_ARG(aligned16(weight) && aligned16(grad_weight) && aligned16(alpha) && aligned16(exp_avg) &&
                      aligned16(exp_avg_sq) && aligned16(grad_alpha),
                  "tensors must be 16-byte aligned");
    MIQ_CHECK_ARG(step >= 1, "Adam step count starts at 1");
    AdamArgs a;
    if (int rc = make_adam(a, reg_param, beta, lr, beta1, beta2, eps, step))
        return rc;
    hipLaunchKernelGGL(bwd_kernel<true>, dim3(vec_blocks(num_element)), dim3(kBlock), 0, (hipStream_t) stream, weight,
                       grad_weight, alpha, exp_avg, exp_avg_sq, grad_alpha, g, a, reg_partial);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_recon_grad_f32(const float* out, const float* target, const int64_t* index, int64_t batch,
                                int64_t num_cached, int64_t per_sample, int activation, float scale, float* grad_out,
                                void* stream)
{
    MIQ_CHECK_ARG(batch >= 0 && batch <= 65535 && per_sample >= 0 && num_cached >= 1, "bad geometry");
    MIQ_CHECK_ARG(activation == 0 || activation == 1, "activation must be 0 (none) or 1 (ReLU)");
    MIQ_CHECK_ARG(index || num_cached >= batch, "without an index the target holds at least `batch` samples");
    if (batch == 0 || per_sample == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(out && target && grad_out, "null tensor pointer");
    const bool vec = per_sample % 4 == 0 && aligned16(out) && aligned16(target) && aligned16(grad_out);
    const int64_t per_block = (int64_t) kBlock * (vec ? 4 : 1);
    int64_t bx = (per_sample + per_block - 1) / per_block;
    bx         = bx > 1024 ? 1024 : bx;
    const dim3 grid((unsigned) bx, (unsigned) batch);
    hipStream_t s = (hipStream_t) stream;
#define MIQ_RECON(R, V)                                                                                                \
    hipLaunchKernelGGL((recon_grad_kernel<R, V>), grid, dim3(kBlock), 0, s, out, target, index, num_cached,            \
                       per_sample, scale, grad_out)
    if (activation == 1)
    {
        if (vec)
            MIQ_RECON(true, true);
        else
            MIQ_RECON(true, false);
    }
    else
    {
        if (vec)
            MIQ_RECON(false, true);
        else
            MIQ_RECON(false, false);
    }
#undef MIQ_RECON
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

int miq_adaround_eval_terms_f32(const float* in, float* out, int64_t num_element, int what, double beta, void* stream)
{
    MIQ_CHECK_ARG(num_element >= 0 && (what == 0 || what == 1), "what must be 0 (terms of alpha) or 1 (terms of h)");
    MIQ_CHECK_ARG(what == 0 || beta >= 1.0, "the regulariser's exponent must be at least 1");
    if (num_element == 0)
        return MIQ_OK;
    MIQ_CHECK_ARG(in && out, "null tensor pointer");
    AdamArgs a;
    if (int rc = make_adam(a, 1.0, beta, 0.0, 0.0, 0.0, 0.0, 0))
        return rc;
    int64_t blocks = (num_element + kBlock - 1) / kBlock;
    if (blocks > 4096)
        blocks = 4096;
    hipLaunchKernelGGL(eval_terms_kernel, dim3((unsigned) blocks), dim3(kBlock), 0, (hipStream_t) stream, in, out,
                       num_element, what, a);
    MIQ_CHECK_LAUNCH();
    return MIQ_OK;
}

}   // extern "C"
