// Per-element arithmetic of AdaRound shared by the elementwise kernels and the MFMA-fused Linear kernels, so that both
// paths produce the same adarounded weight and the same alpha gradient from the same inputs.
//
// Reference arithmetic (ADA = TrainingExtensions/torch/src/python/aimet_torch/v1/adaround):
//   h(alpha) = clamp(sigmoid(alpha) * (zeta - gamma) + gamma, 0, 1)          ADA/adaround_wrapper.py:136-139
//   W' = (clamp(floor(W / delta) + h - offset, clip_min, clip_max) + offset) * delta      :131-147
//   regulariser term 1 - |2h - 1|^beta                                       ADA/adaround_loss.py:100-106
//   Adam: torch.optim.Adam, single-tensor form, no weight decay, no amsgrad
//
// sigmoid and the power use the hardware's base-2 exponential / logarithm / reciprocal instructions (each accurate to
// about one ulp); sigmoid then differs from a libm-based float32 sigmoid by at most a few 1e-8 in absolute terms.  The
// division W / delta and everything that decides a clamp or a floor is IEEE-exact.
#ifndef MIQ_ADAROUND_MATH_H
#define MIQ_ADAROUND_MATH_H

#include "miq_common.h"

namespace miq
{
namespace ada
{
constexpr float kZetaMinusGamma = 1.2f;   // float32(1.1 - (-0.1)) = float32(1.2000000000000002)
constexpr float kGamma          = -0.1f;
constexpr float kLog2e          = 1.44269504088896340736f;

struct AdamArgs
{
    float reg_param;
    float beta;        // exponent of the regulariser; < 0 during warm start (no rounding loss)
    float lr_over_bc1; // lr / (1 - beta1^t)
    float inv_bc2_sqrt; // 1 / sqrt(1 - beta2^t)
    float beta1, beta2, eps;
};

__device__ __forceinline__ float sigmoid(float a)
{
    // 1 / (1 + 2^(-a log2 e)); 2^y overflows to +inf for a < -88 (result 0) and underflows to 0 for a > 88 (result 1)
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * a));
}

// x^p for 0 <= x <= 1 and p > 0
__device__ __forceinline__ float pow01(float x, float p)
{
    return __builtin_amdgcn_exp2f(p * __builtin_amdgcn_logf(x));
}

// h(alpha); `sig` and `inner` are the intermediate values the backward needs
__device__ __forceinline__ float soft_h(float alpha, float& sig, float& inner)
{
    sig   = sigmoid(alpha);
    inner = sig * kZetaMinusGamma + kGamma;
    return fminf(fmaxf(inner, 0.0f), 1.0f);
}

__device__ __forceinline__ float hard_h(float alpha)
{
    return alpha >= 0.0f ? 1.0f : 0.0f;
}

// `f` = floor(w / delta), an IEEE-exact division: it decides the grid point
template <bool SOFT>
__device__ __forceinline__ float adarounded_f(float f, float alpha, float d, float o, float clip_min, float clip_max)
{
    float sig, inner;
    const float h = SOFT ? soft_h(alpha, sig, inner) : hard_h(alpha);
    const float q = fminf(fmaxf(f + h - o, clip_min), clip_max);
    return (q + o) * d;
}

template <bool SOFT>
__device__ __forceinline__ float adarounded(float w, float alpha, float d, float o, float clip_min, float clip_max)
{
    return adarounded_f<SOFT>(floorf(w / d), alpha, d, o, clip_min, clip_max);
}

// dLoss/dalpha of one element from gw = dLoss_recon/dW': chain rule of `adarounded` (closed-interval clamp gradients,
// as torch.clamp) plus the gradient of reg_param * (1 - |2h - 1|^beta); `reg` receives this element's regulariser
// term (0 in warm start)
__device__ __forceinline__ float alpha_grad_f(float f, float gw, float alpha, float d, float o, float clip_min,
                                              float clip_max, const AdamArgs& a, float& reg)
{
    float sig, inner;
    const float h      = soft_h(alpha, sig, inner);
    const float t      = f + h - o;
    const float pass_q = (t >= clip_min && t <= clip_max) ? 1.0f : 0.0f;
    const float pass_h = (inner >= 0.0f && inner <= 1.0f) ? 1.0f : 0.0f;
    const float dsig   = (1.0f - sig) * sig;
    const float dh     = pass_h * kZetaMinusGamma * dsig;
    float grad         = gw * d * pass_q * dh;
    reg                = 0.0f;
    if (a.beta >= 0.0f)
    {
        const float x   = 2.0f * h - 1.0f;
        const float ax  = fabsf(x);
        // one power for both: |x|^beta = |x|^(beta - 1) * |x| (a logarithm and an exponential less per element)
        const float pm1 = (ax > 0.0f) ? pow01(ax, a.beta - 1.0f) : 0.0f;
        reg             = 1.0f - pm1 * ax;
        const float sgn = (x > 0.0f) ? 1.0f : ((x < 0.0f) ? -1.0f : 0.0f);
        const float dp  = a.beta * pm1;
        grad += -a.reg_param * dp * sgn * 2.0f * dh;
    }
    return grad;
}

__device__ __forceinline__ float alpha_grad(float w, float gw, float alpha, float d, float o, float clip_min,
                                            float clip_max, const AdamArgs& a, float& reg)
{
    return alpha_grad_f(floorf(w / d), gw, alpha, d, o, clip_min, clip_max, a, reg);
}

// lerp for the first moment, mul/addcmul for the second, as torch's single-tensor Adam orders them
__device__ __forceinline__ void adam_update(float grad, float& alpha, float& m, float& v, const AdamArgs& a)
{
    m = m + (1.0f - a.beta1) * (grad - m);
    v = v * a.beta2 + (1.0f - a.beta2) * grad * grad;
    // sqrt and the two divisions through the hardware's one-ulp sqrt / reciprocal: the step is lr-sized (1e-3), so the
    // last-bit differences against exact division are ~1e-10 in alpha
    const float denom = __builtin_amdgcn_sqrtf(v) * a.inv_bc2_sqrt + a.eps;
    alpha             = alpha - a.lr_over_bc1 * (m * __builtin_amdgcn_rcpf(denom));
}

// bias corrections in double, as the Python floats of torch.optim.Adam are
int make_adam(AdamArgs& a, float reg_param, float beta, float lr, float beta1, float beta2, float eps, int step);

// sum of `v` over the 256 threads of the block, returned in thread 0 (fixed order: deterministic)
__device__ __forceinline__ float block_sum_256(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o);
    __shared__ float s[4];
    if ((threadIdx.x & 63) == 0)
        s[threadIdx.x >> 6] = v;
    __syncthreads();
    return s[0] + s[1] + s[2] + s[3];
}

}   // namespace ada
}   // namespace miq
#endif
