// Per-element arithmetic of AdaRound shared by the elementwise kernels and the MFMA-fused Linear kernels, so that both
// paths produce the same adarounded weight and the same alpha gradient from the same inputs.
//
// Reference arithmetic (ADA = TrainingExtensions/torch/src/python/aimet_torch/v1/adaround):
//   h(alpha) = clamp(sigmoid(alpha) * (zeta - gamma) + gamma, 0, 1)          ADA/adaround_wrapper.py:136-139
//   W' = (clamp(floor(W / delta) + h - offset, clip_min, clip_max) + offset) * delta      :131-147
//   regulariser term 1 - |2h - 1|^beta                                       ADA/adaround_loss.py:100-106
//   Adam: torch.optim.Adam, single-tensor form, no weight decay, no amsgrad
//
// Accuracy of the transcendental parts against float64 evaluated on the same float32 inputs (measured through
// miq_adaround_eval_terms_f32; tests/test_gpu_adaround.py states the bounds next to what torch's float32 CPU ops reach):
//   h(alpha)         within 1.6 ulp(1) absolutely: sigmoid through the hardware's base-2 exponential and reciprocal
//                    (one ulp each)
//   dh/dalpha        from sigmoid(alpha) sigmoid(-alpha) without the cancellation of (1 - sigmoid) sigmoid
//   |x|^p            <= 2 ulp: log2 |x| in double from a 128-entry table (exact argument reduction m * inv - 1) and a
//                    cubic, p log2 |x| in double, the hardware's base-2 exponential on its fraction.  (The plain
//                    exp2(p log2 x) on float32 is off by up to 150 ulp for p = 19: the logarithm's rounding times p.)
// The division W / delta and everything that decides a clamp or a floor is IEEE-exact.
#ifndef MIQ_ADAROUND_MATH_H
#define MIQ_ADAROUND_MATH_H

#include "miq_common.h"
#include "miq_pow_table.h"

namespace miq
{
namespace ada
{
constexpr float kZetaMinusGamma = 1.2f;   // float32(1.1 - (-0.1)) = float32(1.2000000000000002)
constexpr float kGamma          = -0.1f;

// Hyper-parameters of one launch, prepared on the host (make_adam) as torch's CPU kernels see them: the Python floats
// of torch.optim.Adam stay double until the kernel that uses them casts them to the tensor's float32.
struct AdamArgs
{
    float reg_param;
    float beta;           // exponent of the regulariser; < 0 during warm start (no rounding loss)
    double pow_exp;       // double(float32(beta - 1)): the exponent torch's pow backward uses
    float w1;             // float32(1 - beta1), the weight of exp_avg.lerp_(grad, 1 - beta1)
    float beta2;          // float32(beta2)
    float c2;             // float32(1 - beta2)
    float bc2_sqrt_rcp;   // 1 / float32(sqrt(1 - beta2^t))
    float eps;
    float neg_step;       // float32(-(lr / (1 - beta1^t)))
};

constexpr float kLog2e = 1.44269504088896340736f;

// sigmoid(a) = r = 1 / (1 + e), e = 2^(-a log2 e); e is handed back because sigmoid's derivative is e r r.
// e overflows to +inf for a < -88 (r = 0) and underflows to 0 for a > 88 (r = 1).
__device__ __forceinline__ float sigmoid(float a, float& e)
{
    e = __builtin_amdgcn_exp2f(-kLog2e * a);
    return __builtin_amdgcn_rcpf(1.0f + e);
}

// ---- x^p for 0 < x <= 1 and p > 0 -----------------------------------------------------------------------------------
struct PowEntry
{
    double inv;   // float32(1 / mid_j): m * inv is exact in double for a float32 mantissa m
    double lg;    // log2(inv / 2)
};
static __device__ const PowEntry kPowTable[128] = {MIQ_POW_TABLE_ENTRIES};

// Workgroup-wide copy of the table into LDS (2 KiB); the caller passes a barrier before the first pow01.  The load
// is issued by `request` (place it with the kernel's first loads) and parked by `store`.
struct PowTableLoad
{
    PowEntry e;
    __device__ __forceinline__ void request()
    {
        if (threadIdx.x < 128)
            e = kPowTable[threadIdx.x];
    }
    __device__ __forceinline__ void store(PowEntry* lds) const
    {
        if (threadIdx.x < 128)
            lds[threadIdx.x] = e;
    }
};

// x^p for x = 1 or 2^-24 <= x < 1 (what |2h - 1| can be for a float32 h in [0, 1]) and p >= 1.
// log2 x = -n + log2 2m, x = 2^-n (2m) with m in [0.5, 1) and n >= 0 taken apart by integer operations;
// log2 2m = log2(1 + r) - lg_j, r = m inv_j - 1 (exact), |r| <= 2^-8: the series to r^3 leaves 2^-32 of it.  y = p log2 x in double is split into
// an integer and a fraction of at most one half; the hardware exponential takes the fraction rounded to float32
// (0.35 ulp of the result), ldexp the integer.
__device__ __forceinline__ float pow01(float x, double p, const PowEntry* __restrict__ tab)
{
    constexpr double c1 = 1.4426950408889634074, c2 = -0.7213475204444817037, c3 = 0.4808983469629878025;
    constexpr double kTwo52 = 4503599627370496.0, kRound = 6755399441055744.0;   // 2^52, 2^52 + 2^51
    const uint32_t xb = __float_as_uint(x);
    const PowEntry t  = tab[(xb >> 16) & 127u];
    // (double) m built from the bits (binary64 exponent field 1022)
    const uint32_t m_hi = ((xb & 0x007fffffu) >> 3) | 0x3fe00000u;
    const uint32_t m_lo = xb << 29;
    const double m      = __hiloint2double((int) m_hi, (int) m_lo);
    const int n         = 127 - (int) (xb >> 23);   // 0 for x = 1 (m = 0.5, 2m = 1)
    const double nd     = __hiloint2double(0x43300000, n) - kTwo52;   // (double) n for 0 <= n < 2^32
    const double r      = __builtin_fma(m, t.inv, -1.0);
    const double q      = r * __builtin_fma(r, __builtin_fma(r, c3, c2), c1);
    const double y      = p * ((q - t.lg) - nd);
    const double tt     = y + kRound;
    const double f      = y - (tt - kRound);
    return __builtin_amdgcn_ldexpf(__builtin_amdgcn_exp2f((float) f), __double2loint(tt));
}

// h(alpha); `inner` is the value before the clamp to [0, 1], `e` as sigmoid() returns it
__device__ __forceinline__ float soft_h(float alpha, float& sig, float& inner, float& e)
{
    sig   = sigmoid(alpha, e);
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
    float sig, inner, e;
    const float h = SOFT ? soft_h(alpha, sig, inner, e) : hard_h(alpha);
    const float q = fminf(fmaxf(f + h - o, clip_min), clip_max);
    return (q + o) * d;
}

template <bool SOFT>
__device__ __forceinline__ float adarounded(float w, float alpha, float d, float o, float clip_min, float clip_max)
{
    return adarounded_f<SOFT>(floorf(w / d), alpha, d, o, clip_min, clip_max);
}

// The soft-rounding terms of one element: h(alpha) and dh/dalpha (closed-interval clamp gradient, as torch.clamp).
// sigmoid' = sigmoid(alpha) sigmoid(-alpha) = e r r is formed from the factors themselves: the reference's
// (1 - sigmoid) sigmoid on a float32 sigmoid cancels up to four bits where the clamp is open (sigmoid up to 11/12).
__device__ __forceinline__ float soft_h_grad(float alpha, float& dh)
{
    float sig, inner, e;
    const float h    = soft_h(alpha, sig, inner, e);
    const float dsig = (e * sig) * sig;   // NaN where e is infinite: outside the clamp's open range, dropped below
    dh               = (inner >= 0.0f && inner <= 1.0f) ? kZetaMinusGamma * dsig : 0.0f;
    return h;
}

// The regulariser's terms of one element: returns 1 - |2h - 1|^beta and sets
// dreg = d/dh of it = -beta |2h - 1|^(beta - 1) sgn(2h - 1) 2.  One power serves both: |x|^beta = |x|^(beta - 1) |x|.
__device__ __forceinline__ float reg_terms(float h, const AdamArgs& a, const PowEntry* __restrict__ tab, float& dreg)
{
    const float x   = 2.0f * h - 1.0f;
    const float ax  = fabsf(x);
    const float pm1 = (ax > 0.0f) ? pow01(ax, a.pow_exp, tab) : 0.0f;
    // -(beta pm1) sgn(x) 2: the factors +-1 and 2 are exact; x = 0 gives pm1 = 0
    dreg            = copysignf(a.beta * pm1 * 2.0f, -x);
    return 1.0f - pm1 * ax;
}

// dLoss/dalpha of one element from gw = dLoss_recon/dW': chain rule of `adarounded` (closed-interval clamp gradients,
// as torch.clamp) plus the gradient of reg_param * (1 - |2h - 1|^beta); `reg` receives this element's regulariser
// term (0 in warm start).  `tab`: the workgroup's LDS copy of kPowTable (not read in warm start).
__device__ __forceinline__ float alpha_grad_f(float f, float gw, float alpha, float d, float o, float clip_min,
                                              float clip_max, const AdamArgs& a, const PowEntry* __restrict__ tab,
                                              float& reg)
{
    float dh;
    const float h      = soft_h_grad(alpha, dh);
    const float t      = f + h - o;
    float grad         = (t >= clip_min && t <= clip_max) ? gw * d * dh : 0.0f;
    reg                = 0.0f;
    if (a.beta >= 0.0f)
    {
        float dreg;
        reg = reg_terms(h, a, tab, dreg);
        grad += a.reg_param * dreg * dh;
    }
    return grad;
}

__device__ __forceinline__ float alpha_grad(float w, float gw, float alpha, float d, float o, float clip_min,
                                            float clip_max, const AdamArgs& a, const PowEntry* __restrict__ tab,
                                            float& reg)
{
    return alpha_grad_f(floorf(w / d), gw, alpha, d, o, clip_min, clip_max, a, tab, reg);
}

// torch.optim.Adam's single-tensor update as its CPU kernels evaluate it (torch/optim/adam.py _single_tensor_adam):
//   exp_avg.lerp_(grad, 1 - beta1)                                fma(w, grad - m, m)   (weight < 0.5)
//   exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)  fma(c grad, grad, v beta2)
//   denom = (exp_avg_sq.sqrt() / bias_correction2_sqrt).add_(eps)
//   param.addcdiv_(exp_avg, denom, value=-step_size)              param + (value exp_avg) / denom
// Both moments come out bit for bit.  The square root and the two divisions go through the hardware's one-ulp
// sqrt / reciprocal: that moves the lr-sized step by a few 1e-7 of itself, so alpha equals the exactly divided
// result except where that lands across a rounding boundary of alpha (about one element in a thousand, by one ulp).
// IEEE-exact forms of the three cost 3 us per launch on the [4096, 4096] layer.
__device__ __forceinline__ void adam_update(float grad, float& alpha, float& m, float& v, const AdamArgs& a)
{
    m = fmaf(a.w1, grad - m, m);
    v = fmaf(a.c2 * grad, grad, v * a.beta2);
    const float denom = __builtin_amdgcn_sqrtf(v) * a.bc2_sqrt_rcp + a.eps;
    alpha             = alpha + (a.neg_step * m) * __builtin_amdgcn_rcpf(denom);
}

// bias corrections in double, as the Python floats of torch.optim.Adam are
// `step` < 1: the regulariser's parameters only (no update follows)
int make_adam(AdamArgs& a, double reg_param, double beta, double lr, double beta1, double beta2, double eps, int step);

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
