// getComputedEncodings (ModelOptimizations/DlQuantization/src/quantization_utils.cpp:58-143) in one place for the host
// entry point and for the kernel that computes the encodings of all channels of a tensor on the device.  Every
// operation is an IEEE double operation (add, multiply, divide, floor, ceil, round-half-away, compare), which host and
// device evaluate identically.
#ifndef MIQ_ENCODING_MATH_H
#define MIQ_ENCODING_MATH_H

#include <cmath>

#if defined(__HIPCC__)
#define MIQ_ENC_HD __host__ __device__
#else
#define MIQ_ENC_HD
#endif

namespace miq
{
struct EncodingD
{
    double min, max, delta, offset;
};

MIQ_ENC_HD inline double enc_max2(double a, double b)
{
    return a < b ? b : a;   // std::max(a, b)
}
MIQ_ENC_HD inline double enc_min2(double a, double b)
{
    return b < a ? b : a;   // std::min(a, b)
}

MIQ_ENC_HD inline EncodingD computed_encodings(int bw, double mn, double mx, bool use_symmetric,
                                               bool use_strict_symmetric, bool use_unsigned_symmetric)
{
    const double fmax = 3.4028234663852886e38;   // std::numeric_limits<float>::max()
    double steps      = ldexp(1.0, bw) - 1;      // 2^bw - 1, exact
    if (use_symmetric && use_strict_symmetric)
        steps -= 1;
    EncodingD e;
    // std::isinf of either sign, written as comparisons that host and device compile alike
    const double inf = __builtin_huge_val();
    if (mn == inf || mn == -inf)
        mn = -fmax;
    if (mx == inf || mx == -inf)
        mx = fmax;
    if (use_symmetric && (mn < 0.0 || !use_unsigned_symmetric))
    {
        const double amax        = enc_max2(fabs(mx), fabs(mn));
        const unsigned int n_pos = (unsigned int) floor(steps / 2);
        e.delta                  = amax / n_pos;
        e.offset                 = -ceil(steps / 2);
        e.min                    = enc_max2(e.offset * e.delta, -fmax);
        e.max                    = enc_min2(e.delta * n_pos, fmax);
        return e;
    }
    e.delta = (mx - mn) / steps;
    if (mn < 0 && mx > 0)
    {
        // zero must sit exactly on the grid
        double z = round(-mn / e.delta);
        z        = enc_min2(steps, enc_max2(0.0, z));
        e.offset = -z;
    }
    else
    {
        e.offset = round(mn / e.delta);
        e.min    = mn;
        e.max    = mx;
        return e;
    }
    const double t = e.delta * e.offset;
    e.min          = (t >= -fmax && t <= fmax) ? t : -fmax;
    e.max          = mx - mn + e.min;
    if (e.max > fmax)
        e.max = fmax;
    return e;
}
#if defined(__HIPCC__)
// The float32 parameters the per-channel kernels take, from a channel's encoding in double
// (AimetTensorQuantizer::quantizeDequantizePerChannel, TrainingExtensions/torch/src/AimetTensorQuantizer.cpp:209-227,
// 268-297, on float32(min), float32(max)): zero gated into the range, delta = (max - min) / steps, offset =
// round-half-even(min / delta), with one step less iff channel 0's encoding has min == -max.
struct ChannelKernelParams
{
    float min, max, delta, offset, raw_min, raw_max;
};

__device__ __forceinline__ ChannelKernelParams channel_kernel_params(double enc_min, double enc_max, bool first_is_symmetric,
                                                                     int bw)
{
    ChannelKernelParams p;
    const float num_steps = (float) (ldexp(1.0, bw) - 1.0 - (first_is_symmetric ? 1.0 : 0.0));
    float lo = (float) enc_min, hi = (float) enc_max;
    p.raw_min = lo;
    p.raw_max = hi;
    // torch.minimum / torch.maximum propagate NaN
    lo        = (lo != lo) ? lo : fminf(lo, 0.f);
    hi        = (hi != hi) ? hi : fmaxf(hi, 0.f);
    float eps = lo + 1e-5f;
    hi        = (hi != hi || eps != eps) ? (hi + eps) : fmaxf(hi, eps);
    p.min     = lo;
    p.max     = hi;
    p.delta   = (hi - lo) / num_steps;
    p.offset  = rintf(lo / p.delta);
    return p;
}
#endif
}   // namespace miq

#endif
