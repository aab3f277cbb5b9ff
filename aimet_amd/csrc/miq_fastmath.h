// Division by a launch-invariant divisor, bit-identical to IEEE-754 binary32 division.
//
// With y = RN(1/b) (the correctly rounded reciprocal, computed once per channel), two residual corrections through
// fused multiply-adds yield the correctly rounded quotient: the residual r = a - q*b is exact in an FMA, the first
// correction brings q within one ulp of a/b, and by Markstein's theorem the second one rounds correctly.  Five
// operations replace the eleven of the scaled Newton-Raphson sequence the compiler emits for a / b.
//
// Contract: 2^-64 <= b <= 2^64 and |a| <= 2^60 (so nothing overflows).  The result equals a / b bit for bit
// whenever |a / b| >= 2^-36.  Below that the residual may be inexact (it can fall under the subnormal threshold),
// and the result is only guaranteed to be smaller than 2^-35 in magnitude with the sign of a -- far below anything
// that can change the rounded grid index formed from it.
// The sign of a zero quotient is taken from the dividend (b is positive), as IEEE division does.
// tests/test_fastmath.py compiles this header for the host and checks it against `/` on hundreds of millions of
// operand pairs, including the adversarial ones (divisors with all-ones significands, quotients next to rounding
// midpoints).
#ifndef MIQ_FASTMATH_H
#define MIQ_FASTMATH_H

#if defined(__HIPCC__)
#define MIQ_HD __host__ __device__
#else
#define MIQ_HD
#endif

namespace miq
{
constexpr float kFastDivMinDivisor = 5.421010862427522e-20f;   // 2^-64
constexpr float kFastDivMaxDivisor = 1.8446744073709552e19f;   // 2^64
constexpr float kFastDivMaxDividend = 1.152921504606847e18f;   // 2^60

MIQ_HD inline bool fastdiv_divisor_ok(float b)
{
    return b >= kFastDivMinDivisor && b <= kFastDivMaxDivisor;   // false for NaN
}

MIQ_HD inline float div_by_invariant(float a, float b, float y)
{
    float q = a * y;
    float r = __builtin_fmaf(-q, b, a);
    q       = __builtin_fmaf(r, y, q);
    r       = __builtin_fmaf(-q, b, a);
    q       = __builtin_fmaf(r, y, q);
    return __builtin_copysignf(q, a);
}
// roundf (halves away from zero) in three operations: add the largest float below one half with the sign of x, then
// truncate.  Equal to roundf(x) for every binary32 value (tests/test_fastmath.py walks through all of them below 2^24 in
// both signs; from 2^23 on every float is an integer and comes back unchanged): x + 0.49999997 crosses the next integer
// exactly when the fraction of |x| is at least one half, and the one case where the sum itself rounds (fraction exactly
// one half: 0.5 + 0.49999997 rounds to 1.0) rounds the way roundf does.  The compiler's own expansion of roundf takes six.
MIQ_HD inline float round_half_away(float x)
{
    return __builtin_truncf(x + __builtin_copysignf(0.49999997f, x));
}

// ---- bucket index of the 512-bucket PDF --------------------------------------------------------------------
// Reference arithmetic (DlQuantization/src/math_functions.cpp:375-382), all binary32:
//     q = x / bucket;  t = q - off;  r = roundf(t);  counted in bucket (int) r  iff  0 <= r < buckets
// Three roundings separate t from the real number x / bucket - off, and one fused multiply-add
//     u = fma(x, RN(1 / bucket), RN(1.5 - off))
// lands within  (3 |off| + 2 buckets + 4) 2^-24  of t + 1.5 for every x whose t lies in [-1, buckets + 1]:
//     |q - x/bucket| <= |x/bucket| 2^-24,  |t - (q - off)| <= |t| 2^-24,
//     |x RN(1/bucket) - x/bucket| <= |x/bucket| 2^-24,  |RN(1.5 - off) - (1.5 - off)| <= (|off| + 1.5) 2^-24,
//     |u - (x RN(1/bucket) + RN(1.5 - off))| <= |u| 2^-24,  and |x/bucket| <= |off| + buckets + 1.
// roundf(t) changes only where t + 0.5 crosses an integer, so whenever the fraction of u stays at least
// eps = (|off| + 2 buckets) 2^-21 (more than twice the bound above) away from 0 and 1, floor(u) - 1 is the reference's
// bucket.  Otherwise (a sample within eps of a bucket edge, NaN, infinities, |u| >= 2^23, or a bucket width outside
// the contract of div_by_invariant) the reference sequence itself is evaluated.  Rows: 1 .. buckets are the
// buckets, 0 and buckets + 1 collect what the reference drops.
struct BucketMap
{
    float bucket, rcp, off;   // reference sequence; rcp = RN(1 / bucket) or 0 when div_by_invariant does not apply
    float fast_scale;         // RN(1 / bucket), only read when thr > 0
    float fast_shift;         // RN(1.5 - off)
    float thr;                // 0.5 - eps; not positive: the one-operation path is never taken
};

MIQ_HD inline BucketMap make_bucket_map(float bucket, float off, int buckets)
{
    BucketMap m;
    m.bucket        = bucket;
    m.off           = off;
    const bool ok   = fastdiv_divisor_ok(bucket);
    m.rcp           = ok ? 1.0f / bucket : 0.0f;
    m.fast_scale    = m.rcp;
    m.fast_shift    = 1.5f - off;
    const float eps = (__builtin_fabsf(off) + 2.0f * (float) buckets) * 4.76837158203125e-07f;   // 2^-21
    m.thr           = (ok && eps < 0.25f) ? 0.5f - eps : -1.0f;   // false for a NaN offset
    return m;
}

template <int BUCKETS>
MIQ_HD inline int bucket_row(float x, const BucketMap& m)
{
    const float u  = __builtin_fmaf(x, m.fast_scale, m.fast_shift);
    const float fl = __builtin_floorf(u);
    const float f  = u - fl;   // exact
    if (__builtin_fabsf(f - 0.5f) < m.thr)
    {
        // fl is an integer below 2^23 here (larger floats have no fraction: f == 0 fails the test)
        const int k = (int) fl;
        return k < 0 ? 0 : (k > BUCKETS + 1 ? BUCKETS + 1 : k);
    }
    const float q = (m.rcp != 0.0f && __builtin_fabsf(x) <= kFastDivMaxDividend) ? div_by_invariant(x, m.bucket, m.rcp)
                                                                                 : x / m.bucket;
    const float r = round_half_away(q - m.off);
    return (r >= 0.0f && r < (float) BUCKETS) ? (int) r + 1 : 0;
}

// ---- bin of torch.histc --------------------------------------------------------------------------------------
// torch.histc(x, bins, lo, hi) counts x in bin (int) ((x - lo) * bins / (hi - lo)), all binary32, x == hi in the last
// bin (ATen/native/cuda/SummaryOps.cu getBin; the CPU kernel agrees).  The histogram observer adds: below lo -> first
// bin, above hi -> last bin.  bin() evaluates exactly that sequence (the division through div_by_invariant where its
// contract holds).  Most samples are answered by one fused multiply-add instead,
//     u = fma(x, RN(bins / width), RN(-lo * RN(bins / width))):
// with K = max(|lo|, |hi|) / width, u lies within bins (K + 2) 2^-24 of the real number (x - lo) bins / width (one
// rounding each in the scale, the shift and the result), and the three roundings of the sequence keep it within
// 3 bins 2^-24 of the same number, so the truncated sequence and floor(u) agree whenever the fraction of u stays
// eps = 2 bins (K + 5) 2^-24 (twice the sum of the bounds; in the host check mismatches first appear at three eighths
// of it) away from 0 and 1; u below 0 or from bins on is what the observer's rule for outside values
// maps to the end bins.  A wavefront takes the sequence as soon as one of its lanes does, so eps is kept small.  Samples
// within eps of a bin edge, infinities, NaN (bin -1) and ranges for which eps reaches 1/4 take the sequence.
// tests/test_fastmath.py checks bin() against the plain sequence on ranges over many decades, the floats around every
// bin edge and random samples.
struct HistcBinner
{
    float lo, hi, width, recip, nbf;
    int nb;
    bool divisor_ok;
    float fast_scale, fast_shift, thr;   // thr <= 0: the one-operation path is never taken

    MIQ_HD void init(float lo_, float hi_, int nb_)
    {
        lo         = lo_;
        hi         = hi_;
        nb         = nb_;
        nbf        = (float) nb_;
        width      = hi_ - lo_;
        divisor_ok = fastdiv_divisor_ok(width);
        recip      = divisor_ok ? 1.0f / width : 0.f;
        fast_scale = nbf / width;
        fast_shift = -lo_ * fast_scale;
        const float k   = __builtin_fmaxf(__builtin_fabsf(lo_), __builtin_fabsf(hi_)) / width;
        const float eps = nbf * (k + 5.0f) * 1.1920928955078125e-07f;   // 2^-23
        // (comparisons are false for NaN: a range that is not finite never takes the short path)
        thr = (divisor_ok && eps < 0.25f && __builtin_fabsf(fast_shift) < 1e30f && fast_scale < 1e30f) ? 0.5f - eps
                                                                                                     : -1.0f;
    }

    MIQ_HD int bin_by_sequence(float x) const
    {
        if (x != x)
            return -1;
        if (x < lo)
            return 0;
        if (x > hi)
            return nb - 1;
        const float a = (x - lo) * nbf;
        const float q = (divisor_ok && a <= kFastDivMaxDividend) ? div_by_invariant(a, width, recip) : a / width;
        const int pos = (int) q;
        return pos >= nb ? nb - 1 : pos;
    }

    MIQ_HD int bin(float x) const
    {
        const float u  = __builtin_fmaf(x, fast_scale, fast_shift);
        const float fl = __builtin_floorf(u);
        const float f  = u - fl;   // exact; NaN for infinite u
        if (__builtin_fabsf(f - 0.5f) < thr)
        {
            // |fl| < 2^23 here (larger floats have no fraction: f == 0 fails the test)
            const int k = (int) fl;
            const int below = k < nb - 1 ? k : nb - 1;
            return below > 0 ? below : 0;
        }
        return bin_by_sequence(x);
    }
};
}   // namespace miq
#endif
