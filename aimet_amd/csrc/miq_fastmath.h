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
}   // namespace miq
#endif
