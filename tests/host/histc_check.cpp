// Host check of miq::HistcBinner::bin (aimet_amd/csrc/miq_fastmath.h): the bin it returns must be the one torch.histc's
// float sequence  (int) ((x - lo) * bins / (hi - lo))  selects, with the histogram observer's rule for values outside
// [lo, hi], for every sample.
// Usage: histc_check <ranges>; prints "OK <samples> <share answered by the one-operation path>" or the first mismatches.
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../aimet_amd/csrc/miq_fastmath.h"

static float from_bits(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd()
{
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return (uint32_t) (rng_state >> 16);
}
static float uniform()
{
    return (float) (rnd() >> 8) * (1.0f / 16777216.0f);
}

// the sequence, operation for operation, with plain division
static int reference_bin(float x, float lo, float hi, int nb)
{
    if (x != x)
        return -1;
    if (x < lo)
        return 0;
    if (x > hi)
        return nb - 1;
    volatile float d = x - lo;
    volatile float a = d * (float) nb;
    volatile float w = hi - lo;
    volatile float q = a / w;
    const int pos    = (int) q;
    return pos >= nb ? nb - 1 : pos;
}

static long long failures = 0, checked = 0, fast = 0;
static void check(float x, const miq::HistcBinner& b)
{
    const int got  = b.bin(x);
    const int want = reference_bin(x, b.lo, b.hi, b.nb);
    ++checked;
    const float u = __builtin_fmaf(x, b.fast_scale, b.fast_shift);
    if (std::fabs((u - std::floor(u)) - 0.5f) < b.thr)
        ++fast;
    if (got != want && failures++ < 5)
        printf("MISMATCH x=%a lo=%a hi=%a bins=%d got %d want %d\n", x, b.lo, b.hi, b.nb, got, want);
}

static void check_range(float lo, float hi, int nb)
{
    if (!(lo < hi) || !std::isfinite(lo) || !std::isfinite(hi) || !std::isfinite(hi - lo))
        return;
    miq::HistcBinner b;
    b.init(lo, hi, nb);
    const float w = hi - lo;
    // the floats around every bin edge (of up to 4096 edges), in both formulations of the edge
    const int step = nb > 4096 ? nb / 4096 : 1;
    for (int i = 0; i <= nb; i += step)
    {
        const float edges[2] = {lo + w * ((float) i / (float) nb), lo + (w / (float) nb) * (float) i};
        for (float e : edges)
        {
            float below = e, above = e;
            check(e, b);
            for (int k = 0; k < 6; ++k)
            {
                below = std::nextafterf(below, -INFINITY);
                above = std::nextafterf(above, INFINITY);
                check(below, b);
                check(above, b);
            }
        }
    }
    for (int k = 0; k < 3000; ++k)
    {
        check(lo + w * uniform(), b);                          // inside
        check(lo + w * (3.0f * uniform() - 1.0f), b);          // inside and around
    }
    for (int k = 0; k < 200; ++k)
        check(from_bits(rnd()), b);                            // any bit pattern: NaN, infinities, huge, subnormal
    const float special[] = {lo, hi, 0.0f, -0.0f, INFINITY, -INFINITY, NAN, FLT_MAX, -FLT_MAX, FLT_MIN};
    for (float v : special)
        check(v, b);
}

int main(int argc, char** argv)
{
    const int ranges  = argc > 1 ? atoi(argv[1]) : 1000;
    const int bins[]  = {2048, 512, 100, 4096, 1, 7, 255};
    for (int r = 0; r < ranges; ++r)
    {
        const int nb = bins[r % 7];
        // magnitudes over 60 decades; ranges from zero, around zero, far from zero (narrow and wide), negative
        const float m = std::ldexp(1.0f + uniform(), (int) (rnd() % 200) - 100);
        check_range(0.0f, m, nb);
        check_range(-m * uniform(), m, nb);
        check_range(-m, -m * uniform() * 0.99f, nb);
        check_range(m, m * (1.0f + std::ldexp(1.0f + uniform(), -(int) (rnd() % 20))), nb);
        check_range(m - 1.0f, m + 1.0f, nb);                   // histc's widening of an empty range
        check_range(-m, m * std::ldexp(1.0f, (int) (rnd() % 30)), nb);
    }
    if (failures)
    {
        printf("FAILED %lld of %lld\n", failures, checked);
        return 1;
    }
    printf("OK %lld %.3f\n", checked, (double) fast / (double) checked);
    return 0;
}
