// Host check of miq::bucket_row (aimet_amd/csrc/miq_fastmath.h): the row it returns must be the bucket the reference's
// float sequence  roundf(x / bucket - off)  selects (DlQuantization/src/math_functions.cpp:375-382), for every sample.
// Usage: bucket_check <ranges>; prints "OK <samples> <share answered by the one-operation path>" or the first mismatch.
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../aimet_amd/csrc/miq_fastmath.h"

constexpr int kBuckets = 512;

static float from_bits(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static uint32_t bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static uint64_t rng_state = 0x2545F4914F6CDD1Dull;
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

// the reference, operation for operation
static int reference_row(float x, float bucket, float off)
{
    volatile float q = x / bucket;
    volatile float t = q - off;
    const float r    = roundf(t);
    return (r >= 0.0f && r < (float) kBuckets) ? (int) r + 1 : 0;
}

static long long failures = 0, checked = 0, fast = 0;
static void check(float x, const miq::BucketMap& m)
{
    int got = miq::bucket_row<kBuckets>(x, m);
    if (got == kBuckets + 1)
        got = 0;   // both end rows collect dropped samples
    const int want = reference_row(x, m.bucket, m.off);
    ++checked;
    const float u = __builtin_fmaf(x, m.fast_scale, m.fast_shift);
    if (std::fabs((u - std::floor(u)) - 0.5f) < m.thr)
        ++fast;
    if (got != want && failures++ < 5)
        printf("MISMATCH x=%a bucket=%a off=%a got %d want %d\n", x, m.bucket, m.off, got, want);
}

// range fixed by a first batch with extremes (mn, mx): DlQuantization/src/math_functions.cpp:208-241
static miq::BucketMap map_of(float mn, float mx)
{
    if (mn == mx)
        mx = std::fmax(mx, mn + 0.01f);
    const float c  = (mx + mn) / 2;
    float lo       = c - 3 * (c - mn);
    float hi       = c + 3 * (mx - c);
    lo             = std::fmax(lo, -FLT_MAX);
    hi             = std::fmin(hi, FLT_MAX);
    const double w = ((double) hi - (double) lo) / kBuckets;
    const float bf = (float) ((lo + 1 * w) - (lo + 0 * w));
    return miq::make_bucket_map(bf, lo / bf, kBuckets);
}

int main(int argc, char** argv)
{
    const int ranges = argc > 1 ? atoi(argv[1]) : 2000;
    for (int r = 0; r < ranges; ++r)
    {
        // magnitudes from 1e-30 to 1e30, ranges that straddle zero, one-sided ranges far from zero (large offsets)
        const float scale = std::pow(10.0f, uniform() * 60.0f - 30.0f);
        float mn, mx;
        switch (r % 4)
        {
        case 0: mn = -uniform() * scale; mx = uniform() * scale; break;
        case 1: mn = 0.0f; mx = uniform() * scale; break;
        case 2: mn = scale * (1.0f + uniform()); mx = mn * (1.0f + uniform() * 0.01f); break;   // offset ~ 1e2 .. 1e5
        default: mn = -scale * (1.0f + uniform()); mx = mn * (1.0f - uniform() * 1e-4f); break;  // offset up to ~1e7
        }
        if (!(mn < mx) && !(mn == mx))
            continue;
        const miq::BucketMap m = map_of(mn, mx);
        if (!(m.bucket > 0.0f) || !std::isfinite(m.off))
            continue;
        // every bucket edge, with the floats around it
        for (int k = -2; k <= kBuckets + 1; ++k)
        {
            const double edge = ((double) k - 0.5 + (double) m.off) * (double) m.bucket;
            const float e     = (float) edge;
            if (!std::isfinite(e))
                continue;
            uint32_t b = bits(e);
            for (int d = -48; d <= 48; ++d)
                check(from_bits(b + (uint32_t) d), m);
        }
        // samples inside and around the range
        const double lo = (double) m.off * m.bucket, width = (double) m.bucket * kBuckets;
        for (int i = 0; i < 20000; ++i)
            check((float) (lo + width * (uniform() * 1.2 - 0.1)), m);
        for (int i = 0; i < 2000; ++i)
            check(from_bits(rnd()), m);   // any bit pattern: NaN, infinities, subnormals, huge values
        check(0.0f, m);
        check(-0.0f, m);
        check(INFINITY, m);
        check(-INFINITY, m);
        check(NAN, m);
        check(FLT_MAX, m);
        check(-FLT_MAX, m);
    }
    if (failures)
    {
        printf("FAILED %lld of %lld\n", failures, checked);
        return 1;
    }
    printf("OK %lld %.4f\n", checked, (double) fast / (double) checked);
    return 0;
}
