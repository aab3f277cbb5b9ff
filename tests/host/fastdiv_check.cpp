// Host check of aimet_amd/csrc/miq_fastmath.h: div_by_invariant(a, b, RN(1/b)) == a / b bit for bit.
// Usage: fastdiv_check <pairs_in_millions>; prints "OK <count>" or the first mismatch.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../aimet_amd/csrc/miq_fastmath.h"

static uint32_t bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
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

static long long failures = 0, checked = 0;
static void check(float a, float b)
{
    if (!miq::fastdiv_divisor_ok(b) || !(std::fabs(a) <= miq::kFastDivMaxDividend))
        return;
    const float y    = 1.0f / b;
    const float fast = miq::div_by_invariant(a, b, y);
    const float ref  = a / b;
    ++checked;
    // below 2^-36 the contract only promises a tiny quotient (< 2^-35) of the right sign
    if (std::fabs(ref) < 1.4551915228366852e-11f)
    {
        if (!(std::fabs(fast) < 2.9103830456733704e-11f) || std::signbit(fast) != std::signbit(ref))
        {
            if (failures++ < 5)
                printf("tiny mismatch a=%a b=%a fast=%a ref=%a\n", a, b, fast, ref);
        }
        return;
    }
    if (bits(fast) != bits(ref))
    {
        if (failures++ < 5)
            printf("MISMATCH a=%a b=%a fast=%a ref=%a\n", a, b, fast, ref);
    }
}

int main(int argc, char** argv)
{
    const long long millions = argc > 1 ? atoll(argv[1]) : 50;
    // 1. random significands and exponents inside the contract
    for (long long i = 0; i < millions * 1000000ll; ++i)
    {
        const uint32_t eb = 127 - 64 + rnd() % 129;            // 2^-64 .. 2^64
        const float b     = from_bits((eb << 23) | (rnd() & 0x7fffff));
        const uint32_t ea = 127 - 140 + rnd() % 201;           // 2^-140 .. 2^60
        const float a     = from_bits(((rnd() & 1u) << 31) | (ea << 23) | (rnd() & 0x7fffff));
        check(a, b);
    }
    // 2. adversarial divisors: all-ones / near-one significands, every dividend significand pattern family
    const uint32_t bsig[] = {0x7fffff, 0x7ffffe, 0x000000, 0x000001, 0x400000, 0x3fffff, 0x555555, 0x2aaaaa, 0x7ffffd};
    for (uint32_t sb: bsig)
        for (int e = -60; e <= 60; e += 7)
        {
            const float b = from_bits(((uint32_t) (127 + e) << 23) | sb);
            for (uint32_t sa = 0; sa < (1u << 23); sa += 1)
                check(from_bits((127u << 23) | sa), b);
        }
    // 3. the grid-index regime: a = b * (k + 0.5 +- few ulp), k in [0, 65536]
    for (int rep = 0; rep < 2000; ++rep)
    {
        const float b = from_bits(((uint32_t) (127 - 20 + rnd() % 24) << 23) | (rnd() & 0x7fffff));
        for (int k = 0; k <= 65536; k += 1 + rnd() % 3)
        {
            const float mid = b * ((float) k + 0.5f);
            uint32_t u      = bits(mid);
            for (int d = -3; d <= 3; ++d)
                check(from_bits(u + d), b);
        }
    }
    // 4. zeros and signs
    check(0.0f, 3.0f);
    check(-0.0f, 3.0f);
    if (bits(miq::div_by_invariant(-0.0f, 3.0f, 1.0f / 3.0f)) != bits(-0.0f / 3.0f))
        ++failures;
    if (failures)
    {
        printf("FAILED %lld of %lld\n", failures, checked);
        return 1;
    }
    printf("OK %lld\n", checked);
    return 0;
}
