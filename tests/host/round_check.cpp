// Host check of miq::round_half_away (aimet_amd/csrc/miq_fastmath.h) against roundf: every binary32 value with
// |x| <= 2^24 whose bit pattern is a multiple of `stride` away from a half-integer neighbourhood start, plus, densely,
// every value within 64 ulps of k + 0.5 for k < 2^22, plus specials.  argv[1] = stride (1 = exhaustive).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../aimet_amd/csrc/miq_fastmath.h"

static uint64_t bad = 0;

static void check(float x)
{
    const float a = miq::round_half_away(x), r = roundf(x);
    uint32_t ab, rb;
    memcpy(&ab, &a, 4);
    memcpy(&rb, &r, 4);
    const bool both_nan = (a != a) && (r != r);
    if (ab != rb && !both_nan)
    {
        if (bad < 10)
            printf("x=%.9g got=%.9g want=%.9g\n", x, a, r);
        ++bad;
    }
}

int main(int argc, char** argv)
{
    const uint32_t stride = argc > 1 ? (uint32_t) atoi(argv[1]) : 1;
    for (uint64_t b = 0; b <= 0x4B800000u; b += stride)
    {
        float x;
        const uint32_t bits = (uint32_t) b;
        memcpy(&x, &bits, 4);
        check(x);
        check(-x);
    }
    for (uint32_t k = 0; k < (1u << 22); k += (stride > 1 ? 3 : 1))
    {
        float x = (float) k + 0.5f;
        uint32_t bits;
        memcpy(&bits, &x, 4);
        for (int d = -64; d <= 64; ++d)
        {
            const uint32_t nb = bits + (uint32_t) d;
            float y;
            memcpy(&y, &nb, 4);
            check(y);
            check(-y);
        }
    }
    const float specials[] = {0.0f, -0.0f, 1e-45f, -1e-45f, 1e-38f, 3.4e38f, -3.4e38f, INFINITY, -INFINITY, NAN, 8388607.5f,
                              8388608.0f, 16777216.0f, 33554432.0f, 1e20f};
    for (float v : specials)
        check(v);
    if (bad)
    {
        printf("FAILED: %llu mismatches\n", (unsigned long long) bad);
        return 1;
    }
    printf("OK\n");
    return 0;
}
