// Regenerates n22_mt19937_seed1_6000.f32: the 6000-sample tensor the reference's TF-Enhanced known-answer test
// draws (std::mt19937 generator(1); std::normal_distribution<float>(2, 2); see
// ModelOptimizations/DlQuantization/test/TestTensorQuantizer.cpp:88-103).  libstdc++'s normal_distribution is
// deterministic for a given libstdc++, so the samples are committed as a fixture.
//   g++ -O2 -o /tmp/gen_n22 gen_n22.cpp && /tmp/gen_n22 n22_mt19937_seed1_6000.f32
#include <cstdio>
#include <random>
#include <vector>
int main(int argc, char** argv)
{
    std::normal_distribution<float> distribution(2, 2);
    std::mt19937 generator(1);
    std::vector<float> data(6000);
    for (auto& d: data)
        d = distribution(generator);
    FILE* f = fopen(argc > 1 ? argv[1] : "n22_mt19937_seed1_6000.f32", "wb");
    fwrite(data.data(), sizeof(float), data.size(), f);
    fclose(f);
    return 0;
}
