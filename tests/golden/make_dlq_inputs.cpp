// Writes the pseudo-random inputs that DlQuantization's tests draw with the C++ standard library
// (std::mt19937 seeded with 1, std::normal_distribution<float>; test/TestTfEnhancedEncodingAnalyzer.cpp:25-38,
// test/TestTensorQuantizer.cpp:52-63) as raw float32, so that the Python tests see the same numbers.
// usage: make_dlq_inputs <mean> <stddev> <count> <out.f32>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

int main(int argc, char** argv) {
    if (argc != 5) return 2;
    const float mean = std::atof(argv[1]), stddev = std::atof(argv[2]);
    const unsigned count = std::atoi(argv[3]);
    std::normal_distribution<float> distribution(mean, stddev);
    std::mt19937 generator(1);
    std::vector<float> v(count);
    for (unsigned i = 0; i < count; i++) v[i] = distribution(generator);
    FILE* f = std::fopen(argv[4], "wb");
    if (!f) return 1;
    std::fwrite(v.data(), sizeof(float), v.size(), f);
    std::fclose(f);
    return 0;
}
