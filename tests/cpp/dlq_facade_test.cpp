// Drives include/aimet_amd_dlq.hpp (the BlockTensorQuantizer-shaped C++ facade) on one GPU and prints its results as
// JSON; tests/test_dlq_facade_gpu.py compares them with the CPU oracle.  Inputs follow the reference's own tests
// (test/TestTensorQuantizer.cpp:20-66): 6000 normal(2, 2) draws from std::mt19937(1), and the 60-element ramp.
#include <cstdio>
#include <random>
#include <vector>

#include "aimet_amd_dlq.hpp"

using namespace aimet_amd;

static void printEncodings(const char* name, const Encodings& encs, bool last = false)
{
    std::printf("\"%s\": [", name);
    for (size_t i = 0; i < encs.size(); i++)
        std::printf("%s[%.17g, %.17g, %.17g, %.17g, %d]", i ? ", " : "", encs[i].min, encs[i].max, encs[i].delta,
                    encs[i].offset, encs[i].bw);
    std::printf("]%s\n", last ? "" : ",");
}

static void printFloats(const char* name, const std::vector<float>& v, bool last = false)
{
    std::printf("\"%s\": [", name);
    for (size_t i = 0; i < v.size(); i++)
        std::printf("%s%.9g", i ? ", " : "", v[i]);
    std::printf("]%s\n", last ? "" : ",");
}

int main()
{
    try
    {
        std::vector<float> data4(6000);
        std::normal_distribution<float> distribution(2, 2);
        std::mt19937 generator(1);
        for (auto& d: data4)
            d = distribution(generator);
        std::vector<float> ramp(60);
        float t = -15;
        for (auto& d: ramp)
        {
            d = t;
            t += 0.5;
        }

        float *dIn = nullptr, *dOut = nullptr;
        detail::hipCheck(hipMalloc(&dIn, sizeof(float) * 6000), "hipMalloc");
        detail::hipCheck(hipMalloc(&dOut, sizeof(float) * 6000), "hipMalloc");
        std::printf("{\n");

        // TF-enhanced, per tensor: two batches, asymmetric and symmetric encodings, then quantize-dequantize
        detail::hipCheck(hipMemcpy(dIn, data4.data(), sizeof(float) * 6000, hipMemcpyHostToDevice), "hipMemcpy");
        BlockTensorQuantizer tfe({}, 8, QUANTIZATION_TF_ENHANCED);
        bool threw = false;
        try
        {
            tfe.computeEncodings(false);
        }
        catch (const std::runtime_error&)
        {
            threw = true;
        }
        tfe.updateStats(dIn, {6000}, true);
        tfe.updateStats(dIn, {3000}, true);
        Encodings asym = tfe.computeEncodings(false);
        Encodings sym  = tfe.computeEncodings(true);
        tfe.setEncodings(asym);
        tfe.quantizeDequantize(dIn, dOut, {6000}, true);
        std::vector<float> out(6000);
        detail::hipCheck(hipMemcpy(out.data(), dOut, sizeof(float) * 6000, hipMemcpyDeviceToHost), "hipMemcpy");
        out.resize(64);
        std::printf("\"throws_before_stats\": %s,\n", threw ? "true" : "false");
        printEncodings("tfe_asymmetric", asym);
        printEncodings("tfe_symmetric", sym);
        printFloats("tfe_qdq_head", out);
        std::printf("\"tfe_hist_buckets\": %zu,\n", tfe.getStatsHistogram()[0].size());

        // min/max, one encoding per last-dimension channel of a {1,4,5,3} tensor, strict symmetric on {1,1,5,1}
        detail::hipCheck(hipMemcpy(dIn, ramp.data(), sizeof(float) * 60, hipMemcpyHostToDevice), "hipMemcpy");
        BlockTensorQuantizer tf({3}, 8, QUANTIZATION_TF);
        tf.updateStats(dIn, {1, 4, 5, 3}, true);
        Encodings perChannel = tf.computeEncodings(false);
        tf.setEncodings(perChannel);
        tf.quantizeDequantize(dIn, dOut, {1, 4, 5, 3}, true);
        std::vector<float> out2(60);
        detail::hipCheck(hipMemcpy(out2.data(), dOut, sizeof(float) * 60, hipMemcpyDeviceToHost), "hipMemcpy");
        printEncodings("tf_per_channel", perChannel);
        printFloats("tf_per_channel_qdq", out2);

        BlockTensorQuantizer strict({1, 1, 5, 1}, 8, QUANTIZATION_TF);
        strict.setStrictSymmetric(true);
        strict.updateStats(dIn, {1, 4, 5, 3}, true);
        printEncodings("tf_strict_symmetric", strict.computeEncodings(true));

        // FP8: calibrate per channel on the ramp (E4M3FN), quantize-dequantize; E5M2 per tensor with a fixed scale;
        // the legacy bitwidth field follows setEncodings, the quantization type does not
        BlockTensorQuantizer fp8({3}, QuantizationType::Fp8E4M3FN(), QUANTIZATION_TF);
        fp8.updateStats(dIn, {1, 4, 5, 3}, true);
        Encodings fp8Enc = fp8.computeEncodings(false);
        fp8.setEncodings(fp8Enc);
        fp8.quantizeDequantize(dIn, dOut, {1, 4, 5, 3}, true);
        detail::hipCheck(hipMemcpy(out2.data(), dOut, sizeof(float) * 60, hipMemcpyDeviceToHost), "hipMemcpy");
        printEncodings("fp8_e4m3_per_channel", fp8Enc);
        printFloats("fp8_e4m3_per_channel_qdq", out2);

        detail::hipCheck(hipMemcpy(dIn, data4.data(), sizeof(float) * 6000, hipMemcpyHostToDevice), "hipMemcpy");
        BlockTensorQuantizer e5m2({}, QuantizationType::Fp8E5M2(), QUANTIZATION_TF);
        e5m2.setEncodings({{-57344.0 * 0.3, 57344.0 * 0.3, 0.3, 0.0, 4}});
        e5m2.quantizeDequantize(dIn, dOut, {6000}, true);
        std::vector<float> out3(6000);
        detail::hipCheck(hipMemcpy(out3.data(), dOut, sizeof(float) * 6000, hipMemcpyDeviceToHost), "hipMemcpy");
        out3.resize(256);
        printFloats("fp8_e5m2_qdq_head", out3);
        std::printf("\"fp8_sticky\": [%d, %d, %d]\n", (int) e5m2.getQuantizationType().isFloat(),
                    e5m2.getQuantizationType().bitwidth(), e5m2.bitwidth);
        std::printf("}\n");
        (void) hipFree(dIn);
        (void) hipFree(dOut);
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "facade test failed: %s\n", e.what());
        return 1;
    }
    return 0;
}
