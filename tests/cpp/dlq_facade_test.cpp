// Drives include/aimet_amd_dlq.hpp (the C++ facade with DlQuantization's interface) on one GPU and prints its results
// as JSON; tests/test_dlq_facade_gpu.py compares them with the CPU oracle.
//
// The facade is used the way the reference's ONNX Runtime custom op uses DlQuantization: under the namespace name
// DlQuantization, through modeSpecificActionTensorQuantizer below -- that function is the caller of
// TrainingExtensions/onnx/src/AimetOpUtils.h:46-87 typed out again with its call expressions as they are there
// (updateStats(tensor, shape, useCuda, allocator, stream), quantizeDequantize(in, out, shape, useCuda, stream,
// runner), ...), so it only compiles if the facade binds what that caller binds.  Inputs follow the reference's own
// tests (test/TestTensorQuantizer.cpp:20-66): 6000 normal(2, 2) draws from std::mt19937(1), and the 60-element ramp.
#define AIMET_AMD_AS_DLQUANTIZATION
#include <cstdio>
#include <cstring>
#include <numeric>
#include <random>
#include <vector>

#include "aimet_amd_dlq.hpp"

template <typename T>
void copyInputTensorsToOutputTensors(const T* inTensor, size_t count, T* outTensor, bool useCuda, void* stream)
{
    if (!useCuda)
        throw std::runtime_error("Not compiled for CPU mode.");
    aimet_amd::detail::hipCheck(hipMemcpyAsync(outTensor, inTensor, count * sizeof(T), hipMemcpyDeviceToDevice,
                                               static_cast<hipStream_t>(stream)),
                                "hipMemcpyAsync");
}

template <typename T>
void modeSpecificActionTensorQuantizer(const T* inTensor, T* outTensor, const std::vector<int64_t> inputShape,
                                       DlQuantization::BlockTensorQuantizer* tensorQuantizer,
                                       const DlQuantization::TensorQuantizerOpMode opMode,
                                       const bool useSymmetricEncoding, DlQuantization::IAllocator* allocator,
                                       bool useCuda, void* stream, DlQuantization::IForLoopRunner* runner = nullptr)
{
    int64_t numElements = std::accumulate(inputShape.begin(), inputShape.end(), int64_t(1), std::multiplies<int64_t>());

    switch (opMode)
    {
    case DlQuantization::TensorQuantizerOpMode::oneShotQuantizeDequantize:
    {
        tensorQuantizer->resetEncodingStats();
        tensorQuantizer->updateStats(inTensor, inputShape, useCuda, allocator, stream);
        auto computedEncodings = tensorQuantizer->computeEncodings(useSymmetricEncoding);
        tensorQuantizer->setEncodings(computedEncodings);
    }
    // fall through to quantizeDequantize
    case DlQuantization::TensorQuantizerOpMode::quantizeDequantize:
    {
        tensorQuantizer->quantizeDequantize(inTensor, outTensor, inputShape, useCuda, stream, runner);
        break;
    }
    case DlQuantization::TensorQuantizerOpMode::updateStats:
    {
        tensorQuantizer->updateStats(inTensor, inputShape, useCuda, allocator, stream);
    }
    // fall through to passThrough
    case DlQuantization::TensorQuantizerOpMode::passThrough:
    {
        copyInputTensorsToOutputTensors(inTensor, numElements, outTensor, useCuda, stream);
        break;
    }
    default:
    {
        throw std::exception();
    }
    }
}

using namespace aimet_amd;
using OpMode = DlQuantization::TensorQuantizerOpMode;

// An allocator like the one ONNX Runtime hands to the custom op: counts what goes out and what comes back.
class CountingAllocator : public DlQuantization::IAllocator
{
public:
    void* allocateRaw(size_t bytes) override
    {
        void* p = nullptr;
        detail::hipCheck(hipMalloc(&p, bytes), "hipMalloc");
        ++allocations;
        bytesOut += bytes;
        return p;
    }
    void deleteRaw(void* ptr) override
    {
        ++frees;
        (void) hipFree(ptr);
    }
    int allocations = 0, frees = 0;
    size_t bytesOut = 0;
};

// A loop runner that must never be asked to run anything (there are no host loops to share out).
class IdleRunner : public DlQuantization::IForLoopRunner
{
public:
    void run(std::function<void(size_t)>, size_t) const override { ++calls; }
    mutable int calls = 0;
};

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

template <typename T>
static T* toDevice(const std::vector<T>& host)
{
    T* d = nullptr;
    detail::hipCheck(hipMalloc(reinterpret_cast<void**>(&d), sizeof(T) * host.size()), "hipMalloc");
    detail::hipCheck(hipMemcpy(d, host.data(), sizeof(T) * host.size(), hipMemcpyHostToDevice), "hipMemcpy");
    return d;
}

template <typename T>
static std::vector<T> toHost(const T* d, size_t n)
{
    std::vector<T> host(n);
    detail::hipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");
    detail::hipCheck(hipMemcpy(host.data(), d, sizeof(T) * n, hipMemcpyDeviceToHost), "hipMemcpy");
    return host;
}

static std::vector<half> toHalf(const std::vector<float>& v)
{
    std::vector<half> out(v.size());
    for (size_t i = 0; i < v.size(); i++)
    {
        const _Float16 h = static_cast<_Float16>(v[i]);
        std::memcpy(&out[i].bits, &h, 2);
    }
    return out;
}
static std::vector<float> fromHalf(const std::vector<half>& v)
{
    std::vector<float> out(v.size());
    for (size_t i = 0; i < v.size(); i++)
    {
        _Float16 h;
        std::memcpy(&h, &v[i].bits, 2);
        out[i] = static_cast<float>(h);
    }
    return out;
}
static std::vector<bfloat16> toBfloat16(const std::vector<float>& v)   // round to nearest even
{
    std::vector<bfloat16> out(v.size());
    for (size_t i = 0; i < v.size(); i++)
    {
        uint32_t u;
        std::memcpy(&u, &v[i], 4);
        u += 0x7fffu + ((u >> 16) & 1u);
        out[i].bits = static_cast<uint16_t>(u >> 16);
    }
    return out;
}
static std::vector<float> fromBfloat16(const std::vector<bfloat16>& v)
{
    std::vector<float> out(v.size());
    for (size_t i = 0; i < v.size(); i++)
    {
        const uint32_t u = static_cast<uint32_t>(v[i].bits) << 16;
        std::memcpy(&out[i], &u, 4);
    }
    return out;
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
        hipStream_t stream = nullptr;
        detail::hipCheck(hipStreamCreate(&stream), "hipStreamCreate");
        CountingAllocator allocator;
        IdleRunner runner;
        std::printf("{\n");

        // ---- the reference caller, all four op modes, float tensors, TF-enhanced per tensor, with allocator + runner
        detail::hipCheck(hipMemcpy(dIn, data4.data(), sizeof(float) * 6000, hipMemcpyHostToDevice), "hipMemcpy");
        DlQuantization::BlockTensorQuantizer op({}, 8, DlQuantization::QUANTIZATION_TF_ENHANCED);
        modeSpecificActionTensorQuantizer(dIn, dOut, {6000}, &op, OpMode::oneShotQuantizeDequantize, false, &allocator, true,
                                          stream, &runner);
        printEncodings("op_oneshot_encodings", op.getEncodings());
        {
            auto out = toHost(dOut, 6000);
            out.resize(64);
            printFloats("op_oneshot_qdq_head", out);
        }
        modeSpecificActionTensorQuantizer(dIn, dOut, {6000}, &op, OpMode::updateStats, false, &allocator, true, stream,
                                          &runner);
        {
            const auto out = toHost(dOut, 6000);
            std::printf("\"op_update_passes_through\": %s,\n", out == data4 ? "true" : "false");
        }
        modeSpecificActionTensorQuantizer(dIn, dOut, {3000}, &op, OpMode::updateStats, true, &allocator, true, stream);
        {
            // the statistics now hold the one-shot batch (not reset by updateStats), the same batch again and its first half
            auto enc = op.computeEncodings(true);
            printEncodings("op_after_updates_symmetric", enc);
            op.setEncodings(enc);
        }
        detail::hipCheck(hipMemsetAsync(dOut, 0, sizeof(float) * 6000, stream), "hipMemsetAsync");
        modeSpecificActionTensorQuantizer(dIn, dOut, {6000}, &op, OpMode::quantizeDequantize, true, nullptr, true, stream,
                                          &runner);
        {
            auto out = toHost(dOut, 6000);
            out.resize(64);
            printFloats("op_qdq_head", out);
        }
        modeSpecificActionTensorQuantizer(dIn, dOut, {6000}, &op, OpMode::passThrough, true, nullptr, true, stream);
        {
            const auto out = toHost(dOut, 6000);
            std::printf("\"op_pass_through\": %s,\n", out == data4 ? "true" : "false");
        }
        std::printf("\"allocator\": [%d, %d, %d],\n", allocator.allocations, allocator.frees, allocator.bytesOut > 0 ? 1 : 0);
        std::printf("\"runner_calls\": %d,\n", runner.calls);

        // ---- half and bfloat16 tensors through the same caller: min/max per channel (half), TF-enhanced (bfloat16)
        {
            const std::vector<half> rampH = toHalf(ramp);
            half* hIn                     = toDevice(rampH);
            half* hOut                    = toDevice(rampH);
            DlQuantization::BlockTensorQuantizer q({3}, 8, DlQuantization::QUANTIZATION_TF);
            modeSpecificActionTensorQuantizer(hIn, hOut, {1, 4, 5, 3}, &q, OpMode::oneShotQuantizeDequantize, false, &allocator,
                                              true, stream, &runner);
            printEncodings("half_tf_per_channel", q.getEncodings());
            printFloats("half_tf_per_channel_qdq", fromHalf(toHost(hOut, 60)));
            (void) hipFree(hIn);
            (void) hipFree(hOut);

            const std::vector<bfloat16> dataB = toBfloat16(data4);
            bfloat16* bIn                     = toDevice(dataB);
            bfloat16* bOut                    = toDevice(dataB);
            DlQuantization::BlockTensorQuantizer qb({}, 8, DlQuantization::QUANTIZATION_TF_ENHANCED);
            modeSpecificActionTensorQuantizer(bIn, bOut, {6000}, &qb, OpMode::oneShotQuantizeDequantize, false, &allocator, true,
                                              stream, &runner);
            printEncodings("bf16_tfe", qb.getEncodings());
            auto out = fromBfloat16(toHost(bOut, 6000));
            out.resize(64);
            printFloats("bf16_tfe_qdq_head", out);
            // 16-bit statistics in the min/max scheme fold into float running extrema over two batches
            DlQuantization::BlockTensorQuantizer qt({}, 8, DlQuantization::QUANTIZATION_TF);
            qt.updateStats(bIn, {3000}, true, &allocator, stream);
            qt.updateStats(bIn + 3000, {3000}, true, nullptr, stream);
            printEncodings("bf16_tf_two_batches", qt.computeEncodings(false));
            (void) hipFree(bIn);
            (void) hipFree(bOut);
        }
        std::printf("\"allocator_balanced\": %s,\n", allocator.allocations == allocator.frees ? "true" : "false");

        // ---- free functions and the analyzer factory
        {
            const TfEncoding enc {-5.0, 7.75, 0.05, -100.0, 8};
            DlQuantization::quantizeDequantize(dIn, 6000, enc, dOut, DlQuantization::COMP_MODE_GPU, DlQuantization::ROUND_NEAREST,
                                               stream, &runner);
            auto out = toHost(dOut, 6000);
            out.resize(64);
            printFloats("free_qdq_head", out);
            bool threw = false;
            try
            {
                DlQuantization::quantizeDequantize(dIn, 6000, enc, dOut, DlQuantization::COMP_MODE_CPU,
                                                   DlQuantization::ROUND_NEAREST, stream);
            }
            catch (const std::runtime_error&)
            {
                threw = true;
            }
            std::printf("\"cpu_mode_throws\": %s,\n", threw ? "true" : "false");

            detail::hipCheck(hipMemcpy(dIn, ramp.data(), sizeof(float) * 60, hipMemcpyHostToDevice), "hipMemcpy");
            const Encodings three {{-15.0, 14.0, 29.0 / 255, -132.0, 8}, {-3.0, 3.0, 6.0 / 255, -128.0, 8}, {0.0, 10.0, 10.0 / 255, 0.0, 8}};
            DlQuantization::quantizeDequantizeBroadcast(dIn, dOut, three, {1, 4, 5, 3}, {3}, DlQuantization::COMP_MODE_GPU,
                                                        stream);
            printFloats("free_broadcast_qdq", toHost(dOut, 60));
            const auto spec = QuantizationType::Fp8E4M3FN().floatSpec();
            DlQuantization::quantizeDequantizeFp8(dIn, 60, TfEncoding {-448 * 0.07, 448 * 0.07, 0.07, 0.0, 8}, dOut, spec,
                                                  DlQuantization::COMP_MODE_GPU, stream);
            printFloats("free_fp8_qdq", toHost(dOut, 60));
            const Encodings scales {{0, 0, 0.01, 0, 8}, {0, 0, 0.05, 0, 8}, {0, 0, 0.25, 0, 8}};
            DlQuantization::quantizeDequantizeFp8Broadcast(dIn, dOut, scales, spec, {1, 4, 5, 3}, {3},
                                                           DlQuantization::COMP_MODE_GPU, stream);
            printFloats("free_fp8_broadcast_qdq", toHost(dOut, 60));

            auto analyzer = DlQuantization::getBlockEncodingAnalyzerInstance<float>(DlQuantization::QUANTIZATION_TF, {1, 1, 5, 1});
            analyzer->updateStats(dIn, {1, 4, 5, 3}, DlQuantization::COMP_MODE_GPU, &allocator, stream);
            printEncodings("factory_minmax_strict_symmetric", analyzer->computeEncoding(8, true, true, false, 0.0));
            std::printf("\"factory_observed\": [");
            const auto seen = analyzer->getObservedMinMax();
            for (size_t i = 0; i < seen.size(); i++)
                std::printf("%s[%.9g, %.9g]", i ? ", " : "", std::get<0>(seen[i]), std::get<1>(seen[i]));
            std::printf("],\n");
            detail::hipCheck(hipMemcpy(dIn, data4.data(), sizeof(float) * 6000, hipMemcpyHostToDevice), "hipMemcpy");
        }

        // ---- TF-enhanced, per tensor: two batches, asymmetric and symmetric encodings, then quantize-dequantize
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
        std::vector<float> out = toHost(dOut, 6000);
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
        printEncodings("tf_per_channel", perChannel);
        printFloats("tf_per_channel_qdq", toHost(dOut, 60));

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
        printEncodings("fp8_e4m3_per_channel", fp8Enc);
        printFloats("fp8_e4m3_per_channel_qdq", toHost(dOut, 60));

        detail::hipCheck(hipMemcpy(dIn, data4.data(), sizeof(float) * 6000, hipMemcpyHostToDevice), "hipMemcpy");
        BlockTensorQuantizer e5m2({}, QuantizationType::Fp8E5M2(), QUANTIZATION_TF);
        e5m2.setEncodings({{-57344.0 * 0.3, 57344.0 * 0.3, 0.3, 0.0, 4}});
        e5m2.quantizeDequantize(dIn, dOut, {6000}, true);
        std::vector<float> out3 = toHost(dOut, 6000);
        out3.resize(256);
        printFloats("fp8_e5m2_qdq_head", out3);
        std::printf("\"fp8_sticky\": [%d, %d, %d]\n", (int) e5m2.getQuantizationType().isFloat(),
                    e5m2.getQuantizationType().bitwidth(), e5m2.bitwidth);
        std::printf("}\n");
        (void) hipFree(dIn);
        (void) hipFree(dOut);
        (void) hipStreamDestroy(stream);
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "facade test failed: %s\n", e.what());
        return 1;
    }
    return 0;
}
