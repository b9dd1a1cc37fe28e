// aimet_amd_dlq.hpp -- header-only C++ facade over the C ABI of libaimet_amd.so with the interface a caller of
// DlQuantization binds (paths relative to ModelOptimizations/DlQuantization):
//
//   BlockTensorQuantizer            include/DlQuantization/TensorQuantizer.h:43-199, src/TensorQuantizer.cpp
//   IAllocator, ComputationMode, QuantizationMode, TfEncoding, RoundingMode, TensorDims, Encodings,
//   quantizeDequantizeBroadcast<T>  include/DlQuantization/Quantization.hpp:19-114
//   IForLoopRunner                  include/DlQuantization/IForLoopRunner.h:16-30
//   QuantizationType, FloatQuantizationSpec   include/DlQuantization/QuantizationType.hpp:14-190
//   IBlockEncodingAnalyzer<float>, getBlockEncodingAnalyzerInstance<float>
//                                   include/DlQuantization/IQuantizationEncodingAnalyzer.hpp:102-190,
//                                   include/DlQuantization/QuantizerFactory.hpp:16-19
//   quantizeDequantize<T>, quantizeDequantizeFp8, quantizeDequantizeFp8Broadcast     src/trim_functions.hpp:35-41, 76-79
//
// Same names, argument lists, defaults and exception messages, so the reference's own caller
// (TrainingExtensions/onnx/src/AimetOpUtils.h:46-87) compiles against this header unchanged.  Everything lives in
// namespace aimet_amd; define AIMET_AMD_AS_DLQUANTIZATION before including to get `namespace DlQuantization =
// aimet_amd`.
//
// What differs, all because this implementation is device-only:
//   * tensors must be device pointers: useCuda = false / COMP_MODE_CPU throws "Not compiled for CPU mode";
//   * the IForLoopRunner* argument is accepted and ignored (it parallelises the reference's CPU loops);
//   * IAllocator*: when given, the scratch memory of a call comes from allocateRaw and goes back through deleteRaw
//     before the call returns (the stream is synchronised first, as the reference's GPU analyzers do); when null, the
//     object keeps a scratch buffer of its own that only grows.  The statistics themselves live in device memory owned
//     by the object (hipMalloc in the constructor); the shared library allocates nothing;
//   * 16-bit tensors: aimet_amd::half / aimet_amd::bfloat16 (two-byte structs), Eigen::half / Eigen::bfloat16 (only
//     their names are needed, as in src/trim_functions.hpp:19-23) and _Float16 are accepted element types;
//   * QUANTIZATION_RANGE_LEARNING and ROUND_STOCHASTIC exist as enumerators and are refused at run time.
#ifndef AIMET_AMD_DLQ_HPP
#define AIMET_AMD_DLQ_HPP

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <tuple>
#include <type_traits>
#include <vector>

#include "aimet_amd.h"

namespace Eigen
{
struct half;
struct bfloat16;
}   // namespace Eigen

namespace aimet_amd
{

// ---------------------------------------------------------------------------------------- Quantization.hpp:19-114 --
enum ComputationMode
{
    COMP_MODE_CPU,
    COMP_MODE_GPU
};

class IAllocator
{
public:
    virtual void* allocateRaw(size_t bytes) = 0;
    virtual void deleteRaw(void* ptr)       = 0;
};

enum QuantizationMode
{
    QUANTIZATION_TF,
    QUANTIZATION_TF_ENHANCED,
    QUANTIZATION_RANGE_LEARNING,   // not an analyzer of this library: refused when statistics are asked for
    QUANTIZATION_PERCENTILE,
};

struct TfEncoding
{
    double min;
    double max;
    double delta;
    double offset;
    int bw;
};

enum RoundingMode
{
    ROUND_NEAREST,
    ROUND_STOCHASTIC
};

using TensorDim  = int64_t;
using TensorDims = std::vector<TensorDim>;
using Encodings  = std::vector<TfEncoding>;

// ----------------------------------------------------------------------------------------- IForLoopRunner.h:16-30 --
class IForLoopRunner
{
public:
    virtual ~IForLoopRunner()                                                = default;
    virtual void run(std::function<void(size_t)> fn, size_t numChunks) const = 0;
};

// ------------------------------------------------------------------------------------- TensorQuantizer.h:19-25 --
enum class TensorQuantizerOpMode
{
    updateStats,
    oneShotQuantizeDequantize,
    quantizeDequantize,
    passThrough
};

// -------------------------------------------------------------------------------------- 16-bit element types --
struct half
{
    uint16_t bits;
};
struct bfloat16
{
    uint16_t bits;
};

namespace detail
{
template <typename T>
struct DtypeOf;   // ahq_dtype of a tensor element type; no definition for unsupported types
template <>
struct DtypeOf<float>
{
    static constexpr int32_t value = AHQ_F32;
};
template <>
struct DtypeOf<half>
{
    static constexpr int32_t value = AHQ_F16;
};
template <>
struct DtypeOf<bfloat16>
{
    static constexpr int32_t value = AHQ_BF16;
};
template <>
struct DtypeOf<Eigen::half>
{
    static constexpr int32_t value = AHQ_F16;
};
template <>
struct DtypeOf<Eigen::bfloat16>
{
    static constexpr int32_t value = AHQ_BF16;
};
#ifdef __FLT16_MANT_DIG__
template <>
struct DtypeOf<_Float16>
{
    static constexpr int32_t value = AHQ_F16;
};
#endif

inline void hipCheck(hipError_t e, const char* what)
{
    if (e != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
inline void ahqCheck(int status)
{
    if (status != AHQ_OK)
        throw std::runtime_error(ahq_last_error());
}
inline void requireDevice(ComputationMode mode)
{
    if (mode != COMP_MODE_GPU)
        throw std::runtime_error("Not compiled for CPU mode: tensors must live in device memory");
}
inline int64_t numel(const TensorDims& shape)
{
    int64_t n = 1;
    for (auto d: shape)
        n *= d;
    return n;
}

// A device buffer owned by an object; only ever grows.
struct DeviceBuffer
{
    void* ptr    = nullptr;
    size_t bytes = 0;
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer&)            = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer()
    {
        if (ptr)
            (void) hipFree(ptr);
    }
    void reserve(size_t n)
    {
        if (n <= bytes)
            return;
        if (ptr)
        {
            hipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");   // earlier launches may still read the old one
            hipCheck(hipFree(ptr), "hipFree");
        }
        ptr = nullptr;
        hipCheck(hipMalloc(&ptr, n), "hipMalloc");
        bytes = n;
    }
};

// Scratch memory of one call: from the caller's allocator when there is one (returned in the destructor, after the
// stream has drained), else from the owner's growing buffer.
class Scratch
{
public:
    Scratch(IAllocator* alloc, DeviceBuffer& own, size_t bytes, void* stream) : _alloc(alloc), _stream(stream)
    {
        if (bytes == 0)
            return;
        if (_alloc)
        {
            _ptr = _alloc->allocateRaw(bytes);
            if (!_ptr)
                throw std::runtime_error("IAllocator::allocateRaw returned null");
        }
        else
        {
            own.reserve(bytes);
            _ptr = own.ptr;
        }
    }
    Scratch(const Scratch&)            = delete;
    Scratch& operator=(const Scratch&) = delete;
    ~Scratch()
    {
        if (_alloc && _ptr)
        {
            (void) hipStreamSynchronize(static_cast<hipStream_t>(_stream));
            _alloc->deleteRaw(_ptr);
        }
    }
    void* ptr() const { return _ptr; }

private:
    IAllocator* _alloc;
    void* _stream;
    void* _ptr = nullptr;
};

// getBroadcastableShapes (src/tensor_utils.cpp:28-58) as an ahq_layout: the encoding shape is right-aligned against
// the tensor shape, block size along dim i = tensorShape[i] / encodingShape[i]
inline ahq_layout makeLayout(const TensorDims& tensorShape, const TensorDims& encodingShape)
{
    const size_t nd = tensorShape.size();
    if (encodingShape.size() > nd || nd > AHQ_MAX_DIMS)
        throw std::runtime_error("Cannot interpret tensor and encoding dimensions as broadcastable");
    ahq_layout layout {};
    layout.ndim       = static_cast<int32_t>(nd);
    const size_t lead = nd - encodingShape.size();
    int64_t stride    = 1;
    for (size_t i = nd; i-- > 0;)
    {
        const int64_t d = tensorShape[i];
        const int64_t e = i < lead ? 1 : encodingShape[i - lead];
        if (!(d == e) && (d < e || e <= 0 || d % e != 0))
            throw std::runtime_error("Cannot interpret tensor and encoding dimensions as broadcastable");
        layout.dims[i]       = d;
        layout.block[i]      = e > 1 ? d / e : (d > 0 ? d : 1);
        layout.enc_stride[i] = e > 1 ? stride : 0;
        stride *= e;
    }
    return layout;
}

// delta | offset | min | max as float arrays on the host (QdqEncType is float, src/trim_functions.hpp:30-31)
inline std::vector<float> packEncodings(const Encodings& encodings)
{
    const size_t n = encodings.size();
    std::vector<float> host(4 * n);
    for (size_t e = 0; e < n; e++)
    {
        host[e]         = static_cast<float>(encodings[e].delta);
        host[n + e]     = static_cast<float>(encodings[e].offset);
        host[2 * n + e] = static_cast<float>(encodings[e].min);
        host[3 * n + e] = static_cast<float>(encodings[e].max);
    }
    return host;
}
}   // namespace detail

// ------------------------------------------------------------------------------------ QuantizationType.hpp:14-190 --
enum class QuantizationTypeKind
{
    Int,
    Float,
};

struct IntQuantizationSpec
{
    int bitwidth;
};

struct FloatQuantizationSpec
{
    int bitwidth;
    int exponentBits;
    int mantissaBits;
    int exponentMin;
    double maxValue;
    bool finite;
    bool unsignedZero;
};

class QuantizationType
{
public:
    static QuantizationType Int(int bitwidth)
    {
        if (bitwidth <= 0)
            throw std::invalid_argument("Integer quantization bitwidth must be positive");
        QuantizationType t;
        t._kind    = QuantizationTypeKind::Int;
        t._intSpec = IntQuantizationSpec {bitwidth};
        return t;
    }

    static QuantizationType Float(int bitwidth, int exponentBits, int mantissaBits, int exponentMin, double maxValue,
                                  bool finite, bool unsignedZero)
    {
        if (bitwidth <= 0)
            throw std::invalid_argument("Floating-point quantization bitwidth must be positive");
        if (exponentBits <= 0)
            throw std::invalid_argument("Floating-point quantization exponent bits must be positive");
        if (mantissaBits < 0)
            throw std::invalid_argument("Floating-point quantization mantissa bits must be non-negative");
        if (!(maxValue > 0))
            throw std::invalid_argument("Floating-point quantization max value must be positive");
        QuantizationType t;
        t._kind      = QuantizationTypeKind::Float;
        t._floatSpec = FloatQuantizationSpec {bitwidth, exponentBits, mantissaBits, exponentMin, maxValue, finite,
                                              unsignedZero};
        return t;
    }

    // "fnuz" formats move the bias by one and use the whole top binade; "fn" formats give up only the all-ones
    // mantissa of the top binade; IEEE-like formats give up the top binade (QuantizationType.hpp:88-135).
    static QuantizationType Float(int exponentBits, int mantissaBits, bool finite, bool unsignedZero)
    {
        if (exponentBits <= 0)
            throw std::invalid_argument("Floating-point quantization exponent bits must be positive");
        if (mantissaBits < 0)
            throw std::invalid_argument("Floating-point quantization mantissa bits must be non-negative");
        const int bias    = (1 << (exponentBits - 1)) - 1 + (unsignedZero ? 1 : 0);
        const double unit = std::ldexp(1.0, -mantissaBits);
        const int top     = (1 << exponentBits) - ((unsignedZero || finite) ? 1 : 2) - bias;
        const double man  = (!unsignedZero && finite) ? 2.0 - 2.0 * unit : 2.0 - unit;
        return Float(1 + exponentBits + mantissaBits, exponentBits, mantissaBits, 1 - bias, man * std::ldexp(1.0, top),
                     finite, unsignedZero);
    }

    static QuantizationType Fp8E4M3FN() { return Float(4, 3, true, false); }
    static QuantizationType Fp8E5M2() { return Float(5, 2, false, false); }

    QuantizationTypeKind kind() const { return _kind; }
    bool isInt() const { return _kind == QuantizationTypeKind::Int; }
    bool isFloat() const { return _kind == QuantizationTypeKind::Float; }
    int bitwidth() const { return isInt() ? _intSpec.bitwidth : _floatSpec.bitwidth; }
    const IntQuantizationSpec& intSpec() const
    {
        if (!isInt())
            throw std::logic_error("QuantizationType does not hold an integer spec");
        return _intSpec;
    }
    const FloatQuantizationSpec& floatSpec() const
    {
        if (!isFloat())
            throw std::logic_error("QuantizationType does not hold a floating-point spec");
        return _floatSpec;
    }

    QuantizationType() = default;

private:
    QuantizationTypeKind _kind {QuantizationTypeKind::Int};
    IntQuantizationSpec _intSpec {8};
    FloatQuantizationSpec _floatSpec {8, 4, 3, -6, 448.0, true, false};
};

// ------------------------------------------------------------------- free functions: src/trim_functions.hpp:35-41 --
// quantizeDequantize<DTYPE>(in, cnt, encoding, out, mode, rounding, stream, runner): one encoding for the whole
// tensor, handed to the kernel by value (no device copy, as in the reference's GPU path).
template <typename DTYPE>
void quantizeDequantize(const DTYPE* in, uint64_t cnt, const TfEncoding& encoding, DTYPE* out,
                        ComputationMode mode_cpu_gpu, RoundingMode rounding_mode, void* stream,
                        IForLoopRunner* runner = nullptr)
{
    (void) runner;
    detail::requireDevice(mode_cpu_gpu);
    if (rounding_mode != ROUND_NEAREST)
        throw std::runtime_error("Unknown rounding mode.");   // stochastic rounding is not part of this library
    detail::ahqCheck(ahq_dlq_qdq_per_tensor(detail::DtypeOf<DTYPE>::value, in, out, cnt, encoding.min, encoding.max,
                                            encoding.delta, encoding.offset, stream));
}

inline void quantizeDequantizeFp8(const float* in, uint64_t cnt, const TfEncoding& encoding, float* out,
                                  const FloatQuantizationSpec& fp8Spec, ComputationMode modeCpuGpu,
                                  void* stream = nullptr, IForLoopRunner* runner = nullptr)
{
    (void) runner;
    detail::requireDevice(modeCpuGpu);
    detail::ahqCheck(ahq_dlq_fp8_qdq_per_tensor(AHQ_F32, in, out, cnt, encoding.delta, fp8Spec.mantissaBits,
                                                fp8Spec.exponentMin, static_cast<float>(fp8Spec.maxValue), stream));
}

namespace detail
{
// Broadcast quantize-dequantize with the encodings already on the device (delta | offset | min | max).
template <typename T>
void qdqBroadcastDevice(const T* in, T* out, const float* enc, int64_t numEncodings, const ahq_layout& layout, void* stream)
{
    ahq_grid grid {};
    grid.arith         = AHQ_ARITH_DLQ;
    grid.op            = AHQ_OP_QDQ;
    grid.io_dtype      = DtypeOf<T>::value;
    grid.compute_dtype = AHQ_F32;
    ahqCheck(ahq_qdq_forward(&grid, &layout, in, out, nullptr, enc, enc + numEncodings, enc + 2 * numEncodings,
                             enc + 3 * numEncodings, stream));
}

// Device copy of a packed encoding vector that lives for one call (the reference's broadcast functions also
// allocate and free theirs inside the call, src/trim_functions.cu:230-260).
struct TransientEncodings
{
    float* ptr = nullptr;
    void* stream;
    TransientEncodings(const Encodings& encodings, void* stream_) : stream(stream_)
    {
        const std::vector<float> host = packEncodings(encodings);
        hipCheck(hipMalloc(reinterpret_cast<void**>(&ptr), host.size() * sizeof(float)), "hipMalloc");
        // a pageable-host copy returns once the data has left the host vector
        const hipError_t e = hipMemcpyAsync(ptr, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice,
                                            static_cast<hipStream_t>(stream));
        if (e != hipSuccess)
        {
            (void) hipFree(ptr);
            hipCheck(e, "hipMemcpyAsync");
        }
        hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
    }
    TransientEncodings(const TransientEncodings&)            = delete;
    TransientEncodings& operator=(const TransientEncodings&) = delete;
    ~TransientEncodings()
    {
        (void) hipStreamSynchronize(static_cast<hipStream_t>(stream));
        (void) hipFree(ptr);
    }
};
}   // namespace detail

// Quantization.hpp:106-114
template <typename T>
void quantizeDequantizeBroadcast(const T* inTensor, T* outTensor, const Encodings& encodings, const TensorDims& inputShape,
                                 const TensorDims& encodingShape, ComputationMode mode, void* stream = nullptr,
                                 IForLoopRunner* runner = nullptr)
{
    (void) runner;
    detail::requireDevice(mode);
    const ahq_layout layout = detail::makeLayout(inputShape, encodingShape);
    if (static_cast<int64_t>(encodings.size()) != detail::numel(encodingShape))
        throw std::runtime_error("Length of encoding vector did not match the encoding shape");
    if (detail::numel(inputShape) == 0)
        return;
    detail::TransientEncodings dev(encodings, stream);
    detail::qdqBroadcastDevice(inTensor, outTensor, dev.ptr, static_cast<int64_t>(encodings.size()), layout, stream);
}

// src/trim_functions.hpp:76-79
inline void quantizeDequantizeFp8Broadcast(const float* inTensor, float* outTensor, const Encodings& encodings,
                                           const FloatQuantizationSpec& fp8Spec, const TensorDims& inputShape,
                                           const TensorDims& encodingShape, ComputationMode mode, void* stream = nullptr,
                                           IForLoopRunner* runner = nullptr)
{
    (void) runner;
    detail::requireDevice(mode);
    const ahq_layout layout = detail::makeLayout(inputShape, encodingShape);
    if (static_cast<int64_t>(encodings.size()) != detail::numel(encodingShape))
        throw std::runtime_error("Length of encoding vector did not match the encoding shape");
    if (detail::numel(inputShape) == 0)
        return;
    detail::TransientEncodings dev(encodings, stream);   // the scales are the deltas, first in the packed vector
    detail::ahqCheck(ahq_dlq_fp8_qdq(AHQ_F32, &layout, inTensor, outTensor, dev.ptr, fp8Spec.mantissaBits,
                                     fp8Spec.exponentMin, static_cast<float>(fp8Spec.maxValue), stream));
}

// --------------------------------------------------------- IQuantizationEncodingAnalyzer.hpp:102-190 (block form) --
template <typename DTYPE>
class IBlockEncodingAnalyzer
{
public:
    virtual ~IBlockEncodingAnalyzer() = default;

    virtual void updateStats(const DTYPE* tensor, const TensorDims& tensorShape, ComputationMode tensorCpuGpuMode,
                             IAllocator* allocator = nullptr, void* stream = nullptr) = 0;
    virtual void updateStats(const half* tensor, const TensorDims& tensorShape, ComputationMode tensorCpuGpuMode,
                             IAllocator* allocator = nullptr, void* stream = nullptr)
    {
        (void) tensor, (void) tensorShape, (void) tensorCpuGpuMode, (void) allocator, (void) stream;
        throw std::runtime_error("fp16 calibration not supported for this encoding analyzer");
    }
    virtual void updateStats(const bfloat16* tensor, const TensorDims& tensorShape, ComputationMode tensorCpuGpuMode,
                             IAllocator* allocator = nullptr, void* stream = nullptr)
    {
        (void) tensor, (void) tensorShape, (void) tensorCpuGpuMode, (void) allocator, (void) stream;
        throw std::runtime_error("bf16 calibration not supported for this encoding analyzer");
    }
    virtual void resetStats() = 0;
    virtual std::vector<TfEncoding> computeEncoding(uint8_t bw, bool useSymmetricEncodings, bool useStrictSymmetric,
                                                    bool useUnsignedSymmetric, double zeroPointShift) const = 0;
    virtual std::vector<std::tuple<double, double>> getObservedMinMax() const { return {}; }
    virtual std::vector<std::vector<std::tuple<double, double>>> getStatsHistogram() const = 0;
    virtual void setPercentileValue(float percentile)
    {
        (void) percentile;
        throw std::runtime_error("setPercentileValue is only applicable for percentile encoding analyzers");
    }
    virtual float getPercentileValue()
    {
        throw std::runtime_error("getPercentileValue is only applicable for percentile encoding analyzers");
    }
};

namespace detail
{
// All three analyzers of this library (running min/max; 1536-bucket PDF with the TF-enhanced search or the percentile
// rule) behind the block-analyzer interface: MinMaxEncodingAnalyzer (src/MinMaxEncodingAnalyzer.cpp) and
// EncodingAnalyzerWrapper over TfEnhancedEncodingAnalyzer / PercentileEncodingAnalyzer (src/EncodingAnalyzerWrapper.cpp).
class DeviceBlockAnalyzer : public IBlockEncodingAnalyzer<float>
{
public:
    DeviceBlockAnalyzer(QuantizationMode mode, const TensorDims& shape) : _mode(mode), _shape(shape)
    {
        if (mode != QUANTIZATION_TF && mode != QUANTIZATION_TF_ENHANCED && mode != QUANTIZATION_PERCENTILE)
            throw std::runtime_error("only QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED and QUANTIZATION_PERCENTILE have "
                                     "an encoding analyzer here");
        _numEncodings = numel(_shape);
        if (_mode == QUANTIZATION_TF)
        {
            _min.reserve(sizeof(float) * _numEncodings);
            _max.reserve(sizeof(float) * _numEncodings);
        }
        else
        {
            _xleft.reserve(sizeof(double) * AHQ_DLQ_PDF_SIZE * _numEncodings);
            _pdf.reserve(sizeof(double) * AHQ_DLQ_PDF_SIZE * _numEncodings);
            _meta.reserve(sizeof(int32_t) * 4 * _numEncodings);
        }
        clearStats(false);
    }

    void updateStats(const float* tensor, const TensorDims& tensorShape, ComputationMode mode, IAllocator* allocator = nullptr,
                     void* stream = nullptr) override
    {
        update(tensor, AHQ_F32, tensorShape, mode, allocator, stream);
    }
    void updateStats(const half* tensor, const TensorDims& tensorShape, ComputationMode mode, IAllocator* allocator = nullptr,
                     void* stream = nullptr) override
    {
        update(tensor, AHQ_F16, tensorShape, mode, allocator, stream);
    }
    void updateStats(const bfloat16* tensor, const TensorDims& tensorShape, ComputationMode mode,
                     IAllocator* allocator = nullptr, void* stream = nullptr) override
    {
        update(tensor, AHQ_BF16, tensorShape, mode, allocator, stream);
    }

    // The element type as an ahq_dtype tag: what the typed overloads above and BlockTensorQuantizer::updateStats<T> call.
    void update(const void* tensor, int32_t dtype, const TensorDims& tensorShape, ComputationMode mode, IAllocator* allocator,
                void* stream)
    {
        requireDevice(mode);
        _stream                 = stream;
        const ahq_layout layout = makeLayout(tensorShape, _shape);
        if (numel(tensorShape) == 0)
            return;
        if (_mode == QUANTIZATION_TF)
        {
            const size_t need   = ahq_minmax_workspace_bytes(&layout);
            const size_t offset = (need + 255) & ~size_t(255);
            Scratch scratch(allocator, _workspace, offset + 2 * sizeof(float) * _numEncodings + 512, stream);
            char* w    = static_cast<char*>(scratch.ptr());
            void* bmin = w + offset;
            void* bmax = w + offset + sizeof(float) * _numEncodings;
            if (dtype == AHQ_F32)
            {
                ahqCheck(ahq_minmax(dtype, &layout, tensor, bmin, bmax, _min.ptr, _max.ptr, 2, w, need, stream));
            }
            else
            {
                // extrema in the tensor's own 16-bit type (exact), then the float fold the reference does after
                // widening the tensor
                ahqCheck(ahq_minmax(dtype, &layout, tensor, bmin, bmax, nullptr, nullptr, 2, w, need, stream));
                ahqCheck(ahq_dlq_minmax_fold(dtype, bmin, bmax, _numEncodings, static_cast<float*>(_min.ptr),
                                             static_cast<float*>(_max.ptr), stream));
            }
            return;
        }
        const size_t need = ahq_dlq_pdf_update_workspace_bytes(dtype, &layout);
        {
            Scratch scratch(allocator, _workspace, need, stream);
            ahq_dlq_pdf_state st = pdfState();
            ahqCheck(ahq_dlq_pdf_update(dtype, &layout, tensor, &st, _allInitialized ? 0 : 1, nullptr, scratch.ptr(), need,
                                        stream));
        }
        if (!_allInitialized)
        {
            std::vector<int32_t> meta(4 * _numEncodings);
            hipCheck(hipMemcpyAsync(meta.data(), _meta.ptr, meta.size() * sizeof(int32_t), hipMemcpyDeviceToHost,
                                    static_cast<hipStream_t>(stream)),
                     "hipMemcpyAsync");
            hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
            _allInitialized = true;
            for (int64_t e = 0; e < _numEncodings; e++)
                _allInitialized = _allInitialized && meta[4 * e + 1] != 0;
        }
    }

    void resetStats() override { clearStats(true); }

    // On the stream of the latest updateStats call (the statistics are produced there).
    std::vector<TfEncoding> computeEncoding(uint8_t bw, bool useSymmetricEncodings, bool useStrictSymmetric,
                                            bool useUnsignedSymmetric, double zeroPointShift) const override
    {
        void* stream = _stream;
        _result.reserve(sizeof(double) * 5 * _numEncodings);
        double* out = static_cast<double*>(_result.ptr);
        if (_mode == QUANTIZATION_TF)
        {
            ahqCheck(ahq_dlq_minmax_encodings(static_cast<const float*>(_min.ptr), static_cast<const float*>(_max.ptr),
                                              _numEncodings, bw, useSymmetricEncodings, useStrictSymmetric,
                                              useUnsignedSymmetric, zeroPointShift, out, stream));
        }
        else
        {
            if (zeroPointShift != 0.0)
                throw std::runtime_error("Non-zero zeroPointShift is only supported for min-max quant scheme.");
            ahq_dlq_pdf_state st = pdfState();
            if (_mode == QUANTIZATION_PERCENTILE)
            {
                ahqCheck(ahq_dlq_percentile_encodings(&st, _percentile, bw, useSymmetricEncodings, useStrictSymmetric,
                                                      useUnsignedSymmetric, out, stream));
            }
            else
            {
                const size_t need = ahq_dlq_tfe_encodings_workspace_bytes(static_cast<int32_t>(_numEncodings));
                _workspace.reserve(need);
                ahqCheck(ahq_dlq_tfe_encodings(&st, bw, useSymmetricEncodings, useStrictSymmetric, useUnsignedSymmetric, out,
                                               nullptr, _workspace.ptr, need, stream));
            }
        }
        std::vector<double> host(5 * _numEncodings);
        hipCheck(hipMemcpyAsync(host.data(), out, host.size() * sizeof(double), hipMemcpyDeviceToHost,
                                static_cast<hipStream_t>(stream)),
                 "hipMemcpyAsync");
        hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
        std::vector<TfEncoding> encodings(_numEncodings);
        for (int64_t e = 0; e < _numEncodings; e++)
            encodings[e] = {host[5 * e], host[5 * e + 1], host[5 * e + 2], host[5 * e + 3], static_cast<int>(host[5 * e + 4])};
        return encodings;
    }

    // MinMaxEncodingAnalyzer keeps the raw extrema; the PDF analyzers do not
    std::vector<std::tuple<double, double>> getObservedMinMax() const override
    {
        if (_mode != QUANTIZATION_TF)
            return {};
        std::vector<float> mn(_numEncodings), mx(_numEncodings);
        hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(_stream)), "hipStreamSynchronize");
        hipCheck(hipMemcpy(mn.data(), _min.ptr, sizeof(float) * _numEncodings, hipMemcpyDeviceToHost), "hipMemcpy");
        hipCheck(hipMemcpy(mx.data(), _max.ptr, sizeof(float) * _numEncodings, hipMemcpyDeviceToHost), "hipMemcpy");
        std::vector<std::tuple<double, double>> out(_numEncodings);
        for (int64_t e = 0; e < _numEncodings; e++)
            out[e] = std::make_tuple(static_cast<double>(mn[e]), static_cast<double>(mx[e]));
        return out;
    }

    std::vector<std::vector<std::tuple<double, double>>> getStatsHistogram() const override
    {
        if (_mode == QUANTIZATION_TF)
            throw std::runtime_error("MinMaxEncodingAnalyzer does not have histogram stats");
        const size_t n = static_cast<size_t>(_numEncodings) * AHQ_DLQ_PDF_SIZE;
        std::vector<double> xleft(n), pdf(n);
        std::vector<int32_t> meta(4 * _numEncodings);
        hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(_stream)), "hipStreamSynchronize");
        hipCheck(hipMemcpy(xleft.data(), _xleft.ptr, n * sizeof(double), hipMemcpyDeviceToHost), "hipMemcpy");
        hipCheck(hipMemcpy(pdf.data(), _pdf.ptr, n * sizeof(double), hipMemcpyDeviceToHost), "hipMemcpy");
        hipCheck(hipMemcpy(meta.data(), _meta.ptr, meta.size() * sizeof(int32_t), hipMemcpyDeviceToHost), "hipMemcpy");
        std::vector<std::vector<std::tuple<double, double>>> out(_numEncodings);
        for (int64_t e = 0; e < _numEncodings; e++)
            if (meta[4 * e + 1])
                for (int i = 0; i < AHQ_DLQ_PDF_SIZE; i++)
                    out[e].emplace_back(xleft[e * AHQ_DLQ_PDF_SIZE + i], pdf[e * AHQ_DLQ_PDF_SIZE + i]);
        return out;
    }

    void setPercentileValue(float percentile) override
    {
        if (_mode != QUANTIZATION_PERCENTILE)
            throw std::runtime_error("setPercentileValue is only applicable for percentile encoding analyzers");
        _percentile = percentile;
    }
    float getPercentileValue() override
    {
        if (_mode != QUANTIZATION_PERCENTILE)
            throw std::runtime_error("getPercentileValue is only applicable for percentile encoding analyzers");
        return _percentile;
    }

private:
    ahq_dlq_pdf_state pdfState() const
    {
        ahq_dlq_pdf_state st {};
        st.num_slots = static_cast<int32_t>(_numEncodings);
        st.xleft     = static_cast<double*>(_xleft.ptr);
        st.pdf       = static_cast<double*>(_pdf.ptr);
        st.meta      = static_cast<int32_t*>(_meta.ptr);
        return st;
    }

    void clearStats(bool keepUpdatedFlag)
    {
        hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(_stream)), "hipStreamSynchronize");
        if (_mode == QUANTIZATION_TF)
        {
            // numeric_limits<float>::max() / lowest() (src/MinMaxEncodingAnalyzer.cpp:141-148)
            std::vector<float> hi(_numEncodings, 3.402823466e+38f), lo(_numEncodings, -3.402823466e+38f);
            hipCheck(hipMemcpy(_min.ptr, hi.data(), hi.size() * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy");
            hipCheck(hipMemcpy(_max.ptr, lo.data(), lo.size() * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy");
            return;
        }
        std::vector<int32_t> meta(4 * _numEncodings, 0);
        if (keepUpdatedFlag)   // _statsUpdated survives resetStats (src/TfEnhancedEncodingAnalyzer.cpp:44-50)
        {
            hipCheck(hipMemcpy(meta.data(), _meta.ptr, meta.size() * sizeof(int32_t), hipMemcpyDeviceToHost), "hipMemcpy");
            for (int64_t e = 0; e < _numEncodings; e++)
                meta[4 * e] = meta[4 * e + 1] = 0;
        }
        hipCheck(hipMemset(_xleft.ptr, 0, sizeof(double) * AHQ_DLQ_PDF_SIZE * _numEncodings), "hipMemset");
        hipCheck(hipMemset(_pdf.ptr, 0, sizeof(double) * AHQ_DLQ_PDF_SIZE * _numEncodings), "hipMemset");
        hipCheck(hipMemcpy(_meta.ptr, meta.data(), meta.size() * sizeof(int32_t), hipMemcpyHostToDevice), "hipMemcpy");
        _allInitialized = false;
    }

    QuantizationMode _mode;
    TensorDims _shape;
    int64_t _numEncodings = 1;
    bool _allInitialized  = false;
    float _percentile     = 100;   // src/PercentileEncodingAnalyzer.h:71
    void* _stream         = nullptr;
    DeviceBuffer _min, _max, _xleft, _pdf, _meta;
    mutable DeviceBuffer _workspace, _result;
};
}   // namespace detail

// QuantizerFactory.hpp:16-19, src/QuantizerFactory.cpp:34-42
template <typename DTYPE>
std::unique_ptr<IBlockEncodingAnalyzer<DTYPE>> getBlockEncodingAnalyzerInstance(QuantizationMode quantization_mode,
                                                                                const TensorDims& shape)
{
    static_assert(std::is_same<DTYPE, float>::value, "encoding analyzers keep float statistics");
    return std::unique_ptr<IBlockEncodingAnalyzer<DTYPE>>(new detail::DeviceBlockAnalyzer(quantization_mode, shape));
}

// ------------------------------------------------------------------------------------- TensorQuantizer.h:34-199 --
class BlockTensorQuantizer
{
public:
    BlockTensorQuantizer(TensorDims shape, int bitwidth, QuantizationMode quantScheme) :
        BlockTensorQuantizer(std::move(shape), QuantizationType::Int(bitwidth), quantScheme)
    {
    }

    // src/TensorQuantizer.cpp:22-36.  `bitwidth` is the legacy field setEncodings overwrites; the type stays.
    BlockTensorQuantizer(TensorDims shape, QuantizationType qtype, QuantizationMode quantScheme) :
        isEncodingValid(false), bitwidth(qtype.bitwidth()), _quantScheme(quantScheme), _qtype(qtype), _shape(std::move(shape))
    {
        _encodings.resize(detail::numel(_shape));
        _encodingAnalyzer.reset(new detail::DeviceBlockAnalyzer(quantScheme, _shape));
    }

    Encodings computeEncodings(bool useSymmetricEncodings) const
    {
        if (!_validStats)
            throw std::runtime_error("Cannot compute encodings before updating stats");
        Encodings encodings = _encodingAnalyzer->computeEncoding(static_cast<uint8_t>(bitwidth), useSymmetricEncodings,
                                                                 _useStrictSymmetric, _useUnsignedSymmetric, _zeroPointShift);
        if (!_qtype.isFloat())
            return encodings;
        // src/TensorQuantizer.cpp:182-224: scale = amax / maxValue, from the raw observed extrema where the analyzer
        // keeps them (min/max scheme) and they are not all zero, from the analyzer's range otherwise
        if (_qtype.bitwidth() != 8)
            throw std::runtime_error("BlockTensorQuantizer floating-point encodings currently support FP8 qtypes only");
        const auto observed    = _encodingAnalyzer->getObservedMinMax();
        const bool useObserved = observed.size() == encodings.size();
        const double maxValue  = _qtype.floatSpec().maxValue;
        for (size_t e = 0; e < encodings.size(); e++)
        {
            TfEncoding& enc = encodings[e];
            double amax     = std::max(std::abs(enc.min), std::abs(enc.max));
            if (useObserved)
            {
                const double seen = std::max(std::abs(std::get<0>(observed[e])), std::abs(std::get<1>(observed[e])));
                if (seen > 0.0)
                    amax = seen;
            }
            if (!(amax > 0))
                throw std::invalid_argument("FP8 amax must be positive");   // src/quantization_utils.cpp:186-194
            const double scale = amax / maxValue;
            enc                = {-scale * maxValue, scale * maxValue, scale, 0.0, _qtype.bitwidth()};
        }
        return encodings;
    }

    void resetEncodingStats()
    {
        _validStats     = false;
        isEncodingValid = false;
        _encodingAnalyzer->resetStats();
    }

    template <typename T>
    void quantizeDequantize(const T* input, T* output, const TensorDims& tensorShape, bool useCuda, void* stream = nullptr,
                            IForLoopRunner* runner = nullptr) const
    {
        const ComputationMode mode = useCuda ? COMP_MODE_GPU : COMP_MODE_CPU;
        if (!isEncodingValid)
            throw std::runtime_error("Cannot perform quantization before computing encodings");
        const int64_t numEncodings = detail::numel(_shape);
        if (_qtype.isFloat())
        {
            if (_qtype.bitwidth() != 8)
                throw std::runtime_error("BlockTensorQuantizer floating-point QDQ currently supports FP8 qtypes only");
            if constexpr (std::is_same<T, float>::value)
            {
                if (numEncodings == 1)
                {
                    quantizeDequantizeFp8(input, static_cast<uint64_t>(detail::numel(tensorShape)), _encodings[0], output,
                                          _qtype.floatSpec(), mode, stream, runner);
                }
                else
                {
                    detail::requireDevice(mode);
                    const ahq_layout layout = detail::makeLayout(tensorShape, _shape);
                    const auto& spec        = _qtype.floatSpec();
                    detail::ahqCheck(ahq_dlq_fp8_qdq(AHQ_F32, &layout, input, output, static_cast<const float*>(_encDevice.ptr),
                                                     spec.mantissaBits, spec.exponentMin, static_cast<float>(spec.maxValue),
                                                     stream));
                }
            }
            else
            {
                throw std::runtime_error("BlockTensorQuantizer FP8 QDQ currently supports float tensors only");
            }
            return;
        }
        if (numEncodings == 1)
        {
            // per tensor: the encoding travels by value (src/TensorQuantizer.cpp:106-111)
            aimet_amd::quantizeDequantize(input, static_cast<uint64_t>(detail::numel(tensorShape)), _encodings[0], output, mode,
                                          ROUND_NEAREST, stream, runner);
        }
        else
        {
            detail::requireDevice(mode);
            const ahq_layout layout = detail::makeLayout(tensorShape, _shape);
            if (detail::numel(tensorShape) == 0)
                return;
            detail::qdqBroadcastDevice(input, output, static_cast<const float*>(_encDevice.ptr), numEncodings, layout, stream);
        }
    }

    void updateStats(const float* tensor, const TensorDims& tensorShape, bool useCuda, IAllocator* alloc = nullptr,
                     void* stream = nullptr)
    {
        updateStats<float>(tensor, tensorShape, useCuda, alloc, stream);
    }

    template <typename T>
    void updateStats(const T* tensor, const TensorDims& tensorShape, bool useCuda, IAllocator* alloc = nullptr,
                     void* stream = nullptr)
    {
        _validStats = true;
        _encodingAnalyzer->update(tensor, detail::DtypeOf<T>::value, tensorShape, useCuda ? COMP_MODE_GPU : COMP_MODE_CPU, alloc,
                                  stream);
    }

    void setQuantScheme(QuantizationMode quantScheme)
    {
        // the reference only records the scheme here (src/TensorQuantizer.cpp:126-130); a different scheme needs
        // different statistics, so the analyzer is made anew
        if (quantScheme != _quantScheme)
            _encodingAnalyzer.reset(new detail::DeviceBlockAnalyzer(quantScheme, _shape));
        _quantScheme = quantScheme;
        resetEncodingStats();
    }
    QuantizationMode getQuantScheme() const { return _quantScheme; }
    bool getStrictSymmetric() const { return _useStrictSymmetric; }
    void setStrictSymmetric(bool useStrictSymmetric)
    {
        isEncodingValid     = false;
        _useStrictSymmetric = useStrictSymmetric;
    }
    bool getUnsignedSymmetric() const { return _useUnsignedSymmetric; }
    void setUnsignedSymmetric(bool useUnsignedsymmetric)
    {
        isEncodingValid       = false;
        _useUnsignedSymmetric = useUnsignedsymmetric;
    }
    std::vector<std::vector<std::tuple<double, double>>> getStatsHistogram() const
    {
        return _encodingAnalyzer->getStatsHistogram();
    }
    void setPercentileValue(float percentile) { _encodingAnalyzer->setPercentileValue(percentile); }
    float getPercentileValue() const { return _encodingAnalyzer->getPercentileValue(); }
    bool hasValidStats() { return _validStats; }
    TensorDims getShape() { return _shape; }
    Encodings getEncodings() { return _encodings; }
    QuantizationType getQuantizationType() const { return _qtype; }
    double getZeroPointShift() const { return _zeroPointShift; }
    void setZeroPointShift(double zeroPointShift) { _zeroPointShift = zeroPointShift; }

    void setEncodings(const Encodings& encodings)
    {
        if (static_cast<int64_t>(encodings.size()) != detail::numel(_shape))
            throw std::runtime_error("Length of encoding vector did not match BlockTensorQuantizer shape");
        isEncodingValid = true;
        _encodings      = encodings;
        bitwidth        = encodings[0].bw;
        if (encodings.size() > 1)
        {
            // several blocks: the kernels read the encodings from device memory, so they are put there once, here,
            // instead of in every quantizeDequantize call (a blocking copy: the caller gives no stream)
            const std::vector<float> host = detail::packEncodings(encodings);
            _encDevice.reserve(host.size() * sizeof(float));
            detail::hipCheck(hipDeviceSynchronize(), "hipDeviceSynchronize");   // earlier launches may read the old ones
            detail::hipCheck(hipMemcpy(_encDevice.ptr, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice),
                             "hipMemcpy");
        }
    }

    bool isEncodingValid;
    int bitwidth;

private:
    QuantizationMode _quantScheme;
    QuantizationType _qtype;
    bool _useStrictSymmetric   = false;
    bool _useUnsignedSymmetric = false;
    bool _validStats           = false;
    double _zeroPointShift     = 0.0;
    Encodings _encodings;
    std::unique_ptr<detail::DeviceBlockAnalyzer> _encodingAnalyzer;
    TensorDims _shape;
    detail::DeviceBuffer _encDevice;
};

}   // namespace aimet_amd

#ifdef AIMET_AMD_AS_DLQUANTIZATION
namespace DlQuantization = aimet_amd;
#endif

#endif   // AIMET_AMD_DLQ_HPP
