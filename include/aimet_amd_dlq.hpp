// aimet_amd_dlq.hpp -- header-only C++ facade over the C ABI of libaimet_amd.so with the interface of
// DlQuantization::BlockTensorQuantizer (ModelOptimizations/DlQuantization/include/DlQuantization/TensorQuantizer.h:34-199,
// src/TensorQuantizer.cpp), for the QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED and QUANTIZATION_PERCENTILE schemes on integer grids and FP8 formats.
//
// Differences from the reference class, all forced by "device only":
//   * useCuda must be true: tensors are device pointers (the reference's CPU path has no counterpart here);
//   * the IAllocator* argument is gone: the object owns its device state (hipMalloc in the constructor and on the first
//     call that needs a larger workspace) -- the shared library itself never allocates;
//   * half / bfloat16 tensors are passed as `const void*` with an ahq_dtype tag instead of Eigen types.
// Exceptions and their messages are the reference's (std::runtime_error).
#ifndef AIMET_AMD_DLQ_HPP
#define AIMET_AMD_DLQ_HPP

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "aimet_amd.h"

namespace aimet_amd
{

enum QuantizationMode
{
    QUANTIZATION_TF          = 0,
    QUANTIZATION_TF_ENHANCED = 1,
    QUANTIZATION_PERCENTILE  = 3
};

struct TfEncoding
{
    double min, max, delta, offset;
    int bw;
};

// QuantizationType (DlQuantization/include/DlQuantization/QuantizationType.hpp:36-186): an integer grid of a given
// bitwidth, or a small floating-point format given by its exponent/mantissa layout.
class QuantizationType
{
public:
    static QuantizationType Int(int bitwidth)
    {
        if (bitwidth <= 0)
            throw std::invalid_argument("Integer quantization bitwidth must be positive");
        QuantizationType t;
        t._bitwidth = bitwidth;
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
        QuantizationType t;
        t._isFloat     = true;
        t._bitwidth    = 1 + exponentBits + mantissaBits;
        t.exponentBits = exponentBits;
        t.mantissaBits = mantissaBits;
        t.exponentMin  = 1 - bias;
        t.maxValue     = man * std::ldexp(1.0, top);
        t.finite       = finite;
        t.unsignedZero = unsignedZero;
        return t;
    }

    static QuantizationType Fp8E4M3FN() { return Float(4, 3, true, false); }
    static QuantizationType Fp8E5M2() { return Float(5, 2, false, false); }

    bool isInt() const { return !_isFloat; }
    bool isFloat() const { return _isFloat; }
    int bitwidth() const { return _bitwidth; }

    int exponentBits = 0, mantissaBits = 0, exponentMin = 0;
    double maxValue  = 0.0;
    bool finite = false, unsignedZero = false;

private:
    QuantizationType() = default;
    bool _isFloat = false;
    int _bitwidth = 0;
};

using TensorDim  = int64_t;
using TensorDims = std::vector<TensorDim>;
using Encodings  = std::vector<TfEncoding>;

namespace detail
{
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
// A device buffer that only ever grows.
struct DeviceBuffer
{
    void* ptr    = nullptr;
    size_t bytes = 0;
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer&) = delete;
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
            hipCheck(hipFree(ptr), "hipFree");
        ptr = nullptr;
        hipCheck(hipMalloc(&ptr, n), "hipMalloc");
        bytes = n;
    }
};
}   // namespace detail

class BlockTensorQuantizer
{
public:
    BlockTensorQuantizer(TensorDims shape, int bitwidth, QuantizationMode quantScheme) :
        BlockTensorQuantizer(std::move(shape), QuantizationType::Int(bitwidth), quantScheme)
    {
    }

    // TensorQuantizer.cpp:22-29.  `bitwidth` is the legacy field setEncodings overwrites; the type stays.
    BlockTensorQuantizer(TensorDims shape, QuantizationType qtype, QuantizationMode quantScheme) :
        isEncodingValid(false), bitwidth(qtype.bitwidth()), _quantScheme(quantScheme), _shape(std::move(shape)),
        _qtype(qtype)
    {
        _numEncodings = 1;
        for (auto d: _shape)
            _numEncodings *= d;
        _encodings.resize(_numEncodings);
        allocateStats();
    }

    void resetEncodingStats()
    {
        _validStats     = false;
        isEncodingValid = false;
        clearStats(true);
    }

    // updateStats(tensor, tensorShape, useCuda, alloc, stream) of the reference, for float tensors
    void updateStats(const float* tensor, const TensorDims& tensorShape, bool useCuda, void* stream = nullptr)
    {
        updateStats(tensor, AHQ_F32, tensorShape, useCuda, stream);
    }

    // ... and for half (AHQ_F16) / bfloat16 (AHQ_BF16) tensors
    void updateStats(const void* tensor, int32_t dtype, const TensorDims& tensorShape, bool useCuda, void* stream = nullptr)
    {
        requireDevice(useCuda);
        _validStats             = true;
        const ahq_layout layout = makeLayout(tensorShape);
        if (_quantScheme == QUANTIZATION_TF)
        {
            if (dtype != AHQ_F32)
                throw std::runtime_error("this facade folds running min/max for float tensors only");
            const size_t need = ahq_minmax_workspace_bytes(&layout);
            _workspace.reserve(need + 2 * sizeof(float) * _numEncodings + 512);
            char* w     = static_cast<char*>(_workspace.ptr);
            float* bmin = reinterpret_cast<float*>(w + ((need + 255) & ~size_t(255)));
            float* bmax = bmin + _numEncodings;
            detail::ahqCheck(ahq_minmax(dtype, &layout, tensor, bmin, bmax, _min.ptr, _max.ptr, 2, w, need, stream));
            return;
        }
        const size_t need = ahq_dlq_pdf_update_workspace_bytes(dtype, &layout);
        _workspace.reserve(need);
        ahq_dlq_pdf_state st = pdfState();
        detail::ahqCheck(ahq_dlq_pdf_update(dtype, &layout, tensor, &st, _allInitialized ? 0 : 1, nullptr, _workspace.ptr,
                                            need, stream));
        if (!_allInitialized)
        {
            std::vector<int32_t> meta(4 * _numEncodings);
            detail::hipCheck(hipMemcpyAsync(meta.data(), _meta.ptr, meta.size() * sizeof(int32_t), hipMemcpyDeviceToHost,
                                            static_cast<hipStream_t>(stream)),
                             "hipMemcpyAsync");
            detail::hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
            _allInitialized = true;
            for (int64_t e = 0; e < _numEncodings; e++)
                _allInitialized = _allInitialized && meta[4 * e + 1] != 0;
        }
    }

    Encodings computeEncodings(bool useSymmetricEncodings, void* stream = nullptr) const
    {
        if (!_validStats)
            throw std::runtime_error("Cannot compute encodings before updating stats");
        _result.reserve(sizeof(double) * 5 * _numEncodings);
        double* out = static_cast<double*>(_result.ptr);
        if (_quantScheme == QUANTIZATION_TF)
        {
            detail::ahqCheck(ahq_dlq_minmax_encodings(static_cast<const float*>(_min.ptr), static_cast<const float*>(_max.ptr),
                                                      _numEncodings, bitwidth, useSymmetricEncodings, _useStrictSymmetric,
                                                      _useUnsignedSymmetric, _zeroPointShift, out, stream));
        }
        else if (_quantScheme == QUANTIZATION_PERCENTILE)
        {
            if (_zeroPointShift != 0.0)
                throw std::runtime_error("Non-zero zeroPointShift is only supported for min-max quant scheme.");
            ahq_dlq_pdf_state st = pdfState();
            detail::ahqCheck(ahq_dlq_percentile_encodings(&st, _percentile, bitwidth, useSymmetricEncodings,
                                                          _useStrictSymmetric, _useUnsignedSymmetric, out, stream));
        }
        else
        {
            if (_zeroPointShift != 0.0)
                throw std::runtime_error("Non-zero zeroPointShift is only supported for min-max quant scheme.");
            const size_t need = ahq_dlq_tfe_encodings_workspace_bytes(static_cast<int32_t>(_numEncodings));
            _workspace.reserve(need);
            ahq_dlq_pdf_state st = pdfState();
            detail::ahqCheck(ahq_dlq_tfe_encodings(&st, bitwidth, useSymmetricEncodings, _useStrictSymmetric,
                                                   _useUnsignedSymmetric, out, nullptr, _workspace.ptr, need, stream));
        }
        std::vector<double> host(5 * _numEncodings);
        detail::hipCheck(hipMemcpyAsync(host.data(), out, host.size() * sizeof(double), hipMemcpyDeviceToHost,
                                        static_cast<hipStream_t>(stream)),
                         "hipMemcpyAsync");
        detail::hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
        Encodings encodings(_numEncodings);
        for (int64_t e = 0; e < _numEncodings; e++)
            encodings[e] = {host[5 * e], host[5 * e + 1], host[5 * e + 2], host[5 * e + 3], static_cast<int>(host[5 * e + 4])};
        if (_qtype.isFloat())
            toFp8Encodings(encodings, stream);
        return encodings;
    }

    void setEncodings(const Encodings& encodings, void* stream = nullptr)
    {
        if (static_cast<int64_t>(encodings.size()) != _numEncodings)
            throw std::runtime_error("Length of encoding vector did not match BlockTensorQuantizer shape");
        isEncodingValid = true;
        _encodings      = encodings;
        bitwidth        = encodings[0].bw;
        // delta | offset | min | max as float arrays (QdqEncType is float, trim_functions.hpp:30-31)
        std::vector<float> host(4 * _numEncodings);
        for (int64_t e = 0; e < _numEncodings; e++)
        {
            host[e]                     = static_cast<float>(encodings[e].delta);
            host[_numEncodings + e]     = static_cast<float>(encodings[e].offset);
            host[2 * _numEncodings + e] = static_cast<float>(encodings[e].min);
            host[3 * _numEncodings + e] = static_cast<float>(encodings[e].max);
        }
        _encDevice.reserve(host.size() * sizeof(float));
        detail::hipCheck(hipMemcpyAsync(_encDevice.ptr, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice,
                                        static_cast<hipStream_t>(stream)),
                         "hipMemcpyAsync");
        detail::hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
    }

    void quantizeDequantize(const float* input, float* output, const TensorDims& tensorShape, bool useCuda,
                            void* stream = nullptr) const
    {
        quantizeDequantize(input, output, AHQ_F32, tensorShape, useCuda, stream);
    }

    void quantizeDequantize(const void* input, void* output, int32_t dtype, const TensorDims& tensorShape, bool useCuda,
                            void* stream = nullptr) const
    {
        requireDevice(useCuda);
        if (!isEncodingValid)
            throw std::runtime_error("Cannot perform quantization before computing encodings");
        const ahq_layout layout = makeLayout(tensorShape);
        if (_qtype.isFloat())
        {
            if (_qtype.bitwidth() != 8)
                throw std::runtime_error("BlockTensorQuantizer floating-point QDQ currently supports FP8 qtypes only");
            if (dtype != AHQ_F32)
                throw std::runtime_error("BlockTensorQuantizer FP8 QDQ currently supports float tensors only");
            detail::ahqCheck(ahq_dlq_fp8_qdq(dtype, &layout, input, output, static_cast<const float*>(_encDevice.ptr),
                                             _qtype.mantissaBits, _qtype.exponentMin, static_cast<float>(_qtype.maxValue),
                                             stream));
            return;
        }
        ahq_grid grid{};
        grid.arith         = AHQ_ARITH_DLQ;
        grid.op            = AHQ_OP_QDQ;
        grid.io_dtype      = dtype;
        grid.compute_dtype = AHQ_F32;
        const float* enc   = static_cast<const float*>(_encDevice.ptr);
        detail::ahqCheck(ahq_qdq_forward(&grid, &layout, input, output, nullptr, enc, enc + _numEncodings,
                                         enc + 2 * _numEncodings, enc + 3 * _numEncodings, stream));
    }

    std::vector<std::vector<std::tuple<double, double>>> getStatsHistogram() const
    {
        if (_quantScheme == QUANTIZATION_TF)
            throw std::runtime_error("MinMaxEncodingAnalyzer does not have histogram stats");
        const size_t n = static_cast<size_t>(_numEncodings) * AHQ_DLQ_PDF_SIZE;
        std::vector<double> xleft(n), pdf(n);
        std::vector<int32_t> meta(4 * _numEncodings);
        detail::hipCheck(hipMemcpy(xleft.data(), _xleft.ptr, n * sizeof(double), hipMemcpyDeviceToHost), "hipMemcpy");
        detail::hipCheck(hipMemcpy(pdf.data(), _pdf.ptr, n * sizeof(double), hipMemcpyDeviceToHost), "hipMemcpy");
        detail::hipCheck(hipMemcpy(meta.data(), _meta.ptr, meta.size() * sizeof(int32_t), hipMemcpyDeviceToHost), "hipMemcpy");
        std::vector<std::vector<std::tuple<double, double>>> out(_numEncodings);
        for (int64_t e = 0; e < _numEncodings; e++)
            if (meta[4 * e + 1])
                for (int i = 0; i < AHQ_DLQ_PDF_SIZE; i++)
                    out[e].emplace_back(xleft[e * AHQ_DLQ_PDF_SIZE + i], pdf[e * AHQ_DLQ_PDF_SIZE + i]);
        return out;
    }

    void setQuantScheme(QuantizationMode quantScheme)
    {
        _quantScheme = quantScheme;
        allocateStats();
        resetEncodingStats();
    }
    QuantizationMode getQuantScheme() const { return _quantScheme; }
    bool getStrictSymmetric() const { return _useStrictSymmetric; }
    void setStrictSymmetric(bool v)
    {
        isEncodingValid     = false;
        _useStrictSymmetric = v;
    }
    bool getUnsignedSymmetric() const { return _useUnsignedSymmetric; }
    void setUnsignedSymmetric(bool v)
    {
        isEncodingValid       = false;
        _useUnsignedSymmetric = v;
    }
    void setPercentileValue(float percentile)
    {
        if (_quantScheme != QUANTIZATION_PERCENTILE)
            throw std::runtime_error("percentile is only used by the percentile quantization scheme");
        _percentile = percentile;
    }
    float getPercentileValue() const
    {
        if (_quantScheme != QUANTIZATION_PERCENTILE)
            throw std::runtime_error("percentile is only used by the percentile quantization scheme");
        return _percentile;
    }
    bool hasValidStats() const { return _validStats; }
    TensorDims getShape() const { return _shape; }
    Encodings getEncodings() const { return _encodings; }
    QuantizationType getQuantizationType() const { return _qtype; }
    double getZeroPointShift() const { return _zeroPointShift; }
    void setZeroPointShift(double v) { _zeroPointShift = v; }

    bool isEncodingValid;
    int bitwidth;

private:
    // TensorQuantizer.cpp:182-224: scale = amax / maxValue, from the raw observed extrema where the analyzer keeps
    // them (min/max scheme) and they are not all zero, from the analyzer's range otherwise; delta carries the scale.
    void toFp8Encodings(Encodings& encodings, void* stream) const
    {
        if (_qtype.bitwidth() != 8)
            throw std::runtime_error("BlockTensorQuantizer floating-point encodings currently support FP8 qtypes only");
        std::vector<float> seenMin, seenMax;
        if (_quantScheme == QUANTIZATION_TF)
        {
            seenMin.resize(_numEncodings);
            seenMax.resize(_numEncodings);
            detail::hipCheck(hipMemcpyAsync(seenMin.data(), _min.ptr, sizeof(float) * _numEncodings, hipMemcpyDeviceToHost,
                                            static_cast<hipStream_t>(stream)), "hipMemcpyAsync");
            detail::hipCheck(hipMemcpyAsync(seenMax.data(), _max.ptr, sizeof(float) * _numEncodings, hipMemcpyDeviceToHost,
                                            static_cast<hipStream_t>(stream)), "hipMemcpyAsync");
            detail::hipCheck(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
        }
        for (int64_t e = 0; e < _numEncodings; e++)
        {
            TfEncoding& enc = encodings[e];
            double amax     = std::max(std::abs(enc.min), std::abs(enc.max));
            if (!seenMin.empty())
            {
                const double seen = std::max(std::abs(static_cast<double>(seenMin[e])), std::abs(static_cast<double>(seenMax[e])));
                if (seen > 0.0)
                    amax = seen;
            }
            if (!(amax > 0))
                throw std::invalid_argument("FP8 amax must be positive");   // quantization_utils.cpp:186-194
            const double scale = amax / _qtype.maxValue;
            enc                = {-scale * _qtype.maxValue, scale * _qtype.maxValue, scale, 0.0, _qtype.bitwidth()};
        }
    }

    static void requireDevice(bool useCuda)
    {
        if (!useCuda)
            throw std::runtime_error("Not compiled for CPU mode: tensors must live in device memory");
    }

    // getBroadcastableShapes (tensor_utils.cpp:28-58) as an ahq_layout: the quantizer shape is right-aligned against
    // the tensor shape, block size along dim i = tensorShape[i] / shape[i]
    ahq_layout makeLayout(const TensorDims& tensorShape) const
    {
        const size_t nd = tensorShape.size();
        if (_shape.size() > nd || nd > AHQ_MAX_DIMS)
            throw std::runtime_error("Cannot interpret tensor and encoding dimensions as broadcastable");
        ahq_layout layout{};
        layout.ndim       = static_cast<int32_t>(nd);
        const size_t lead = nd - _shape.size();
        int64_t stride    = 1;
        for (size_t i = nd; i-- > 0;)
        {
            const int64_t d = tensorShape[i];
            const int64_t e = i < lead ? 1 : _shape[i - lead];
            if (!(d == e) && (d < e || d % e != 0))
                throw std::runtime_error("Cannot interpret tensor and encoding dimensions as broadcastable");
            layout.dims[i]       = d;
            layout.block[i]      = e > 1 ? d / e : (d > 0 ? d : 1);
            layout.enc_stride[i] = e > 1 ? stride : 0;
            stride *= e;
        }
        return layout;
    }

    ahq_dlq_pdf_state pdfState() const
    {
        ahq_dlq_pdf_state st{};
        st.num_slots = static_cast<int32_t>(_numEncodings);
        st.xleft     = static_cast<double*>(_xleft.ptr);
        st.pdf       = static_cast<double*>(_pdf.ptr);
        st.meta      = static_cast<int32_t*>(_meta.ptr);
        return st;
    }

    void allocateStats()
    {
        if (_quantScheme == QUANTIZATION_TF)
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

    void clearStats(bool keepUpdatedFlag)
    {
        if (_quantScheme == QUANTIZATION_TF)
        {
            // numeric_limits<float>::max() / lowest() (MinMaxEncodingAnalyzer.cpp:141-148)
            std::vector<float> hi(_numEncodings, 3.402823466e+38f), lo(_numEncodings, -3.402823466e+38f);
            detail::hipCheck(hipMemcpy(_min.ptr, hi.data(), hi.size() * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy");
            detail::hipCheck(hipMemcpy(_max.ptr, lo.data(), lo.size() * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy");
            return;
        }
        std::vector<int32_t> meta(4 * _numEncodings, 0);
        if (keepUpdatedFlag)   // _statsUpdated survives resetStats (TfEnhancedEncodingAnalyzer.cpp:44-50)
        {
            detail::hipCheck(hipMemcpy(meta.data(), _meta.ptr, meta.size() * sizeof(int32_t), hipMemcpyDeviceToHost), "hipMemcpy");
            for (int64_t e = 0; e < _numEncodings; e++)
                meta[4 * e] = meta[4 * e + 1] = 0;
        }
        detail::hipCheck(hipMemset(_xleft.ptr, 0, sizeof(double) * AHQ_DLQ_PDF_SIZE * _numEncodings), "hipMemset");
        detail::hipCheck(hipMemset(_pdf.ptr, 0, sizeof(double) * AHQ_DLQ_PDF_SIZE * _numEncodings), "hipMemset");
        detail::hipCheck(hipMemcpy(_meta.ptr, meta.data(), meta.size() * sizeof(int32_t), hipMemcpyHostToDevice), "hipMemcpy");
        _allInitialized = false;
    }

    QuantizationMode _quantScheme;
    bool _useStrictSymmetric   = false;
    bool _useUnsignedSymmetric = false;
    bool _validStats           = false;
    bool _allInitialized       = false;
    double _zeroPointShift     = 0.0;
    float _percentile          = 100;
    Encodings _encodings;
    TensorDims _shape;
    QuantizationType _qtype;
    int64_t _numEncodings = 1;
    detail::DeviceBuffer _min, _max, _xleft, _pdf, _meta, _encDevice;
    mutable detail::DeviceBuffer _workspace, _result;
};

}   // namespace aimet_amd

#endif   // AIMET_AMD_DLQ_HPP
