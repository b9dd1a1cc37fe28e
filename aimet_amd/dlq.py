"""DlQuantization's block tensor quantizer on the HIP library.

Mirrors ``DlQuantization::BlockTensorQuantizer`` (ModelOptimizations/DlQuantization/include/DlQuantization/
TensorQuantizer.h:34-199, src/TensorQuantizer.cpp) method for method, for the two integer calibration schemes on the
hot path: ``QUANTIZATION_TF`` (running min/max per block), ``QUANTIZATION_TF_ENHANCED`` (1536-bucket PDF per block
and the (delta, offset) grid search) and ``QUANTIZATION_PERCENTILE`` (the same PDF, clipped at a percentile), on
integer grids and on the FP8 formats (fake-cast with a per-block scale).  Tensors are torch tensors on a HIP device; statistics stay on the device, and
``computeEncodings`` returns host-side ``TfEncoding`` tuples like the reference.  There is no CPU path.
"""

from __future__ import annotations

from collections import namedtuple
from typing import List, Optional, Sequence

import torch

from . import _lib
from .quantization.affine.backends import hip as _hip

QUANTIZATION_TF = 0           # DlQuantization::QuantizationMode (Quantization.hpp)
QUANTIZATION_TF_ENHANCED = 1
QUANTIZATION_PERCENTILE = 3
_SCHEMES = (QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED, QUANTIZATION_PERCENTILE)
PDF_SIZE = _lib.DLQ_PDF_SIZE

TfEncoding = namedtuple("TfEncoding", ["min", "max", "delta", "offset", "bw"])


class QuantizationType:
    """DlQuantization::QuantizationType (include/DlQuantization/QuantizationType.hpp:36-186): an integer grid of a
    given bitwidth, or a small floating-point format described by its exponent/mantissa layout."""

    __slots__ = ("_float", "_bitwidth", "exponentBits", "mantissaBits", "exponentMin", "maxValue", "finite",
                 "unsignedZero")

    def __init__(self):
        raise TypeError("use QuantizationType.Int / Float / Fp8E4M3FN / Fp8E5M2")

    @classmethod
    def Int(cls, bitwidth: int) -> "QuantizationType":
        if bitwidth <= 0:
            raise ValueError("Integer quantization bitwidth must be positive")
        t = object.__new__(cls)
        t._float, t._bitwidth = False, int(bitwidth)
        t.exponentBits = t.mantissaBits = t.exponentMin = 0
        t.maxValue, t.finite, t.unsignedZero = 0.0, False, False
        return t

    @classmethod
    def Float(cls, exponentBits: int, mantissaBits: int, finite: bool, unsignedZero: bool) -> "QuantizationType":
        """Bitwidth, minimum normal exponent and largest value follow from the layout
        (QuantizationType.hpp:88-135): "fnuz" formats move the bias by one and use the whole top binade, "fn"
        formats give up only the all-ones mantissa of the top binade, IEEE-like formats give up the top binade."""
        if exponentBits <= 0:
            raise ValueError("Floating-point quantization exponent bits must be positive")
        if mantissaBits < 0:
            raise ValueError("Floating-point quantization mantissa bits must be non-negative")
        bias = (1 << (exponentBits - 1)) - 1 + (1 if unsignedZero else 0)
        unit = 2.0 ** -mantissaBits
        if unsignedZero:
            max_exponent, max_mantissa = (1 << exponentBits) - 1 - bias, 2.0 - unit
        elif finite:
            max_exponent, max_mantissa = (1 << exponentBits) - 1 - bias, 2.0 - 2.0 * unit
        else:
            max_exponent, max_mantissa = (1 << exponentBits) - 2 - bias, 2.0 - unit
        t = object.__new__(cls)
        t._float, t._bitwidth = True, 1 + exponentBits + mantissaBits
        t.exponentBits, t.mantissaBits, t.exponentMin = int(exponentBits), int(mantissaBits), 1 - bias
        t.maxValue, t.finite, t.unsignedZero = max_mantissa * 2.0 ** max_exponent, bool(finite), bool(unsignedZero)
        return t

    @classmethod
    def Fp8E4M3FN(cls) -> "QuantizationType":
        return cls.Float(4, 3, True, False)

    @classmethod
    def Fp8E5M2(cls) -> "QuantizationType":
        return cls.Float(5, 2, False, False)

    def isInt(self) -> bool:
        return not self._float

    def isFloat(self) -> bool:
        return self._float

    def bitwidth(self) -> int:
        return self._bitwidth

_FLT_MAX = torch.finfo(torch.float32).max


def _numel(shape: Sequence[int]) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


class BlockTensorQuantizer:
    """Simulated blocked quantization: the block size along tensor dimension i is tensor_shape[i] / shape[i], the
    quantizer shape being right-aligned against the tensor shape (tensor_utils.cpp:28-58)."""

    def __init__(self, shape: Sequence[int], bitwidth, quantScheme: int, device="cuda"):
        """``bitwidth``: an int (integer grid) or a QuantizationType (TensorQuantizer.cpp:17-29)."""
        if quantScheme not in _SCHEMES:
            raise ValueError("only QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED and QUANTIZATION_PERCENTILE are implemented")
        self._percentile = 100.0  # PercentileEncodingAnalyzer.h:71
        self._shape = tuple(int(d) for d in shape)
        self._qtype = bitwidth if isinstance(bitwidth, QuantizationType) else QuantizationType.Int(int(bitwidth))
        self.bitwidth = self._qtype.bitwidth()  # legacy field; setEncodings overwrites it, the qtype stays
        self.isEncodingValid = False
        self._quantScheme = quantScheme
        self._useStrictSymmetric = False
        self._useUnsignedSymmetric = False
        self._validStats = False
        self._zeroPointShift = 0.0
        self._device = torch.device(device)
        _lib.require_device(torch.empty(0, device=self._device), "BlockTensorQuantizer")
        self._E = _numel(self._shape)
        self._encodings: List[Optional[TfEncoding]] = [None] * self._E
        self._enc_dev = None  # (delta, offset, min, max) float32 device tensors of `shape`
        self._allocate_stats()

    # ------------------------------------------------------------------------------------------------ statistics --
    def _allocate_stats(self):
        E, dev = self._E, self._device
        if self._quantScheme == QUANTIZATION_TF:
            # numeric_limits<float>::max() / lowest() (MinMaxEncodingAnalyzer.cpp:141-148)
            self._min = torch.full((E,), _FLT_MAX, dtype=torch.float32, device=dev)
            self._max = torch.full((E,), -_FLT_MAX, dtype=torch.float32, device=dev)
        else:
            self._xleft = torch.zeros(E, PDF_SIZE, dtype=torch.float64, device=dev)
            self._pdf = torch.zeros(E, PDF_SIZE, dtype=torch.float64, device=dev)
            self._meta = torch.zeros(E, 4, dtype=torch.int32, device=dev)
            self._all_initialized = False

    def resetEncodingStats(self):
        self._validStats = False
        self.isEncodingValid = False
        if self._quantScheme == QUANTIZATION_TF:
            self._min.fill_(_FLT_MAX)
            self._max.fill_(-_FLT_MAX)
        else:
            self._xleft.zero_()
            self._pdf.zero_()
            self._meta[:, :2].zero_()  # _statsUpdated survives a reset (TfEnhancedEncodingAnalyzer.cpp:44-50)
            self._all_initialized = False

    def _layout(self, tensor: torch.Tensor):
        shape = tuple(tensor.shape)
        if len(self._shape) > len(shape):
            raise RuntimeError("Cannot interpret tensor and encoding dimensions as broadcastable")
        lead = len(shape) - len(self._shape)
        if any(d < 1 for d in shape[:lead]):  # leading encoding dims are padded with 1 (tensor_utils.cpp:12-26)
            raise RuntimeError("Cannot interpret tensor and encoding dimensions as broadcastable")
        block = []
        for k, e in enumerate(self._shape):
            d = shape[lead + k]
            if d < e or d % e != 0:
                raise RuntimeError("Cannot interpret tensor and encoding dimensions as broadcastable")
            block.append(d // e)
        return _hip._prepare(tensor, self._shape, tuple(block) if block else None)

    def updateStats(self, tensor: torch.Tensor, return_histogram: bool = False):
        """updateStats(tensor, tensorShape, useCuda=true): the tensor carries its own shape and lives on the GPU."""
        _lib.require_device(tensor, "tensor")
        if tensor.dtype not in _lib.DTYPE_CODE:
            raise TypeError("BlockTensorQuantizer::updateStats only supports float, half and bfloat16")
        lib = _lib.load()
        self._validStats = True
        x, layout = self._layout(tensor)
        code = _lib.DTYPE_CODE[x.dtype]
        stream = _lib.current_stream(x.device)
        if self._quantScheme == QUANTIZATION_TF:
            if x.numel() == 0:
                return None
            nbytes = lib.ahq_minmax_workspace_bytes(layout)
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
            if x.dtype == torch.float32:
                mn = torch.empty(self._E, dtype=torch.float32, device=x.device)
                mx = torch.empty_like(mn)
                _lib.check(lib.ahq_minmax(code, layout, x.data_ptr(), mn.data_ptr(), mx.data_ptr(), self._min.data_ptr(),
                                          self._max.data_ptr(), 2, ws.data_ptr(), nbytes, stream), "ahq_minmax")
            else:
                # 16-bit tensors: extrema in the tensor's dtype, widened, then the same std::min / std::max fold
                mn = torch.empty(self._E, dtype=x.dtype, device=x.device)
                mx = torch.empty_like(mn)
                _lib.check(lib.ahq_minmax(code, layout, x.data_ptr(), mn.data_ptr(), mx.data_ptr(), None, None, 2,
                                          ws.data_ptr(), nbytes, stream), "ahq_minmax")
                _lib.check(lib.ahq_dlq_minmax_fold(code, mn.data_ptr(), mx.data_ptr(), self._E, self._min.data_ptr(),
                                                   self._max.data_ptr(), stream), "ahq_dlq_minmax_fold")
            return None
        state = self._pdf_state()
        nbytes = lib.ahq_dlq_pdf_update_workspace_bytes(code, layout)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        hist = torch.empty(self._E, PDF_SIZE, dtype=torch.int32, device=x.device) if return_histogram else None
        with_init = 0 if self._all_initialized else 1
        _lib.check(lib.ahq_dlq_pdf_update(code, layout, x.data_ptr(), state, with_init, _lib.ptr(hist), ws.data_ptr(),
                                          nbytes, stream), "ahq_dlq_pdf_update")
        if not self._all_initialized:
            # one small read-back while the histogram range is still open; none once every block has its range
            self._all_initialized = bool((self._meta[:, 1] != 0).all().item())
        return hist

    def _pdf_state(self) -> _lib.DlqPdfState:
        st = _lib.DlqPdfState()
        st.num_slots = self._E
        st.xleft = self._xleft.data_ptr()
        st.pdf = self._pdf.data_ptr()
        st.meta = self._meta.data_ptr()
        return st

    def hasValidStats(self) -> bool:
        return self._validStats

    def getStatsHistogram(self):
        """List (one per block) of (left edge, probability) pairs."""
        if self._quantScheme == QUANTIZATION_TF:
            raise RuntimeError("MinMaxEncodingAnalyzer does not have histogram stats")
        xl, pdf, meta = self._xleft.cpu(), self._pdf.cpu(), self._meta.cpu()
        out = []
        for e in range(self._E):
            out.append(list(zip(xl[e].tolist(), pdf[e].tolist())) if meta[e, 1] else [])
        return out

    def setPercentileValue(self, percentile: float):
        if self._quantScheme != QUANTIZATION_PERCENTILE:
            raise RuntimeError("percentile is only used by the percentile quantization scheme")
        self._percentile = float(percentile)

    def getPercentileValue(self) -> float:
        if self._quantScheme != QUANTIZATION_PERCENTILE:
            raise RuntimeError("percentile is only used by the percentile quantization scheme")
        return self._percentile

    # ------------------------------------------------------------------------------------------------- encodings --
    def computeEncodings(self, useSymmetricEncodings: bool) -> List[TfEncoding]:
        if not self._validStats:
            raise RuntimeError("Cannot compute encodings before updating stats")
        lib = _lib.load()
        dev = self._device
        stream = _lib.current_stream(dev)
        out = torch.empty(self._E, 5, dtype=torch.float64, device=dev)
        sym = 1 if useSymmetricEncodings else 0
        if self._quantScheme == QUANTIZATION_TF:
            status = lib.ahq_dlq_minmax_encodings(self._min.data_ptr(), self._max.data_ptr(), self._E, self.bitwidth, sym,
                                                  int(self._useStrictSymmetric), int(self._useUnsignedSymmetric),
                                                  float(self._zeroPointShift), out.data_ptr(), stream)
            if status != _lib.AHQ_OK:
                raise RuntimeError(lib.ahq_last_error().decode())
        elif self._quantScheme == QUANTIZATION_PERCENTILE:
            if self._zeroPointShift != 0.0:
                raise RuntimeError("Non-zero zeroPointShift is only supported for min-max quant scheme.")
            _lib.check(lib.ahq_dlq_percentile_encodings(self._pdf_state(), self._percentile, self.bitwidth, sym,
                                                        int(self._useStrictSymmetric), int(self._useUnsignedSymmetric),
                                                        out.data_ptr(), stream), "ahq_dlq_percentile_encodings")
        else:
            if self._zeroPointShift != 0.0:
                raise RuntimeError("Non-zero zeroPointShift is only supported for min-max quant scheme.")
            nbytes = lib.ahq_dlq_tfe_encodings_workspace_bytes(self._E)
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
            self._last_best = torch.empty(self._E, 2, dtype=torch.int32, device=dev)
            _lib.check(lib.ahq_dlq_tfe_encodings(self._pdf_state(), self.bitwidth, sym, int(self._useStrictSymmetric),
                                                 int(self._useUnsignedSymmetric), out.data_ptr(),
                                                 self._last_best.data_ptr(), ws.data_ptr(), nbytes, stream),
                       "ahq_dlq_tfe_encodings")
        rows = out.cpu().tolist()
        if self._qtype.isFloat():
            return self._fp8_encodings(rows)
        return [TfEncoding(r[0], r[1], r[2], r[3], int(r[4])) for r in rows]

    def _fp8_encodings(self, rows) -> List[TfEncoding]:
        """TensorQuantizer.cpp:182-224: scale = amax / maxValue, with the raw observed extrema in place of the
        grid-snapped ones where the analyzer keeps them (min/max scheme only); delta carries the scale."""
        if self._qtype.bitwidth() != 8:
            raise RuntimeError("BlockTensorQuantizer floating-point encodings currently support FP8 qtypes only")
        observed = None
        if self._quantScheme == QUANTIZATION_TF:
            observed = torch.stack([self._min, self._max], dim=1).double().cpu().tolist()
        max_value = self._qtype.maxValue
        out = []
        for idx, r in enumerate(rows):
            amax = max(abs(r[0]), abs(r[1]))
            if observed is not None:
                seen = max(abs(observed[idx][0]), abs(observed[idx][1]))
                if seen > 0.0:
                    amax = seen
            if not amax > 0:
                raise ValueError("FP8 amax must be positive")  # computeFp8Scale, quantization_utils.cpp:186-194
            scale = amax / max_value
            out.append(TfEncoding(-scale * max_value, scale * max_value, scale, 0.0, self._qtype.bitwidth()))
        return out

    def setEncodings(self, encodings: Sequence[TfEncoding]):
        if len(encodings) != self._E:
            raise RuntimeError("Length of encoding vector did not match BlockTensorQuantizer shape")
        self.isEncodingValid = True
        self._encodings = [TfEncoding(*e) for e in encodings]
        self.bitwidth = int(self._encodings[0].bw)
        # the kernels take the encodings as float (QdqEncType, trim_functions.hpp:30-31): doubles narrowed once here
        t = torch.tensor([[e.delta, e.offset, e.min, e.max] for e in self._encodings], dtype=torch.float64)
        t = t.to(torch.float32).t().contiguous().to(self._device)
        self._enc_dev = t

    def getEncodings(self) -> List[Optional[TfEncoding]]:
        return list(self._encodings)

    def quantizeDequantize(self, input: torch.Tensor, output: Optional[torch.Tensor] = None) -> torch.Tensor:
        if not self.isEncodingValid:
            raise RuntimeError("Cannot perform quantization before computing encodings")
        _lib.require_device(input, "input")
        if input.dtype not in _lib.DTYPE_CODE:
            raise TypeError("quantizeDequantize only supports float, half and bfloat16")
        if self._qtype.isFloat():
            if self._qtype.bitwidth() != 8:
                raise RuntimeError("BlockTensorQuantizer floating-point QDQ currently supports FP8 qtypes only")
            if input.dtype != torch.float32:
                raise RuntimeError("BlockTensorQuantizer FP8 QDQ currently supports float tensors only")
        lib = _lib.load()
        x, layout = self._layout(input)
        y = torch.empty_like(x) if output is None else output
        if y.shape != x.shape or y.dtype != x.dtype or y.stride() != x.stride():
            raise RuntimeError("output must match the input's shape, dtype and memory layout")
        if self._qtype.isFloat():
            t = self._qtype
            _lib.check(lib.ahq_dlq_fp8_qdq(_lib.DTYPE_CODE[x.dtype], layout, x.data_ptr(), y.data_ptr(),
                                           self._enc_dev[0].data_ptr(), t.mantissaBits, t.exponentMin,
                                           float(t.maxValue), _lib.current_stream(x.device)), "ahq_dlq_fp8_qdq")
            return y
        grid = _hip._grid(_lib.AHQ_ARITH_DLQ, _lib.AHQ_OP_QDQ, x.dtype, torch.float32, 0, 0, 0.0)
        d, o, mn, mx = self._enc_dev
        _lib.check(lib.ahq_qdq_forward(grid, layout, x.data_ptr(), y.data_ptr(), None, d.data_ptr(), o.data_ptr(),
                                       mn.data_ptr(), mx.data_ptr(), _lib.current_stream(x.device)), "ahq_qdq_forward")
        return y

    # --------------------------------------------------------------------------------------------------- settings --
    def setQuantScheme(self, quantScheme: int):
        if quantScheme not in _SCHEMES:
            raise ValueError("only QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED and QUANTIZATION_PERCENTILE are implemented")
        self._quantScheme = quantScheme
        self._allocate_stats()
        self._validStats = False
        self.isEncodingValid = False

    def getQuantScheme(self) -> int:
        return self._quantScheme

    def getStrictSymmetric(self) -> bool:
        return self._useStrictSymmetric

    def setStrictSymmetric(self, useStrictSymmetric: bool):
        self.isEncodingValid = False
        self._useStrictSymmetric = bool(useStrictSymmetric)

    def getUnsignedSymmetric(self) -> bool:
        return self._useUnsignedSymmetric

    def setUnsignedSymmetric(self, useUnsignedSymmetric: bool):
        self.isEncodingValid = False
        self._useUnsignedSymmetric = bool(useUnsignedSymmetric)

    def getZeroPointShift(self) -> float:
        return self._zeroPointShift

    def setZeroPointShift(self, zeroPointShift: float):
        self._zeroPointShift = float(zeroPointShift)

    def getShape(self):
        return self._shape

    def getQuantizationType(self) -> QuantizationType:
        return self._qtype


def quantizeDequantizeBroadcast(input: torch.Tensor, encodings: Sequence[TfEncoding], encodingShape: Sequence[int]):
    """DlQuantization::quantizeDequantizeBroadcast (Quantization.hpp:106-114, trim_functions.cpp:909-948)."""
    q = BlockTensorQuantizer(encodingShape, int(encodings[0].bw) if encodings[0].bw else 8, QUANTIZATION_TF,
                             device=input.device)
    q.setEncodings(encodings)
    return q.quantizeDequantize(input)
