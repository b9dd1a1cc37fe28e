"""DlQuantization's block tensor quantizer on the HIP library.

Mirrors ``DlQuantization::BlockTensorQuantizer`` (ModelOptimizations/DlQuantization/include/DlQuantization/
TensorQuantizer.h:34-199, src/TensorQuantizer.cpp) method for method, for the two integer calibration schemes on the
hot path: ``QUANTIZATION_TF`` (running min/max per block) and ``QUANTIZATION_TF_ENHANCED`` (1536-bucket PDF per block
and the (delta, offset) grid search).  Tensors are torch tensors on a HIP device; statistics stay on the device, and
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

_FLT_MAX = torch.finfo(torch.float32).max


def _numel(shape: Sequence[int]) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


class BlockTensorQuantizer:
    """Simulated blocked quantization: the block size along tensor dimension i is tensor_shape[i] / shape[i], the
    quantizer shape being right-aligned against the tensor shape (tensor_utils.cpp:28-58)."""

    def __init__(self, shape: Sequence[int], bitwidth: int, quantScheme: int, device="cuda"):
        if quantScheme not in _SCHEMES:
            raise ValueError("only QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED and QUANTIZATION_PERCENTILE are implemented")
        self._percentile = 100.0  # PercentileEncodingAnalyzer.h:71
        self._shape = tuple(int(d) for d in shape)
        self.bitwidth = int(bitwidth)
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
                torch.minimum(self._min, mn.float(), out=self._min)
                torch.maximum(self._max, mx.float(), out=self._max)
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
        return [TfEncoding(r[0], r[1], r[2], r[3], int(r[4])) for r in rows]

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
        lib = _lib.load()
        x, layout = self._layout(input)
        y = torch.empty_like(x) if output is None else output
        if y.shape != x.shape or y.dtype != x.dtype or y.stride() != x.stride():
            raise RuntimeError("output must match the input's shape, dtype and memory layout")
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


def quantizeDequantizeBroadcast(input: torch.Tensor, encodings: Sequence[TfEncoding], encodingShape: Sequence[int]):
    """DlQuantization::quantizeDequantizeBroadcast (Quantization.hpp:106-114, trim_functions.cpp:909-948)."""
    q = BlockTensorQuantizer(encodingShape, int(encodings[0].bw) if encodings[0].bw else 8, QUANTIZATION_TF,
                             device=input.device)
    q.setEncodings(encodings)
    return q.quantizeDequantize(input)
