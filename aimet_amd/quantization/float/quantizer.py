"""Float fake-cast quantizer on the HIP library.

Counterpart of aimet_torch/quantization/float/quantizer.py:44-538 (``FloatQuantizeDequantize``) and of its functional
form ``_float_quantize_dequantize`` (:634-716).  The element-wise work -- divide by the scale, clamp to the format's
range, round onto the format's grid, multiply by the scale, each step rounded to the tensor's dtype -- is one kernel
(``ahq_float_qdq``); the scale itself (2^(log2|maxval| - log2 max)) and the calibration statistics are small
``shape``-sized tensors handled by torch and the min/max analyzer.  Not mirrored: the MXFP4 / NVFP4 subclasses and
ONNX export hooks.
"""

from __future__ import annotations

import functools
import math
from contextlib import contextmanager, nullcontext
from typing import Dict, List, Optional

import torch

from aimet_amd import _lib
from aimet_amd.quantization._utils import _is_expandable, patch_attr
from aimet_amd.quantization.affine.backends import hip as _hip
from aimet_amd.quantization.base.quantizer import QuantizerBase
from aimet_amd.quantization.encoding_analyzer import (EncodingAnalyzer, MinMaxEncodingAnalyzer, StatisticsNotFoundError,
                                                      _flag_extreme_min_max)
from aimet_amd.quantization.tensor import DequantizedTensor
from ._finfo import _finfo, _float4_e2m1fn, _torch_dtype_to_finfo
from .encoding import FloatEncoding

__all__ = ["FloatQuantizeDequantize", "QuantizeDequantize", "float_quantize_dequantize", "float_quantize",
           "float_dequantize"]


_TABLE_BYTES = {}


def _table_bytes(dtype_code: int, layout) -> int:
    """ahq_float_cast_workspace_bytes, asked once per (dtype, layout object): layouts are cached by shape."""
    key = (dtype_code, id(layout))
    held = _TABLE_BYTES.get(key)
    if held is None or held[0] is not layout:
        held = _TABLE_BYTES[key] = (layout, int(_lib.load().ahq_float_cast_workspace_bytes(dtype_code, layout)))
    return held[1]


def _launch(x: torch.Tensor, finfo: _finfo, scale: torch.Tensor, block_size, entry: str = "ahq_float_qdq") -> torch.Tensor:
    lib = _lib.load()
    x, layout = _hip._prepare(x, scale.shape, block_size)  # pylint: disable=protected-access
    y = torch.empty_like(x)
    if x.numel():
        mbits, emin, mx, overflow_nan, uz = finfo.kernel_format()
        s = _hip._enc_f32(scale)  # pylint: disable=protected-access
        # a format without a storage type goes through the reference's logarithm formula, whose steps round to the
        # tensor's dtype: on 16-bit tensors that differs from an exact cast next to binade boundaries
        log_form = finfo.to_torch_dtype() is None and x.dtype != torch.float32
        # large 16-bit tensors with one encoding go through a table of the cast's 65536 values, which lives in a
        # workspace (0 bytes: the table does not apply)
        nbytes = _table_bytes(_lib.DTYPE_CODE[x.dtype], layout) if scale.numel() == 1 else 0
        ws = _hip._workspace(nbytes, x.device) if nbytes else None  # pylint: disable=protected-access
        _lib.check(getattr(lib, entry)(_lib.DTYPE_CODE[x.dtype], layout, x.data_ptr(), y.data_ptr(), s.data_ptr(), mbits,
                                       emin, mx, int(overflow_nan), int(uz), int(log_form),
                                       ws.data_ptr() if ws is not None else None, nbytes,
                                       _lib.current_stream(x.device)),
                   entry)
    return y


def _checked_operands(input: torch.Tensor, scale: torch.Tensor):  # pylint: disable=redefined-builtin
    _lib.require_device(input, "input")
    dtype = torch.result_type(input, scale)
    if dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"float fake-cast computes in float32, float16 or bfloat16; got {dtype}")
    return (input if input.dtype == dtype else input.to(dtype)).detach(), scale.to(input.device)


def float_quantize(input: torch.Tensor, finfo: _finfo, scale: torch.Tensor, block_size=None) -> torch.Tensor:  # pylint: disable=redefined-builtin
    """_float_quantize (float/quantizer.py:687-706): ``cast(clamp(input / scale, -max, max))``, i.e. the value the
    simulated format stores.  No gradient is formed (FloatEncoding.quantize is its only caller)."""
    if finfo.to_torch_dtype() is None and finfo.unsigned_zero:
        raise NotImplementedError(f"Fake-casting to {finfo.to_str()} is not implemented")
    x, scale = _checked_operands(input, scale)
    if finfo.max > torch.finfo(x.dtype).max:
        raise RuntimeError(f"value cannot be converted to type {x.dtype} without overflow")
    return _launch(x, finfo, scale, tuple(block_size) if block_size else None, "ahq_float_quantize")


def float_dequantize(input: torch.Tensor, scale: torch.Tensor, block_size=None) -> torch.Tensor:  # pylint: disable=redefined-builtin
    """FloatEncoding.dequantize (float/encoding.py:154-165): ``input * scale`` blockwise."""
    x, scale = _checked_operands(input, scale)
    lib = _lib.load()
    x, layout = _hip._prepare(x, scale.shape, tuple(block_size) if block_size else None)  # pylint: disable=protected-access
    y = torch.empty_like(x)
    if x.numel():
        s = _hip._enc_f32(scale)  # pylint: disable=protected-access
        _lib.check(lib.ahq_float_dequantize(_lib.DTYPE_CODE[x.dtype], layout, x.data_ptr(), y.data_ptr(), s.data_ptr(),
                                            _lib.current_stream(x.device)), "ahq_float_dequantize")
    return y


class _FloatQdqFunction(torch.autograd.Function):
    """Forward: one kernel.  Backward: what autograd derives for the reference's composition (float/quantizer.py:634-710)
    -- g * scale, converted to the storage type and back (the backward of the two conversions: the gradient lands on
    the simulated format's grid), passed by the clamp where |x / scale| <= max, divided by the scale -- in one kernel;
    the rounding of the logarithm-based cast (formats without a storage type) has a zero derivative."""

    @staticmethod
    def forward(ctx, x, scale, finfo, block_size):
        ctx.finfo, ctx.block_size = finfo, block_size
        ctx.save_for_backward(x, scale)
        return _launch(x, finfo, scale, block_size)

    @staticmethod
    def backward(ctx, grad):
        x, scale = ctx.saved_tensors
        if ctx.finfo.to_torch_dtype() is None:
            # the logarithm formula rounds with torch.round: zero gradient everywhere
            return torch.zeros_like(grad), None, None, None
        # what autograd derives for div, clamp, .to(storage type).to(dtype), mul -- the casts' backward rounds the
        # gradient onto the format's grid -- in one pass (ahq_float_qdq_backward)
        lib = _lib.load()
        x, layout = _hip._prepare(x, scale.shape, ctx.block_size)  # pylint: disable=protected-access
        g = _hip._like(x, grad)  # pylint: disable=protected-access
        gx = torch.empty_like(x)
        if x.numel():
            mbits, emin, mx, overflow_nan, uz = ctx.finfo.kernel_format()
            s = _hip._enc_f32(scale)  # pylint: disable=protected-access
            _lib.check(lib.ahq_float_qdq_backward(_lib.DTYPE_CODE[x.dtype], layout, g.data_ptr(), x.data_ptr(),
                                                  gx.data_ptr(), s.data_ptr(), mbits, emin, mx, int(overflow_nan),
                                                  int(uz), _lib.current_stream(x.device)),
                       "ahq_float_qdq_backward")
        return gx, None, None, None


def float_quantize_dequantize(input: torch.Tensor, finfo: _finfo, scale: torch.Tensor,  # pylint: disable=redefined-builtin
                              block_size=None) -> torch.Tensor:
    """_float_quantize_dequantize (float/quantizer.py:634-656).  The result has the dtype torch's type promotion gives
    ``input / scale`` (a per-tensor scale leaves a 16-bit input in its dtype, a per-channel float32 scale widens it)."""
    _lib.require_device(input, "input")
    if finfo.to_torch_dtype() is None and finfo.unsigned_zero:
        raise NotImplementedError(f"Fake-casting to {finfo.to_str()} is not implemented")
    dtype = torch.result_type(input, scale)
    if dtype not in _lib.DTYPE_CODE:
        raise RuntimeError(f"float fake-cast computes in float32, float16 or bfloat16; got {dtype}")
    if finfo.max > torch.finfo(dtype).max:
        # the reference's clamp(-max, max) refuses a bound the tensor's dtype cannot hold
        raise RuntimeError(f"value cannot be converted to type {dtype} without overflow")
    x = input if input.dtype == dtype else input.to(dtype)
    scale = scale.to(x.device)
    if torch.is_grad_enabled() and x.requires_grad:
        return _FloatQdqFunction.apply(x, scale, finfo, tuple(block_size) if block_size else None)
    return _launch(x.detach(), finfo, scale, tuple(block_size) if block_size else None)


class FloatQuantizeDequantize(QuantizerBase):  # pylint: disable=abstract-method
    """Simulates quantization by fake-casting the input to a floating-point format given either as a torch dtype or
    by its exponent / mantissa bits (float/quantizer.py:44-171).  Sub-16-bit formats calibrate ``maxval`` (the value
    mapped to the format's largest one) with a min/max analyzer; 16-bit formats stay at scale 1."""

    maxval: torch.Tensor

    def __init__(self, exponent_bits: Optional[int] = None, mantissa_bits: Optional[int] = None,
                 finite: Optional[bool] = None, unsigned_zero: Optional[bool] = None,
                 dtype: Optional[torch.dtype] = None, shape=None, block_size=None,
                 encoding_analyzer: Optional[EncodingAnalyzer] = None):
        super().__init__()
        if dtype is None:
            if exponent_bits is None or mantissa_bits is None:
                raise ValueError('Neither "dtype" nor "exponent/mantissa_bits" was specified.')
            finite = False if finite is None else finite
            unsigned_zero = False if unsigned_zero is None else unsigned_zero
        else:
            if any(v is not None for v in (exponent_bits, mantissa_bits, finite, unsigned_zero)):
                raise ValueError(
                    'Argument "dtype" is mutually exclusive with "exponent/mantissa_bits/finite/unsigned_zero".')
            exponent_bits, mantissa_bits, finite, unsigned_zero = _finfo.from_torch_dtype(dtype)
        self._finfo = _finfo(exponent_bits, mantissa_bits, finite, unsigned_zero)
        if shape is None:
            self.shape = tuple(encoding_analyzer.observer.shape) if encoding_analyzer else ()
        else:
            self.shape = tuple(shape)
        self.block_size = tuple(block_size) if block_size else None
        if self.bitwidth < 16 and encoding_analyzer is None:
            encoding_analyzer = MinMaxEncodingAnalyzer(self.shape, self.block_size)
        self.encoding_analyzer = encoding_analyzer
        if encoding_analyzer and not _is_expandable(tuple(encoding_analyzer.observer.shape), self.shape):
            raise RuntimeError(f"Encoding analyzer of shape {encoding_analyzer.observer.shape} "
                               f"is incompatible with quantizer of shape {self.shape}.")
        self.register_buffer("maxval", torch.full(self.shape, self._finfo.max))
        self._is_overwrite_allowed.update({"maxval": True})
        self._assert_supported_dtype()

    def _assert_supported_dtype(self):
        fi = self._finfo
        if fi != _float4_e2m1fn and (fi.finite or fi.unsigned_zero) and fi.to_torch_dtype() is None:
            special = [d for d in _torch_dtype_to_finfo if d not in (torch.float16, torch.bfloat16)]
            raise RuntimeError("finite/unsigned_zero floating point has limited support. "
                               f"Expected PyTorch built-in data types, such as {special}; got '{fi.to_str()}'")

    # ------------------------------------------------------------------------------------------------- format --
    @property
    def exponent_bits(self) -> int:
        return self._finfo.exponent_bits

    @exponent_bits.setter
    def exponent_bits(self, exponent_bits: int):
        self._finfo = self._finfo._replace(exponent_bits=exponent_bits)

    @property
    def mantissa_bits(self) -> int:
        return self._finfo.mantissa_bits

    @mantissa_bits.setter
    def mantissa_bits(self, mantissa_bits: int):
        self._finfo = self._finfo._replace(mantissa_bits=mantissa_bits)

    @property
    def bitwidth(self) -> int:
        return self.exponent_bits + self.mantissa_bits + 1

    def is_float16(self) -> bool:
        return self._finfo.is_float16()

    def is_bfloat16(self) -> bool:
        return self._finfo.is_bfloat16()

    # ------------------------------------------------------------------------------------------ checkpointing --
    def get_extra_state(self):
        state = super().get_extra_state()
        fi = self._finfo
        state.update({"exponent_bits": torch.tensor(fi.exponent_bits), "mantissa_bits": torch.tensor(fi.mantissa_bits),
                      "finite": torch.tensor(fi.finite), "unsigned_zero": torch.tensor(fi.unsigned_zero),
                      "block_size": torch.tensor(self.block_size or ())})
        return state

    def set_extra_state(self, state):
        block_size = tuple(int(b) for b in state.get("block_size", self.block_size or ()))
        self.block_size = block_size or None
        fi = self._finfo
        self._finfo = _finfo(int(state.get("exponent_bits", fi.exponent_bits)),
                             int(state.get("mantissa_bits", fi.mantissa_bits)),
                             bool(state.get("finite", fi.finite)), bool(state.get("unsigned_zero", fi.unsigned_zero)))
        super().set_extra_state(state)

    def load_state_dict(self, state_dict, *args, **kwargs):  # pylint: disable=arguments-differ
        if "maxval" in state_dict:
            if self.maxval is None or self.maxval.shape != state_dict["maxval"].shape:
                del self.maxval
                self.register_buffer("maxval", state_dict["maxval"])
        elif self.maxval is not None:
            del self.maxval
            self.register_buffer("maxval", None)
        ret = super().load_state_dict(state_dict, *args, **kwargs)
        if self.maxval is not None:
            self.shape = tuple(self.maxval.shape)
        return ret

    def get_legacy_encodings(self) -> Optional[List[Dict]]:
        return [{"bitwidth": self.bitwidth, "dtype": "float"}]

    def set_legacy_encodings(self, encodings: List[Dict]):
        if encodings[0]["bitwidth"] != 16:
            raise RuntimeError(f"{self.__class__} can only import 16-bit legay encodings.")
        self.exponent_bits = 5
        self.mantissa_bits = 10

    # ---------------------------------------------------------------------------------------------- encodings --
    def get_scale(self) -> torch.Tensor:
        """2^(log2|maxval| - log2 max) (float/quantizer.py:336-342).  The reference evaluates this in float32 with the
        host's log2f / powf, which no other math library reproduces bit for bit; here the exponent is formed in
        float64 on the device and the result rounded to maxval's dtype once, which is exact whenever maxval / max is
        (in particular 1.0 for an uncalibrated quantizer) and otherwise within a few float32 ulps of the reference."""
        return (2 ** self._get_log2_scale()).to(self.maxval.dtype)

    def _get_log2_scale(self) -> torch.Tensor:
        return torch.log2(self.maxval.abs().double()) - math.log2(self._finfo.max)

    def get_encodings(self) -> Optional[FloatEncoding]:
        if not self.is_initialized():
            return None
        fi = self._finfo
        mv = self.maxval
        # the scale is six small launches' worth of arithmetic on maxval: derived once per value of maxval unless a
        # gradient has to flow through the derivation (the key follows the tensor object, its version and its memory)
        reuse = (type(self).get_scale is FloatQuantizeDequantize.get_scale and isinstance(mv, torch.Tensor)
                 and not (torch.is_grad_enabled() and mv.requires_grad))
        if reuse:
            key = (id(mv), mv._version, mv.data_ptr(), tuple(fi), self.block_size)  # pylint: disable=protected-access
            held = self.__dict__.get("_encoding_cache")
            if held is not None and held[0] == key:
                return held[1]
        enc = FloatEncoding(fi.mantissa_bits, fi.exponent_bits, fi.finite, fi.unsigned_zero, self.get_scale(),
                            block_size=self.block_size, producer=self)
        if reuse:
            self.__dict__["_encoding_cache"] = (key, enc)
        return enc

    def _get_dummy_encoding(self) -> FloatEncoding:
        fi = self._finfo
        scale = torch.ones((), dtype=torch.float32, device=self.maxval.device)
        return FloatEncoding(fi.mantissa_bits, fi.exponent_bits, fi.finite, fi.unsigned_zero, scale, block_size=None,
                             producer=self)

    @classmethod
    def from_encodings(cls, encodings: FloatEncoding) -> "FloatQuantizeDequantize":
        if not isinstance(encodings, FloatEncoding):
            raise TypeError(f"Expected {FloatEncoding}; got {type(encodings)}")
        qtzr = cls(*encodings._finfo, shape=encodings.scale.shape, block_size=encodings.block_size)  # pylint: disable=protected-access
        if not (encodings.scale.numel() == 1 and encodings.scale.item() == 1):
            qtzr.maxval = encodings.maxval.clone().detach()
        return qtzr

    # -------------------------------------------------------------------------------------------- calibration --
    @contextmanager
    def compute_encodings(self):
        """Observe inputs and set ``maxval`` from their statistics on exit; inside the context the forward pass uses
        the statistics of the current input (float/quantizer.py:363-431)."""
        with self._compute_encodings(passthrough=False):
            yield

    @contextmanager
    def _compute_encodings(self, passthrough: bool = False):
        if not self.encoding_analyzer or not any(self._is_overwrite_allowed.values()):
            yield
            return
        inner_forward = torch.Tensor.clone if passthrough else self.forward
        num_steps = math.pow(2, self.bitwidth) - 1

        @functools.wraps(inner_forward)
        def observing_forward(input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
            if type(input) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
                input = input.as_subclass(torch.Tensor)
            if input.numel() == 0:
                return inner_forward(input)
            stats = self.encoding_analyzer.update_stats(input)
            lo, hi = self.encoding_analyzer.compute_encodings_from_stats(stats, num_steps, is_symmetric=False)
            absmax = torch.maximum(lo.abs(), hi.abs())
            absmax = absmax.to(dtype=self.maxval.dtype, device=self.maxval.device).expand_as(self.maxval)
            with patch_attr(self, "maxval", absmax):
                return inner_forward(input)

        self.encoding_analyzer.reset_stats()
        with patch_attr(self, "forward", observing_forward):
            yield
        try:
            lo, hi = self.encoding_analyzer.compute_encodings(num_steps, is_symmetric=False)
            _flag_extreme_min_max(lo, hi)
        except StatisticsNotFoundError:
            return
        if lo is None or hi is None:
            return
        absmax = torch.maximum(lo.abs(), hi.abs()).expand_as(self.maxval)
        with torch.no_grad():
            self.maxval.copy_(absmax.to(dtype=self.maxval.dtype, device=self.maxval.device))

    @contextmanager
    def _precompute_encodings(self, dtype: Optional[torch.dtype] = None):
        enc = self.get_encodings()
        if enc is not None:
            enc = enc.to(dtype=dtype) if dtype is not None else enc
            enc.scale = enc.scale.detach()
        with (patch_attr(self, "get_encodings", lambda *a, **k: enc),
              patch_attr(self, "is_initialized", lambda *a, **k: enc is not None)) if enc is not None else nullcontext():
            yield

    # ------------------------------------------------------------------------------------------------ forward --
    def forward(self, input: torch.Tensor):  # pylint: disable=redefined-builtin
        if not input.is_floating_point():
            return input
        self._assert_supported_dtype()
        encoding = self.get_encodings()
        if encoding is None:
            if input.numel() == 0:
                encoding = self._get_dummy_encoding()
            else:
                raise RuntimeError(
                    "Failed to run FloatQuantizeDequantize since quantization parameters are not initialized."
                    " Please initialize the quantization parameters using `compute_encodings()`.")
        if type(input) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        output = float_quantize_dequantize(input, self._finfo, encoding.scale, encoding.block_size)
        output = output.as_subclass(DequantizedTensor)
        output.encoding = encoding
        return output

    def extra_repr(self) -> str:
        torch_dtype = self._finfo.to_torch_dtype()
        if torch_dtype is not None:
            parts = [f"dtype={torch_dtype}"]
        else:
            e, m, fn, uz = self._finfo
            parts = [f"exponent_bits={e}", f"mantissa_bits={m}", f"finite={fn}", f"unsigned_zero={uz}"]
        if self.shape:
            parts.append(f"shape={self.shape}")
        if self.block_size:
            parts.append(f"block_size={self.block_size}")
        return ", ".join(parts)


class QuantizeDequantize(FloatQuantizeDequantize):
    """Alias of FloatQuantizeDequantize (float/quantizer.py:540-543)."""
