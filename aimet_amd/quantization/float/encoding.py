"""Encoding of a float fake-cast (counterpart of aimet_torch/quantization/float/encoding.py:24-190)."""

from __future__ import annotations

from typing import Optional

import torch
from torch._C._nn import _parse_to as parse_to_args

from aimet_amd.quantization.base.encoding import EncodingBase
from ._finfo import _finfo

__all__ = ["FloatEncoding"]


class FloatEncoding(EncodingBase):
    def __init__(self, mantissa_bits: int, exponent_bits: int, finite: bool, unsigned_zero: bool, scale: torch.Tensor,
                 block_size=None, *, producer=None):
        if scale is None:
            raise ValueError("scale cannot be None for FloatEncoding")
        self._finfo = _finfo(exponent_bits, mantissa_bits, finite, unsigned_zero)
        self.scale = scale
        self.block_size = tuple(block_size) if block_size else None
        self.producer = producer

    @property
    def mapping(self) -> str:
        return "float"

    @property
    def mantissa_bits(self) -> int:
        return self._finfo.mantissa_bits

    @property
    def exponent_bits(self) -> int:
        return self._finfo.exponent_bits

    @property
    def finite(self) -> bool:
        return self._finfo.finite

    @property
    def unsigned_zero(self) -> bool:
        return self._finfo.unsigned_zero

    @property
    def maxval(self) -> torch.Tensor:
        """Largest representable value of the dequantized tensor."""
        return self.scale * self._finfo.max

    @property
    def bitwidth(self) -> int:
        return self.mantissa_bits + self.exponent_bits + 1

    @property
    def granularity(self) -> str:
        if self.scale.dim() == 0 or self.scale.numel() == 1:
            return "pertensor"
        if self.block_size:
            return "blockwise"
        non_singleton = [d for d in self.scale.shape if d > 1]
        return "perchannel" if len(non_singleton) <= 1 else "unknown"

    def to(self, *args, **kwargs) -> "FloatEncoding":
        device, dtype, _, _ = parse_to_args(*args, **kwargs)
        dtype = dtype or self.scale.dtype
        device = device or self.scale.device
        if dtype == self.scale.dtype and device == self.scale.device:
            return self
        if not dtype.is_floating_point:
            raise RuntimeError(f"Cannot change encoding data dtype to {dtype}, only floating point data types are supported")
        return FloatEncoding(self.mantissa_bits, self.exponent_bits, self.finite, self.unsigned_zero,
                             self.scale.to(dtype=dtype, device=device), self.block_size, producer=self.producer)

    def quantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        """float/encoding.py:140-152: the values the format stores, ``cast(clamp(input / scale))``."""
        from .quantizer import float_quantize

        if type(input) is not torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        return float_quantize(input, self._finfo, self.scale, self.block_size)

    def dequantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        """float/encoding.py:154-165: ``input * scale`` blockwise."""
        from .quantizer import float_dequantize

        if type(input) is not torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        return float_dequantize(input, self.scale, self.block_size)

    def quantize_dequantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        """float/encoding.py:167-178."""
        from .quantizer import float_quantize_dequantize

        if type(input) is not torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        return float_quantize_dequantize(input, self._finfo, self.scale, self.block_size)
