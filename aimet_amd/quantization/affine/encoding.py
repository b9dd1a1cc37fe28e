"""Affine encodings: the (scale, offset, grid) description attached to quantizer outputs.

Counterpart of aimet_torch/quantization/affine/encoding.py:33-331 and :579-619 (the export formats are not part of
this package).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from aimet_amd.quantization.base.encoding import EncodingBase
from aimet_amd.quantization.affine._utils import _GridMixin
from aimet_amd.quantization.affine.backends import quantize, dequantize, quantize_dequantize, _derive_qmin_qmax

__all__ = ["AffineEncoding", "GroupedBlockEncoding"]


class AffineEncoding(EncodingBase, _GridMixin):
    """AffineEncoding(scale, offset, qmin, qmax, symmetry=False, block_size=None, zero_point_shift=None) or
    AffineEncoding(scale, offset, bitwidth, signed=False, symmetry=False, block_size=None, zero_point_shift=None)."""

    def __init__(self, scale: torch.Tensor, offset: torch.Tensor, *args, **kwargs):
        self.scale = scale
        self.offset = offset
        pos = tuple(args) + (None,) * (5 - len(args))
        first = kwargs.pop("qmin", kwargs.pop("bitwidth", pos[0]))
        second = kwargs.pop("qmax", kwargs.pop("signed", pos[1]))
        symmetry = kwargs.pop("symmetry", pos[2])
        block_size = kwargs.pop("block_size", pos[3])
        zero_point_shift = kwargs.pop("zero_point_shift", pos[4])
        self.producer = kwargs.pop("producer", None)
        if kwargs:
            raise TypeError(f"{type(self).__qualname__}.__init__ got unexpected keyword argument: {', '.join(kwargs)}")
        if first is None:
            raise TypeError("expected (qmin, qmax) or (bitwidth[, signed]) after scale and offset")
        if second is None or isinstance(second, bool):
            qmin, qmax = _derive_qmin_qmax(bitwidth=first, signed=bool(second))
        else:
            qmin, qmax = first, second
        if qmin >= qmax:
            raise ValueError(f"qmax should be strictly larger than qmin. Got qmax={qmax}, qmin={qmin}")
        self.qmin = qmin
        self.qmax = qmax
        self._symmetry = bool(symmetry)
        self.block_size = block_size
        self._zero_point_shift = zero_point_shift or 0.0
        if self._zero_point_shift not in (0.0, 0.5):
            raise ValueError(f"zero_point_shift should be 0.0 or 0.5. Got {self._zero_point_shift}")

    @property
    def mapping(self) -> str:
        return "affine"

    @property
    def granularity(self) -> str:
        if self.scale.dim() == 0:
            return "pertensor"
        if self.block_size is not None:
            return "blockwise"
        non_singleton = [d for d in self.scale.shape if d > 1]
        if len(non_singleton) <= 1:
            return "perchannel"
        return "unknown"

    @property
    def num_steps(self) -> int:
        return self.qmax - self.qmin

    @property
    def min(self) -> torch.Tensor:
        return (self.offset + self.qmin) * self.scale

    @property
    def max(self) -> torch.Tensor:
        return (self.offset + self.qmax) * self.scale

    @property
    def symmetry(self) -> bool:
        return self._symmetry

    @property
    def zero_point_shift(self) -> float:
        return self._zero_point_shift

    @property
    def bitwidth(self) -> int:
        return self._get_bitwidth()

    @property
    def signed(self) -> bool:
        return self._get_signed()

    def to(self, *args, **kwargs):
        """Same encoding with scale/offset moved to another device and/or floating-point dtype."""
        scale = self.scale.to(*args, **kwargs)
        if scale is self.scale:
            return self
        if not scale.dtype.is_floating_point:
            raise RuntimeError(f"Cannot change encoding data dtype to {scale.dtype}, must be a floating point dtype")
        return self._rebuilt(scale, self.offset.to(*args, **kwargs))

    def _rebuilt(self, scale, offset):
        return AffineEncoding(scale, offset, self.qmin, self.qmax, self._symmetry, self.block_size,
                              self._zero_point_shift, producer=self.producer)

    def quantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        return quantize(input, self.scale, self.offset, self.qmin, self.qmax, block_size=self.block_size)

    def dequantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        return dequantize(input, self.scale, self.offset, block_size=self.block_size)

    def quantize_dequantize(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        return quantize_dequantize(input, self.scale, self.offset, self.qmin, self.qmax, block_size=self.block_size,
                                   zero_point_shift=self._zero_point_shift)


class GroupedBlockEncoding(AffineEncoding):
    """Blockwise encoding whose block scales are integer multiples of a per-channel scale (LPBQ)."""

    def __init__(self, scale, offset, bitwidth: int, signed=False, symmetry=False,
                 block_size: Optional[Tuple[int, ...]] = None, block_grouping: Optional[Tuple[int, ...]] = None,
                 decompressed_bw: Optional[int] = None, per_channel_scale: Optional[torch.Tensor] = None, **kwargs):
        super().__init__(scale, offset, bitwidth, signed, symmetry, block_size, **kwargs)
        self.block_grouping = block_grouping
        self.decompressed_bw = decompressed_bw
        self.per_channel_scale = per_channel_scale

    @property
    def per_block_int_scale(self) -> torch.Tensor:
        """Integer multipliers m with scale = m * per_channel_scale (1 <= m <= 2^(decompressed_bw - bitwidth))."""
        return quantize(self.scale, scale=self.per_channel_scale, offset=torch.zeros_like(self.per_channel_scale),
                        qmin=1, qmax=2 ** (self.decompressed_bw - self.bitwidth), block_size=self.block_grouping)

    def _rebuilt(self, scale, offset):
        return GroupedBlockEncoding(scale, offset, self.bitwidth, self.signed, self._symmetry, self.block_size,
                                    self.block_grouping, self.decompressed_bw,
                                    self.per_channel_scale.to(device=scale.device, dtype=scale.dtype),
                                    zero_point_shift=self._zero_point_shift, producer=self.producer)
