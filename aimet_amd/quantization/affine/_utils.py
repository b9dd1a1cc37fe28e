"""Quantization-grid helpers shared by encodings and quantizers (bitwidth / signed views of (qmin, qmax)).

Counterpart of aimet_torch/quantization/affine/_utils.py:19-175.
"""

from __future__ import annotations

import math


class _GridMixin:
    qmin: int
    qmax: int

    def _is_standard_grid(self) -> bool:
        return self.qmin + self.qmax == -1 or self.qmin == 0

    def _undefined(self, what: str) -> RuntimeError:
        return RuntimeError(
            f"{type(self).__qualname__}.{what} is undefined for qmin={self.qmin}, qmax={self.qmax}: "
            f"{what} only exists for grids [0, 2^B - 1] and [-2^(B-1), 2^(B-1) - 1]"
        )

    def _get_centroid(self) -> int:
        return math.ceil((self.qmax + self.qmin) / 2)

    def _get_bitwidth(self) -> int:
        """B such that the grid is [0, 2^B - 1] or [-2^(B-1), 2^(B-1) - 1]; RuntimeError otherwise."""
        if self._is_standard_grid():
            bits = math.log2(self.qmax - self.qmin + 1)
            if bits == int(bits):
                return int(bits)
        raise self._undefined("bitwidth")

    def _set_bitwidth(self, bitwidth: int):
        if bitwidth != int(bitwidth):
            raise TypeError(f"Setting bitwidth to a non-integer value {bitwidth} is not supported; set qmin/qmax instead")
        bitwidth = int(bitwidth)
        if bitwidth < 1:
            raise ValueError(f"Bitwidth can't be smaller than 1. Got {bitwidth}")
        if self.qmin + self.qmax == -1:
            self.qmin, self.qmax = -(2 ** (bitwidth - 1)), 2 ** (bitwidth - 1) - 1
        elif self.qmin == 0:
            self.qmax = 2 ** bitwidth - 1
        else:
            raise self._undefined("bitwidth")

    def _get_signed(self) -> bool:
        if self._is_standard_grid():
            return self.qmin < 0 <= self.qmax
        raise self._undefined("signed")

    def _set_signed(self, signed: bool):
        if not self._is_standard_grid():
            raise self._undefined("signed")
        was = self._get_signed()
        if was and not signed:
            shift = self.qmin
        elif signed and not was:
            shift = math.ceil((self.qmax + self.qmin) / 2)
        else:
            shift = 0
        self.qmin -= shift
        self.qmax -= shift
