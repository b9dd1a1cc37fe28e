"""Description of a simulated floating-point format (counterpart of aimet_torch/quantization/float/_finfo.py)."""

from __future__ import annotations

import math
from collections import namedtuple
from typing import Mapping, Optional

import torch


class _finfo(namedtuple("_finfo", ("exponent_bits", "mantissa_bits", "finite", "unsigned_zero"))):
    def to_torch_dtype(self) -> Optional[torch.dtype]:
        return _finfo_to_torch_dtype.get(self)

    @classmethod
    def from_torch_dtype(cls, dtype: torch.dtype) -> "_finfo":
        try:
            return _torch_dtype_to_finfo[dtype]
        except KeyError as e:
            raise ValueError(f"Expected dtype to be one of {list(_torch_dtype_to_finfo.keys())}; got {dtype}") from e

    def to_str(self) -> str:
        torch_dtype = self.to_torch_dtype()
        if torch_dtype:
            return str(torch_dtype).split(".")[1]
        e, m, fn, uz = self
        return f"float{e + m + 1}_e{e}m{m}{'fn' if fn else ''}{'uz' if uz else ''}"

    def is_float16(self) -> bool:
        return self == _float16

    def is_bfloat16(self) -> bool:
        return self == _bfloat16

    @property
    def max(self) -> float:
        """Largest representable value (_finfo.py:66-86)."""
        torch_dtype = self.to_torch_dtype()
        if torch_dtype:
            return torch.finfo(torch_dtype).max
        if self == _float4_e2m1fn:
            return 6.0
        if not self.finite and not self.unsigned_zero:
            exponent_max = 2 ** self.exponent_bits - 1
            return (2 - 2 ** -self.mantissa_bits) * 2 ** (exponent_max - exponent_max // 2 - 1)
        raise RuntimeError(f"Maximum representable value of {self.to_str()} is unkown")

    def kernel_format(self):
        """(mantissa bits, exponent of the smallest normal binade, largest value, overflow-to-NaN, unsigned zero) as
        the HIP fake-cast takes them.  Storage types of torch use their own exponent bias; any other layout follows
        the reference's formula (aimet_torch/fp_quantization.py:177-201), whose bias 2^E - floor(log2(max)) - 1 puts
        the smallest normal binade at 1 - bias."""
        mx = self.max
        torch_dtype = self.to_torch_dtype()
        if torch_dtype is not None:
            emin = round(math.log2(torch.finfo(torch_dtype).smallest_normal))
            overflow_nan = self.finite
        else:
            emin = 1 - (2 ** self.exponent_bits - math.floor(math.log2(mx)) - 1)
            overflow_nan = False  # cannot happen: max is on the grid and exactly representable in every input dtype
        return self.mantissa_bits, emin, float(mx), bool(overflow_nan), bool(self.unsigned_zero)


_float16 = _finfo(exponent_bits=5, mantissa_bits=10, finite=False, unsigned_zero=False)
_bfloat16 = _finfo(exponent_bits=8, mantissa_bits=7, finite=False, unsigned_zero=False)
_float8_e4m3fn = _finfo(exponent_bits=4, mantissa_bits=3, finite=True, unsigned_zero=False)
_float8_e4m3fnuz = _finfo(exponent_bits=4, mantissa_bits=3, finite=True, unsigned_zero=True)
_float8_e5m2 = _finfo(exponent_bits=5, mantissa_bits=2, finite=False, unsigned_zero=False)
_float8_e5m2fnuz = _finfo(exponent_bits=5, mantissa_bits=2, finite=True, unsigned_zero=True)
_float4_e2m1fn = _finfo(exponent_bits=2, mantissa_bits=1, finite=True, unsigned_zero=False)

_finfo_to_torch_dtype: Mapping[_finfo, torch.dtype] = {
    _float16: torch.float16,
    _bfloat16: torch.bfloat16,
    _float8_e4m3fn: torch.float8_e4m3fn,
    _float8_e4m3fnuz: torch.float8_e4m3fnuz,
    _float8_e5m2: torch.float8_e5m2,
    _float8_e5m2fnuz: torch.float8_e5m2fnuz,
}
_torch_dtype_to_finfo: Mapping[torch.dtype, _finfo] = {dt: fi for fi, dt in _finfo_to_torch_dtype.items()}
