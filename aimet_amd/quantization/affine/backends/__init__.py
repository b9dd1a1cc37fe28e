"""Functional affine quantization API dispatched to the active backend.

Counterpart of aimet_torch/quantization/affine/backends/__init__.py:50-445: three call forms
``(bitwidth[, signed])``, ``(num_steps=, signed=)`` and ``(qmin, qmax)``, optional ``block_size`` and
``zero_point_shift``.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from aimet_amd.quantization.affine.backends import hip
from aimet_amd.quantization.affine.backends.utils import set_backend, get_backend, add_backend

__all__ = ["quantize", "quantize_dequantize", "dequantize", "set_backend", "get_backend", "add_backend"]


def _derive_qmin_qmax(*, bitwidth: int = None, num_steps: int = None, signed: bool):
    if bitwidth is not None:
        num_steps = 2 ** bitwidth - 1
    if signed:
        return -math.ceil(num_steps / 2), math.floor(num_steps / 2)
    return 0, num_steps


def _parse_args(args, kwargs) -> Tuple[int, int, Optional[Tuple[int, ...]], float]:
    """Sort out the three overloads (backends/__init__.py:408-431)."""
    pos = tuple(args) + (None,) * (4 - len(args))
    first = kwargs.get("qmin", kwargs.get("bitwidth", pos[0]))
    second = kwargs.get("qmax", kwargs.get("signed", pos[1]))
    block_size = kwargs.get("block_size", None) or pos[2]
    zero_point_shift = pos[3] or kwargs.get("zero_point_shift", 0.0)

    if first is None:
        qmin, qmax = _derive_qmin_qmax(num_steps=kwargs["num_steps"], signed=kwargs["signed"])
    elif second is None or isinstance(second, bool):
        qmin, qmax = _derive_qmin_qmax(bitwidth=first, signed=bool(second))
    else:
        qmin, qmax = first, second
    assert qmin is not None and qmax is not None
    return qmin, qmax, block_size, zero_point_shift


def quantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, *args, **kwargs):
    r"""out = clamp(round(tensor / scale) - offset, qmin, qmax)"""
    qmin, qmax, block_size, zero_point_shift = _parse_args(args, kwargs)
    if zero_point_shift != 0.0:
        raise RuntimeError("Nonzero zero_point_shift not supported for quantize()")
    return get_backend().quantize(tensor, scale, offset, qmin, qmax, block_size)


def quantize_dequantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, *args, **kwargs):
    r"""out = (clamp(round(tensor / scale) - offset, qmin, qmax) + offset) * scale"""
    qmin, qmax, block_size, zero_point_shift = _parse_args(args, kwargs)
    return get_backend().quantize_dequantize(tensor, scale, offset, qmin, qmax, block_size, zero_point_shift)


def dequantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor,
               block_size: Optional[Tuple[int, ...]] = None):
    r"""out = (tensor + offset) * scale"""
    return get_backend().dequantize(tensor, scale, offset, block_size)
