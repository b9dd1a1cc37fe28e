"""Encoding base class (counterpart of aimet_torch/quantization/base/encoding.py)."""

from __future__ import annotations

import abc

import torch


class EncodingBase(abc.ABC):
    """Describes how a tensor was (or is to be) quantized."""

    @property
    @abc.abstractmethod
    def granularity(self) -> str: ...

    @abc.abstractmethod
    def quantize(self, input: torch.Tensor) -> torch.Tensor: ...  # pylint: disable=redefined-builtin

    @abc.abstractmethod
    def dequantize(self, input: torch.Tensor) -> torch.Tensor: ...  # pylint: disable=redefined-builtin

    @abc.abstractmethod
    def to(self, *args, **kwargs) -> "EncodingBase": ...
