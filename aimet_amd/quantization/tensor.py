"""Tensor subclasses that carry the encoding they were produced with.

Only what the quantizers' outputs need (aimet_torch/quantization/tensor.py:570-690 holds the reference classes):
``QuantizedTensor`` stores integer codes in a floating-point tensor, ``DequantizedTensor`` stores fake-quantized
values; both expose ``.encoding``, ``quantize()`` / ``dequantize()`` and ``quantized_repr()``.
"""

from __future__ import annotations

import torch

__all__ = ["QuantizedTensorBase", "QuantizedTensor", "DequantizedTensor"]


class QuantizedTensorBase(torch.Tensor):
    encoding = None

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        # results of arbitrary torch operations are plain tensors: an encoding only describes the tensor it was made for
        ret = super().__torch_function__(func, types, args, kwargs or {})
        if func in (torch.Tensor.clone, torch.Tensor.detach, torch.Tensor.to, torch.Tensor.as_subclass):
            src = args[0]
            if isinstance(ret, QuantizedTensorBase) and isinstance(src, QuantizedTensorBase):
                ret.encoding = src.encoding
            return ret
        if isinstance(ret, QuantizedTensorBase) and func not in (torch.Tensor.requires_grad_,):
            return ret.as_subclass(torch.Tensor)
        return ret


class QuantizedTensor(QuantizedTensorBase):
    """Integer codes on the encoding's grid."""

    def quantize(self) -> "QuantizedTensor":
        return self

    def dequantize(self) -> "DequantizedTensor":
        out = self.encoding.dequantize(self.as_subclass(torch.Tensor)).as_subclass(DequantizedTensor)
        out.encoding = self.encoding
        return out

    def quantized_repr(self) -> torch.Tensor:
        enc = self.encoding
        if enc.qmin >= 0:
            dtype = torch.uint8 if enc.qmax < 2 ** 8 else torch.int32
        elif enc.qmin >= -(2 ** 7) and enc.qmax < 2 ** 7:
            dtype = torch.int8
        elif enc.qmin >= -(2 ** 15) and enc.qmax < 2 ** 15:
            dtype = torch.int16
        else:
            dtype = torch.int32
        return self.as_subclass(torch.Tensor).to(dtype)


class DequantizedTensor(QuantizedTensorBase):
    """Values that lie on the encoding's grid in floating point."""

    def dequantize(self) -> "DequantizedTensor":
        return self

    def quantize(self) -> QuantizedTensor:
        out = self.encoding.quantize(self.as_subclass(torch.Tensor)).as_subclass(QuantizedTensor)
        out.encoding = self.encoding
        return out

    def quantized_repr(self) -> torch.Tensor:
        return self.quantize().quantized_repr()
