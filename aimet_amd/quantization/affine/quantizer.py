"""Affine quantizer modules: ``Quantize``, ``QuantizeDequantize``, ``Dequantize``, ``GroupedBlockQuantizeDequantize``.

API-compatible counterparts of aimet_torch/quantization/affine/quantizer.py (constructor overloads, learnable
``min`` / ``max`` parameters, ``get_scale`` / ``get_offset`` / ``get_min`` / ``get_max`` / ``set_range`` /
``get_encodings``, the ``compute_encodings()`` context manager, ``allow_overwrite``, extra state for checkpoints).
Tensor work is done by the HIP backend and the HIP encoding analyzers.  Quantizers here are parametrised by min/max;
the reference's alternative scale/offset parametrisation is not part of this package.
"""

# pylint: disable=redefined-builtin

from __future__ import annotations

import functools
import math
from contextlib import contextmanager, nullcontext
from typing import Any, NamedTuple, Optional, Protocol, Tuple, runtime_checkable

import torch
from torch import nn

from aimet_amd import _lib
from aimet_amd.quantization._utils import (
    StatisticsNotFoundError,
    _get_minimum_scale,
    _is_expandable,
    concretize_block_size,
    interleave,
    patch_attr,
    ste_round,
    true_divide,
)
from aimet_amd.quantization.affine._utils import _GridMixin
from aimet_amd.quantization.affine.backends import quantize, quantize_dequantize, dequantize, _derive_qmin_qmax, get_backend
from aimet_amd.quantization.affine.backends import hip as _hip_backend
from aimet_amd.quantization.affine.backends.hip import _build_layout
from aimet_amd.quantization.affine.encoding import AffineEncoding, GroupedBlockEncoding
from aimet_amd.quantization.base.quantizer import QuantizerBase
from aimet_amd.quantization.encoding_analyzer import EncodingAnalyzer, MinMaxEncodingAnalyzer, _flag_extreme_min_max
from aimet_amd.quantization.tensor import QuantizedTensor, DequantizedTensor

__all__ = ["AffineQuantizerBase", "MinMaxQuantizer", "ScaleOffsetQuantizer", "Quantize", "QuantizeDequantize",
           "Dequantize", "GroupedBlockQuantizeDequantize"]


def _symmetric_offset(qmin: int, qmax: int, shape, dtype, device) -> torch.Tensor:
    """Constant offset of a symmetric grid (quantizer.py:843-850).  The value is also attached as a Python attribute
    so that the backend can reason about it without reading device memory."""
    value = -round((qmin + qmax) / 2)
    off = torch.full(tuple(shape), fill_value=value, requires_grad=False, dtype=dtype, device=device)
    off._ahq_constant = value  # pylint: disable=protected-access
    return off


class _RangeToScaleOffset(torch.autograd.Function):
    """(min, max) -> (scale, offset) in float32 with one launch each way (ahq_range_to_scale_offset /
    ahq_range_backward) instead of the dozen elementwise operations of get_scale / _get_offset and the dozen autograd
    nodes behind them (quantizer.py:319-376); the same float32 operations, so the same bits."""

    @staticmethod
    def forward(ctx, mn, mx, qmin, qmax, symmetric, constant_offset):  # pylint: disable=arguments-differ
        lib = _lib.load()
        scale = torch.empty(mn.shape, dtype=torch.float32, device=mn.device)
        offset = constant_offset if symmetric else torch.empty(mn.shape, dtype=torch.float32, device=mn.device)
        _lib.check(
            lib.ahq_range_to_scale_offset(_lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(), mn.numel(), qmin, qmax,
                                          _get_minimum_scale(qmax - qmin), scale.data_ptr(),
                                          None if symmetric else offset.data_ptr(), _lib.current_stream(mn.device)),
            "ahq_range_to_scale_offset")
        ctx.save_for_backward(mn, mx)
        ctx.grid = (qmin, qmax, symmetric)
        ctx.set_materialize_grads(False)  # an output nobody used arrives as None, not as zeros
        if symmetric:
            ctx.mark_non_differentiable(offset)
        return scale, offset

    @staticmethod
    def backward(ctx, gscale, goffset):  # pylint: disable=arguments-differ
        mn, mx = ctx.saved_tensors
        qmin, qmax, symmetric = ctx.grid
        if gscale is None and (symmetric or goffset is None):
            return None, None, None, None, None, None
        shape, device = mn.shape, mn.device
        if gscale is None:
            gscale = torch.zeros(shape, dtype=torch.float32, device=device)
        # an offset that nothing downstream used has no gradient path at all (a zero gradient would still meet
        # infinite factors on its way)
        symmetric = symmetric or goffset is None
        gscale = gscale.to(torch.float32).contiguous()
        if not symmetric:
            goffset = goffset.to(torch.float32).contiguous()
        gmin, gmax = torch.empty((2,) + tuple(mn.shape), dtype=mn.dtype, device=mn.device).unbind(0)
        _lib.check(
            _lib.load().ahq_range_backward(_lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(), mn.numel(), qmin, qmax,
                                           _get_minimum_scale(qmax - qmin), gscale.data_ptr(),
                                           None if symmetric else goffset.data_ptr(), gmin.data_ptr(), gmax.data_ptr(),
                                           _lib.current_stream(device)),
            "ahq_range_backward")
        return gmin, gmax, None, None, None, None


class _QdqFromRange(torch.autograd.Function):
    """QuantizeDequantize.forward with learned min / max as one autograd node: (x, min, max) -> (y, scale, offset).
    Forward: ahq_range_to_scale_offset, then ahq_qdq_forward; backward: ahq_qdq_backward (input, scale and offset
    gradients in one launch), then ahq_range_backward.  The same four launches as _RangeToScaleOffset followed by the
    backend's quantize_dequantize, so the same bits; one node, one apply() and one encoding object less per step of a
    host-bound training loop.  scale and offset are outputs too, for whoever differentiates through the encoding the
    output tensor carries; offset is None on a symmetric grid (the caller holds the constant)."""

    @staticmethod
    def forward(ctx, x, mn, mx, qmin, qmax, symmetric, constant_offset, block_size, zps, compute_dtype):  # pylint: disable=arguments-differ
        from aimet_amd.quantization.affine.backends import hip as _hip

        if symmetric:
            scale, offset = torch.empty(mn.shape, dtype=torch.float32, device=mn.device), constant_offset
        else:
            scale, offset = torch.empty((2,) + tuple(mn.shape), dtype=torch.float32, device=mn.device).unbind(0)
        _lib.check(
            _lib.load().ahq_range_to_scale_offset(_lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(), mn.numel(),
                                                  qmin, qmax, _get_minimum_scale(qmax - qmin), scale.data_ptr(),
                                                  None if symmetric else offset.data_ptr(),
                                                  _lib.current_stream(mn.device)),
            "ahq_range_to_scale_offset")
        y, xd, s, o, grid, layout = _hip._launch_forward(  # pylint: disable=protected-access
            x, scale, offset, _lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QDQ, compute_dtype, qmin, qmax, block_size, zps)
        ctx.save_for_backward(xd, s, o, mn, mx)
        ctx.grid, ctx.layout, ctx.range_grid = grid, layout, (qmin, qmax, symmetric)
        ctx.set_materialize_grads(False)  # an output nobody used arrives as None, not as zeros
        return y, scale, (None if symmetric else offset)

    @staticmethod
    def backward(ctx, gy, gscale, goffset):  # pylint: disable=arguments-differ
        from aimet_amd.quantization.affine.backends import hip as _hip

        xd, s, o, mn, mx = ctx.saved_tensors
        qmin, qmax, symmetric = ctx.range_grid
        need_x, need_mn, need_mx = ctx.needs_input_grad[:3]
        none7 = (None,) * 7
        want_pg = need_mn or need_mx
        gx = gs = go = None
        if gy is not None and (need_x or want_pg):
            gx, gs, go = _hip._launch_backward(ctx.grid, ctx.layout, xd, s, o, gy, need_x, want_pg)  # pylint: disable=protected-access
        if not want_pg:
            return (gx, None, None) + none7
        # gradients that reached scale / offset through the encoding object add to the kernel's
        if gscale is not None:
            gscale = gscale.to(torch.float32).reshape(s.shape)
            gs = gscale if gs is None else gs + gscale
        if goffset is not None and not symmetric:
            goffset = goffset.to(torch.float32).reshape(s.shape)
            go = goffset if go is None else go + goffset
        if gs is None and (symmetric or go is None):
            return (gx, None, None) + none7
        if gs is None:
            gs = torch.zeros(s.shape, dtype=torch.float32, device=s.device)
        # an offset that nothing downstream used has no gradient path at all (a zero gradient would still meet
        # infinite factors on its way)
        symmetric = symmetric or go is None
        gmin, gmax = torch.empty((2,) + tuple(mn.shape), dtype=mn.dtype, device=mn.device).unbind(0)
        _lib.check(
            _lib.load().ahq_range_backward(_lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(), mn.numel(), qmin, qmax,
                                           _get_minimum_scale(qmax - qmin), gs.contiguous().data_ptr(),
                                           None if symmetric else go.contiguous().data_ptr(), gmin.data_ptr(),
                                           gmax.data_ptr(), _lib.current_stream(mn.device)),
            "ahq_range_backward")
        return (gx, gmin if need_mn else None, gmax if need_mx else None) + none7


def _lpbq_forward_launch(x, mn, mx, qmin, qmax, block_size, group, group_shape, multipliers, offset):
    """ahq_lpbq_qdq_forward on a plain tensor: (status, y, x dense in memory, scale, per-channel scale, grid, layout).
    ``offset``: the quantizer's constant float32 offset (not passed to the kernel when it is zero)."""
    from aimet_amd.quantization.affine.backends import hip as _hip

    x, layout = _hip._prepare(x.detach(), tuple(mn.shape), block_size)  # pylint: disable=protected-access
    grid = _hip._grid(_lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QDQ, x.dtype, x.dtype, qmin, qmax, 0.0)  # pylint: disable=protected-access
    y = torch.empty_like(x)
    scale = torch.empty(mn.shape, dtype=torch.float32, device=x.device)
    per_channel = torch.empty(group_shape, dtype=torch.float32, device=x.device)
    offset_ptr = None if getattr(offset, "_ahq_constant", None) == 0 else offset.data_ptr()
    status = _lib.load().ahq_lpbq_qdq_forward(
        grid, layout, x.data_ptr(), y.data_ptr(), None, _lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(), group,
        _get_minimum_scale(qmax - qmin), multipliers, offset_ptr, scale.data_ptr(), per_channel.data_ptr(),
        _lib.current_stream(x.device))
    return status, y, x, scale, per_channel, grid, layout


class _LpbqQdqFromRange(torch.autograd.Function):
    """GroupedBlockQuantizeDequantize.forward with gradients as one autograd node: (x, min, max) -> (y, block scales,
    per-channel scales) with ahq_lpbq_qdq_forward; backward: ahq_qdq_backward (input and scale gradients in one
    launch), then ahq_lpbq_scale_backward down to min / max.  The launches compute what _LpbqScale followed by the
    backend's quantize_dequantize computes, bit for bit."""

    @staticmethod
    def forward(ctx, x, mn, mx, qmin, qmax, block_size, group, group_shape, multipliers, offset, group_layout):  # pylint: disable=arguments-differ
        status, y, xd, scale, per_channel, grid, layout = _lpbq_forward_launch(
            x, mn, mx, qmin, qmax, block_size, group, group_shape, multipliers, offset)
        _lib.check(status, "ahq_lpbq_qdq_forward")
        ctx.save_for_backward(xd, scale, mn, mx)
        ctx.grid, ctx.layout, ctx.offset = grid, layout, offset
        ctx.args = (qmin, qmax, multipliers, group_layout)
        ctx.set_materialize_grads(False)
        return y, scale, per_channel

    @staticmethod
    def backward(ctx, gy, gscale, gper_channel):  # pylint: disable=arguments-differ
        from aimet_amd.quantization.affine.backends import hip as _hip

        xd, s, mn, mx = ctx.saved_tensors
        qmin, qmax, multipliers, group_layout = ctx.args
        need_x, need_mn, need_mx = ctx.needs_input_grad[:3]
        none8 = (None,) * 8
        want_pg = need_mn or need_mx
        gx = gs = None
        if gy is not None and (need_x or want_pg):
            gx, gs, _ = _hip._launch_backward(ctx.grid, ctx.layout, xd, s.detach(), ctx.offset, gy, need_x, want_pg)  # pylint: disable=protected-access
        if not want_pg:
            return (gx, None, None) + none8
        if gscale is not None:
            gscale = gscale.to(torch.float32).reshape(s.shape)
            gs = gscale if gs is None else gs + gscale
        if gs is None and gper_channel is None:
            return (gx, None, None) + none8
        if gs is None:
            gs = torch.zeros(s.shape, dtype=torch.float32, device=s.device)
        if gper_channel is not None:
            gper_channel = gper_channel.to(torch.float32).contiguous()
        gmin, gmax = torch.empty((2,) + tuple(mn.shape), dtype=mn.dtype, device=mn.device).unbind(0)
        _lib.check(
            _lib.load().ahq_lpbq_scale_backward(_lib.DTYPE_CODE[mn.dtype], group_layout, mn.data_ptr(), mx.data_ptr(),
                                                qmin, qmax, _get_minimum_scale(qmax - qmin), multipliers,
                                                gs.contiguous().data_ptr(), _lib.ptr(gper_channel), gmin.data_ptr(),
                                                gmax.data_ptr(), _lib.current_stream(mn.device)),
            "ahq_lpbq_scale_backward")
        return (gx, gmin if need_mn else None, gmax if need_mx else None) + none8


class _LpbqScale(torch.autograd.Function):
    """(min, max) -> (LPBQ block scales, per-group scales) in float32 with one launch each way (ahq_lpbq_scale /
    ahq_lpbq_scale_backward) instead of the reference's sequence -- get_scale, group maximum, division,
    quantize-dequantize of the block scales (quantizer.py:1363-1399) -- and the autograd nodes behind it."""

    @staticmethod
    def forward(ctx, mn, mx, qmin, qmax, multipliers, layout, group_shape):  # pylint: disable=arguments-differ
        scale = torch.empty(mn.shape, dtype=torch.float32, device=mn.device)
        per_channel = torch.empty(group_shape, dtype=torch.float32, device=mn.device)
        _lib.check(
            _lib.load().ahq_lpbq_scale(_lib.DTYPE_CODE[mn.dtype], layout, mn.data_ptr(), mx.data_ptr(), qmin, qmax,
                                       _get_minimum_scale(qmax - qmin), multipliers, scale.data_ptr(),
                                       per_channel.data_ptr(), _lib.current_stream(mn.device)),
            "ahq_lpbq_scale")
        ctx.save_for_backward(mn, mx)
        ctx.args = (qmin, qmax, multipliers, layout)
        ctx.set_materialize_grads(False)
        return scale, per_channel

    @staticmethod
    def backward(ctx, gscale, gper_channel):  # pylint: disable=arguments-differ
        mn, mx = ctx.saved_tensors
        qmin, qmax, multipliers, layout = ctx.args
        if gscale is None and gper_channel is None:
            return (None,) * 7
        if gscale is None:
            gscale = torch.zeros(mn.shape, dtype=torch.float32, device=mn.device)
        gscale = gscale.to(torch.float32).contiguous()
        if gper_channel is not None:
            gper_channel = gper_channel.to(torch.float32).contiguous()
        gmin, gmax = torch.empty((2,) + tuple(mn.shape), dtype=mn.dtype, device=mn.device).unbind(0)
        _lib.check(
            _lib.load().ahq_lpbq_scale_backward(_lib.DTYPE_CODE[mn.dtype], layout, mn.data_ptr(), mx.data_ptr(), qmin,
                                                qmax, _get_minimum_scale(qmax - qmin), multipliers, gscale.data_ptr(),
                                                _lib.ptr(gper_channel), gmin.data_ptr(), gmax.data_ptr(),
                                                _lib.current_stream(mn.device)),
            "ahq_lpbq_scale_backward")
        return gmin, gmax, None, None, None, None, None


def _get_scale_offset(min: torch.Tensor, max: torch.Tensor, qmin: int, qmax: int, symmetric: bool):
    """scale = (max - min) / (qmax - qmin); offset = round(min / scale) - qmin, or the symmetric constant
    (quantizer.py:876-900)."""
    num_steps = qmax - qmin
    if not isinstance(min, torch.Tensor):
        min = torch.tensor(min, dtype=torch.float32)
    if not isinstance(max, torch.Tensor):
        max = torch.tensor(max, dtype=torch.float32)
    out_dtype = min.dtype
    min = min.to(torch.float32)
    max = max.to(torch.float32)
    scale = true_divide(max - min, num_steps)
    if symmetric:
        offset = _symmetric_offset(qmin, qmax, min.shape, min.dtype, min.device)
    else:
        offset = ste_round(min / scale) - qmin
    return scale.to(out_dtype), offset.to(out_dtype)


def _get_min_max(scale, offset, qmin: int, qmax: int):
    """min = scale * (offset + qmin), max = scale * (offset + qmax) in float32, offsets as int32
    (quantizer.py:853-873); offset None: the symmetric constant."""
    if not isinstance(scale, torch.Tensor):
        scale = torch.tensor(scale, dtype=torch.float32)
    if offset is None:
        offset = _symmetric_offset(qmin, qmax, scale.shape, torch.int32, scale.device)
    if not isinstance(offset, torch.Tensor):
        offset = torch.tensor(offset, dtype=torch.int32)
    out_dtype = scale.dtype
    scale = scale.to(torch.float32)
    offset = offset.to(torch.int32)
    return (scale * (offset + qmin)).to(out_dtype), (scale * (offset + qmax)).to(out_dtype)


class AffineQuantizerBase(QuantizerBase, _GridMixin):
    """Base class of the affine quantizers.

    ``(shape, bitwidth, symmetric, encoding_analyzer=None, block_size=None, zero_point_shift=None)`` or
    ``(shape, qmin, qmax, symmetric, encoding_analyzer=None, block_size=None, zero_point_shift=None)``.
    """

    def __init__(self, shape, *args, **kwargs):
        super().__init__()
        if isinstance(shape, int):
            shape = (shape,)
        self.shape = tuple(shape)
        pos = tuple(args) + (None,) * (6 - len(args))
        first = kwargs.pop("qmin", kwargs.pop("bitwidth", pos[0]))
        second = kwargs.pop("qmax", pos[1])
        if second is not None and not isinstance(second, bool):
            qmin, qmax = first, second
            symmetric = kwargs.pop("symmetric", pos[2])
            rest = pos[3:6]
        else:
            symmetric = kwargs.pop("symmetric", pos[1])
            if first is None or symmetric is None:
                raise TypeError("expected (shape, bitwidth, symmetric, ...) or (shape, qmin, qmax, symmetric, ...)")
            qmin, qmax = _derive_qmin_qmax(bitwidth=first, signed=symmetric)
            rest = pos[2:5]
        if qmin is None or qmax is None or symmetric is None:
            raise TypeError("expected (shape, bitwidth, symmetric, ...) or (shape, qmin, qmax, symmetric, ...)")
        encoding_analyzer = kwargs.pop("encoding_analyzer", rest[0])
        block_size = kwargs.pop("block_size", rest[1])
        zero_point_shift = kwargs.pop("zero_point_shift", rest[2])
        if kwargs:
            raise TypeError(f"{type(self).__qualname__}.__init__ got unexpected keyword argument: {', '.join(kwargs)}")
        if qmin >= qmax:
            raise ValueError(f"qmax should be strictly larger than qmin. Got qmax={qmax}, qmin={qmin}")

        self.qmin = qmin
        self.qmax = qmax
        self._symmetric = symmetric
        self.block_size = block_size
        self.zero_point_shift = zero_point_shift or 0.0
        if self.zero_point_shift not in (0.0, 0.5):
            raise ValueError(f"zero_point_shift should be 0.0 or 0.5. Got {self.zero_point_shift}")

        self.encoding_analyzer: EncodingAnalyzer = encoding_analyzer or MinMaxEncodingAnalyzer(
            shape=self.shape, block_size=self.block_size
        )
        if not _is_expandable(self.encoding_analyzer.observer.shape, self.shape):
            raise RuntimeError(
                f"Encoding analyzer of shape {self.encoding_analyzer.observer.shape} "
                f"is incompatible with quantizer of shape {self.shape}."
            )

        self._reparametrize_to_min_max()
        self._is_overwrite_allowed.update({"min": True, "max": True})

    # ------------------------------------------------------------------- which parameters hold the encoding --
    def _is_scale_offset_quantizer(self) -> bool:
        return "scale" in self._parameters and "offset" in self._parameters

    def _is_min_max_quantizer(self) -> bool:
        return "min" in self._parameters and "max" in self._parameters

    def __getattr__(self, name: str):
        try:
            return super().__getattr__(name)
        except AttributeError as e:
            if ((name in ("min", "max") and self._is_scale_offset_quantizer())
                    or (name in ("scale", "offset") and self._is_min_max_quantizer())):
                param_names = "/".join(self._parameters.keys())
                raise AttributeError(
                    f"'{type(self).__qualname__}' object has no attribute '{name}' "
                    f"because it's parametrized with {param_names}. "
                    f"To get '{name}' of this quantizer, use qtzr.get_{name}() instead. "
                    "To assign a new input range to this quantizer, use qtzr.set_range() instead") from e
            raise e

    def _forget_derived_encodings(self) -> None:
        """Everything kept from earlier calls that was derived from the parameters being replaced."""
        for key in ("_encoding_cache", "_forward_plan", "_forward_seen", "_calibrate_qdq_plan"):
            self.__dict__.pop(key, None)

    def _reparametrize_to_scale_offset(self):
        """The encoding held as (scale, offset) instead of (min, max) (quantizer.py:225-261): scale and offset are
        float32 on the device of min / max, learnable if min or max was, and -- if the quantizer was initialised --
        hold the values get_scale() / get_offset() gave.  A symmetric quantizer holds no offset (None)."""
        if self._is_scale_offset_quantizer():
            return
        was_initialized = self.is_initialized()
        self._forget_derived_encodings()
        self.register_quantization_parameter("scale", nn.Parameter(torch.ones(self.shape)))
        self.register_quantization_parameter(
            "offset",
            None if self.symmetric
            else nn.Parameter(_symmetric_offset(self.qmin, self.qmax, self.shape, torch.float32, "cpu")))
        if self._is_min_max_quantizer():
            mn = self._parameters.pop("min")
            mx = self._parameters.pop("max")
            self._initial_parameters.pop("min", None)
            self._initial_parameters.pop("max", None)
            self.requires_grad_(mn.requires_grad or mx.requires_grad)
            # the device of min / max is followed, their dtype is not: scale and offset stay float32
            self.to(device=mn.device, dtype=torch.float32)
            if was_initialized:
                self.set_range(mn, mx)
        # the marker the runtime-checkable protocols below look for (quantizer.py:252-254)
        self.__dict__.pop("_is_min_max", None)
        self.__dict__["_is_scale_offset"] = True

    def _reparametrize_to_min_max(self):
        """The encoding held as (min, max) (quantizer.py:263-285), the form every quantizer starts in."""
        if self._is_min_max_quantizer():
            return
        was_initialized = self.is_initialized()
        self._forget_derived_encodings()
        self.register_quantization_parameter("min", nn.Parameter(-torch.ones(self.shape)))
        self.register_quantization_parameter("max", nn.Parameter(torch.ones(self.shape)))
        if self._is_scale_offset_quantizer():
            self._symmetric = self._parameters["offset"] is None
            scale = self._parameters.pop("scale")
            offset = self._parameters.pop("offset")
            self._initial_parameters.pop("scale", None)
            self._initial_parameters.pop("offset", None)
            self.requires_grad_(scale.requires_grad or getattr(offset, "requires_grad", False))
            self.to(device=scale.device, dtype=scale.dtype)
            if was_initialized:
                mn, mx = _get_min_max(scale.detach(), None if offset is None else offset.detach(), self.qmin, self.qmax)
                self.set_range(mn, mx)
        self.__dict__.pop("_is_scale_offset", None)
        self.__dict__["_is_min_max"] = True

    # ------------------------------------------------------------------------------------- derived quantities --
    def get_scale(self, dtype=None) -> Optional[torch.Tensor]:
        """|max - min| / (qmax - qmin), or the scale parameter, floored at the minimum scale; None before
        initialisation (quantizer.py:319-342)."""
        if not self.is_initialized():
            return None
        dtype = dtype or torch.float32
        num_steps = self.qmax - self.qmin
        if self._is_scale_offset_quantizer():
            # (abs() makes a new tensor, so that the in-place clamp below never touches the parameter)
            return self.scale.abs().clamp_min_(_get_minimum_scale(num_steps)).to(dtype)
        scale = true_divide(self.max.to(dtype) - self.min.to(dtype), num_steps)
        return scale.abs().clamp_min_(_get_minimum_scale(num_steps)).to(dtype)

    def get_offset(self, dtype=None) -> Optional[torch.Tensor]:
        return self._get_offset(dtype=dtype)

    def _get_offset(self, scale=None, dtype=None) -> Optional[torch.Tensor]:
        """clamp(round(min / scale) - qmin, -qmax, -qmin), or the symmetric constant (quantizer.py:357-376)."""
        if not self.is_initialized():
            return None
        dtype = dtype or torch.float32
        if self.symmetric:
            device = next(p.device for p in self._parameters.values() if p is not None)
            return _symmetric_offset(self.qmin, self.qmax, self.shape, dtype, device)
        if self._is_scale_offset_quantizer():
            return ste_round(self.offset).to(dtype)
        scale = scale if scale is not None else self.get_scale(dtype)
        offset = torch.clamp(ste_round(self.min / scale) - self.qmin, -self.qmax, -self.qmin)
        return offset.to(dtype)

    def get_min(self, dtype=None) -> Optional[torch.Tensor]:
        if not self.is_initialized():
            return None
        return self.get_scale(dtype) * (self.get_offset(dtype) + self.qmin + self.zero_point_shift)

    def get_max(self, dtype=None) -> Optional[torch.Tensor]:
        if not self.is_initialized():
            return None
        return self.get_scale(dtype) * (self.get_offset(dtype) + self.qmax + self.zero_point_shift)

    @torch.no_grad()
    def set_range(self, min, max):
        """Assign the encoding range; ``None`` leaves that end untouched (quantizer.py:378-438)."""
        if min is None and max is None:
            return
        if min is not None and not isinstance(min, torch.Tensor):
            min = torch.tensor(min)
        if max is not None and not isinstance(max, torch.Tensor):
            max = torch.tensor(max)
        if self._is_min_max_quantizer():
            if min is not None:
                self.min.copy_(min)
            if max is not None:
                self.max.copy_(max)
            return
        if min is None:
            min = self.get_min()
        if max is None:
            max = self.get_max()
        if min is None or max is None:
            raise ValueError(
                f"{type(self).__name__}.set_range(...) with partial input, "
                "such as `set_range(min=0.0, max=None)` or `set_range(min=None, max=1.0), "
                "cannot be supported for quantizers parametrized with scale & offset.")
        # scale / offset are derived in float32
        scale, offset = _get_scale_offset(min.to(torch.float32), max.to(torch.float32), qmin=self.qmin, qmax=self.qmax,
                                          symmetric=self.symmetric)
        self.scale.copy_(scale)
        if not self.symmetric:
            self.offset.copy_(offset)

    def get_encodings(self) -> Optional[AffineEncoding]:
        # When no gradient can flow into min/max, scale and offset are constants of the current parameter values:
        # they are derived once and reused until min or max is written again (their version counters change) or
        # moved.  A whole-model forward calls this once per quantizer, and the half-dozen tiny kernels behind
        # get_scale()/get_offset() would otherwise cost more than the quantize-dequantize kernel itself.
        # Deviation from the reference, which recomputes scale and offset on every call: a write through `.data`
        # (`q.min.data.copy_(...)`, `q.min.data.fill_(...)`) changes neither the version counter nor the address and
        # is not seen here; such callers follow the write with invalidate_encoding_cache().  set_range(), copy_(),
        # load_state_dict() and optimizer steps all bump the version counter and need nothing.
        if not self._is_min_max_quantizer():
            return self._derive_encodings()  # held as scale / offset: nothing to derive but a clamp and a rounding
        if torch.is_grad_enabled() and (self.min.requires_grad or self.max.requires_grad):
            return self._derive_encodings()
        key = self._encoding_cache_key()
        cached = self.__dict__.get("_encoding_cache")
        if cached is not None and cached[0] == key:
            return cached[1]
        with torch.no_grad():
            enc = self._derive_encodings()
        if enc is not None:
            self.__dict__["_encoding_cache"] = (key, enc)
        return enc

    def invalidate_encoding_cache(self) -> None:
        """Forget the scale / offset derived from min / max.  Needed only after a write that bypasses torch's version
        counter (through ``.data``); every tracked in-place write invalidates the cache by itself."""
        self.__dict__.pop("_encoding_cache", None)

    def _fused_scale_offset(self):
        """get_scale(float32) and _get_offset(float32) of a quantizer that holds min / max on a GPU in one launch
        (ahq_range_to_scale_offset; as an autograd node with a one-launch backward when min / max are learned); None
        when that does not apply (a subclass with its own scale, parameters that are not on a GPU or not contiguous)
        and the step-by-step form has to run."""
        cls = type(self)
        if (cls.get_scale is not AffineQuantizerBase.get_scale or cls._get_offset is not AffineQuantizerBase._get_offset
                or not self._is_min_max_quantizer()):
            return None
        mn, mx = self.min, self.max
        if not (mn.is_cuda and mx.device == mn.device and mn.dtype == mx.dtype and mn.dtype in _lib.DTYPE_CODE
                and mn.shape == mx.shape and mn.is_contiguous() and mx.is_contiguous()):
            return None
        if torch.is_grad_enabled() and (mn.requires_grad or mx.requires_grad):
            # learned ranges: the same kernel as one autograd node, with a one-launch backward
            return _RangeToScaleOffset.apply(mn, mx, self.qmin, self.qmax, bool(self.symmetric),
                                             self._constant_offset(mn.device) if self.symmetric else None)
        lib = _lib.load()
        scale = torch.empty(mn.shape, dtype=torch.float32, device=mn.device)
        if self.symmetric:
            offset = self._constant_offset(mn.device)
        else:
            offset = torch.empty(mn.shape, dtype=torch.float32, device=mn.device)
        _lib.check(
            lib.ahq_range_to_scale_offset(_lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(), mn.numel(), self.qmin,
                                          self.qmax, _get_minimum_scale(self.qmax - self.qmin), scale.data_ptr(),
                                          None if self.symmetric else offset.data_ptr(), _lib.current_stream(mn.device)),
            "ahq_range_to_scale_offset",
        )
        return scale, offset

    def _constant_offset(self, device) -> torch.Tensor:
        """The float32 offset of a symmetric grid, made once per (grid, shape, device)."""
        key = (self.qmin, self.qmax, tuple(self.shape), device)
        held = self.__dict__.get("_sym_offset")
        if held is None or held[0] != key:
            held = (key, _symmetric_offset(self.qmin, self.qmax, self.shape, torch.float32, device))
            self.__dict__["_sym_offset"] = held
        return held[1]

    def _encoding_cache_key(self):
        mn, mx = self.min, self.max
        return (id(mn), mn._version, mn.data_ptr(), id(mx), mx._version, mx.data_ptr(),  # pylint: disable=protected-access
                self.qmin, self.qmax, self._symmetric, self.block_size, self.zero_point_shift)

    def _finalize_from_minmax(self) -> bool:
        """The end of a min/max calibration -- statistics to range, range into min / max, scale and offset for the
        next forward -- in one launch (ahq_minmax_finalize) instead of the analyzer's kernel, two copies and, on the
        next forward, the scale / offset kernel.  False when that does not apply and the step-by-step form has to
        run: another analyzer, a subclass with its own scale, an end that may not be overwritten, statistics or
        parameters that are not contiguous 16/32-bit floats on one GPU."""
        an = self.encoding_analyzer
        cls = type(self)
        if (type(an) is not MinMaxEncodingAnalyzer  # pylint: disable=unidiomatic-typecheck
                or cls.get_scale is not AffineQuantizerBase.get_scale
                or cls._get_offset is not AffineQuantizerBase._get_offset
                or cls.set_range is not AffineQuantizerBase.set_range
                or not self._is_min_max_quantizer()
                or not all(self._is_overwrite_allowed.values())):
            return False
        mn, mx = self.min, self.max
        num_steps = self._num_steps_for_calibration()
        if (not mn.is_cuda or mx.device != mn.device or mn.dtype not in _lib.DTYPE_CODE or mx.dtype != mn.dtype
                or mn.shape != mx.shape or not (mn.is_contiguous() and mx.is_contiguous())
                or num_steps <= 0 or num_steps > (1 << 24)):
            return False
        # a single encoding observed through observe_and_clone(): the running extrema still lie in the observer's
        # slots, and the launch folds them itself (the observer is left as it is and folds them if anybody asks)
        slots = an.observer.live_slots()
        if slots is not None and (slots[1] != mn.device or mn.numel() != 1):
            slots = None
        if slots is None:
            stats = an.observer.get_stats()
            smin, smax = stats.min, stats.max
            if (smin is None or smax is None or smin.dtype not in _lib.DTYPE_CODE or smax.dtype != smin.dtype
                    or smin.device != mn.device or smax.device != mn.device or smin.shape != smax.shape
                    or mn.numel() != smin.numel() or not (smin.is_contiguous() and smax.is_contiguous())):
                return False
            stat_dtype = smin.dtype
        else:
            stat_dtype = slots[0]
        from aimet_amd.quantization.encoding_analyzer import _scalar_constants, _range_flags_buffer, _report_range_flags

        device = mn.device
        consts = _scalar_constants(stat_dtype, _get_minimum_scale(num_steps))
        scale = torch.empty(mn.shape, dtype=torch.float32, device=device)
        offset = self._constant_offset(device) if self.symmetric else torch.empty(mn.shape, dtype=torch.float32,
                                                                                  device=device)
        flags, own = _range_flags_buffer(device)
        if slots is not None:
            _lib.check(
                _lib.load().ahq_minmax_slots_finalize(
                    _lib.DTYPE_CODE[stat_dtype], slots[2].data_ptr(), num_steps, 1 if self.symmetric else 0,
                    consts[0], consts[1], consts[2], consts[3], flags.data_ptr(), _lib.DTYPE_CODE[mn.dtype],
                    mn.data_ptr(), mx.data_ptr(), self.qmin, self.qmax, _get_minimum_scale(self.qmax - self.qmin),
                    scale.data_ptr(), None if self.symmetric else offset.data_ptr(), _lib.current_stream(device)),
                "ahq_minmax_slots_finalize")
        else:
            _lib.check(
                _lib.load().ahq_minmax_finalize(
                    _lib.DTYPE_CODE[stat_dtype], smin.data_ptr(), smax.data_ptr(), smin.numel(), num_steps,
                    1 if self.symmetric else 0, consts[0], consts[1], consts[2], consts[3], flags.data_ptr(),
                    _lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(), self.qmin, self.qmax,
                    _get_minimum_scale(self.qmax - self.qmin), scale.data_ptr(),
                    None if self.symmetric else offset.data_ptr(), _lib.current_stream(device)),
                "ahq_minmax_finalize")
        self._finalize_adopt(scale, offset)
        if own:
            _report_range_flags(flags)
        return True

    def _finalize_adopt(self, scale: torch.Tensor, offset: torch.Tensor) -> None:
        """What follows a finalize launch on the host: min / max were written behind torch's back (tell autograd, and
        everyone who keys on the version counters), and the encodings the next forward would derive are at hand."""
        torch.autograd.graph.increment_version((self.min, self.max))
        self._mark_offset_in_grid(offset)
        enc = AffineEncoding(scale, offset, self.qmin, self.qmax, self._symmetric, self.block_size,
                             self.zero_point_shift, producer=self)
        self.__dict__["_encoding_cache"] = (self._encoding_cache_key(), enc)

    def _slots_finalize_item(self):
        """The arguments of ahq_minmax_slots_finalize for this quantizer as (item fields..., scale, offset), for a
        caller that finalizes many quantizers with one call (aimet_amd.nn.compute_encodings); None where
        _set_range_from_statistics() has to run: the conditions of _finalize_from_minmax(), with the running extrema
        of a single encoding in the observer's slots."""
        an = self.encoding_analyzer
        cls = type(self)
        if (type(an) is not MinMaxEncodingAnalyzer  # pylint: disable=unidiomatic-typecheck
                or cls.get_scale is not AffineQuantizerBase.get_scale
                or cls._get_offset is not AffineQuantizerBase._get_offset
                or cls.set_range is not AffineQuantizerBase.set_range
                or not self._is_min_max_quantizer()
                or not all(self._is_overwrite_allowed.values())):
            return None
        mn, mx = self.min, self.max
        num_steps = self._num_steps_for_calibration()
        slots = an.observer.live_slots()
        if (slots is None or mn.numel() != 1 or not mn.is_cuda or slots[1] != mn.device or mx.device != mn.device
                or mn.dtype not in _lib.DTYPE_CODE or mx.dtype != mn.dtype or mn.shape != mx.shape
                or num_steps <= 0 or num_steps > (1 << 24)):
            return None
        return slots[0], slots[2], num_steps

    def _derive_encodings(self) -> Optional[AffineEncoding]:
        if not self.is_initialized():
            return None
        fused = self._fused_scale_offset()
        if fused is not None:
            scale, offset = fused
        else:
            scale = self.get_scale(dtype=torch.float32)
            offset = self._get_offset(scale=scale, dtype=torch.float32)
        if scale is None or offset is None:
            return None
        self._mark_offset_in_grid(offset)
        return AffineEncoding(scale, offset, self.qmin, self.qmax, self.symmetric, self.block_size,
                              self.zero_point_shift, producer=self)

    def _mark_offset_in_grid(self, offset: torch.Tensor) -> None:
        """An asymmetric offset derived from min / max is clamp(round(min / scale) - qmin, -qmax, -qmin)
        (_get_offset, and the kernels that compute the same): its zero point lies in [qmin, qmax] by construction,
        which is what the backend would otherwise read back from the device before it chooses the arithmetic."""
        if (not self.symmetric and self._is_min_max_quantizer()
                and type(self)._get_offset is AffineQuantizerBase._get_offset  # pylint: disable=protected-access
                and getattr(offset, "_ahq_constant", None) is None):
            offset._ahq_in_grid = (self.qmin, self.qmax)  # pylint: disable=protected-access

    @classmethod
    def from_encodings(cls, encodings: AffineEncoding) -> "AffineQuantizerBase":
        if not isinstance(encodings, AffineEncoding):
            raise TypeError(f"Expected {AffineEncoding}; got {type(encodings)}")
        qtzr = cls(shape=encodings.scale.shape, qmin=encodings.qmin, qmax=encodings.qmax,
                   symmetric=encodings.symmetry, block_size=encodings.block_size,
                   zero_point_shift=encodings.zero_point_shift)
        qtzr.to(encodings.scale.device)
        qtzr.set_range(encodings.min, encodings.max)
        return qtzr

    @torch.no_grad()
    def get_legacy_encodings(self) -> Optional[list]:
        """The encodings as a list of dictionaries, one per channel (min, max, scale, offset, bitwidth, dtype,
        is_symmetric); None before initialisation (quantizer.py:480-489)."""
        if not self.is_initialized():
            return None
        return self.get_encodings()._to_legacy_format()  # pylint: disable=protected-access

    @torch.no_grad()
    def set_legacy_encodings(self, encodings: list):
        """Take the grid and the range from a list in the form get_legacy_encodings() gives (quantizer.py:491-523).
        That form knows two grids: unsigned asymmetric and signed symmetric."""
        flag = encodings[0]["is_symmetric"].lower()
        if flag not in ("true", "false"):
            raise ValueError(f"is_symmetric must be 'True' or 'False'; got {encodings[0]['is_symmetric']!r}")
        symmetric = flag == "true"
        self.qmin, self.qmax = _derive_qmin_qmax(bitwidth=encodings[0]["bitwidth"], signed=symmetric)
        self.symmetric = symmetric
        self.zero_point_shift = encodings[0].get("zero_point_shift", 0.0)
        min_ = torch.tensor([e["min"] for e in encodings]).view(self.shape)
        max_ = torch.tensor([e["max"] for e in encodings]).view(self.shape)
        self.set_range(min_, max_)

    def extra_repr(self) -> str:
        parts = [f"shape={self.shape}"]
        if self.block_size:
            parts.append(f"block_size={self.block_size}")
        parts += [f"qmin={self.qmin}", f"qmax={self.qmax}", f"symmetric={self.symmetric}"]
        if self.zero_point_shift:
            parts.append(f"zero_point_shift={self.zero_point_shift}")
        return ", ".join(parts)

    @property
    def symmetric(self) -> bool:
        """A quantizer held as scale / offset is symmetric exactly when it holds no offset (quantizer.py:540-571)."""
        if self._is_min_max_quantizer():
            return self._symmetric
        return self.offset is None

    @symmetric.setter
    def symmetric(self, symmetric: bool):
        self._symmetric = symmetric
        if self._is_min_max_quantizer():
            return
        was_symmetric = self.offset is None
        if symmetric and not was_symmetric:
            self._forget_derived_encodings()
            self.offset = None
        elif not symmetric and was_symmetric:
            self._forget_derived_encodings()
            scale = self.scale
            self.offset = nn.Parameter(_symmetric_offset(self.qmin, self.qmax, self.shape, scale.dtype, scale.device),
                                       requires_grad=scale.requires_grad)

    @property
    def bitwidth(self) -> int:
        return self._get_bitwidth()

    @bitwidth.setter
    def bitwidth(self, bitwidth: int):
        self._set_bitwidth(bitwidth)

    @property
    def signed(self) -> bool:
        return self._get_signed()

    @signed.setter
    def signed(self, signed: bool):
        self._set_signed(signed)

    # --------------------------------------------------------------------------------------------- calibration --
    @contextmanager
    def compute_encodings(self):
        """Observe inputs and set min/max from their statistics on exit.  Inside the context the forward pass
        quantizes dynamically with the statistics of the current input (quantizer.py:591-599)."""
        with self._compute_encodings(passthrough=False):
            yield

    def _num_steps_for_calibration(self) -> int:
        n = self.qmax - self.qmin
        return n - 1 if self.zero_point_shift == 0.5 else n

    @contextmanager
    def _compute_encodings(self, passthrough: bool = False):
        """passthrough=True: inputs are observed and returned unquantized (what a whole-model calibration uses)
        (quantizer.py:601-698)."""
        if not any(self._is_overwrite_allowed.values()):
            yield
            return
        inner_forward = torch.Tensor.clone if passthrough else self.forward
        shape = self.shape
        dtype, device = next((p.dtype, p.device) for p in self._parameters.values() if p is not None)

        def observing_forward(input: torch.Tensor) -> torch.Tensor:
            if type(input) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
                input = input.as_subclass(torch.Tensor)
            if input.numel() == 0:
                return inner_forward(input)
            batch_stats = self.encoding_analyzer.update_stats(input)
            lo, hi = self.encoding_analyzer.compute_encodings_from_stats(
                batch_stats, self._num_steps_for_calibration(), self.symmetric
            )
            if self.block_size is not None:
                lo, hi = lo.view(shape), hi.view(shape)
            lo = lo.to(dtype=dtype, device=device).expand(shape)
            hi = hi.to(dtype=dtype, device=device).expand(shape)
            scale, offset = _get_scale_offset(lo.to(torch.float32), hi.to(torch.float32), qmin=self.qmin,
                                              qmax=self.qmax, symmetric=self.symmetric)
            encoding = AffineEncoding(scale, offset, self.qmin, self.qmax, self.symmetric, self.block_size,
                                      self.zero_point_shift, producer=self)
            with self._set_encodings(encoding):
                ret = inner_forward(input)
            if not hasattr(ret, "encoding"):
                ret.encoding = encoding
            return ret

        if passthrough:
            observing_forward = self._observe_passthrough
        if not passthrough:  # (a whole-model calibration enters hundreds of these contexts: nothing it does not need)
            functools.update_wrapper(observing_forward, inner_forward)
        self.encoding_analyzer.reset_stats()
        # (patch_attr(self, "forward", ...) without its generality: a plain function goes into the instance's own
        # dictionary, which is where Module.__setattr__ would put it after its checks)
        own = self.__dict__
        outer = own.get("forward")
        own["forward"] = observing_forward
        try:
            yield
        finally:
            if outer is None:
                del own["forward"]
            else:
                own["forward"] = outer
        self._set_range_from_statistics()

    def _observe_passthrough(self, input: torch.Tensor) -> torch.Tensor:
        """The forward pass of a whole-model calibration (quantizer.py:601-640 with passthrough): the input is only
        observed and comes back as a copy; the dynamic encodings of this batch would go unused.  A min/max analyzer
        writes the copy from the pass that reads the tensor."""
        if type(input) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        if input.numel() == 0:
            return input.clone()
        fused = getattr(self.encoding_analyzer, "observe_and_clone", None)
        if (fused is not None and input.is_cuda and input.dtype in _lib.DTYPE_CODE and input.is_contiguous()
                and not (torch.is_grad_enabled() and input.requires_grad)):
            return fused(input)
        self.encoding_analyzer.update_stats(input)
        return input.clone()

    def _begin_passthrough_calibration(self) -> bool:
        """Entering ``_compute_encodings(passthrough=True)`` without the context manager around it, for a caller
        that enters hundreds of them and leaves them together (aimet_amd.nn.compute_encodings): statistics reset,
        forward replaced by the observing one.  False, with nothing changed, when no end may be overwritten.  The
        caller ends with _end_passthrough_calibration() and sets the range (_set_range_from_statistics(), or a
        launch of its own that does the same for many quantizers)."""
        if not any(self._is_overwrite_allowed.values()):
            return False
        self.encoding_analyzer.reset_stats()
        own = self.__dict__
        own["_forward_before_calibration"] = own.get("forward")
        own["forward"] = self._observe_passthrough
        return True

    def _end_passthrough_calibration(self) -> None:
        own = self.__dict__
        outer = own.pop("_forward_before_calibration", None)
        if outer is None:
            own.pop("forward", None)
        else:
            own["forward"] = outer

    def _calibrate_on(self, tensor: torch.Tensor) -> None:
        """``with self._compute_encodings(passthrough=True): self(tensor)`` for a caller that drops the result (the
        calibration of a parameter, nn/base.py:378-383): the statistics are reset, the tensor is observed and the range
        set, without the pass-through copy of the tensor and without patching the forward method."""
        if not any(self._is_overwrite_allowed.values()):
            return
        self.encoding_analyzer.reset_stats()
        if type(tensor) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            tensor = tensor.as_subclass(torch.Tensor)
        if tensor.numel():
            self.encoding_analyzer.update_stats(tensor.detach())
        self._set_range_from_statistics()

    def _set_range_from_statistics(self) -> None:
        """What leaving compute_encodings() does (quantizer.py:678-698)."""
        shape = self.shape
        if self._finalize_from_minmax():
            return
        try:
            lo, hi = self.encoding_analyzer.compute_encodings(self._num_steps_for_calibration(), self.symmetric)
            if self.block_size is not None:
                # the views are new tensor objects: hand on the range flags the kernel has already evaluated
                flags = getattr(lo, "_ahq_range_flags", None)
                same = flags is not None and getattr(hi, "_ahq_range_flags", None) is flags
                lo, hi = lo.view(shape), hi.view(shape)
                if same:
                    lo._ahq_range_flags = hi._ahq_range_flags = flags  # pylint: disable=protected-access
            _flag_extreme_min_max(lo, hi)
        except StatisticsNotFoundError:
            return
        if not self._is_overwrite_allowed["min"]:
            lo = None
        if not self._is_overwrite_allowed["max"]:
            hi = None
        self.set_range(lo, hi)

    @contextmanager
    def _set_encodings(self, enc: Optional[AffineEncoding]):
        """Temporarily make ``get_encodings()`` return ``enc`` (quantizer.py:806-821)."""
        with (
            patch_attr(self, "get_encodings", lambda *a, **k: enc),
            patch_attr(self, "is_initialized", lambda *a, **k: enc is not None),
        ):
            yield

    @contextmanager
    def _precompute_encodings(self, dtype: Optional[torch.dtype] = None):
        """Evaluate the encodings once and reuse them for every forward inside the context (quantizer.py:790-804)."""
        enc = self.get_encodings()
        if enc is not None:
            with torch.no_grad():
                enc = enc.to(dtype=dtype) if dtype is not None else enc
                const = getattr(enc.offset, "_ahq_constant", None)
                enc.scale = enc.scale.detach()
                enc.offset = enc.offset.detach()
                if const is not None:
                    enc.offset._ahq_constant = const  # pylint: disable=protected-access
        with self._set_encodings(enc) if enc is not None else nullcontext():
            yield

    def _get_dummy_encoding(self) -> AffineEncoding:
        device = next(p.device for p in self._parameters.values() if p is not None)
        return AffineEncoding(torch.ones((), device=device), torch.zeros((), device=device), self.qmin, self.qmax,
                              self.symmetric, block_size=None, zero_point_shift=self.zero_point_shift, producer=self)

    def _forward_encoding(self, input: torch.Tensor, what: str) -> AffineEncoding:
        encoding = self.get_encodings()
        if encoding is None:
            if input.numel() == 0:
                return self._get_dummy_encoding()
            raise RuntimeError(
                f"Failed to run {what} since quantization parameters are not initialized."
                " Please initialize the quantization parameters using `compute_encodings()`."
            )
        return encoding

    # ----------------------------------------------------------------------------------------- checkpointing --
    def get_extra_state(self):
        state = super().get_extra_state()
        state.update({
            "qmin": torch.tensor(self.qmin),
            "qmax": torch.tensor(self.qmax),
            "symmetric": torch.tensor(self.symmetric),
            "block_size": torch.tensor(self.block_size or ()),
            "zero_point_shift": torch.tensor(self.zero_point_shift),
        })
        return state

    def set_extra_state(self, state):
        state = dict(state)
        grid = {k: state.pop(k) for k in ("qmin", "qmax", "symmetric", "block_size", "zero_point_shift") if k in state}
        super().set_extra_state(state)
        if "qmin" in grid:
            self.qmin = grid["qmin"].item()
        if "qmax" in grid:
            self.qmax = grid["qmax"].item()
        if "symmetric" in grid:
            self.symmetric = grid["symmetric"].item()
        if "block_size" in grid:
            self.block_size = tuple(int(b) for b in grid["block_size"]) or None
        if "zero_point_shift" in grid:
            self.zero_point_shift = grid["zero_point_shift"].item()
        self.shape = tuple(self.min.shape if self._is_min_max_quantizer() else self.scale.shape)

    def load_state_dict(self, state_dict, strict: bool = True, **kwargs):  # pylint: disable=arguments-differ
        if not strict:
            # a non-strict load may change the shape of the encodings, never their parametrisation
            # (quantizer.py:700-751)
            if "min" in state_dict or "max" in state_dict:
                names = ("min", "max")
            elif "scale" in state_dict or "offset" in state_dict:
                names = ("scale", "offset")
            else:
                return super().load_state_dict(state_dict, strict, **kwargs)  # malformed: the base class says how
            if self._is_min_max_quantizer() != (names == ("min", "max")):
                raise RuntimeError(
                    f"state dict holds {'/'.join(names)} but this quantizer is parametrized with "
                    f"{'/'.join(self._parameters.keys())}")
            self._forget_derived_encodings()
            for name in names:
                new = state_dict.get(name)
                cur = self._parameters[name]
                if new is None:
                    continue
                if cur is None:  # the offset of a symmetric scale/offset quantizer
                    ref = self.scale
                    setattr(self, name, nn.Parameter(new.clone().to(device=ref.device, dtype=ref.dtype)))
                elif new.shape != cur.shape:
                    setattr(self, name, nn.Parameter(new.clone().to(device=cur.device, dtype=cur.dtype)))
        return super().load_state_dict(state_dict, strict, **kwargs)


@runtime_checkable
class MinMaxQuantizer(Protocol):
    """An affine quantizer that holds its encoding as min and max (quantizer.py:903-914): isinstance() looks for the
    marker the reparametrisation leaves."""

    _is_min_max: Any

    shape: Tuple[int, ...]
    qmin: int
    qmax: int
    symmetric: bool


@runtime_checkable
class ScaleOffsetQuantizer(Protocol):
    """An affine quantizer that holds its encoding as scale and offset (quantizer.py:917-928)."""

    _is_scale_offset: Any

    shape: Tuple[int, ...]
    qmin: int
    qmax: int
    symmetric: bool


class Quantize(AffineQuantizerBase):
    r"""out = clamp(round(input / scale) - offset, qmin, qmax), returned as a :class:`QuantizedTensor`."""

    def __init__(self, shape, *args, **kwargs):
        super().__init__(shape, *args, **kwargs)
        if self.zero_point_shift != 0.0:
            raise RuntimeError("Nonzero quant shift not supported for Quantize")

    def forward(self, input: torch.Tensor) -> QuantizedTensor:
        encoding = self._forward_encoding(input, "Quantize")
        if type(input) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        output = quantize(input, encoding.scale, encoding.offset, encoding.qmin, encoding.qmax,
                          block_size=encoding.block_size)
        output = output.as_subclass(QuantizedTensor)
        output.encoding = encoding
        return output


class _ForwardPlan(NamedTuple):
    """What a forward pass without gradients can take over from an earlier one (QuantizeDequantize._forward_steady)."""
    encoding: AffineEncoding   # the encodings last checked against the rest
    shape: torch.Size          # of the input
    dtype: torch.dtype
    device: torch.device
    grid: "_lib.Grid"
    layout: "_lib.Layout"
    grid_key: tuple            # (qmin, qmax, symmetry, block_size, zero_point_shift) the grid and layout were made for
    enc_shape: torch.Size      # of scale and offset
    needs_constant: bool       # the arithmetic was chosen knowing that the offsets are the grid's constant


class QuantizeDequantize(AffineQuantizerBase):
    r"""out = (clamp(round(input / scale) - offset, qmin, qmax) + offset) * scale, returned as a
    :class:`DequantizedTensor`; scale and offset derive from the learnable ``min`` / ``max``."""

    def __init__(self, shape, *args, **kwargs):  # pylint: disable=useless-parent-delegation
        super().__init__(shape, *args, **kwargs)

    def _forward_from_range(self, input: torch.Tensor) -> Optional[DequantizedTensor]:
        """The forward pass with learned min / max as one autograd node (_QdqFromRange); None when that does not
        apply (nothing learned, a subclass or a patched get_encodings(), another backend, tensors the library does
        not take, a grid that needs another compute dtype check) and the step-by-step form has to run."""
        if not torch.is_grad_enabled():
            return None
        from aimet_amd.quantization.affine.backends import get_backend, hip as _hip

        cls = type(self)
        if not self._is_min_max_quantizer():
            return None
        mn, mx = self.min, self.max
        if not (mn.requires_grad or mx.requires_grad):
            return None
        if (cls.get_scale is not AffineQuantizerBase.get_scale or cls._get_offset is not AffineQuantizerBase._get_offset
                or cls.get_encodings is not AffineQuantizerBase.get_encodings or "get_encodings" in self.__dict__
                or get_backend() is not _hip or not self.is_initialized()):
            return None
        if not (input.is_cuda and input.dtype in _lib.DTYPE_CODE and input.numel() > 0 and mn.device == input.device
                and mx.device == input.device and mn.dtype == mx.dtype and mn.dtype in _lib.DTYPE_CODE
                and mn.shape == mx.shape and mn.is_contiguous() and mx.is_contiguous()):
            return None
        cd = _hip._internal_dtype(input.dtype, self.qmin, self.qmax)  # pylint: disable=protected-access
        if cd == torch.float64 or not _hip._is_grid_representable(cd, self.qmin, self.qmax):  # pylint: disable=protected-access
            return None  # the step-by-step form raises what the reference raises
        x = input if type(input) == torch.Tensor else input.as_subclass(torch.Tensor)  # pylint: disable=unidiomatic-typecheck
        _hip._validate_arguments(x, mn, self.qmin, self.qmax, self.block_size)  # pylint: disable=protected-access
        symmetric = bool(self.symmetric)
        constant = self._constant_offset(mn.device) if symmetric else None
        bs = tuple(self.block_size) if self.block_size else None
        y, scale, offset = _QdqFromRange.apply(x, mn, mx, self.qmin, self.qmax, symmetric, constant, bs,
                                               float(self.zero_point_shift or 0.0), cd)
        encoding = AffineEncoding(scale, constant if symmetric else offset, self.qmin, self.qmax, self._symmetric,
                                  self.block_size, self.zero_point_shift, producer=self)
        output = y.as_subclass(DequantizedTensor)
        output.encoding = encoding
        return output

    def _calibrate_qdq_prepare(self, tensor: torch.Tensor):
        """Whether calibration on `tensor` followed by its quantize-dequantize can be one library call
        (ahq_minmax_calibrate_qdq), and with which arguments: (tensor as the library takes it, grid, layout, workspace
        bytes, calibration steps, symmetric).  None when the two steps have to run: gradients switched on, a subclass
        or a patched method, hooks on the quantizer, another backend or analyzer, an end that may not be overwritten,
        tensors the library does not take, or an arithmetic that would depend on the offsets' values."""
        if torch.is_grad_enabled() or type(self) is not QuantizeDequantize:  # pylint: disable=unidiomatic-typecheck
            return None
        from aimet_amd.quantization._stats import _check_reducible
        from aimet_amd.quantization.affine.backends import get_backend, hip as _hip
        from torch.nn.modules import module as _module

        an = self.encoding_analyzer
        if not self._is_min_max_quantizer():
            return None
        mn, mx = self.min, self.max
        own = self.__dict__
        if (type(an) is not MinMaxEncodingAnalyzer  # pylint: disable=unidiomatic-typecheck
                or not all(self._is_overwrite_allowed.values()) or get_backend() is not _hip
                or "forward" in own or "get_encodings" in own or "is_initialized" in own
                or self._forward_hooks or self._forward_pre_hooks
                or _module._global_forward_hooks or _module._global_forward_pre_hooks):  # pylint: disable=protected-access
            return None
        x = tensor.detach()
        if type(x) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            x = x.as_subclass(torch.Tensor)
        num_steps = self._num_steps_for_calibration()
        if not (x.is_cuda and x.dtype in _lib.DTYPE_CODE and x.is_contiguous() and x.numel() > 0
                and mn.device == x.device and mx.device == x.device and mn.dtype == mx.dtype
                and mn.dtype in _lib.DTYPE_CODE and mn.shape == mx.shape and mn.is_contiguous() and mx.is_contiguous()
                and 0 < num_steps <= (1 << 24)):
            return None
        symmetric = bool(self.symmetric)
        zps = float(self.zero_point_shift or 0.0)
        bs = tuple(self.block_size) if self.block_size else None
        held = own.get("_calibrate_qdq_plan")
        key = (tuple(x.shape), x.dtype, x.device, tuple(mn.shape), self.qmin, self.qmax, symmetric, bs, zps)
        if held is None or held[0] != key:
            try:
                _check_reducible(x, tuple(self.shape), bs)
                _hip._validate_arguments(x, mn, self.qmin, self.qmax, bs)  # pylint: disable=protected-access
            except RuntimeError:
                return None  # the step-by-step form raises what the reference raises
            # the arithmetic the forward pass would choose (backends/hip.py: quantize_dequantize)
            per_tensor = mn.numel() == 1
            if bs is None and zps == 0.0 and (per_tensor or symmetric):
                aten = per_tensor or _hip._aten_arithmetic_applies(  # pylint: disable=protected-access
                    x, mn, self._constant_offset(x.device), self.qmin, self.qmax)
            elif bs is None and zps == 0.0:
                return None  # per-channel, asymmetric: the choice looks at the offsets
            else:
                aten = False
            if aten:
                arith, cd = _lib.AHQ_ARITH_ATEN, torch.float32
            else:
                arith, cd = _lib.AHQ_ARITH_AUTOGRAD, _hip._internal_dtype(x.dtype, self.qmin, self.qmax)  # pylint: disable=protected-access
                if cd == torch.float64 or not _hip._is_grid_representable(cd, self.qmin, self.qmax):  # pylint: disable=protected-access
                    return None
            grid = _hip._grid(arith, _lib.AHQ_OP_QDQ, x.dtype, cd, self.qmin, self.qmax, 0.0 if aten else zps)  # pylint: disable=protected-access
            layout = _build_layout(tuple(x.shape), tuple(range(x.dim())), tuple(mn.shape), None if aten else bs)
            nbytes = _lib.load().ahq_minmax_calibrate_qdq_workspace_bytes(_lib.DTYPE_CODE[x.dtype], layout)
            held = own["_calibrate_qdq_plan"] = (key, grid, layout, nbytes)
        _, grid, layout, nbytes = held
        return x, grid, layout, nbytes, num_steps, symmetric

    def _calibrate_qdq_adopt(self, y: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor) -> DequantizedTensor:
        """What follows the launches of ahq_minmax_calibrate_qdq on the host: min / max were written behind torch's
        back, the encodings the next forward would derive are at hand, and `y` is the quantizer's output."""
        torch.autograd.graph.increment_version((self.min, self.max))
        self._mark_offset_in_grid(offset)
        enc = AffineEncoding(scale, offset, self.qmin, self.qmax, self._symmetric, self.block_size,
                             self.zero_point_shift, producer=self)
        self.__dict__["_encoding_cache"] = (self._encoding_cache_key(), enc)
        output = y.as_subclass(DequantizedTensor)
        output.encoding = enc
        return output

    def _calibrate_and_quantize(self, tensor: torch.Tensor) -> Optional[DequantizedTensor]:
        """``self._calibrate_on(tensor)`` followed by ``self(tensor)`` -- what a quantized module does with each of
        its parameters when a calibration starts (nn/base.py:331-386, 296-324) -- as one library call
        (ahq_minmax_calibrate_qdq: the three launches of the step-by-step form, same results).  None, with nothing
        changed, when that does not apply and the two steps have to run (see _calibrate_qdq_prepare)."""
        from aimet_amd.quantization.encoding_analyzer import _scalar_constants, _range_flags_buffer, _report_range_flags

        plan = self._calibrate_qdq_prepare(tensor)
        if plan is None:
            return None
        x, grid, layout, nbytes, num_steps, symmetric = plan
        mn, mx = self.min, self.max
        device = x.device
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device)  # two statistics per encoding: not kept
        self.encoding_analyzer.reset_stats()
        consts = _scalar_constants(x.dtype, _get_minimum_scale(num_steps))
        y = torch.empty_like(x)
        scale = torch.empty(mn.shape, dtype=torch.float32, device=device)
        offset = self._constant_offset(device) if symmetric else torch.empty(mn.shape, dtype=torch.float32,
                                                                             device=device)
        flags, own_flags = _range_flags_buffer(device)
        _lib.check(
            _lib.load().ahq_minmax_calibrate_qdq(
                grid, layout, x.data_ptr(), y.data_ptr(), num_steps, 1 if symmetric else 0, consts[0], consts[1],
                consts[2], consts[3], flags.data_ptr(), _lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr(),
                _get_minimum_scale(self.qmax - self.qmin), scale.data_ptr(), offset.data_ptr(), ws.data_ptr(), nbytes,
                _lib.current_stream(device)),
            "ahq_minmax_calibrate_qdq")
        output = self._calibrate_qdq_adopt(y, scale, offset)
        if own_flags:
            _report_range_flags(flags)
        return output

    def _forward_steady(self, input: torch.Tensor) -> Optional[DequantizedTensor]:
        """The forward pass of an inference loop -- no gradients, cached encodings, an input of the shape seen before:
        the library call of the step-by-step form with the grid and layout of an earlier call, and nothing else (a
        whole-model forward makes hundreds of these calls and is bound by their host time).  Grid and layout depend
        on the quantizer's grid and on shapes, not on the encodings' values, so they outlive a new calibration.  None
        whenever anything differs; the step-by-step form then runs."""
        own = self.__dict__
        plan = own.get("_forward_plan")
        if plan is None or torch.is_grad_enabled():
            return None
        borrowed = "get_encodings" in own  # precomputed encodings, or the dynamic ones of a calibration batch
        if borrowed:
            enc = self.get_encodings()
            if enc is None:
                return None
        else:
            cached = own.get("_encoding_cache")
            if cached is None or cached[0] != self._encoding_cache_key():
                return None
            enc = cached[1]
        x = input if type(input) == torch.Tensor else input.as_subclass(torch.Tensor)  # pylint: disable=unidiomatic-typecheck
        if (plan.shape != x.shape or plan.dtype != x.dtype or plan.device != x.device or not x.is_contiguous()
                or get_backend() is not _hip_backend):
            return None
        scale, offset = enc.scale, enc.offset
        if plan.encoding is not enc:
            # other encodings than last time (a calibration, a new range): they have to fit the plan as they are
            f32 = torch.float32
            if (plan.grid_key != (enc.qmin, enc.qmax, enc.symmetry, enc.block_size, enc.zero_point_shift)
                    or scale.dtype != f32 or offset.dtype != f32 or scale.shape != plan.enc_shape
                    or offset.shape != plan.enc_shape or not (scale.is_contiguous() and offset.is_contiguous())
                    or scale.device != x.device or offset.device != x.device or scale.requires_grad
                    or offset.requires_grad
                    or (plan.needs_constant and getattr(offset, "_ahq_constant", None) is None
                        and getattr(offset, "_ahq_in_grid", None) != (enc.qmin, enc.qmax))):
                if not borrowed:
                    del own["_forward_plan"]
                return None
            own["_forward_plan"] = plan._replace(encoding=enc)
        y = torch.empty_like(x)
        status = _lib.load().ahq_qdq_forward(plan.grid, plan.layout, x.data_ptr(), y.data_ptr(), None, scale.data_ptr(),
                                             offset.data_ptr(), None, None, _lib.current_stream(x.device))
        if status:
            _lib.check(status, "ahq_qdq_forward")
        output = y.as_subclass(DequantizedTensor)
        output.encoding = enc
        return output

    def _plan_steady_forward(self, input: torch.Tensor, encoding: AffineEncoding) -> None:
        """After a step-by-step forward pass without gradients, the second in a row with the same input shape: keep
        what the next one can reuse (see _forward_steady).  Nothing is kept where the choice of the arithmetic looks
        at tensor values, where scale or offset would have to be converted or broadcast first, or for anything but
        the plain class on this backend."""
        _hip = _hip_backend
        own = self.__dict__
        if "get_encodings" in own:
            return  # a pass with borrowed encodings (dynamic ones of a calibration batch, precomputed ones)
        own.pop("_forward_plan", None)
        seen = own.get("_forward_seen")
        if seen is None or seen[0] != input.shape or seen[1] != input.dtype:
            own["_forward_seen"] = (input.shape, input.dtype)
            return
        cached = own.get("_encoding_cache")
        scale, offset = encoding.scale, encoding.offset
        if (type(self) is not QuantizeDequantize  # pylint: disable=unidiomatic-typecheck
                or cached is None or cached[1] is not encoding or get_backend() is not _hip
                or not (input.is_cuda and input.is_contiguous() and input.numel() > 0 and input.dtype in _lib.DTYPE_CODE)
                or scale.dtype != torch.float32 or offset.dtype != torch.float32 or scale.shape != offset.shape
                or not (scale.is_contiguous() and offset.is_contiguous())
                or scale.device != input.device or offset.device != input.device
                or scale.requires_grad or offset.requires_grad):
            return
        bs = tuple(encoding.block_size) if encoding.block_size else None
        zps = float(encoding.zero_point_shift or 0.0)
        qmin, qmax = encoding.qmin, encoding.qmax
        aten = needs_constant = False
        if bs is None and zps == 0.0:
            needs_constant = scale.numel() != 1
            if (needs_constant and getattr(offset, "_ahq_constant", None) is None
                    and getattr(offset, "_ahq_in_grid", None) != (qmin, qmax)):
                return  # per-channel with offsets of unknown range: the choice reads them on every call
            aten = _hip._aten_arithmetic_applies(input, scale, offset, qmin, qmax)  # pylint: disable=protected-access
        if aten:
            arith, cd = _lib.AHQ_ARITH_ATEN, torch.float32
        else:
            arith, cd = _lib.AHQ_ARITH_AUTOGRAD, _hip._internal_dtype(input.dtype, qmin, qmax)  # pylint: disable=protected-access
            if cd == torch.float64 or not _hip._is_grid_representable(cd, qmin, qmax):  # pylint: disable=protected-access
                return
        grid = _hip._grid(arith, _lib.AHQ_OP_QDQ, input.dtype, cd, qmin, qmax, 0.0 if aten else zps)  # pylint: disable=protected-access
        layout = _build_layout(tuple(input.shape), tuple(range(input.dim())), tuple(scale.shape), None if aten else bs)
        own["_forward_plan"] = _ForwardPlan(
            encoding, input.shape, input.dtype, input.device, grid, layout,
            (qmin, qmax, encoding.symmetry, encoding.block_size, encoding.zero_point_shift), scale.shape, needs_constant)

    def forward(self, input: torch.Tensor) -> DequantizedTensor:
        steady = self._forward_steady(input)
        if steady is not None:
            return steady
        fused = self._forward_from_range(input)
        if fused is not None:
            return fused
        encoding = self._forward_encoding(input, "QuantizeDequantize")
        if type(input) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        output = quantize_dequantize(input, encoding.scale, encoding.offset, encoding.qmin, encoding.qmax,
                                     block_size=encoding.block_size, zero_point_shift=encoding.zero_point_shift)
        if not torch.is_grad_enabled():
            self._plan_steady_forward(input, encoding)
        output = output.as_subclass(DequantizedTensor)
        output.encoding = encoding
        return output


class Dequantize(AffineQuantizerBase):
    r"""out = (input + offset) * scale"""

    def forward(self, input):
        if self.zero_point_shift != 0.0:
            raise RuntimeError("Nonzero quant shift not supported for Dequantize")
        encoding = self._forward_encoding(input, "Dequantize")
        if type(input) != torch.Tensor:  # pylint: disable=unidiomatic-typecheck
            input = input.as_subclass(torch.Tensor)
        output = dequantize(input, encoding.scale, encoding.offset, block_size=encoding.block_size)
        output = output.as_subclass(DequantizedTensor)
        output.encoding = encoding
        return output


class GroupedBlockQuantizeDequantize(QuantizeDequantize):
    """Blockwise quantize-dequantize whose block scales are snapped to integer multiples (1 .. 2^(decompressed_bw -
    bitwidth)) of a scale shared by each group of blocks -- LPBQ (quantizer.py:1270-1440)."""

    def __init__(self, shape, bitwidth: int, symmetric: bool, decompressed_bw: int,
                 encoding_analyzer: EncodingAnalyzer = None, block_size: Optional[Tuple[int, ...]] = None,
                 block_grouping: Optional[Tuple[int, ...]] = None):
        super().__init__(shape, bitwidth, symmetric, encoding_analyzer, block_size)
        self.decompressed_bw = decompressed_bw
        self.block_grouping = block_grouping
        if self.block_grouping is None:
            self.block_grouping = tuple(1 for _ in self.shape)
        if block_grouping is not None:
            if len(block_grouping) != len(self.shape):
                raise RuntimeError(f"Length of block grouping {block_grouping} must equal length of shape {shape}.")
            for dim, group in zip(self.shape, block_grouping):
                if group != -1 and dim % group != 0:
                    raise RuntimeError(
                        f"Quantizer shape dimensions must divide evenly with corresponding block "
                        f"grouping values for shapes {shape} and block grouping {block_grouping}."
                    )
        if self.decompressed_bw < self.bitwidth:
            raise RuntimeError(
                f"Decompressed bitwidth {decompressed_bw} cannot be smaller than self.bitwidth {bitwidth}"
            )
        if not symmetric:
            raise RuntimeError("GroupedBlockQuantizeDequantize only supports symmetric quantization.")

    def get_scale(self, dtype=None) -> Optional[torch.Tensor]:
        return self._get_scale(dtype)[0]

    def get_per_channel_scale(self, dtype=None) -> Optional[torch.Tensor]:
        raw = super().get_scale(dtype)
        return None if raw is None else self._get_per_channel_scale(raw)

    def _fused_lpbq_scale(self):
        """(scale, per-channel scale) in float32 from one launch of ahq_lpbq_scale -- as an autograd node with a
        one-launch backward when min / max are learned; None when that does not apply (parameters not on a GPU,
        groups that are not runs of neighbouring blocks, the encoding held as scale / offset) and the step-by-step
        form has to run."""
        if not self._is_min_max_quantizer():
            return None
        mn, mx = self.min, self.max
        if not (mn.is_cuda and mx.device == mn.device and mn.dtype == mx.dtype and mn.dtype in _lib.DTYPE_CODE
                and mn.shape == mx.shape and mn.is_contiguous() and mx.is_contiguous() and mn.numel() > 0):
            return None
        if type(self).get_scale is not GroupedBlockQuantizeDequantize.get_scale:
            return None
        shape = tuple(mn.shape)
        group_shape = tuple(d // g if g != -1 else 1 for d, g in zip(shape, self.block_grouping))
        layout = _build_layout(shape, tuple(range(len(shape))), group_shape, tuple(self.block_grouping))
        multipliers = 2 ** (self.decompressed_bw - self.bitwidth)
        unsupported = self.__dict__.get("_lpbq_unsupported")
        if unsupported == (shape, tuple(self.block_grouping)):
            return None
        if torch.is_grad_enabled() and (mn.requires_grad or mx.requires_grad):
            # the library refuses some groupings; find out once, outside autograd
            if self.__dict__.get("_lpbq_supported") != (shape, tuple(self.block_grouping)):
                with torch.no_grad():
                    if self._fused_lpbq_scale() is None:
                        return None
            return _LpbqScale.apply(mn, mx, self.qmin, self.qmax, multipliers, layout, group_shape)
        lib = _lib.load()
        scale = torch.empty(shape, dtype=torch.float32, device=mn.device)
        per_channel = torch.empty(group_shape, dtype=torch.float32, device=mn.device)
        status = lib.ahq_lpbq_scale(_lib.DTYPE_CODE[mn.dtype], layout, mn.data_ptr(), mx.data_ptr(), self.qmin, self.qmax,
                                    _get_minimum_scale(self.qmax - self.qmin), multipliers,
                                    scale.data_ptr(), per_channel.data_ptr(), _lib.current_stream(mn.device))
        if status == _lib.AHQ_ERR_UNSUPPORTED:
            self.__dict__["_lpbq_unsupported"] = (shape, tuple(self.block_grouping))
            return None
        _lib.check(status, "ahq_lpbq_scale")
        self.__dict__["_lpbq_supported"] = (shape, tuple(self.block_grouping))
        return scale, per_channel

    def _blocks_per_group(self) -> Optional[int]:
        """Blocks per group when every group is a run of neighbouring blocks in the flat order of the scale array
        (grouping 1 on leading dimensions, any divisor on one, whole dimensions after it); else None."""
        shape = tuple(self.shape)
        grouping = tuple(d if g == -1 else g for d, g in zip(shape, self.block_grouping))
        first = 0
        while first < len(shape) and grouping[first] == 1:
            first += 1
        if any(grouping[k] != shape[k] for k in range(first + 1, len(shape))):
            return None
        return math.prod(grouping[first:])

    def forward(self, input: torch.Tensor) -> DequantizedTensor:
        out = self._fused_forward(input)
        return out if out is not None else super().forward(input)

    def _fused_forward(self, input: torch.Tensor) -> Optional[DequantizedTensor]:
        """The whole forward pass -- block scales from min / max, snapped to the group's multiples, then
        quantize-dequantize -- in one launch (ahq_lpbq_qdq_forward), as one autograd node (_LpbqQdqFromRange) when a
        gradient is wanted; None when that does not apply and get_encodings() followed by quantize_dequantize() has
        to run."""
        from aimet_amd.quantization.affine.backends import get_backend, hip as _hip

        cls = type(self)
        if (cls.get_scale is not GroupedBlockQuantizeDequantize.get_scale
                or cls.get_encodings is not GroupedBlockQuantizeDequantize.get_encodings
                or "get_encodings" in self.__dict__ or not self.is_initialized() or self.zero_point_shift
                or get_backend() is not _hip or not self._is_min_max_quantizer()):
            return None
        mn, mx = self.min, self.max
        if not (input.is_cuda and input.dtype in _lib.DTYPE_CODE and input.numel() > 0 and mn.device == input.device
                and mx.device == input.device and mn.dtype == mx.dtype and mn.dtype in _lib.DTYPE_CODE
                and mn.shape == mx.shape and mn.is_contiguous() and mx.is_contiguous()):
            return None
        shape = tuple(mn.shape)
        key = (tuple(input.shape), input.dtype, shape, self.block_size, tuple(self.block_grouping))
        if self.__dict__.get("_lpbq_forward_unsupported") == key:
            return None
        group = self._blocks_per_group()
        if group is None or _hip._internal_dtype(input.dtype, self.qmin, self.qmax) != input.dtype:  # pylint: disable=protected-access
            return None
        x = input if type(input) == torch.Tensor else input.as_subclass(torch.Tensor)  # pylint: disable=unidiomatic-typecheck
        _hip._validate_arguments(x, mn, self.qmin, self.qmax, self.block_size)  # pylint: disable=protected-access
        offset = self._constant_offset(x.device)  # symmetric grid (the constructor accepts no other)
        if not (offset.is_contiguous() and offset.numel() == mn.numel() and offset.dtype == torch.float32):
            return None
        group_shape = tuple(d // g if g != -1 else 1 for d, g in zip(shape, self.block_grouping))
        multipliers = 2 ** (self.decompressed_bw - self.bitwidth)
        bs = tuple(self.block_size) if self.block_size else None
        if torch.is_grad_enabled() and (input.requires_grad or mn.requires_grad or mx.requires_grad):
            # the library refuses some layouts and groupings: find out once per shape, outside autograd
            if self.__dict__.get("_lpbq_forward_supported") != key:
                with torch.no_grad():
                    if self._fused_forward(x.detach()) is None or self._fused_lpbq_scale() is None:
                        self.__dict__["_lpbq_forward_unsupported"] = key
                        return None
            group_layout = _build_layout(shape, tuple(range(len(shape))), group_shape, tuple(self.block_grouping))
            y, scale, per_channel = _LpbqQdqFromRange.apply(x, mn, mx, self.qmin, self.qmax, bs, group, group_shape,
                                                            multipliers, offset, group_layout)
        else:
            status, y, _, scale, per_channel, _, _ = _lpbq_forward_launch(x, mn, mx, self.qmin, self.qmax, bs, group,
                                                                          group_shape, multipliers, offset)
            if status == _lib.AHQ_ERR_UNSUPPORTED:
                self.__dict__["_lpbq_forward_unsupported"] = key
                return None
            _lib.check(status, "ahq_lpbq_qdq_forward")
            self.__dict__["_lpbq_forward_supported"] = key
        encoding = GroupedBlockEncoding(scale=scale, offset=offset, bitwidth=self.bitwidth, signed=self.signed,
                                        symmetry=self.symmetric, block_size=self.block_size,
                                        block_grouping=self.block_grouping, decompressed_bw=self.decompressed_bw,
                                        per_channel_scale=per_channel, zero_point_shift=self.zero_point_shift,
                                        producer=self)
        out = y.as_subclass(DequantizedTensor)
        out.encoding = encoding
        return out

    def _get_scale(self, dtype=None):
        if dtype in (None, torch.float32) and self.is_initialized():
            fused = self._fused_lpbq_scale()
            if fused is not None:
                return fused
        raw = None
        mn, mx = (self.min, self.max) if self._is_min_max_quantizer() else (None, None)
        if (mn is not None and dtype in (None, torch.float32) and self.is_initialized() and torch.is_grad_enabled()
                and (mn.requires_grad or mx.requires_grad) and mn.is_cuda and mx.device == mn.device
                and mn.dtype == mx.dtype and mn.dtype in _lib.DTYPE_CODE and mn.shape == mx.shape
                and mn.is_contiguous() and mx.is_contiguous()):
            # learned ranges: the block scales before snapping as one autograd node (see _RangeToScaleOffset)
            raw = _RangeToScaleOffset.apply(mn, mx, self.qmin, self.qmax, True, self._constant_offset(mn.device))[0]
        if raw is None:
            raw = super().get_scale(dtype)
        if raw is None:
            return None, None
        per_channel = self._get_per_channel_scale(raw)
        snapped = quantize_dequantize(raw, per_channel, torch.zeros_like(per_channel), 1,
                                      2 ** (self.decompressed_bw - self.bitwidth), block_size=self.block_grouping)
        return snapped, per_channel

    def _get_per_channel_scale(self, raw_scale: torch.Tensor) -> torch.Tensor:
        """Largest block scale of each group divided by the number of integer multipliers (quantizer.py:1382-1399)."""
        group_shape = [d // g if g != -1 else 1 for d, g in zip(raw_scale.shape, self.block_grouping)]
        grouping = concretize_block_size(raw_scale.shape, group_shape, self.block_grouping)
        view = raw_scale.reshape(*interleave(group_shape, grouping))
        largest = torch.amax(view, dim=tuple(range(1, view.dim(), 2)))
        return true_divide(largest, 2 ** (self.decompressed_bw - self.bitwidth))

    def get_encodings(self) -> Optional[GroupedBlockEncoding]:
        if not self.is_initialized():
            return None
        scale, per_channel = self._get_scale(dtype=torch.float32)
        return GroupedBlockEncoding(scale=scale, offset=self.get_offset(dtype=torch.float32), bitwidth=self.bitwidth,
                                    signed=self.signed, symmetry=self.symmetric, block_size=self.block_size,
                                    block_grouping=self.block_grouping, decompressed_bw=self.decompressed_bw,
                                    per_channel_scale=per_channel, zero_point_shift=self.zero_point_shift,
                                    producer=self)

    @classmethod
    def from_encodings(cls, encodings: GroupedBlockEncoding) -> "GroupedBlockQuantizeDequantize":
        if not isinstance(encodings, GroupedBlockEncoding):
            raise TypeError(f"Expected {GroupedBlockEncoding}; got {type(encodings)}")
        qtzr = cls(shape=encodings.scale.shape, bitwidth=encodings.bitwidth, symmetric=encodings.symmetry,
                   decompressed_bw=encodings.decompressed_bw, block_size=encodings.block_size,
                   block_grouping=encodings.block_grouping)
        qtzr.to(encodings.scale.device)
        qtzr.set_range(encodings.min, encodings.max)
        return qtzr
