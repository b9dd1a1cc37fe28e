"""HIP quantization backend: ``quantize`` / ``dequantize`` / ``quantize_dequantize`` on MI355X.

Satisfies the reference's backend protocol (aimet_torch/quantization/affine/backends/utils.py:16-44) and reproduces the
decisions of its default backend (aimet_torch/quantization/affine/backends/torch_builtins.py):

* argument validation and error types                         torch_builtins.py:119-162
* compute-dtype promotion (bf16 up to 4-bit, fp16 up to 8-bit)  torch_builtins.py:49-116, 193-196, 274-281
* the choice between the ATen fake-quantize arithmetic and the composed autograd arithmetic
                                                              torch_builtins.py:243-266, 335-431
* straight-through gradients for input, scale and offset      torch_builtins.py:588-831

Every tensor pass runs in a hand-written HIP kernel reached through the C ABI of libaimet_amd.so.  There is no
fallback: CPU tensors, float64 grids and missing libraries raise ``RuntimeError``.
"""

from __future__ import annotations

import functools
from typing import List, Optional, Tuple

import torch

from aimet_amd import _lib
from aimet_amd._lib import HipLibraryError
from aimet_amd.quantization._utils import interleave, concretize_block_size, _is_expandable

__all__ = ["quantize", "dequantize", "quantize_dequantize"]

_MANTISSA_BITS = {torch.float32: 23, torch.float16: 10, torch.bfloat16: 7, torch.float64: 52}


# ------------------------------------------------------------------------------------------------- dtype guards --
def _is_value_representable(dtype: torch.dtype, value: int) -> bool:
    """Whether the integer ``value`` is exact in ``dtype`` (torch_builtins.py:49-83)."""
    if dtype not in _MANTISSA_BITS:
        raise ValueError(f"Expected dtype to be one of float32, float16, bfloat16, or float64; got {dtype}")
    finfo = torch.finfo(dtype)
    if not finfo.min <= value <= finfo.max:
        return False
    msb = max(0, value.bit_length() - 1)
    lsb = max(0, (value & -value).bit_length() - 1)
    return msb - lsb <= _MANTISSA_BITS[dtype]


@functools.lru_cache(None)
def _is_grid_representable(dtype: torch.dtype, qmin: int, qmax: int) -> bool:
    """torch_builtins.py:86-96"""
    return all(_is_value_representable(dtype, v) for v in (qmax, qmax - 1, qmin + 1, qmin))


@functools.lru_cache(None)
def _is_numerically_stable(dtype: torch.dtype, qmin: int, qmax: int) -> bool:
    """torch_builtins.py:99-116"""
    if not _is_grid_representable(dtype, qmin, qmax):
        return False
    if qmin == qmax:
        return True
    return not torch.finfo(dtype).eps > 0.25 / (qmax - qmin)


def _internal_dtype(dtype: torch.dtype, qmin: int, qmax: int) -> torch.dtype:
    if _is_numerically_stable(dtype, qmin, qmax):
        return dtype
    if _is_numerically_stable(torch.float32, qmin, qmax):
        return torch.float32
    return torch.float64


def _validate_arguments(tensor, scale, qmin=None, qmax=None, block_size=None):
    """Same checks and messages as torch_builtins.py:119-162."""
    if block_size is not None:
        if len(scale.shape) != len(block_size):
            raise RuntimeError(f"Length of scale shape {scale.shape} must equal length of block size {block_size}")
        for i in range(1, len(block_size) + 1):
            if block_size[-i] == -1:
                if tensor.shape[-i] % scale.shape[-i] != 0:
                    raise RuntimeError(
                        f"Each tensor dimension size for tensor shape {tensor.shape} must divide "
                        f"evenly with corresponding scale dimension value for scale shape {scale.shape}"
                    )
            elif block_size[-i] * scale.shape[-i] != tensor.shape[-i]:
                raise RuntimeError(
                    f"Each tensor dimension size for tensor shape {tensor.shape} must equal the "
                    f"corresponding scale dimension size * block size for scale shape {scale.shape} "
                    f"and block size {block_size}"
                )
    elif not _is_expandable(scale.shape, tensor.shape):
        msg = f"Scale of shape {scale.shape} cannot be expanded like input tensor of shape {tensor.shape}. "
        if tensor.numel() == 0:
            msg += (
                "Detected that the tensor is empty, which may be caused by the following reasons: "
                "1. The input tensor is incorrect. "
                "2. Improper use of model inference without initializing DeepSpeed after offloading parameters."
            )
        raise RuntimeError(msg)
    if qmin is not None and qmax is not None and qmin > qmax:
        raise RuntimeError(f"qmin ({qmin}) must be smaller than or equal to qmax ({qmax})")


def _check_devices(tensor, scale, offset):
    _lib.require_device(tensor, "input tensor")
    if scale.device != tensor.device or offset.device != tensor.device:
        raise RuntimeError(
            f"Expected all tensors to be on the same device, but found input on {tensor.device}, "
            f"scale on {scale.device} and offset on {offset.device}"
        )
    if tensor.dtype not in _lib.DTYPE_CODE:
        raise HipLibraryError(f"the HIP backend handles float32, float16 and bfloat16 tensors; got {tensor.dtype}")


# ------------------------------------------------------------------------------------------------------ layout --
def _dense_order(t: torch.Tensor) -> Optional[Tuple[int, ...]]:
    """Dimension order (outermost first) in which ``t`` is dense in memory, or None if it is not dense."""
    if t.is_contiguous():
        return tuple(range(t.dim()))
    order = sorted(range(t.dim()), key=lambda d: (-t.stride(d), d))
    expect = 1
    for d in reversed(order):
        if t.shape[d] != 1 and t.stride(d) != expect:
            return None
        expect *= t.shape[d]
    return tuple(order)


@functools.lru_cache(maxsize=4096)
def _build_layout(shape: Tuple[int, ...], order: Tuple[int, ...], enc_shape: Tuple[int, ...],
                  block_size: Optional[Tuple[int, ...]]):
    """ahq_layout of a tensor whose memory order is ``order`` and whose encodings have shape ``enc_shape``."""
    nd = len(shape)
    block = [shape[d] if shape[d] > 0 else 1 for d in range(nd)]
    stride = [0] * nd
    lead = nd - len(enc_shape)
    if block_size is not None:
        bs = concretize_block_size(shape, enc_shape, block_size)
    else:
        bs = tuple(1 if e > 1 else (shape[lead + k] or 1) for k, e in enumerate(enc_shape))
    run = 1
    enc_strides = []
    for e in reversed(enc_shape):
        enc_strides.append(run)
        run *= e
    enc_strides.reverse()
    for k, e in enumerate(enc_shape):
        d = lead + k
        if e > 1:
            block[d] = bs[k]
            stride[d] = enc_strides[k]
    dims = [shape[d] for d in order]
    return _lib.make_layout(dims, [block[d] for d in order], [stride[d] for d in order])


def _prepare(tensor: torch.Tensor, enc_shape, block_size):
    """Returns (tensor dense in memory, layout)."""
    order = _dense_order(tensor)
    if order is None:
        tensor = tensor.contiguous()
        order = tuple(range(tensor.dim()))
    bs = tuple(block_size) if block_size else None
    return tensor, _build_layout(tuple(tensor.shape), order, tuple(enc_shape), bs)


def _enc_f32(t: torch.Tensor) -> torch.Tensor:
    t = t.detach()
    if t.dtype != torch.float32:
        t = t.to(torch.float32)
    return t.contiguous()


def _like(ref: torch.Tensor, t: torch.Tensor) -> torch.Tensor:
    """``t`` with the memory layout of ``ref`` (same shape)."""
    if t.stride() == ref.stride() and t.dtype == ref.dtype:
        return t
    out = torch.empty_like(ref)
    out.copy_(t)
    return out


@functools.lru_cache(maxsize=1024)
def _grid(arith, op, io_dtype, compute_dtype, qmin, qmax, zps) -> _lib.Grid:
    """The ahq_grid of a call; shared between calls with the same arguments, so nobody writes into it."""
    g = _lib.Grid()
    g.arith = arith
    g.op = op
    g.io_dtype = _lib.DTYPE_CODE[io_dtype]
    g.compute_dtype = _lib.DTYPE_CODE[compute_dtype]
    g.qmin = qmin
    g.qmax = qmax
    g.zero_point_shift = zps
    return g


_WORKSPACES = {}  # (device, stream, bytes) -> tensor
_BACKWARD_BYTES = {}  # (id(grid), id(layout), parameter gradients wanted) -> (grid, layout, bytes)


def _workspace(nbytes: int, device) -> Optional[torch.Tensor]:
    """Scratch of ``nbytes`` for a launch on the current stream of ``device``.  The library neither expects anything
    in a workspace nor leaves anything there for a later call, and launches on one stream run in order, so one buffer
    per (device, stream, size) serves every call (a step of a training loop asks for the same size again and
    again); a handful of sizes are kept."""
    if nbytes == 0:
        return None
    key = (device, _lib.current_stream(device), nbytes)
    ws = _WORKSPACES.get(key)
    if ws is None:
        if len(_WORKSPACES) >= 64:
            _WORKSPACES.clear()
        ws = _WORKSPACES[key] = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return ws


def _backward_workspace_bytes(grid, layout, want_pg: bool) -> int:
    """ahq_qdq_backward_workspace_bytes, asked once per (grid, layout): both objects come out of caches and live on."""
    key = (id(grid), id(layout), want_pg)
    held = _BACKWARD_BYTES.get(key)
    if held is None or held[0] is not grid or held[1] is not layout:
        if len(_BACKWARD_BYTES) >= 4096:
            _BACKWARD_BYTES.clear()
        held = _BACKWARD_BYTES[key] = (grid, layout,
                                       _lib.load().ahq_qdq_backward_workspace_bytes(grid, layout, 1 if want_pg else 0))
    return held[2]


def _launch_forward(tensor, scale, offset, arith, op, compute_dtype, qmin, qmax, block_size, zps):
    lib = _lib.load()
    x, layout = _prepare(tensor.detach(), scale.shape, block_size)
    s = _enc_f32(scale)
    o = _enc_f32(offset)
    grid = _grid(arith, op, x.dtype, compute_dtype, qmin, qmax, zps)
    y = torch.empty_like(x)
    if x.numel():
        _lib.check(
            lib.ahq_qdq_forward(grid, layout, x.data_ptr(), y.data_ptr(), None, s.data_ptr(), o.data_ptr(),
                                None, None, _lib.current_stream(x.device)),
            "ahq_qdq_forward",
        )
    return y, x, s, o, grid, layout


# ---------------------------------------------------------------------------------------------- autograd function --
class _HipAffineFunction(torch.autograd.Function):
    """One fused kernel forward, one fused kernel backward (input, scale and offset gradients together)."""

    @staticmethod
    def forward(ctx, tensor, scale, offset, arith, op, compute_dtype, qmin, qmax, block_size, zps):
        y, x, s, o, grid, layout = _launch_forward(tensor, scale, offset, arith, op, compute_dtype, qmin, qmax,
                                                   block_size, zps)
        ctx.grid = grid
        ctx.layout = layout
        ctx.save_for_backward(x, s, o)
        ctx.enc_shapes = (scale.shape, offset.shape, scale.dtype, offset.dtype)
        return y

    @staticmethod
    def backward(ctx, grad):
        x, s, o = ctx.saved_tensors
        need_x, need_s, need_o = ctx.needs_input_grad[:3]
        none7 = (None,) * 7
        if not (need_x or need_s or need_o):
            return (None, None, None) + none7
        want_pg = (need_s or need_o) and ctx.grid.arith == _lib.AHQ_ARITH_AUTOGRAD
        gx, gs, go = _launch_backward(ctx.grid, ctx.layout, x, s, o, grad, need_x, want_pg)
        s_shape, o_shape, s_dtype, o_dtype = ctx.enc_shapes
        gs_out = gs.view(s_shape).to(s_dtype) if (need_s and want_pg) else None
        go_out = go.view(o_shape).to(o_dtype) if (need_o and want_pg) else None
        return (gx, gs_out, go_out) + none7


def _launch_backward(grid, layout, x, s, o, grad, need_x: bool, want_pg: bool):
    """One launch for the input gradient and (``want_pg``) the float32 gradients of scale and offset; x, s, o as
    _launch_forward returned them."""
    lib = _lib.load()
    g = _like(x, grad)
    gx = torch.empty_like(x) if need_x else None
    gs = go = None
    if want_pg:
        gs, go = torch.empty((2,) + tuple(s.shape), dtype=torch.float32, device=x.device).unbind(0)
    if x.numel() == 0:
        if want_pg:
            gs.zero_()
            go.zero_()
    else:
        nbytes = _backward_workspace_bytes(grid, layout, want_pg)
        ws = _workspace(nbytes, x.device)
        _lib.check(
            lib.ahq_qdq_backward(grid, layout, g.data_ptr(), x.data_ptr(), _lib.ptr(gx), _lib.ptr(gs),
                                 _lib.ptr(go), s.data_ptr(), o.data_ptr(), _lib.ptr(ws), nbytes,
                                 _lib.current_stream(x.device)),
            "ahq_qdq_backward",
        )
    return gx, gs, go


def _broadcast_encodings(scale: torch.Tensor, offset: torch.Tensor, block_size):
    """Scale and offset expanded to one common shape, the way the reference's elementwise arithmetic broadcasts them
    against each other (torch_builtins.py:727-773: ``tensor / scale - offset``).  The kernels index both arrays with
    the same encoding index, so a scalar offset next to a per-channel scale has to be materialised; ``expand`` is
    differentiable, so autograd sums the gradient back to the operand's own shape."""
    if offset.shape == scale.shape:
        return scale, offset
    try:
        shape = torch.broadcast_shapes(scale.shape, offset.shape)
    except RuntimeError as e:
        raise RuntimeError(
            f"Offset of shape {tuple(offset.shape)} cannot be broadcast with scale of shape {tuple(scale.shape)}"
        ) from e
    if block_size is not None and len(shape) != len(scale.shape):
        raise RuntimeError(
            f"Offset of shape {tuple(offset.shape)} has more dimensions than scale of shape {tuple(scale.shape)}, "
            f"which block size {tuple(block_size)} describes"
        )
    if block_size is not None and tuple(shape) != tuple(scale.shape):
        raise RuntimeError(
            f"Offset of shape {tuple(offset.shape)} cannot be expanded to scale of shape {tuple(scale.shape)}"
        )
    return scale.expand(shape), offset.expand(shape)


def _apply(tensor, scale, offset, arith, op, compute_dtype, qmin, qmax, block_size, zps):
    bs = tuple(block_size) if block_size else None
    if offset.shape != scale.shape:
        scale, offset = _broadcast_encodings(scale, offset, bs)
        if bs is None and not _is_expandable(scale.shape, tensor.shape):
            raise RuntimeError(
                f"Encodings of shape {tuple(scale.shape)} cannot be expanded like input tensor of shape "
                f"{tuple(tensor.shape)}"
            )
    if not torch.is_grad_enabled() or not (tensor.requires_grad or scale.requires_grad or offset.requires_grad):
        # nothing to differentiate: skip the autograd bookkeeping (a whole-model forward makes hundreds of these calls)
        return _launch_forward(tensor, scale, offset, arith, op, compute_dtype, qmin, qmax, bs, zps)[0]
    return _HipAffineFunction.apply(tensor, scale, offset, arith, op, compute_dtype, qmin, qmax, bs, zps)


# --------------------------------------------------------------------------------------- ATen-arithmetic decision --
def _offsets_fit_grid(offset: torch.Tensor, qmin: int, qmax: int) -> bool:
    """ATen's per-channel fake-quantize refuses zero points outside [qmin, qmax]; the reference then leaves the fast
    path (torch_builtins.py:425-429).  Quantizer-made offsets say so themselves -- symmetric ones carry their constant
    value, those derived from a min / max pair the grid they were clamped into -- so that this needs no device read
    (a read is a synchronisation: 78 instead of 43 us for a no-grad forward over 134 MB)."""
    const = getattr(offset, "_ahq_constant", None)
    if const is not None:
        return qmin <= -int(const) <= qmax
    if getattr(offset, "_ahq_in_grid", None) == (qmin, qmax):
        return True  # derived from a min / max pair by a formula that ends in clamp(., -qmax, -qmin)
    # the answer is kept on the tensor object, for the version of its contents that was read (like autograd, this
    # follows writes torch knows of; a write through .data or by a foreign kernel into the same memory is not seen)
    key = (offset._version, offset.data_ptr(), qmin, qmax)  # pylint: disable=protected-access
    held = getattr(offset, "_ahq_fit_checked", None)
    if held is not None and held[0] == key:
        return held[1]
    zp = -offset.detach().to(torch.int32)
    fits = bool(((zp >= qmin) & (zp <= qmax)).all())
    try:
        offset._ahq_fit_checked = (key, fits)  # pylint: disable=protected-access
    except (AttributeError, RuntimeError):
        pass
    return fits


def _aten_arithmetic_applies(tensor, scale, offset, qmin, qmax) -> bool:
    """Mirror of `_torch_fake_quantize` (torch_builtins.py:335-431): per-tensor, or per-channel on exactly one axis."""
    if scale.numel() == 1 and offset.numel() == 1:
        return True
    sshape = (1,) * (tensor.dim() - scale.dim()) + tuple(scale.shape)
    oshape = (1,) * (tensor.dim() - offset.dim()) + tuple(offset.shape)
    if sshape != oshape:
        return False
    if not all(sd in (1, td) for sd, td in zip(sshape, tensor.shape)):
        return False
    if sum(1 for sd in sshape if sd != 1) != 1:
        return False
    return _offsets_fit_grid(offset, qmin, qmax)


# ------------------------------------------------------------------------------------------------- public entry --
def quantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int, qmax: int,
             block_size: Optional[List] = None) -> torch.Tensor:
    """clamp(round(tensor / scale) - offset, qmin, qmax), differentiable (torch_builtins.py:166-212)."""
    _validate_arguments(tensor, scale, qmin, qmax, block_size)
    _check_devices(tensor, scale, offset)
    if not _is_grid_representable(tensor.dtype, qmin, qmax):
        raise RuntimeError(f"{tensor.dtype} is unable to represent quantized output of range [{qmin}, {qmax}].")
    cd = _internal_dtype(tensor.dtype, qmin, qmax)
    if cd == torch.float64:
        raise HipLibraryError(f"a grid of [{qmin}, {qmax}] needs float64 arithmetic, which the HIP backend does not have")
    return _apply(tensor, scale, offset, _lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QUANTIZE, cd, qmin, qmax, block_size, 0.0)


def quantize_dequantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int, qmax: int,
                        block_size: Optional[List] = None, zero_point_shift: float = 0.0) -> torch.Tensor:
    """(clamp(round(tensor / scale) - offset, qmin, qmax) + offset) * scale, differentiable
    (torch_builtins.py:216-302)."""
    _validate_arguments(tensor, scale, qmin, qmax, block_size)
    _check_devices(tensor, scale, offset)
    zero_point_shift = zero_point_shift or 0.0

    fast = (
        block_size is None
        and (not scale.requires_grad and not offset.requires_grad or not torch.is_grad_enabled())
        and zero_point_shift == 0.0
        and _aten_arithmetic_applies(tensor, scale, offset, qmin, qmax)
    )
    if fast:
        return _apply(tensor, scale, offset, _lib.AHQ_ARITH_ATEN, _lib.AHQ_OP_QDQ, torch.float32, qmin, qmax, None, 0.0)

    cd = _internal_dtype(tensor.dtype, qmin, qmax)
    if cd == torch.float64:
        raise HipLibraryError(f"a grid of [{qmin}, {qmax}] needs float64 arithmetic, which the HIP backend does not have")
    if not _is_grid_representable(cd, qmin, qmax):
        raise RuntimeError(f"{cd} is unable to represent quantized output of range [{qmin}, {qmax}].")
    return _apply(tensor, scale, offset, _lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QDQ, cd, qmin, qmax, block_size,
                  float(zero_point_shift))


def dequantize(tensor: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor,
               block_size: Optional[List] = None) -> torch.Tensor:
    """(tensor + offset) * scale, differentiable (torch_builtins.py:537-571)."""
    _validate_arguments(tensor, scale, block_size=block_size)
    _check_devices(tensor, scale, offset)
    return _apply(tensor, scale, offset, _lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_DEQUANTIZE, tensor.dtype, 0, 0,
                  block_size, 0.0)
