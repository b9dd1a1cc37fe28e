"""Thin Python wrappers over the statistics entry points of libaimet_amd.so."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from aimet_amd import _lib
from aimet_amd._lib import HipLibraryError
from aimet_amd.quantization._utils import _is_expandable
from aimet_amd.quantization.affine.backends.hip import _prepare


def _check_reducible(x: torch.Tensor, shape: Tuple[int, ...], block_size) -> None:
    if block_size is not None:
        if len(block_size) != len(shape):
            raise RuntimeError(f"Length of shape {shape} must equal length of block size {block_size}")
        if x.dim() < len(shape):
            raise RuntimeError(f"Input of shape {list(x.shape)} can't be reduced to shape {list(shape)}")
        for i in range(1, len(shape) + 1):
            b, s, d = block_size[-i], shape[-i], x.shape[-i]
            ok = (d % s == 0) if b == -1 else (b * s == d)
            if not ok:
                raise RuntimeError(f"Input of shape {list(x.shape)} can't be reduced to shape {list(shape)}")
    elif not _is_expandable(shape, x.shape):
        raise RuntimeError(f"Input of shape {list(x.shape)} can't be reduced to shape {list(shape)}")


def reduce_min_max(x: torch.Tensor, shape: Tuple[int, ...], block_size=None, *, finite_only: bool = False,
                   running: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                   copy_to: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-encoding minimum and maximum of ``x`` in one pass (both extrema from a single read of the tensor).

    Equivalent of ``reduce(x, shape, torch.amin, block_size)`` and ``reduce(x, shape, torch.amax, block_size)``
    (aimet_torch/utils.py:1115-1148, aimet_torch/quantization/encoding_analyzer.py:80-94).  The batch result is
    returned; with ``running`` it is also folded into the given (min, max) tensors in place, as
    ``_MinMaxObserver.merge_stats`` does.  ``copy_to``: a contiguous tensor of ``x``'s shape and dtype that receives a
    copy of ``x`` from the same pass (``ahq_minmax_copy``).
    """
    _lib.require_device(x, "input tensor")
    if x.dtype not in _lib.DTYPE_CODE:
        raise HipLibraryError(f"min/max statistics support float32, float16 and bfloat16; got {x.dtype}")
    shape = tuple(shape)
    _check_reducible(x, shape, block_size)
    if x.numel() == 0:
        raise RuntimeError("cannot reduce an empty tensor")
    lib = _lib.load()
    xd, layout = _prepare(x.detach(), shape, block_size)
    rmn = rmx = None
    if running is not None:
        rmn, rmx = running
        for r in (rmn, rmx):
            if r.dtype != x.dtype or not r.is_contiguous() or tuple(r.shape) != shape or r.device != x.device:
                raise RuntimeError("running statistics must be contiguous tensors of the observer shape, on the "
                                   "input's device and of its dtype")
    mn = torch.empty(shape, dtype=x.dtype, device=x.device)
    mx = torch.empty(shape, dtype=x.dtype, device=x.device)
    nbytes = lib.ahq_minmax_workspace_bytes(layout)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device) if nbytes else None
    if copy_to is not None:
        if (copy_to.dtype != x.dtype or copy_to.device != x.device or copy_to.shape != x.shape
                or not copy_to.is_contiguous()):
            raise RuntimeError("copy_to must be a contiguous tensor of the input's shape, dtype and device")
        _lib.check(
            lib.ahq_minmax_copy(_lib.DTYPE_CODE[x.dtype], layout, xd.data_ptr(), copy_to.data_ptr(), mn.data_ptr(),
                                mx.data_ptr(), _lib.ptr(rmn), _lib.ptr(rmx), 1 if finite_only else 0, _lib.ptr(ws),
                                nbytes, _lib.current_stream(x.device)),
            "ahq_minmax_copy",
        )
        return mn, mx
    _lib.check(
        lib.ahq_minmax(_lib.DTYPE_CODE[x.dtype], layout, xd.data_ptr(), mn.data_ptr(), mx.data_ptr(),
                       _lib.ptr(rmn), _lib.ptr(rmx), 1 if finite_only else 0, _lib.ptr(ws), nbytes,
                       _lib.current_stream(x.device)),
        "ahq_minmax",
    )
    return mn, mx
