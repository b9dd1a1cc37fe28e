"""Shape helpers and small utilities shared by the backend, the quantizers and the analyzers.

Behavioural counterparts in the reference: aimet_torch/quantization/_utils.py:11-62 (interleave,
concretize_block_size), aimet_torch/utils.py:1094-1113 (_is_expandable), :1176-1254 (patch_attr, ste_round),
_aimet_common/quantsim.py:538-559 (_get_minimum_scale).
"""

from __future__ import annotations

import functools
from typing import Any, Callable, Sequence, Tuple

import torch


class StatisticsNotFoundError(RuntimeError):
    """compute_encodings() was asked for encodings before any statistics were observed."""


def interleave(first, second) -> Tuple[int, ...]:
    """(a0, b0, a1, b1, ...); an int argument is repeated to the other's length."""
    if isinstance(first, int) and isinstance(second, int):
        raise ValueError("At least one of the inputs must be a sequence.")
    if isinstance(first, int):
        first = (first,) * len(second)
    if isinstance(second, int):
        second = (second,) * len(first)
    if len(first) != len(second):
        raise ValueError("Both sequences must have the same length to interleave.")
    out = []
    for a, b in zip(first, second):
        out += [a, b]
    return tuple(out)


def concretize_block_size(input_shape: Sequence[int], scale_shape: Sequence[int],
                          block_size: Sequence[int]) -> Tuple[int, ...]:
    """Resolve -1 wildcards and pad missing leading entries so that there is one block size per scale dimension."""
    if len(input_shape) < len(scale_shape):
        raise ValueError(
            f"Input shape {input_shape} must have at least as many dimensions as scale shape {scale_shape}."
        )
    if len(scale_shape) < len(block_size):
        raise ValueError(
            f"Scale shape {scale_shape} must have at least as many dimensions as block size {block_size}."
        )
    n = len(scale_shape)
    trailing = tuple(input_shape)[len(input_shape) - n:] if n else ()
    missing = n - len(block_size)
    padded = [1 if scale_shape[i] > 1 else -1 for i in range(missing)] + list(block_size)
    return tuple(padded[i] if padded[i] != -1 else trailing[i] // scale_shape[i] for i in range(n))


def _is_expandable(src_shape: Sequence[int], target_shape: Sequence[int]) -> bool:
    """True if a tensor of ``src_shape`` broadcasts to ``target_shape``."""
    if len(src_shape) > len(target_shape):
        return False
    return all(s in (1, t) for s, t in zip(reversed(tuple(src_shape)), reversed(tuple(target_shape))))


@functools.lru_cache(None)
def _get_minimum_scale(num_steps: int) -> float:
    """Largest s <= float32 eps whose grid of ``num_steps`` steps stays inside [-0.005, 0.005]."""
    return min(float(torch.finfo(torch.float32).eps), 0.01 / num_steps)


class _ContextManager:
    """Runs ``action`` on entry and ``cleanup`` on exit; also usable as a decorator."""

    def __init__(self, action: Callable[[], Any], cleanup: Callable[[], Any]):
        self._action = action
        self._cleanup = cleanup

    def __enter__(self):
        self._action()
        return self

    def __exit__(self, *_):
        self._cleanup()

    def __call__(self, fn: Callable):
        @functools.wraps(fn)
        def wrapped(*args, **kwargs):
            with self:
                return fn(*args, **kwargs)

        return wrapped


_MISSING = object()


def patch_attr(obj, name: str, value) -> _ContextManager:
    """Temporarily replace ``obj.name`` (parameters and buffers of a module are swapped inside their containers)."""
    if isinstance(obj, torch.nn.Module):
        for container in (obj._parameters, obj._buffers):  # pylint: disable=protected-access
            if name in container:
                saved = container[name]
                return _ContextManager(lambda c=container: c.update({name: value}),
                                       lambda c=container: c.update({name: saved}))

    saved = getattr(obj, name, _MISSING)

    def restore():
        try:
            delattr(obj, name)
        except AttributeError:
            pass
        if saved is not _MISSING and not hasattr(obj, name):
            setattr(obj, name, saved)

    return _ContextManager(lambda: setattr(obj, name, value), restore)


class _RoundSTE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):  # pylint: disable=arguments-differ
        return torch.round(x)

    @staticmethod
    def backward(ctx, grad):  # pylint: disable=arguments-differ
        return grad


def ste_round(x: torch.Tensor) -> torch.Tensor:
    """round() whose gradient is the identity."""
    return _RoundSTE.apply(x)


def true_divide(t: torch.Tensor, value: float) -> torch.Tensor:
    """``t / value`` with IEEE division on any device.

    Dividing a GPU tensor by a Python number is evaluated by torch as a multiplication with the reciprocal, which is
    one unit in the last place off for some operands; dividing by a 0-dim device tensor is a true division.  16-bit
    tensors are divided in float32 and rounded once, which is what the CPU path does for ``tensor / number``.
    """
    divisor = torch.full((), float(value), dtype=torch.float32, device=t.device)
    if t.dtype == torch.float32:
        return t / divisor
    return (t.to(torch.float32) / divisor).to(t.dtype)
