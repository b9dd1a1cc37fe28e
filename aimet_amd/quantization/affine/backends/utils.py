"""Backend registry: the plug-in boundary of the affine quantization functions.

Same contract as aimet_torch/quantization/affine/backends/utils.py:16-114: a backend is any object with
``quantize``, ``dequantize`` and ``quantize_dequantize``; ``set_backend`` switches globally and, used as a context
manager, switches back on exit; ``add_backend`` registers a new one.  The only built-in backend here is ``"hip"``.
"""

from __future__ import annotations

from typing import List, Optional, Protocol

import torch

from aimet_amd.quantization._utils import _ContextManager
from aimet_amd.quantization.affine.backends import hip


class _QuantizationBackendProtocol(Protocol):
    def quantize(self, input: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int, qmax: int,
                 block_size: Optional[List] = None) -> torch.Tensor: ...

    def dequantize(self, input: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor,
                   block_size: Optional[List] = None) -> torch.Tensor: ...

    def quantize_dequantize(self, input: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int,
                            qmax: int, block_size: Optional[List] = None,
                            zero_point_shift: float = 0.0) -> torch.Tensor: ...


_CURRENT_BACKEND = "hip"
_SUPPORTED_BACKENDS = {"hip": hip}


def set_backend(name: str) -> _ContextManager:
    """Select the backend used by quantize / dequantize / quantize_dequantize.  ``with set_backend(name): ...``
    restores the previous backend on exit."""
    global _CURRENT_BACKEND  # pylint: disable=global-statement
    if name not in _SUPPORTED_BACKENDS:
        raise RuntimeError(
            f"Backend '{name}' is not supported. Please choose one of: {', '.join(_SUPPORTED_BACKENDS)}"
        )
    previous = _CURRENT_BACKEND
    _CURRENT_BACKEND = name

    def restore():
        global _CURRENT_BACKEND  # pylint: disable=global-statement
        _CURRENT_BACKEND = previous

    return _ContextManager(action=lambda: None, cleanup=restore)


def get_backend() -> _QuantizationBackendProtocol:
    return _SUPPORTED_BACKENDS[_CURRENT_BACKEND]


def add_backend(name: str, module: _QuantizationBackendProtocol):
    """Register ``module`` under ``name``.  An existing name is left untouched and an error object is returned
    (not raised), as the reference does (backends/utils.py:110-114)."""
    if name in _SUPPORTED_BACKENDS:
        return RuntimeError(f"Backend {name} already exists.")
    _SUPPORTED_BACKENDS[name] = module
    return None


__all__ = ["set_backend", "get_backend", "add_backend"]
