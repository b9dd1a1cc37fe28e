"""ctypes binding of libaimet_amd.so (the C ABI declared in include/aimet_amd.h).

The library is the only compute path of this package: if it is missing, or a tensor does not live on a HIP device,
the callers raise -- there is no CPU or eager-PyTorch fallback.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence

import torch

AHQ_MAX_DIMS = 8

AHQ_OK, AHQ_ERR_INVALID, AHQ_ERR_UNSUPPORTED, AHQ_ERR_LAUNCH, AHQ_ERR_WORKSPACE = 0, 1, 2, 3, 4
AHQ_F32, AHQ_F16, AHQ_BF16 = 0, 1, 2
AHQ_ARITH_ATEN, AHQ_ARITH_AUTOGRAD, AHQ_ARITH_DLQ = 1, 2, 3
AHQ_OP_QDQ, AHQ_OP_QUANTIZE, AHQ_OP_DEQUANTIZE = 0, 1, 2

DTYPE_CODE = {torch.float32: AHQ_F32, torch.float16: AHQ_F16, torch.bfloat16: AHQ_BF16}

MINMAX_SLOTS_BYTES = 12 * 512  # AHQ_MINMAX_SLOTS_BYTES
LIB_NAME = "libaimet_amd.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)


class Layout(ctypes.Structure):
    _fields_ = [
        ("ndim", ctypes.c_int32),
        ("dims", ctypes.c_int64 * AHQ_MAX_DIMS),
        ("block", ctypes.c_int64 * AHQ_MAX_DIMS),
        ("enc_stride", ctypes.c_int64 * AHQ_MAX_DIMS),
    ]


class Grid(ctypes.Structure):
    _fields_ = [
        ("arith", ctypes.c_int32),
        ("op", ctypes.c_int32),
        ("io_dtype", ctypes.c_int32),
        ("compute_dtype", ctypes.c_int32),
        ("qmin", ctypes.c_int64),
        ("qmax", ctypes.c_int64),
        ("zero_point_shift", ctypes.c_double),
    ]


class HistState(ctypes.Structure):
    _fields_ = [
        ("num_slots", ctypes.c_int32),
        ("num_bins", ctypes.c_int32),
        ("growth_limit", ctypes.c_float),
        ("hist", ctypes.c_void_p),
        ("edges", ctypes.c_void_p),
        ("minmax", ctypes.c_void_p),
        ("limits", ctypes.c_void_p),
        ("new_hist", ctypes.c_void_p),
        ("new_edges", ctypes.c_void_p),
        ("new_minmax", ctypes.c_void_p),
    ]


class SqnrParams(ctypes.Structure):
    _fields_ = [
        ("num_slots", ctypes.c_int32),
        ("num_bins", ctypes.c_int32),
        ("num_deltas", ctypes.c_int32),
        ("num_offsets", ctypes.c_int32),
        ("symmetric", ctypes.c_int32),
        ("stat_dtype", ctypes.c_int32),
        ("num_steps", ctypes.c_int64),
        ("minimum_scale", ctypes.c_double),
        ("gamma", ctypes.c_double),
        ("p", ctypes.c_double),
    ]


class DlqPdfState(ctypes.Structure):
    """ahq_dlq_pdf_state"""

    _fields_ = [
        ("num_slots", ctypes.c_int32),
        ("xleft", ctypes.c_void_p),
        ("pdf", ctypes.c_void_p),
        ("meta", ctypes.c_void_p),
    ]


class GridProbeItem(ctypes.Structure):
    """ahq_grid_probe_item"""

    _fields_ = [("dtype", ctypes.c_int32), ("layout", Layout), ("x", ctypes.c_void_p), ("num_levels", ctypes.c_int64)]


class CalibrateQdqItem(ctypes.Structure):
    """ahq_calibrate_qdq_item"""

    _fields_ = [
        ("grid", Grid), ("layout", Layout), ("x", ctypes.c_void_p), ("y", ctypes.c_void_p),
        ("num_steps", ctypes.c_int64), ("symmetric", ctypes.c_int32),
        ("minimum_scale_in_dtype", ctypes.c_float), ("minimum_scale", ctypes.c_float), ("dtype_max", ctypes.c_float),
        ("near_max_threshold", ctypes.c_float), ("param_dtype", ctypes.c_int32),
        ("param_min", ctypes.c_void_p), ("param_max", ctypes.c_void_p), ("grid_minimum_scale", ctypes.c_double),
        ("scale", ctypes.c_void_p), ("offset", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
    ]


class SlotsFinalizeItem(ctypes.Structure):
    """ahq_slots_finalize_item"""

    _fields_ = [
        ("stat_dtype", ctypes.c_int32), ("symmetric", ctypes.c_int32), ("slots", ctypes.c_void_p),
        ("num_steps", ctypes.c_int64),
        ("minimum_scale_in_dtype", ctypes.c_float), ("minimum_scale", ctypes.c_float), ("dtype_max", ctypes.c_float),
        ("near_max_threshold", ctypes.c_float), ("param_dtype", ctypes.c_int32), ("reserved", ctypes.c_int32),
        ("param_min", ctypes.c_void_p), ("param_max", ctypes.c_void_p), ("qmin", ctypes.c_int64), ("qmax", ctypes.c_int64),
        ("grid_minimum_scale", ctypes.c_double), ("scale", ctypes.c_void_p), ("offset", ctypes.c_void_p),
    ]


DLQ_PDF_SIZE = 1536


class HipLibraryError(RuntimeError):
    """Raised when libaimet_amd.so is missing or one of its entry points reports an error."""


_lib: Optional[ctypes.CDLL] = None

# name -> (restype, argtypes); every symbol include/aimet_amd.h declares
_P = ctypes.c_void_p
_SIGNATURES = {
    "ahq_last_error": (ctypes.c_char_p, []),
    "ahq_version": (ctypes.c_int, []),
    "ahq_qdq_forward": (ctypes.c_int, [ctypes.POINTER(Grid), ctypes.POINTER(Layout), _P, _P, _P, _P, _P, _P, _P, _P]),
    "ahq_qdq_backward_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(Grid), ctypes.POINTER(Layout), ctypes.c_int]),
    "ahq_qdq_backward": (ctypes.c_int, [ctypes.POINTER(Grid), ctypes.POINTER(Layout), _P, _P, _P, _P, _P, _P, _P, _P,
                                        ctypes.c_size_t, _P]),
    "ahq_minmax_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(Layout)]),
    "ahq_minmax": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, _P, _P, ctypes.c_int, _P,
                                  ctypes.c_size_t, _P]),
    "ahq_minmax_copy": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, _P, _P, _P, ctypes.c_int, _P,
                                       ctypes.c_size_t, _P]),
    "ahq_minmax_static": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, _P, _P, ctypes.c_int, _P]),
    "ahq_minmax_to_encodings": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32,
                                               ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, _P, _P, _P,
                                               _P]),
    "ahq_lpbq_scale_backward": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, ctypes.c_int64,
                                               ctypes.c_int64, ctypes.c_double, ctypes.c_int32, _P, _P, _P, _P, _P]),
    "ahq_range_backward": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                          ctypes.c_double, _P, _P, _P, _P, _P]),
    "ahq_minmax_accumulate": (ctypes.c_int, [ctypes.c_int32, _P, ctypes.c_int64, _P, _P, _P, ctypes.c_int32, _P]),
    "ahq_minmax_slots_to_encodings": (ctypes.c_int, [ctypes.c_int32, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_float,
                                                     ctypes.c_float, ctypes.c_float, ctypes.c_float, _P, _P, _P, _P, _P,
                                                     _P]),
    "ahq_minmax_slots_read": (ctypes.c_int, [ctypes.c_int32, _P, _P, _P, _P]),
    "ahq_minmax_finalize": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32,
                                           ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, _P,
                                           ctypes.c_int32, _P, _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_double, _P,
                                           _P, _P]),
    "ahq_minmax_slots_finalize": (ctypes.c_int, [ctypes.c_int32, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_float,
                                                 ctypes.c_float, ctypes.c_float, ctypes.c_float, _P, ctypes.c_int32, _P,
                                                 _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_double, _P, _P, _P]),
    "ahq_minmax_calibrate_qdq_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32, ctypes.POINTER(Layout)]),
    "ahq_minmax_calibrate_qdq": (ctypes.c_int, [ctypes.POINTER(Grid), ctypes.POINTER(Layout), _P, _P, ctypes.c_int64,
                                                ctypes.c_int32, ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                                ctypes.c_float, _P, ctypes.c_int32, _P, _P, ctypes.c_double, _P, _P, _P,
                                                ctypes.c_size_t, _P]),
    "ahq_range_to_scale_offset": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                                 ctypes.c_double, _P, _P, _P]),
    "ahq_lpbq_scale": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, ctypes.c_int64, ctypes.c_int64,
                                      ctypes.c_double, ctypes.c_int32, _P, _P, _P]),
    "ahq_lpbq_qdq_forward": (ctypes.c_int, [ctypes.POINTER(Grid), ctypes.POINTER(Layout), _P, _P, _P, ctypes.c_int32, _P,
                                            _P, ctypes.c_int64, ctypes.c_double, ctypes.c_int32, _P, _P, _P, _P]),
    "ahq_grid_probe": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, ctypes.c_int64, _P, _P]),
    "ahq_grid_probe_many": (ctypes.c_int, [ctypes.POINTER(GridProbeItem), ctypes.c_int64, _P, _P, _P]),
    "ahq_minmax_calibrate_qdq_many": (ctypes.c_int, [ctypes.POINTER(CalibrateQdqItem), ctypes.c_int64, _P, _P]),
    "ahq_minmax_slots_finalize_many": (ctypes.c_int, [ctypes.POINTER(SlotsFinalizeItem), ctypes.c_int64, _P, _P]),
    "ahq_hist_update_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32, ctypes.POINTER(Layout), ctypes.c_int32]),
    "ahq_hist_table_min_numel": (ctypes.c_int64, [ctypes.c_int64]),
    "ahq_hist_update": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, ctypes.POINTER(HistState),
                                       ctypes.c_int, _P, ctypes.c_size_t, _P]),
    "ahq_sqnr_search": (ctypes.c_int, [ctypes.POINTER(SqnrParams), _P, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "ahq_dlq_minmax_encodings": (ctypes.c_int, [_P, _P, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                                ctypes.c_int32, ctypes.c_double, _P, _P]),
    "ahq_dlq_qdq_per_tensor": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_uint64, ctypes.c_double, ctypes.c_double,
                                              ctypes.c_double, ctypes.c_double, _P]),
    "ahq_dlq_fp8_qdq_per_tensor": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_uint64, ctypes.c_double, ctypes.c_int32,
                                                  ctypes.c_int32, ctypes.c_float, _P]),
    "ahq_dlq_minmax_fold": (ctypes.c_int, [ctypes.c_int32, _P, _P, ctypes.c_int64, _P, _P, _P]),
    "ahq_dlq_pdf_update_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32, ctypes.POINTER(Layout)]),
    "ahq_dlq_pdf_update": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, ctypes.POINTER(DlqPdfState),
                                          ctypes.c_int32, _P, _P, ctypes.c_size_t, _P]),
    "ahq_dlq_tfe_encodings_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32]),
    "ahq_dlq_fp8_qdq": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, ctypes.c_int32, ctypes.c_int32,
                                       ctypes.c_float, _P]),
    "ahq_float_cast_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int32, ctypes.POINTER(Layout)]),
    "ahq_float_qdq": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, ctypes.c_int32, ctypes.c_int32,
                                     ctypes.c_float, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, _P, ctypes.c_size_t,
                                     _P]),
    "ahq_float_quantize": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, ctypes.c_int32,
                                          ctypes.c_int32, ctypes.c_float, ctypes.c_int32, ctypes.c_int32,
                                          ctypes.c_int32, _P, ctypes.c_size_t, _P]),
    "ahq_float_dequantize": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, _P]),
    "ahq_float_qdq_backward": (ctypes.c_int, [ctypes.c_int32, ctypes.POINTER(Layout), _P, _P, _P, _P, ctypes.c_int32,
                                              ctypes.c_int32, ctypes.c_float, ctypes.c_int32, ctypes.c_int32, _P]),
    "ahq_diag_read": (ctypes.c_int, [_P, ctypes.c_size_t, ctypes.c_int32, ctypes.c_int32, _P, _P]),
    "ahq_diag_copy": (ctypes.c_int, [_P, _P, ctypes.c_size_t, ctypes.c_int32, _P]),
    "ahq_dlq_percentile_encodings": (ctypes.c_int, [ctypes.POINTER(DlqPdfState), ctypes.c_float, ctypes.c_int32,
                                                    ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, _P, _P]),
    "ahq_dlq_tfe_encodings": (ctypes.c_int, [ctypes.POINTER(DlqPdfState), ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                             ctypes.c_int32, _P, _P, _P, ctypes.c_size_t, _P]),
}


def exported_symbols() -> Sequence[str]:
    return tuple(_SIGNATURES)


def load() -> ctypes.CDLL:
    """Load the shared library (once).  Raises HipLibraryError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipLibraryError(
            f"{LIB_PATH} not found: build it with `python -m aimet_amd.csrc.build` "
            "(this package has no fallback implementation)"
        )
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:
        raise HipLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    for name, (res, args) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise HipLibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from e
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, where: str) -> None:
    if status != AHQ_OK:
        msg = load().ahq_last_error()
        raise HipLibraryError(f"{where} failed ({status}): {msg.decode() if msg else 'unknown error'}")


def make_layout(dims: Sequence[int], block: Sequence[int], enc_stride: Sequence[int]) -> Layout:
    n = len(dims)
    if n > AHQ_MAX_DIMS:
        raise HipLibraryError(f"tensors of more than {AHQ_MAX_DIMS} dimensions are not supported (got {n})")
    lay = Layout()
    lay.ndim = n
    for i in range(n):
        lay.dims[i] = int(dims[i])
        lay.block[i] = int(block[i])
        lay.enc_stride[i] = int(enc_stride[i])
    return lay


def require_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise HipLibraryError(
            f"{what} lives on '{t.device}': the HIP backend only runs on GPU tensors and has no CPU fallback"
        )


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # pylint: disable=protected-access


def current_stream(device: torch.device) -> int:
    """Handle of torch's current stream on ``device`` (the library launches on the stream it is given)."""
    if _raw_stream is not None:
        # the same value without building a torch.cuda.Stream object (about 2 us per call, once per launch)
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream
