"""The quantized-module glue a whole-model calibration needs, for ``nn.Linear`` only.

Counterpart of the reference's ``BaseQuantizationMixin`` as used by ``QuantizedLinear``
(aimet_torch/nn/base.py:228-427, aimet_torch/nn/fake_quant.py): one input quantizer, one output quantizer, a weight
quantizer; ``compute_encodings()`` calibrates the weight quantizer from the weight once and puts the activation
quantizers into observe-and-pass-through mode (nn/base.py:392-427); outside that context the forward pass
quantize-dequantizes input, weight and output.  The GEMM itself is ``torch.nn.functional.linear``.

``fold_param_quantizers`` / ``inference_mode`` are the two ways the reference avoids re-quantizing weights on every
forward pass (nn/base.py:1103-1151, utils.py:1653-1684).

A weight that already lies on a symmetric integer grid keeps that grid (nn/base.py:355-383): the cheap test for it
-- do the first blocks hold more distinct magnitudes than the grid has levels? -- runs on every weight, as one kernel,
and only a weight that passes goes through the recovery of its per-block scale
(aimet_amd/quantization/_decompose.py); every trained or random weight goes straight to min/max calibration.
"""

from __future__ import annotations

import contextlib
import math
from typing import Iterable, Optional

import torch
from torch import nn
from torch.nn import functional as F

from aimet_amd.quantization._decompose import _DecompositionError, _decompose_prequantized_tensor
from aimet_amd.quantization._utils import concretize_block_size, patch_attr
from aimet_amd.quantization.affine.quantizer import AffineQuantizerBase, GroupedBlockQuantizeDequantize
from aimet_amd.quantization.base.quantizer import QuantizerBase

__all__ = ["QuantizedLinear", "compute_encodings", "quantized_linears", "fold_param_quantizers", "inference_mode",
           "remove_input_quantizers", "remove_output_quantizers", "remove_param_quantizers",
           "remove_activation_quantizers", "remove_all_quantizers"]


def _grid_probe(param: torch.Tensor, qtzr: AffineQuantizerBase, num_levels: int):
    """The same test in one launch (ahq_grid_probe) for a contiguous GPU parameter; None where the library does not
    cover the case (blocks along several dimensions, grids above 13 bits) and the torch form has to run."""
    from aimet_amd import _lib
    from aimet_amd.quantization.affine.backends.hip import _prepare

    if not (param.is_cuda and param.dtype in _lib.DTYPE_CODE and param.is_contiguous() and param.numel() > 0):
        return None
    shape = tuple(qtzr.shape)
    block_elems = param.numel() // max(1, math.prod(shape))
    if block_elems <= num_levels:
        return True
    if num_levels > 4096:
        return None
    xd, layout = _prepare(param, shape, qtzr.block_size)
    out = torch.empty((), dtype=torch.bool, device=param.device)
    status = _lib.load().ahq_grid_probe(_lib.DTYPE_CODE[param.dtype], layout, xd.data_ptr(), num_levels, out.data_ptr(),
                                        _lib.current_stream(param.device))
    if status == _lib.AHQ_ERR_UNSUPPORTED:
        return None
    _lib.check(status, "ahq_grid_probe")
    return out


def _may_be_prequantized(param: torch.Tensor, qtzr: AffineQuantizerBase, on_device: bool = True):
    """The early exit of _decompose_prequantized_tensor (aimet_torch/utils.py:2098-2118): the first 64 blocks, first
    2 * num_levels elements each; more distinct magnitudes than grid levels means the tensor is not on a grid.
    Returns True, or a 0-dim bool tensor on the parameter's device (not yet read back)."""
    num_levels = max(abs(qtzr.qmax), abs(qtzr.qmin)) + 1
    shape = tuple(qtzr.shape)
    verdict = _grid_probe(param, qtzr, num_levels) if on_device else None
    if verdict is not None:
        return verdict
    block = concretize_block_size(tuple(param.shape), shape, qtzr.block_size or tuple(-1 for _ in shape))
    block = (*param.shape[: param.dim() - len(block)], *block)
    split = []
    for d, b in zip(param.shape, block):
        split += [d // b, b]
    nd = len(split)
    x = param.reshape(split).permute(*range(0, nd, 2), *range(1, nd, 2))
    nblocks = math.prod(split[0::2])
    x = x.reshape(nblocks, -1)
    if x.shape[1] <= num_levels:
        return True
    xs = x[:64, : num_levels * 2].float().abs().sort(dim=1).values
    distinct = (xs[:, 1:] != xs[:, :-1]).sum(dim=1) + 1
    return ~torch.any(distinct > num_levels)


class _Removed:
    """Quantizers taken out of a ModuleList / ModuleDict at once (aimet_torch/nn/base.py:1240-1265 with
    utils._ContextManager): the slots read None from the moment of the call; leaving a ``with`` block puts them back,
    a bare call leaves them out for good."""

    def __init__(self, container, keys):
        slots = container._modules  # pylint: disable=protected-access
        self._restore = [(slots, k, slots[k]) for k in keys]
        for k in keys:
            slots[k] = None

    @classmethod
    def both(cls, first: "_Removed", second: "_Removed") -> "_Removed":
        merged = cls.__new__(cls)
        merged._restore = first._restore + second._restore  # pylint: disable=protected-access
        return merged

    def _cleanup(self):
        for slots, k, q in self._restore:
            slots[k] = q

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self._cleanup()
        return False


class QuantizedLinear(nn.Linear):
    """``nn.Linear`` with quantizers at its input, weight and output (any of them may be None)."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.input_quantizers = nn.ModuleList([None])
        self.output_quantizers = nn.ModuleList([None])
        self.param_quantizers = nn.ModuleDict({"weight": None, "bias": None})

    @classmethod
    def from_module(cls, linear: nn.Linear) -> "QuantizedLinear":
        """Wraps an existing layer; the parameters are shared, not copied."""
        q = cls.__new__(cls)
        nn.Module.__init__(q)
        q.in_features, q.out_features = linear.in_features, linear.out_features
        q.weight, q.bias = linear.weight, linear.bias
        q.input_quantizers = nn.ModuleList([None])
        q.output_quantizers = nn.ModuleList([None])
        q.param_quantizers = nn.ModuleDict({"weight": None, "bias": None})
        return q

    def __call__(self, *args, **kwargs):
        self._compute_param_encodings(overwrite=False)  # nn/base.py:262-265
        return super().__call__(*args, **kwargs)

    def forward(self, input: torch.Tensor) -> torch.Tensor:  # pylint: disable=redefined-builtin
        iq, oq = self.input_quantizers[0], self.output_quantizers[0]
        wq, bq = self.param_quantizers["weight"], self.param_quantizers["bias"]
        if iq is not None:
            input = iq(input)
        weight = self.weight if wq is None else wq(self.weight)
        bias = self.bias if (bq is None or self.bias is None) else bq(self.bias)
        out = F.linear(input.as_subclass(torch.Tensor), weight.as_subclass(torch.Tensor),
                       None if bias is None else bias.as_subclass(torch.Tensor))
        if oq is not None:
            out = oq(out)
        return out

    def _params_to_calibrate(self, overwrite: bool):
        for name, qtzr in self.param_quantizers.items():
            if qtzr is None or not qtzr.is_overwrite_allowed():
                continue
            if qtzr.is_initialized() and not overwrite:
                continue
            param = getattr(self, name)
            if param is not None:
                yield name, qtzr, param

    @staticmethod
    def _wants_grid_recovery(qtzr) -> bool:
        """The parameters whose grid the reference would first try to recover (nn/base.py:355-383)."""
        return (isinstance(qtzr, AffineQuantizerBase) and not isinstance(qtzr, GroupedBlockQuantizeDequantize)
                and bool(qtzr.symmetric) and math.ceil((qtzr.qmin + qtzr.qmax) / 2) == 0)

    def _prequantized_verdicts(self, overwrite: bool):
        """name -> True / device flag for the parameters whose grid the reference would first try to recover."""
        out = {}
        for name, qtzr, param in self._params_to_calibrate(overwrite):
            if self._wants_grid_recovery(qtzr):
                out[name] = _may_be_prequantized(param.detach(), qtzr)
        return out

    def _compute_param_encodings(self, overwrite: bool, verdicts=None, quantized=None):
        """nn/base.py:331-383.  ``verdicts``: already read-back results of _prequantized_verdicts().  ``quantized``:
        a dictionary that receives, by name, the quantize-dequantized parameters that came out of the calibration
        itself (one library call for both, where the quantizer offers it), for a caller that wants them next."""
        todo = list(self._params_to_calibrate(overwrite))
        if not todo:
            return
        if verdicts is None:
            verdicts = {k: bool(v) for k, v in self._prequantized_verdicts(overwrite).items()}
        for name, qtzr, param in todo:
            if quantized is not None and name in quantized:
                continue  # calibrated and quantize-dequantized already (aimet_amd.nn.compute_encodings)
            if verdicts.get(name, False):
                try:
                    _, scale = _decompose_prequantized_tensor(
                        param.detach(), qtzr.qmin, qtzr.qmax, scale_shape=tuple(qtzr.shape),
                        block_size=qtzr.block_size, zero_point_shift=qtzr.zero_point_shift, return_input_q=False,
                        _probed=True)
                except _DecompositionError:
                    pass  # on no grid after all: calibrate
                else:
                    with torch.no_grad():
                        qtzr.set_range(scale * qtzr.qmin, scale * qtzr.qmax)
                    continue
            if isinstance(qtzr, AffineQuantizerBase):
                fused = getattr(qtzr, "_calibrate_and_quantize", None) if quantized is not None else None
                out = fused(param) if fused is not None else None
                if out is not None:
                    quantized[name] = out
                else:
                    qtzr._calibrate_on(param)  # pylint: disable=protected-access
            else:
                with qtzr._compute_encodings(passthrough=True):  # pylint: disable=protected-access
                    _ = qtzr(param)
            if getattr(qtzr, "encoding_analyzer", None) is not None:
                qtzr.encoding_analyzer.reset_stats()  # nn/base.py:385-386

    def _patch_quantized_parameters(self, param_names: Optional[Iterable[str]] = None, _quantized=None):
        """nn/base.py:296-324: a context in which the named parameters (all by default) hold their
        quantize-dequantized values, computed once on entry (``_quantized``: those already at hand, by name)."""
        names = self.param_quantizers.keys() if param_names is None else param_names
        stack = contextlib.ExitStack()
        for name in names:
            qtzr = self.param_quantizers[name]
            param = getattr(self, name)
            if qtzr is None or param is None:
                continue
            if _quantized and name in _quantized:
                param = _quantized[name]
            elif qtzr.is_initialized():
                param = qtzr(param)
            stack.enter_context(patch_attr(self, name, param))
        return stack

    def _params_quantized_once(self):
        """Names of the parameters whose quantize-dequantized value may be formed once for a whole calibration context
        instead of in every pass: the quantizer holds encodings, and no gradient can be wanted through it (gradients
        are switched off, or neither the parameter nor the quantizer learns).  Every other parameter quantizer stays
        in place and runs in every pass, as in the reference (nn/base.py:392-427): a pass then builds its own graph,
        and a quantizer without encodings raises in forward."""
        names = []
        grad = torch.is_grad_enabled()
        for name, qtzr in self.param_quantizers.items():
            param = getattr(self, name)
            if qtzr is None or param is None or not qtzr.is_initialized():
                continue
            if grad and (param.requires_grad or any(p.requires_grad for p in qtzr.parameters())):
                continue
            names.append(name)
        return names

    def _remove_input_quantizers(self, indices=None):
        """nn/base.py:983-993: the input quantizers (all, one index or several) are taken out at once; used as a
        context manager, the call puts them back on leaving."""
        if isinstance(indices, int):
            indices = [indices]
        elif indices is None:
            indices = list(range(len(self.input_quantizers)))
        return _Removed(self.input_quantizers, [str(i) for i in indices])

    def _remove_param_quantizers(self, keys=None):
        """nn/base.py:995-1005."""
        keys = list(self.param_quantizers.keys()) if keys is None else ([keys] if isinstance(keys, str) else list(keys))
        return _Removed(self.param_quantizers, keys)

    def _remove_output_quantizers(self, indices=None):
        """nn/base.py:1007-1017."""
        if isinstance(indices, int):
            indices = [indices]
        elif indices is None:
            indices = list(range(len(self.output_quantizers)))
        return _Removed(self.output_quantizers, [str(i) for i in indices])

    def _remove_activation_quantizers(self):
        """nn/base.py:1019-1026."""
        return _Removed.both(self._remove_output_quantizers(), self._remove_input_quantizers())

    def _remove_all_quantizers(self):
        """nn/base.py:1028-1035."""
        return _Removed.both(self._remove_activation_quantizers(), self._remove_param_quantizers())

    def compute_param_encodings(self):
        """Compute the encodings of the parameter quantizers (nn/base.py:388-390)."""
        self._compute_param_encodings(overwrite=True)

    def export_input_encodings(self, encoding_version: str):
        """One exported dictionary (or None) per input quantizer (nn/base.py:527-539)."""
        return [q.get_encodings().to_qnn_encoding_dict(encoding_version)
                if isinstance(q, QuantizerBase) and q.is_initialized() else None for q in self.input_quantizers]

    def export_output_encodings(self, encoding_version: str):
        """nn/base.py:586-598."""
        return [q.get_encodings().to_qnn_encoding_dict(encoding_version)
                if isinstance(q, QuantizerBase) and q.is_initialized() else None for q in self.output_quantizers]

    def export_param_encodings(self, encoding_version: str):
        """{parameter name: exported dictionary or None} (nn/base.py:645-678); a parameter that is an already
        quantized tensor without a quantizer exports the encoding it carries."""
        from aimet_amd.quantization.tensor import QuantizedTensorBase

        out = {}
        for name, q in self.param_quantizers.items():
            param = getattr(self, name)
            if isinstance(q, QuantizerBase):
                out[name] = (q.get_encodings()._hint_input_shape(param.shape).to_qnn_encoding_dict(encoding_version)  # pylint: disable=protected-access
                             if q.is_initialized() else None)
            elif isinstance(param, QuantizedTensorBase) and param.encoding is not None:
                out[name] = param.encoding._hint_input_shape(param.shape).to_qnn_encoding_dict(encoding_version)  # pylint: disable=protected-access
            else:
                out[name] = None
        return out

    def get_original_module(self) -> nn.Linear:
        """The floating-point layer with the quantizers removed; parameters are shared (nn/base.py:757-794)."""
        orig = nn.Linear.__new__(nn.Linear)
        orig.__dict__ = self.__dict__.copy()
        orig.__dict__.pop("forward", None)
        orig._parameters = self._parameters.copy()  # pylint: disable=protected-access
        orig._buffers = self._buffers.copy()  # pylint: disable=protected-access
        orig._modules = {k: v for k, v in self._modules.items()  # pylint: disable=protected-access
                         if k not in ("input_quantizers", "output_quantizers", "param_quantizers")}
        return orig

    def fold_param_quantizers(self):
        """nn/base.py:1103-1151: bake each parameter quantizer into its parameter (the parameter becomes the
        quantize-dequantized tensor, the quantizer is dropped), so later forward passes skip that work."""
        self._compute_param_encodings(overwrite=False)
        for name, qtzr in self.param_quantizers.items():
            if not qtzr:
                continue
            param = getattr(self, name)
            if param is None:
                continue
            with torch.no_grad():
                qdq = qtzr(param).dequantize()
            setattr(self, name, nn.Parameter(qdq, requires_grad=param.requires_grad))
            self.param_quantizers[name] = None

    @contextlib.contextmanager
    def compute_encodings(self, _verdicts=None):
        """nn/base.py:392-427: weights are calibrated on entry; activation quantizers observe their inputs and pass
        them through unquantized, and set their ranges on exit."""
        quantized = {}
        self._compute_param_encodings(overwrite=True, verdicts=_verdicts, quantized=quantized)
        with contextlib.ExitStack() as stack:
            # Neither the parameters nor their (just computed) encodings change inside the context, so where no
            # gradient can be wanted the quantize-dequantized parameters are the same in every calibration pass: they
            # are formed once here and the passes use them (the reference calls the parameter quantizers again in
            # every pass, with the same result; its own _patch_quantized_parameters / fold_param_quantizers,
            # nn/base.py:296-324, 1103-1151, are the same trade).  A caller that modifies such a parameter in place
            # inside the context sees the old values, and reads None for its quantizer.
            once = self._params_quantized_once()
            if once:
                stack.enter_context(self._patch_quantized_parameters(once, _quantized=quantized))
                stack.enter_context(self._remove_param_quantizers(once))
            for qtzr in list(self.input_quantizers) + list(self.output_quantizers):
                if not isinstance(qtzr, QuantizerBase) or not qtzr.is_overwrite_allowed():
                    continue
                stack.enter_context(qtzr._compute_encodings(passthrough=True))  # pylint: disable=protected-access
            yield


def quantized_linears(model: nn.Module) -> Iterable[QuantizedLinear]:
    return (m for m in model.modules() if isinstance(m, QuantizedLinear))


def _probe_parameters_together(candidates):
    """_may_be_prequantized() for many (parameter, quantizer) pairs with one library call (ahq_grid_probe_many) and
    one read-back.  Returns the verdicts as Python booleans, in order."""
    import ctypes

    from aimet_amd import _lib
    from aimet_amd.quantization.affine.backends.hip import _prepare

    verdicts = [None] * len(candidates)
    batched = []  # (index, item fields)
    for i, (param, qtzr) in enumerate(candidates):
        num_levels = max(abs(qtzr.qmax), abs(qtzr.qmin)) + 1
        p = param.detach()
        shape = tuple(qtzr.shape)
        if (p.is_cuda and p.dtype in _lib.DTYPE_CODE and p.is_contiguous() and p.numel() > 0 and num_levels <= 4096
                and p.numel() // max(1, math.prod(shape)) > num_levels):
            xd, layout = _prepare(p, shape, qtzr.block_size)
            batched.append((i, _lib.DTYPE_CODE[p.dtype], layout, xd, num_levels))
        else:
            verdicts[i] = _may_be_prequantized(p, qtzr)
    by_device = {}
    for entry in batched:
        by_device.setdefault(entry[3].device, []).append(entry)
    pending = []
    for device, entries in by_device.items():
        items = (_lib.GridProbeItem * len(entries))()
        for it, (_, code, layout, xd, num_levels) in zip(items, entries):
            it.dtype, it.layout, it.x, it.num_levels = code, layout, xd.data_ptr(), num_levels
        out = torch.empty(len(entries), dtype=torch.bool, device=device)
        unsupported = (ctypes.c_uint8 * len(entries))()
        with torch.cuda.device(device):
            _lib.check(_lib.load().ahq_grid_probe_many(items, len(entries), out.data_ptr(), unsupported,
                                                       _lib.current_stream(device)), "ahq_grid_probe_many")
        pending.append((entries, out, unsupported))
    for entries, out, unsupported in pending:
        answers = out.tolist()
        for (i, *_), answer, skipped in zip(entries, answers, unsupported):
            verdicts[i] = _may_be_prequantized(candidates[i][0].detach(), candidates[i][1], on_device=False) if skipped else answer
    return [bool(v) for v in verdicts]


def _calibrate_parameters_together(work):
    """Calibration and first quantize-dequantize of many parameters with one library call
    (ahq_minmax_calibrate_qdq_many).  ``work``: (module, name, quantizer, parameter) of parameters that are not on a
    grid already.  Returns {id(module): {name: quantize-dequantized parameter}} for those the call covered; the
    others are left to QuantizedLinear._compute_param_encodings()."""
    from aimet_amd import _lib
    from aimet_amd.quantization._utils import _get_minimum_scale
    from aimet_amd.quantization.encoding_analyzer import _scalar_constants, _range_flags_buffer, _report_range_flags

    done = {}
    if torch.is_grad_enabled():
        return done
    by_device = {}
    for module, name, qtzr, param in work:
        prepare = getattr(qtzr, "_calibrate_qdq_prepare", None)
        plan = prepare(param) if prepare is not None else None
        if plan is not None:
            by_device.setdefault(plan[0].device, []).append((module, name, qtzr, plan))
    for device, entries in by_device.items():
        n = len(entries)
        items = (_lib.CalibrateQdqItem * n)()
        # one allocation each for the scales, the offsets of asymmetric grids and the workspaces of all parameters
        enc_sizes = [q.min.numel() for _, _, q, _ in entries]
        ws_sizes = [(max(plan[3], 16) + 255) // 256 * 256 for *_, plan in entries]
        scales = torch.empty(sum(enc_sizes), dtype=torch.float32, device=device)
        offsets = torch.empty(sum(e for e, (*_, plan) in zip(enc_sizes, entries) if not plan[5]) or 1,
                              dtype=torch.float32, device=device)
        ws = torch.empty(sum(ws_sizes), dtype=torch.uint8, device=device)
        flags, own_flags = _range_flags_buffer(device)
        outputs = []
        s_at = o_at = w_at = 0
        for it, (module, name, qtzr, plan), ne, nw in zip(items, entries, enc_sizes, ws_sizes):
            x, grid, layout, nbytes, num_steps, symmetric = plan
            mn, mx = qtzr.min, qtzr.max
            consts = _scalar_constants(x.dtype, _get_minimum_scale(num_steps))
            y = torch.empty_like(x)
            scale = scales[s_at:s_at + ne].view(mn.shape)
            s_at += ne
            if symmetric:
                offset = qtzr._constant_offset(device)  # pylint: disable=protected-access
            else:
                offset = offsets[o_at:o_at + ne].view(mn.shape)
                o_at += ne
            qtzr.encoding_analyzer.reset_stats()
            it.grid, it.layout, it.x, it.y = grid, layout, x.data_ptr(), y.data_ptr()
            it.num_steps, it.symmetric = num_steps, 1 if symmetric else 0
            it.minimum_scale_in_dtype, it.minimum_scale, it.dtype_max, it.near_max_threshold = consts
            it.param_dtype, it.param_min, it.param_max = _lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr()
            it.grid_minimum_scale = _get_minimum_scale(qtzr.qmax - qtzr.qmin)
            it.scale, it.offset = scale.data_ptr(), offset.data_ptr()
            it.workspace, it.workspace_bytes = ws.data_ptr() + w_at, nbytes
            w_at += nw
            outputs.append((y, scale, offset))
        with torch.cuda.device(device):
            _lib.check(_lib.load().ahq_minmax_calibrate_qdq_many(items, n, flags.data_ptr(), _lib.current_stream(device)),
                       "ahq_minmax_calibrate_qdq_many")
        for (module, name, qtzr, _), (y, scale, offset) in zip(entries, outputs):
            done.setdefault(id(module), {})[name] = qtzr._calibrate_qdq_adopt(y, scale, offset)  # pylint: disable=protected-access
            qtzr.encoding_analyzer.reset_stats()  # nn/base.py:385-386
        if own_flags:
            _report_range_flags(flags)
    return done


def _finalize_together(quantizers):
    """What leaving their compute_encodings() contexts does for many activation quantizers
    (_set_range_from_statistics), with one library call for all per-tensor min/max quantizers whose running extrema
    lie in their observers' slots (ahq_minmax_slots_finalize_many); the others one by one."""
    from aimet_amd import _lib
    from aimet_amd.quantization._utils import _get_minimum_scale
    from aimet_amd.quantization.encoding_analyzer import _scalar_constants, _range_flags_buffer, _report_range_flags

    by_device = {}
    for q in quantizers:
        item = q._slots_finalize_item() if hasattr(q, "_slots_finalize_item") else None  # pylint: disable=protected-access
        if item is None:
            q._set_range_from_statistics()  # pylint: disable=protected-access
        else:
            by_device.setdefault(q.min.device, []).append((q, item))
    for device, entries in by_device.items():
        n = len(entries)
        items = (_lib.SlotsFinalizeItem * n)()
        scales = torch.empty(n, dtype=torch.float32, device=device)
        n_asym = sum(1 for q, _ in entries if not q.symmetric)
        offsets = torch.empty(max(n_asym, 1), dtype=torch.float32, device=device)
        flags, own_flags = _range_flags_buffer(device)
        s_ptr, o_ptr = scales.data_ptr(), offsets.data_ptr()
        scale_views, offset_views = scales.unbind(0), offsets.unbind(0)  # all 0-dim views with one call each
        outputs = []
        o_at = 0
        for k, (it, (q, (stat_dtype, slots, num_steps))) in enumerate(zip(items, entries)):
            mn, mx = q.min, q.max
            symmetric = bool(q.symmetric)
            consts = _scalar_constants(stat_dtype, _get_minimum_scale(num_steps))
            it.stat_dtype, it.symmetric, it.slots, it.num_steps = _lib.DTYPE_CODE[stat_dtype], 1 if symmetric else 0, slots.data_ptr(), num_steps
            it.minimum_scale_in_dtype, it.minimum_scale, it.dtype_max, it.near_max_threshold = consts
            it.param_dtype, it.param_min, it.param_max = _lib.DTYPE_CODE[mn.dtype], mn.data_ptr(), mx.data_ptr()
            it.qmin, it.qmax, it.grid_minimum_scale = q.qmin, q.qmax, _get_minimum_scale(q.qmax - q.qmin)
            it.scale = s_ptr + 4 * k
            scale = scale_views[k] if mn.dim() == 0 else scale_views[k].view(mn.shape)
            if symmetric:
                it.offset = None
                offset = q._constant_offset(device)  # pylint: disable=protected-access
            else:
                it.offset = o_ptr + 4 * o_at
                offset = offset_views[o_at] if mn.dim() == 0 else offset_views[o_at].view(mn.shape)
                o_at += 1
            outputs.append((scale, offset))
        with torch.cuda.device(device):
            _lib.check(_lib.load().ahq_minmax_slots_finalize_many(items, n, flags.data_ptr(), _lib.current_stream(device)),
                       "ahq_minmax_slots_finalize_many")
        for (q, _), (scale, offset) in zip(entries, outputs):
            q._finalize_adopt(scale, offset)  # pylint: disable=protected-access
        if own_flags:
            _report_range_flags(flags)


@contextlib.contextmanager
def compute_encodings(model: nn.Module):
    """aimet_torch.nn.compute_encodings (nn/base.py): the compute_encodings context of every quantized module.  The
    modules enter and leave together, so the work of all their quantizers is handed to the library in three calls
    (the "already on a grid?" test of every weight, calibration + quantize-dequantize of every weight, the ranges of
    all per-tensor activation quantizers at the end); whatever those calls do not cover goes the quantizer's own way,
    with the same results."""
    from aimet_amd.quantization.encoding_analyzer import deferred_range_warnings

    modules = list(quantized_linears(model))
    with deferred_range_warnings(), contextlib.ExitStack() as stack:
        # 1. parameters: the reference's early exit of the grid recovery, then min/max calibration (nn/base.py:331-386)
        todo = [(m, name, qtzr, param) for m in modules for name, qtzr, param in m._params_to_calibrate(True)]  # pylint: disable=protected-access
        probe = [k for k, (m, name, qtzr, param) in enumerate(todo) if m._wants_grid_recovery(qtzr)]  # pylint: disable=protected-access
        answers = _probe_parameters_together([(todo[k][3], todo[k][2]) for k in probe])
        verdicts = {id(m): {} for m in modules}
        for k, answer in zip(probe, answers):
            verdicts[id(todo[k][0])][todo[k][1]] = answer
        plain = [w for w in todo if not verdicts[id(w[0])].get(w[1], False) and isinstance(w[2], AffineQuantizerBase)]
        quantized = _calibrate_parameters_together(plain)
        for m in modules:
            mine = quantized.get(id(m), {})
            m._compute_param_encodings(overwrite=True, verdicts=verdicts[id(m)], quantized=mine)  # pylint: disable=protected-access
            once = m._params_quantized_once()  # pylint: disable=protected-access
            if once:
                stack.enter_context(m._patch_quantized_parameters(once, _quantized=mine))  # pylint: disable=protected-access
                stack.enter_context(m._remove_param_quantizers(once))  # pylint: disable=protected-access
        # 2. activations: observed and passed through unquantized; ranges set on leaving (nn/base.py:392-427)
        observing = []
        for m in modules:
            for qtzr in list(m.input_quantizers) + list(m.output_quantizers):
                if not isinstance(qtzr, QuantizerBase) or not qtzr.is_overwrite_allowed():
                    continue
                begin = getattr(qtzr, "_begin_passthrough_calibration", None)
                if begin is not None and "forward" not in qtzr.__dict__:
                    if begin():
                        observing.append(qtzr)
                else:
                    stack.enter_context(qtzr._compute_encodings(passthrough=True))  # pylint: disable=protected-access
        try:
            yield
        finally:
            for qtzr in observing:
                qtzr._end_passthrough_calibration()  # pylint: disable=protected-access
            _finalize_together(observing)


def fold_param_quantizers(model: nn.Module):
    """QuantizationSimModel.fold_param_quantizers (quantsim/quantsim.py:930-960)."""
    for m in quantized_linears(model):
        m.fold_param_quantizers()


def _remove_from_all(model, method: str) -> _Removed:
    removed = None
    for m in quantized_linears(model):
        one = getattr(m, method)()
        removed = one if removed is None else _Removed.both(removed, one)
    return removed if removed is not None else _Removed(nn.ModuleList(), [])


def remove_input_quantizers(model: nn.Module) -> _Removed:
    """aimet_torch.utils.remove_input_quantizers (utils.py:1305-1347) for the quantized modules of ``model``: taken
    out at the call, put back on leaving a ``with`` block."""
    return _remove_from_all(model, "_remove_input_quantizers")


def remove_output_quantizers(model: nn.Module) -> _Removed:
    """aimet_torch.utils.remove_output_quantizers (utils.py:1350-1392)."""
    return _remove_from_all(model, "_remove_output_quantizers")


def remove_param_quantizers(model: nn.Module) -> _Removed:
    """aimet_torch.utils.remove_param_quantizers (utils.py:1395-1437)."""
    return _remove_from_all(model, "_remove_param_quantizers")


def remove_activation_quantizers(model: nn.Module) -> _Removed:
    """aimet_torch.utils.remove_activation_quantizers (utils.py:1440-1491)."""
    return _remove_from_all(model, "_remove_activation_quantizers")


def remove_all_quantizers(model: nn.Module) -> _Removed:
    """aimet_torch.utils.remove_all_quantizers (utils.py:1494-1540)."""
    return _remove_from_all(model, "_remove_all_quantizers")


@contextlib.contextmanager
def inference_mode(model: nn.Module, prequantize_parameters: bool = True):
    """aimet_torch.utils._inference_mode (utils.py:1653-1684): every quantizer's encodings are evaluated once and
    reused by all forward passes inside the context; with ``prequantize_parameters`` the parameters are
    quantize-dequantized once on entry and their quantizers are skipped inside."""
    with contextlib.ExitStack() as stack:
        for q in model.modules():
            if isinstance(q, QuantizerBase):
                import itertools

                dtype = next(p.dtype for p in itertools.chain(q.parameters(), q.buffers()))
                stack.enter_context(q._precompute_encodings(dtype=dtype))  # pylint: disable=protected-access
        if prequantize_parameters:
            with torch.no_grad():
                for m in quantized_linears(model):
                    stack.enter_context(m._patch_quantized_parameters())  # pylint: disable=protected-access
            stack.enter_context(remove_param_quantizers(model))
        # quantized parameters enter the GEMM as plain tensors
        for m in quantized_linears(model):
            for name, param in list(m.named_parameters(recurse=False)):
                if type(param) not in (torch.Tensor, nn.Parameter):
                    stack.enter_context(patch_attr(m, name, param.as_subclass(torch.Tensor)))
        yield


def wrap_linears(model: nn.Module, make_quantizers) -> int:
    """Replaces every nn.Linear in ``model`` by a QuantizedLinear sharing its parameters.  ``make_quantizers(name,
    linear)`` returns (input quantizer, weight quantizer, output quantizer), any of them None."""
    count = 0
    for parent_name, parent in list(model.named_modules()):
        for child_name, child in list(parent.named_children()):
            if type(child) is nn.Linear:  # pylint: disable=unidiomatic-typecheck
                q = QuantizedLinear.from_module(child)
                full = f"{parent_name}.{child_name}" if parent_name else child_name
                iq, wq, oq = make_quantizers(full, child)
                q.input_quantizers[0] = iq
                q.param_quantizers["weight"] = wq
                q.output_quantizers[0] = oq
                setattr(parent, child_name, q)
                count += 1
    return count
