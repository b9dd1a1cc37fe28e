"""CPU restatement of the aimet_torch fake-quant and calibration path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``aimet_amd/`` may import this module;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` use it, and there only as the checker.

Every function issues, on CPU tensors, the same sequence of torch operations
that the reference issues, so the result is produced by the same ATen CPU
kernels.  Reference files followed (paths relative to the reference checkout,
``AT`` = TrainingExtensions/torch/src/python/aimet_torch):

* AT/quantization/affine/backends/torch_builtins.py   (QDQ arithmetic, dtype guards)
* AT/quantization/_utils.py                            (block-size helpers)
* AT/quantization/encoding_analyzer.py                 (observers and analyzers)
* AT/quantization/affine/quantizer.py                  (scale/offset derivation, LPBQ)
* AT/utils.py:1115-1148                                (reduce)
* TrainingExtensions/common/src/python/_aimet_common/quantsim.py:538-559 (minimum scale)

Pinning status (which independent check pins which function) is listed in
``tests/test_oracle_golden.py``.  Functions whose end-to-end result on realistic
data no reference fixture covers are marked "parity unpinned" below:

* ``hist_merge`` on arbitrary data (the reference tests hold four small cases,
  all reproduced in the tests) -- pinned on those cases plus integer-count
  conservation; beyond that: parity unpinned.
* ``sqnr_encodings`` on realistic data -- pinned by the uniform-distribution
  closed form, the candidate-grid structure checks and a brute-force Python
  float enumeration on tiny inputs; beyond that: parity unpinned.
"""

from __future__ import annotations

import itertools
import math
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import torch

_MANTISSA_BITS = {
    torch.float32: 23,
    torch.float16: 10,
    torch.bfloat16: 7,
    torch.float64: 52,
}


# --------------------------------------------------------------------------- #
# dtype guards (torch_builtins.py:49-116)
# --------------------------------------------------------------------------- #
def value_representable(dtype: torch.dtype, value: int) -> bool:
    """torch_builtins.py:49-83"""
    if dtype not in _MANTISSA_BITS:
        raise ValueError(f"unsupported dtype {dtype}")
    info = torch.finfo(dtype)
    if not info.min <= value <= info.max:
        return False
    top = max(0, value.bit_length() - 1)
    low = max(0, (value & -value).bit_length() - 1)
    return top - low <= _MANTISSA_BITS[dtype]


def grid_representable(dtype: torch.dtype, qmin: int, qmax: int) -> bool:
    """torch_builtins.py:86-96"""
    return all(
        value_representable(dtype, v) for v in (qmax, qmax - 1, qmin + 1, qmin)
    )


def numerically_stable(dtype: torch.dtype, qmin: int, qmax: int) -> bool:
    """torch_builtins.py:99-116"""
    if not grid_representable(dtype, qmin, qmax):
        return False
    if qmin == qmax:
        return True
    return not torch.finfo(dtype).eps > 0.25 / (qmax - qmin)


def internal_dtype(dtype: torch.dtype, qmin: int, qmax: int) -> torch.dtype:
    """Promotion rule of torch_builtins.py:193-196 / 274-277."""
    if numerically_stable(dtype, qmin, qmax):
        return dtype
    if numerically_stable(torch.float32, qmin, qmax):
        return torch.float32
    return torch.float64


def minimum_scale(num_steps: int) -> float:
    """_aimet_common/quantsim.py:538-559"""
    return min(float(torch.finfo(torch.float32).eps), 0.01 / num_steps)


# --------------------------------------------------------------------------- #
# block helpers (quantization/_utils.py:11-62)
# --------------------------------------------------------------------------- #
def interleave(a, b) -> Tuple[int, ...]:
    if isinstance(a, int):
        a = (a,) * len(b)
    if isinstance(b, int):
        b = (b,) * len(a)
    assert len(a) == len(b)
    return tuple(v for pair in zip(a, b) for v in pair)


def concrete_block_size(in_shape, enc_shape, block_size) -> Tuple[int, ...]:
    """quantization/_utils.py:30-62"""
    in_shape = tuple(in_shape)[-len(enc_shape):] if len(enc_shape) else ()
    lead = len(enc_shape) - len(block_size)
    full = [1 if d > 1 else -1 for d in enc_shape[:lead]] + list(block_size)
    return tuple(
        full[i] if full[i] != -1 else in_shape[i] // enc_shape[i]
        for i in range(len(enc_shape))
    )


def _blocked_views(x, scale, offset, block_size):
    """torch_builtins.py:285-289: the interleaved reshape used for block quantization."""
    if not block_size:
        return x, scale, offset
    bs = concrete_block_size(x.shape, scale.shape, block_size)
    x = x.reshape(-1, *interleave(scale.shape, bs))
    scale = scale.view(interleave(scale.shape, 1))
    if offset is not None:
        offset = offset.view(interleave(offset.shape, 1))
    return x, scale, offset


# --------------------------------------------------------------------------- #
# V1: ATen fake-quantize fast path (torch_builtins.py:335-431)
# --------------------------------------------------------------------------- #
def qdq_v1(x: torch.Tensor, scale: torch.Tensor, offset: torch.Tensor, qmin: int, qmax: int):
    """Calls the installed ATen CPU kernels exactly as torch_builtins.py:485-491 / 526-533 do.

    Returns ``(y, mask)`` where ``mask`` is the cachemask ATen uses for the backward
    (``gx = g * mask``).  Returns ``None`` when the reference would leave the fast path
    (torch_builtins.py:388-431).
    """
    scale = scale.to(torch.float32)
    if scale.numel() == 1 and offset.numel() == 1:
        zp = -offset.to(torch.int32)
        y, mask = torch._fake_quantize_per_tensor_affine_cachemask_tensor_qparams(
            x, scale.view(()), zp.view(()), torch.ones((), dtype=torch.long), qmin, qmax
        )
        return y, mask
    sshape = (1,) * (x.dim() - scale.dim()) + tuple(scale.shape)
    oshape = (1,) * (x.dim() - offset.dim()) + tuple(offset.shape)
    if sshape != oshape or not all(s in (1, t) for s, t in zip(sshape, x.shape)):
        return None
    axes = [i for i, s in enumerate(sshape) if s != 1]
    if len(axes) != 1:
        return None
    zp = -offset.to(torch.int32)
    y, mask = torch.ops.aten.fake_quantize_per_channel_affine_cachemask(
        x, scale.flatten(), zp.flatten(), axes[0], qmin, qmax
    )
    return y, mask


# --------------------------------------------------------------------------- #
# V2: composed elementwise path (torch_builtins.py:727-831)
# --------------------------------------------------------------------------- #
@dataclass
class QdqTrace:
    y: torch.Tensor            # output in x.dtype, x.shape
    mask: torch.Tensor         # in-range mask, x.shape (bool)
    dtype: torch.dtype         # internal dtype D


def qdq_v2_forward(x, scale, offset, qmin, qmax, block_size=None, zero_point_shift=0.0) -> QdqTrace:
    """torch_builtins.py:268-302 + 727-751."""
    D = internal_dtype(x.dtype, qmin, qmax)
    if not grid_representable(D, qmin, qmax):
        raise RuntimeError(f"{D} is unable to represent quantized output of range [{qmin}, {qmax}].")
    shape = x.shape
    xb, sb, ob = _blocked_views(x, scale, offset, block_size)
    sb = sb.to(D)
    ob = ob.to(D)
    t = xb.to(D) / sb
    if zero_point_shift != 0:
        t = t - zero_point_shift
    r = torch.round_(t).sub_(ob)
    mask = (qmin <= r) & (r <= qmax)
    q = r.clamp_(qmin, qmax)
    y = q.add_(ob if zero_point_shift == 0 else ob + zero_point_shift).mul_(sb)
    return QdqTrace(y.to(x.dtype).view(shape), mask.view(shape), D)


def qdq_v2_backward(g, x, scale, offset, qmin, qmax, block_size=None, zero_point_shift=0.0):
    """torch_builtins.py:779-831 followed by the autograd sum-to-size and the cast of the
    scale/offset gradients back to the fp32 parameters.  Returns (gx, gscale, goffset)."""
    D = internal_dtype(x.dtype, qmin, qmax)
    shape = x.shape
    xb, sb, ob = _blocked_views(x, scale, offset, block_size)
    sb = sb.to(D)
    ob = ob.to(D)
    # the output cast `.to(output_dtype)` back-propagates as a cast of g to D
    gb = g.to(D).reshape(xb.shape)

    t = xb.to(D) / sb
    if zero_point_shift != 0:
        t = t - zero_point_shift
    r = torch.round(t).sub_(ob)
    mask = (qmin <= r) & (r <= qmax)

    x_scaled = xb.to(D) / sb - zero_point_shift
    x_rounded = torch.round(x_scaled)
    err = x_rounded - x_scaled
    x_rounded.clamp_(ob + qmin, ob + qmax)
    if zero_point_shift != 0.0:
        x_rounded.add_(zero_point_shift)
    gs_full = gb * torch.where(mask, err, x_rounded)
    goff_full = torch.where(mask, 0, gb * sb)
    gx = torch.where(mask, gb, 0).to(x.dtype).view(shape)
    gs = gs_full.sum_to_size(sb.shape).to(scale.dtype).view(scale.shape)
    goff = goff_full.sum_to_size(ob.shape).to(offset.dtype).view(offset.shape)
    return gx, gs, goff


def quantize_forward(x, scale, offset, qmin, qmax, block_size=None):
    """torch_builtins.py:166-212 + 610-632.  Returns (codes in x.dtype, in-range mask)."""
    if not grid_representable(x.dtype, qmin, qmax):
        raise RuntimeError(f"{x.dtype} is unable to represent quantized output of range [{qmin}, {qmax}].")
    D = internal_dtype(x.dtype, qmin, qmax)
    shape = x.shape
    xb, sb, ob = _blocked_views(x, scale, offset, block_size)
    sb = sb.to(D)
    ob = ob.to(D)
    r = torch.round_(xb.to(D) / sb).sub_(ob)
    mask = (r >= qmin) * (r <= qmax)
    return r.clamp_(qmin, qmax).to(x.dtype).view(shape), mask.view(shape)


def quantize_backward(g, x, scale, offset, qmin, qmax, block_size=None):
    """torch_builtins.py:637-655 (+ sum-to-size).  Returns (gx, gscale, goffset)."""
    D = internal_dtype(x.dtype, qmin, qmax)
    shape = x.shape
    xb, sb, ob = _blocked_views(x, scale, offset, block_size)
    sb = sb.to(D)
    ob = ob.to(D)
    gb = g.to(D).reshape(xb.shape)
    r = torch.round_(xb.to(D) / sb).sub_(ob)
    mask = (r >= qmin) * (r <= qmax)
    mg = gb * mask
    gx = (mg / sb).to(x.dtype).view(shape)
    gs = (-(mg / sb) * (xb.to(D) / sb)).sum_to_size(sb.shape).to(scale.dtype).view(scale.shape)
    goff = (-mg).sum_to_size(ob.shape).to(offset.dtype).view(offset.shape)
    return gx, gs, goff


def dequantize_forward(x, scale, offset, block_size=None):
    """torch_builtins.py:537-571 + 674-686 (internal dtype = x.dtype)."""
    shape = x.shape
    xb, sb, ob = _blocked_views(x, scale, offset, block_size)
    return (xb + ob.to(x.dtype)).mul_(sb.to(x.dtype)).view(shape)


def dequantize_backward(g, x, scale, offset, block_size=None):
    """torch_builtins.py:691-701 (+ sum-to-size).  Returns (gx, gscale, goffset)."""
    shape = x.shape
    xb, sb, ob = _blocked_views(x, scale, offset, block_size)
    sb = sb.to(x.dtype)
    ob = ob.to(x.dtype)
    gb = g.reshape(xb.shape)
    gx_full = gb * sb
    gs = (gb * (xb + ob)).sum_to_size(sb.shape).to(scale.dtype).view(scale.shape)
    goff = gx_full.sum_to_size(ob.shape).to(offset.dtype).view(offset.shape)
    return gx_full.view(shape), gs, goff


# --------------------------------------------------------------------------- #
# scale / offset derivation (quantizer.py:319-376, 843-900, 1363-1399)
# --------------------------------------------------------------------------- #
def scale_from_minmax(mn, mx, qmin, qmax):
    """quantizer.py:333-342 (min/max-parametrised quantizer, dtype float32)."""
    n = qmax - qmin
    s = (mx.to(torch.float32) - mn.to(torch.float32)) / n
    return s.abs().clamp_min_(minimum_scale(n)).to(torch.float32)


def offset_from_minmax(mn, scale, qmin, qmax, symmetric):
    """quantizer.py:357-376."""
    if symmetric:
        return torch.full(mn.shape, -round((qmin + qmax) / 2), dtype=torch.float32)
    return torch.clamp(torch.round(mn / scale) - qmin, -qmax, -qmin).to(torch.float32)


def scale_offset_dynamic(mn, mx, qmin, qmax, symmetric):
    """quantizer.py:876-900 (`_get_scale_offset`)."""
    n = qmax - qmin
    mn = mn.to(torch.float32)
    mx = mx.to(torch.float32)
    s = (mx - mn).div_(n)
    if symmetric:
        off = torch.full_like(mn, -round((qmin + qmax) / 2))
    else:
        off = torch.round(mn / s) - qmin
    return s, off


def lpbq_scale(raw_scale, bitwidth, decompressed_bw, block_grouping):
    """quantizer.py:1363-1399: returns (lpbq_scale, per_channel_scale)."""
    pcs_shape = [d // g if g != -1 else 1 for d, g in zip(raw_scale.shape, block_grouping)]
    grouping = concrete_block_size(raw_scale.shape, pcs_shape, block_grouping)
    resh = raw_scale.reshape(*interleave(pcs_shape, grouping))
    mx = torch.amax(resh, dim=tuple(range(1, resh.dim(), 2)))
    pcs = mx / 2 ** (decompressed_bw - bitwidth)
    tr = qdq_v2_forward(raw_scale, pcs, torch.zeros_like(pcs), 1, 2 ** (decompressed_bw - bitwidth),
                        block_size=block_grouping)
    return tr.y, pcs


# --------------------------------------------------------------------------- #
# min/max observer + encodings (AT/utils.py:1115-1148, encoding_analyzer.py:80-112, 425-481)
# --------------------------------------------------------------------------- #
def reduce_minmax(x, shape, block_size=None):
    out_shape = tuple(shape)
    if block_size is not None:
        bs = concrete_block_size(x.shape, shape, block_size)
        x = x.reshape(-1, *interleave(shape, bs))
        shape = interleave(shape, 1)
    padded = (1,) * (x.dim() - len(shape)) + tuple(shape)
    red = tuple(a for a, d in enumerate(padded) if d == 1)
    keep = tuple(a for a, d in enumerate(padded) if d > 1)
    flat = x.permute(red + keep).reshape(-1, *out_shape)
    return torch.amin(flat, dim=0), torch.amax(flat, dim=0)


def minmax_encodings(mn, mx, num_steps, symmetric):
    """encoding_analyzer.py:425-481."""
    if num_steps <= 0:
        raise ValueError("The number of quantization bins cannot be less than or equal to 0.")
    ms = minimum_scale(num_steps)
    lo = torch.clamp(mn, max=0)
    hi = torch.clamp(mx, min=0)
    diff = (hi - lo) / num_steps
    adj = ms * (diff < ms)
    if symmetric:
        up = hi + math.floor(num_steps / 2) * adj
        dn = lo - math.ceil(num_steps / 2) * adj
        pos = math.floor(num_steps / 2)
        neg = math.ceil(num_steps / 2)
        extra = 1 if num_steps == 3 else 0
        delta = torch.maximum(up / (pos + extra), -dn / neg)
        dn = (-1 * neg) * delta
        up = pos * delta
    else:
        up = hi + num_steps * adj
        dn = lo
    up = torch.clamp(up, max=torch.finfo(mn.dtype).max).to(mn.dtype)
    dn = torch.clamp(dn, min=torch.finfo(mx.dtype).min).to(mx.dtype)
    return dn, up


# --------------------------------------------------------------------------- #
# histogram observer (encoding_analyzer.py:121-338)
# --------------------------------------------------------------------------- #
@dataclass
class Hist:
    histogram: torch.Tensor = None
    bin_edges: torch.Tensor = None
    min: Optional[torch.Tensor] = None
    max: Optional[torch.Tensor] = None


def bin_edges(lo, hi, num_bins):
    """encoding_analyzer.py:221-229."""
    lo, hi = (
        torch.where(lo == hi, lo - 0.5, lo).float(),
        torch.where(lo == hi, hi + 0.5, hi).float(),
    )
    step = (hi - lo) / num_bins
    return torch.arange(0, num_bins + 1) * step + lo


def hist_slices(x, shape, block_size=None):
    """encoding_analyzer.py:148-187: the per-encoding slices in histogram order."""
    hshape = tuple(shape)
    if block_size is not None:
        bs = concrete_block_size(x.shape, shape, block_size)
        x = x.reshape(-1, *interleave(shape, bs))
        hshape = interleave(shape, 1)
    padded = (1,) * (x.dim() - len(hshape)) + tuple(hshape)
    count = 1
    for d in shape:
        count *= d
    for i in range(count):
        cur = x
        for axis, dim in enumerate(padded):
            if dim == 1:
                continue
            inner = 1
            for d in padded[axis + 1:]:
                inner *= d
            cur = torch.unsqueeze(torch.select(cur, axis, (i // inner) % dim), axis)
        yield cur


def hist_collect_one(sl, num_bins) -> Hist:
    """encoding_analyzer.py:193-209 for one slice."""
    fin = sl.isfinite()
    lo = torch.where(fin, sl, float("inf")).min()
    hi = torch.where(fin, sl, -float("inf")).max()
    edges = bin_edges(lo, hi, num_bins)
    h = torch.histc(sl.to(torch.float), bins=num_bins, min=edges[0], max=edges[-1])
    h[0] += torch.sum(sl < edges[0])
    h[-1] += torch.sum(sl > edges[-1])
    return Hist(h, edges, lo, hi)


def hist_collect(x, shape, num_bins, block_size=None) -> List[Hist]:
    return [hist_collect_one(sl, num_bins) for sl in hist_slices(x, shape, block_size)]


def _bin_num(width, lo, data, num_bins):
    """encoding_analyzer.py:231-234."""
    cap = torch.full(data.shape, num_bins - 1)
    return torch.minimum(((data - lo) / width).to(torch.int32), cap)


class HistObserver:
    """State machine of `_HistogramObserver` (encoding_analyzer.py:121-338)."""

    def __init__(self, shape, num_bins, growth_limit=None, block_size=None):
        if isinstance(shape, int):
            shape = (shape,)
        self.shape = tuple(shape)
        self.block_size = block_size
        self.num_bins = num_bins
        n = 1
        for d in self.shape:
            n *= d
        self.stats = [Hist() for _ in range(n)]
        self.growth_limit = float("inf") if growth_limit is None else growth_limit
        if self.growth_limit < 1.0:
            raise RuntimeError(f"Growth limit must be at least 1.0. Got {growth_limit}")
        self.limit = None

    def update(self, x) -> List[Hist]:
        new = hist_collect(x, self.shape, self.num_bins, self.block_size)
        self.merge(new, x)
        return new

    def merge(self, new: List[Hist], x):
        """encoding_analyzer.py:238-332."""
        B = self.num_bins
        if self.stats[0].histogram is None:
            self.stats = new
            lo0 = torch.tensor([h.bin_edges[0] for h in new])
            hi0 = torch.tensor([h.bin_edges[-1] for h in new])
            rng = hi0 - lo0
            left = (lo0 - rng * self.growth_limit / 2).flatten()
            right = (hi0 + rng * self.growth_limit / 2).flatten()
            self.limit = torch.stack((left, right), dim=1)
            return
        for k, (nw, sl) in enumerate(zip(new, hist_slices(x, self.shape, self.block_size))):
            cur = self.stats[k]
            left, right = self.limit[k]
            lo = nw.min.clamp(left, cur.bin_edges[0])
            hi = nw.max.clamp(cur.bin_edges[-1], right)
            if lo == cur.min and hi == cur.max:
                carried = cur.histogram
            else:
                dst_w = (hi - lo) / B
                src_w = cur.bin_edges[1] - cur.bin_edges[0]
                carried = torch.zeros(B)
                src_start = cur.bin_edges[:-1]
                dst_idx = _bin_num(dst_w, lo, src_start, B)
                dst_end = lo + dst_w * (dst_idx + 1)
                part = torch.round(((dst_end - src_start) / src_w) * cur.histogram)
                first = torch.minimum(part, cur.histogram)
                carried.index_add_(dim=0, index=dst_idx, source=first)
                split = (first < cur.histogram).nonzero().flatten()
                oth_idx = _bin_num(dst_w, lo, src_start + dst_w, B)
                rest = cur.histogram - first
                carried.index_add_(dim=0, index=oth_idx[split], source=rest[split])
            h = torch.histc(sl.to(torch.float), bins=B, min=lo, max=hi)
            h += carried
            h[0] += torch.sum(sl < lo)
            h[-1] += torch.sum(sl > hi)
            self.stats[k] = Hist(h, bin_edges(lo, hi, B), lo, hi)


# --------------------------------------------------------------------------- #
# percentile (encoding_analyzer.py:501-534, 600-650)
# --------------------------------------------------------------------------- #
def adjust_min_max(lo, hi, num_steps, symmetric):
    """encoding_analyzer.py:501-534 (operates on 0-d tensors)."""
    ms = minimum_scale(num_steps)
    lo = torch.minimum(lo, torch.zeros_like(lo))
    hi = torch.maximum(hi, torch.zeros_like(hi))
    lo.clamp_(min=torch.finfo(hi.dtype).min, max=0)
    hi.clamp_(min=0, max=torch.finfo(hi.dtype).max)
    thr = (hi - lo) / num_steps
    if symmetric:
        lo[thr < ms] -= ms * math.ceil(num_steps / 2)
        hi[thr < ms] += ms * math.floor(num_steps / 2)
    else:
        hi[thr < ms] += ms * num_steps
    if symmetric:
        pos = math.floor(num_steps / 2)
        neg = math.ceil(num_steps / 2)
        delta = max(hi / pos, -lo / neg)
        lo = (-1 * neg) * delta
        hi = pos * delta
    return lo, hi


def percentile_encodings(stats: List[Hist], shape, percentile, num_steps, symmetric):
    """encoding_analyzer.py:600-650."""
    los, his = [], []
    for st in stats:
        cs = torch.cumsum(st.histogram, dim=0)
        hi_i = torch.searchsorted(cs, cs[-1] * percentile / 100)
        lo_i = torch.searchsorted(cs, cs[-1] * (1 - percentile / 100))
        if percentile == 100:
            lo_i, hi_i = 0, -1
        lo, hi = adjust_min_max(st.bin_edges[lo_i], st.bin_edges[hi_i], num_steps, symmetric)
        los.append(lo)
        his.append(hi)
    lo = torch.tensor(los, dtype=stats[0].min.dtype).reshape(shape)
    hi = torch.tensor(his, dtype=stats[0].max.dtype).reshape(shape)
    return lo, hi


# --------------------------------------------------------------------------- #
# SQNR / TF-enhanced search (encoding_analyzer.py:695-899)
# --------------------------------------------------------------------------- #
def _clamp_candidates(lo, hi, num_steps, deltas, offsets):
    """encoding_analyzer.py:797-820."""
    ms = minimum_scale(num_steps)
    tmin = deltas[:, :, None] * offsets[:, None, :]
    tmax = tmin + deltas[:, :, None] * num_steps
    tmin = torch.max(lo[:, None, None], tmin)
    tmax = torch.min(hi[:, None, None], tmax)
    d = (tmax - tmin) / num_steps
    d = torch.max(d, torch.tensor([ms], dtype=d.dtype))
    return d, torch.round(tmin / d)


def sqnr_candidates(stats: List[Hist], num_steps, symmetric, asym_deltas, sym_deltas, num_offsets):
    """encoding_analyzer.py:728-795: returns (deltas, offsets) as (H,D,O) tensors
    (or (H,D,1)/(1,1,1) in symmetric mode)."""
    ms = minimum_scale(num_steps)
    lo = torch.stack([s.min for s in stats])
    hi = torch.stack([s.max for s in stats])
    lo = torch.min(lo, torch.zeros_like(lo))
    hi = torch.max(hi, torch.zeros_like(hi))
    hi = torch.max(hi, lo + ms * num_steps)
    if symmetric:
        dmax = 2 * torch.max(hi, -lo).to(torch.float32) / num_steps
        offs = torch.full((1,), (-num_steps) // 2, dtype=torch.float32)
        space = torch.arange(1, 1 + sym_deltas, 1, dtype=torch.float32)
        d = dmax[:, None] * space[None, :] / (sym_deltas - 1)
        d = torch.max(d, torch.tensor([ms], dtype=torch.float32))
        return d[:, :, None], offs[:, None, None]
    dmax = (hi - lo).to(torch.float32) / num_steps
    obs_off = torch.round(lo / dmax)
    obs_min = dmax * obs_off
    obs_max = obs_min + dmax * num_steps
    space = torch.arange(1, 1 + asym_deltas, 1, dtype=torch.float32)
    d = dmax[:, None] * space[None, :] / (asym_deltas - 1)
    n_off = min(num_steps + 2, num_offsets)
    step = num_steps / (n_off - 2)
    offs = torch.round(torch.arange(-num_steps, step, step, dtype=torch.float32))
    offs = offs[None, :].expand(lo.shape[0], -1)
    offs = torch.concat((offs, obs_off[:, None]), dim=1)
    return _clamp_candidates(obs_min, obs_max, num_steps, d, offs)


def sqnr_noise(stats: List[Hist], deltas, offsets, num_steps, p=2.0, gamma=3.0):
    """encoding_analyzer.py:842-899: (H,D,O) noise tensor."""
    hists = torch.stack([s.histogram for s in stats])
    edges = torch.stack([s.bin_edges for s in stats])
    w = edges[:, 1] - edges[:, 0]
    k = torch.arange(0, edges.shape[1] - 1, dtype=deltas.dtype)
    mids = (edges[:, 0] + w / 2)[:, None] + w[:, None] * k[None, :]
    ob = offsets[:, :, :, None]
    db = deltas[:, :, :, None]
    q = mids[:, None, None, :].div(db).sub(ob).round()
    if gamma != 1.0:
        clipped = torch.logical_or(q < 0, q > num_steps)
    q = q.clamp_(0, num_steps).add_(ob).mul_(db)
    err = torch.abs(q.sub_(mids[:, None, None, :])).pow_(p).mul_(hists[:, None, None, :])
    if gamma != 1.0:
        err = torch.where(clipped, err * gamma, err)
    return torch.sum(err, dim=-1)


def sqnr_encodings(stats: List[Hist], shape, num_steps, symmetric, *, asym_deltas=17, sym_deltas=101,
                   num_offsets=21, gamma=3.0, p=2.0, max_parallelism=64):
    """encoding_analyzer.py:695-726 + 822-839.  Returns (min, max, best_delta, best_offset, argmin)."""
    if num_steps <= 0:
        raise ValueError("The number of quantization bins cannot be less than or equal to 0.")
    bd, bo, bi = [], [], []
    for c in range(0, len(stats), max_parallelism):
        chunk = stats[c:c + max_parallelism]
        d, o = sqnr_candidates(chunk, num_steps, symmetric, asym_deltas, sym_deltas, num_offsets)
        noise = sqnr_noise(chunk, d, o, num_steps, p, gamma)
        _, idx = torch.min(noise.flatten(start_dim=1), dim=1)
        bd.append(torch.gather(d.flatten(start_dim=1), 1, idx[:, None]))
        bo.append(o if o.numel() == 1 else torch.gather(o.flatten(start_dim=1), 1, idx[:, None]))
        bi.append(idx)
    off = bo[0] if symmetric else torch.cat(bo)
    delta = torch.cat(bd)
    lo = off * delta
    hi = lo + num_steps * delta
    lo = lo.to(stats[0].min.dtype)
    hi = hi.to(stats[0].max.dtype)
    return lo.view(shape), hi.view(shape), delta, off, torch.cat(bi)


# --------------------------------------------------------------------------- #
# Float fake-cast (quantization/float/quantizer.py:634-716, fp_quantization.py:148-214)
# --------------------------------------------------------------------------- #
FLOAT_TORCH_DTYPES = {
    (5, 10, False, False): torch.float16,
    (8, 7, False, False): torch.bfloat16,
    (4, 3, True, False): torch.float8_e4m3fn,
    (4, 3, True, True): torch.float8_e4m3fnuz,
    (5, 2, False, False): torch.float8_e5m2,
    (5, 2, True, True): torch.float8_e5m2fnuz,
}


def float_max(exponent_bits, mantissa_bits, finite, unsigned_zero) -> float:
    """_finfo.max (float/_finfo.py:66-86)."""
    key = (exponent_bits, mantissa_bits, finite, unsigned_zero)
    if key in FLOAT_TORCH_DTYPES:
        return torch.finfo(FLOAT_TORCH_DTYPES[key]).max
    if key == (2, 1, True, False):
        return 6.0
    if not finite and not unsigned_zero:
        exponent_max = 2 ** exponent_bits - 1
        return (2 - 2 ** -mantissa_bits) * 2 ** (exponent_max - exponent_max // 2 - 1)
    raise RuntimeError("Maximum representable value of this format is unknown")


def fake_cast_to_ieee_float(x, maxval, exponent_bits, mantissa_bits, finite=True):
    """fp_quantization.py:148-214, for a tensor x and a Python-float maxval."""
    import numpy as np

    maxval = torch.tensor(maxval, dtype=torch.float64)
    bias = 2 ** exponent_bits - torch.log2(maxval) + np.log2(2 - 2 ** (-mantissa_bits)) - 1
    xc = x.clamp(-maxval, maxval)
    log_scales = torch.floor(torch.log2(torch.abs(xc)) + bias).detach()
    log_scales = torch.clamp(log_scales, 1.0)
    scales = 2.0 ** (log_scales - mantissa_bits - bias)
    out = torch.round(xc / scales) * scales
    if not finite:
        out = torch.where(x.isinf(), x, out)
    return out.to(x.dtype)


def float_quantize(x, scale, exponent_bits, mantissa_bits, finite, unsigned_zero, block_size=None):
    """_float_quantize (float/quantizer.py:687-706): divide, clamp, fake-cast, every step a torch op on the promoted
    dtype of (x, scale)."""
    key = (exponent_bits, mantissa_bits, finite, unsigned_zero)
    mx = float_max(*key)
    shape = x.shape
    xb, sb, _ = _blocked_views(x, scale, None, block_size)
    t = torch.div(xb, sb).reshape(shape) if block_size else torch.div(x, scale)
    t = t.clamp(-mx, mx)
    if key in FLOAT_TORCH_DTYPES:
        return t.to(FLOAT_TORCH_DTYPES[key]).to(t.dtype)
    if not unsigned_zero:
        return fake_cast_to_ieee_float(t, mx, exponent_bits, mantissa_bits, finite=finite)
    raise NotImplementedError("Fake-casting to this format is not implemented")


def float_dequantize(t, scale, block_size=None):
    """FloatEncoding.dequantize (float/encoding.py:154-165): blockwise torch.mul."""
    if block_size:
        tb, sb, _ = _blocked_views(t, scale, None, block_size)
        return torch.mul(tb, sb).reshape(t.shape)
    return torch.mul(t, scale)


def float_qdq(x, scale, exponent_bits, mantissa_bits, finite, unsigned_zero, block_size=None):
    """_float_quantize_dequantize (float/quantizer.py:634-656): quantize, then multiply by the scale."""
    t = float_quantize(x, scale, exponent_bits, mantissa_bits, finite, unsigned_zero, block_size)
    return float_dequantize(t, scale, block_size)
