"""Recovering the grid of a tensor that was quantized before it got here.

Counterpart of ``_decompose_prequantized_tensor`` and its helpers (aimet_torch/utils.py:1687-2300): a weight that
already lies on a symmetric integer grid, ``w = (code + shift) * scale`` per block, is taken apart into the codes and
the per-block scale, so that its quantizer can be given exactly that grid instead of one calibrated from min/max
(nn/base.py:355-383).  A tensor that does not lie on such a grid raises ``_DecompositionError`` and the caller
calibrates as usual.

The computation, per block of the scale's layout (all of it in float32 whatever the tensor's dtype):

1.  A cheap refusal: 64 blocks, ``2 * levels`` elements each; more distinct magnitudes than the grid has levels and
    the tensor cannot be on it (utils.py:2098-2118).
2.  Two guesses of ``k = anchor / step`` (anchor: largest magnitude, doubled on the half-integer grid): from the
    smallest non-zero magnitude and from the smallest gap between sorted magnitudes (utils.py:1842-1880).  The
    candidate divisors of the whole tensor are the integers within 2 of any block's rounded guess, plus 1 and the
    largest possible one (utils.py:1779-1808).
3.  Every candidate is scored per block by the share of non-zero elements off its grid -- further from a grid point
    than three storage roundings of the element's own magnitude -- and by the mean distance to the grid; the smallest
    divisor among those that fit about as well as the best one wins (utils.py:1883-1963).  Storage rounding is read
    off the bit patterns: float32 values whose low 16 (13) mantissa bits are all zero were bfloat16 (float16) once
    (utils.py:1741-1776).
4.  The scale is re-estimated as the median of ``|w| / |code + shift|`` and polished by alternating between codes and
    the least-squares scale for them, keeping per block whatever reconstructs best (utils.py:1966-2022).
5.  The tensor is accepted if at least 90 % of its blocks fit some grid and the relative reconstruction error is at
    the level of the storage rounding (utils.py:2255-2283).

Blocks are independent but for the candidate list, the storage precision and the final verdict, so the rows are
worked through in slabs of bounded size; within a slab several candidates are scored per pass, as many as a fixed
element budget allows.  Everything runs as torch operations on the tensor's own device; the host reads back four
small results (refusal flag, bit fingerprint, candidate list, verdict).
"""

from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

from aimet_amd.quantization._utils import _get_minimum_scale, concretize_block_size

__all__ = ["_DecompositionError", "_decompose_prequantized_tensor"]


class _DecompositionError(RuntimeError):
    """The tensor does not lie on a grid of the requested kind (utils.py:1687)."""


# utils.py:1691-1738
_HALF_ULP = {"bf16": 2.0 ** -8, "fp16": 2.0 ** -11, "fp32": 2.0 ** -20}
_NOISE_ROUNDINGS = 3.0       # an element may be this many storage roundings away from its grid point
_OFFGRID_SLACK = 0.005       # candidates this close to the best off-grid share stay in the race
_FIT_SLACK = 0.5             # ... and of those, the ones whose mean distance is within 1.5 x the best
_OFFGRID_LIMIT = 0.05        # a block whose winner still has more than this share off the grid is not on a grid
_MIN_MATCHED_BLOCKS = 0.90
_RELRMS_ROUNDINGS = 5.0
_RELRMS_FLOOR = 1e-3
_POLISH_ROUNDS = 4
_TINY = 1e-12
# rows are worked through in slabs of at most this many elements (utils.py:1736-1738) ...
_DECOMPOSE_CHUNK_NUMEL = 2 ** 24
# ... and candidates are scored in groups whose [rows, candidates, elements] temporaries stay below this many elements
_SCORE_GROUP_NUMEL = 2 ** 25


class _Blocks:
    """The tensor seen as ``[blocks, elements per block]`` in the order of the scale's elements, and the way back."""

    def __init__(self, t: torch.Tensor, scale_shape: Sequence[int], block_size: Optional[Sequence[int]]):
        inner = concretize_block_size(tuple(t.shape), tuple(scale_shape), block_size or tuple(-1 for _ in scale_shape))
        per_dim = (*t.shape[: t.dim() - len(inner)], *inner)
        split: List[int] = []
        for extent, b in zip(t.shape, per_dim):
            split += [extent // b, b]
        nd = len(split)
        self._order = (*range(0, nd, 2), *range(1, nd, 2))
        self._shape = tuple(t.shape)
        moved = t.reshape(split).permute(self._order)
        self._moved_shape = tuple(moved.shape)
        self.count = math.prod(split[0::2])
        self.rows = moved.reshape(self.count, -1)

    def restore(self, rows: torch.Tensor) -> torch.Tensor:
        back = [0] * len(self._order)
        for pos, axis in enumerate(self._order):
            back[axis] = pos
        return rows.reshape(self._moved_shape).permute(back).reshape(self._shape)


def _too_many_magnitudes(rows: torch.Tensor, levels: int) -> torch.Tensor:
    """0-dim bool: one of the first 64 blocks shows more than ``levels`` distinct magnitudes among its first
    ``2 * levels`` elements (utils.py:2104-2118)."""
    head = rows[:64, : 2 * levels].float().abs().sort(dim=1).values
    distinct = (head[:, 1:] != head[:, :-1]).sum(dim=1) + 1
    return (distinct > levels).any()


def _anchor(absmax: torch.Tensor, shift: float) -> torch.Tensor:
    # on the half-integer grid the stored values are odd multiples of half a step
    return absmax * 2.0 if shift == 0.5 else absmax


def _survey(x: torch.Tensor, shift: float):
    """Per block of one float32 slab: largest magnitude, smallest non-zero magnitude, the two divisor guesses; and
    the slab's bit fingerprint (any non-zero, any of the low 16 bits set, any of the low 13 bits set)."""
    mag = x.abs()
    absmax = mag.amax(dim=1)
    smallest = torch.where(mag > 0, mag, mag.new_full((), math.inf)).amin(dim=1)
    anchor = _anchor(absmax, shift)
    by_smallest = absmax / smallest.clamp(min=_TINY)
    fallback = anchor.clamp(min=_TINY)
    if x.shape[1] > 1:
        mag = mag.sort(dim=1).values
        gap = mag[:, 1:] - mag[:, :-1]
        gap = torch.where(gap > _TINY, gap, gap.new_full((), math.inf)).amin(dim=1)
        gap = torch.where(torch.isfinite(gap), gap, fallback)  # all magnitudes equal: one step
    else:
        gap = fallback
    by_gap = anchor / gap.clamp(min=_TINY)
    bits = x.contiguous().view(torch.int32)
    fingerprint = torch.stack([(x != 0).any(), (bits & 0xFFFF).ne(0).any(), (bits & 0x1FFF).ne(0).any()])
    return absmax, smallest, by_smallest, by_gap, fingerprint


def _storage_half_ulp(fingerprint: Sequence[bool]) -> float:
    """utils.py:1741-1776, from the fingerprint of the whole tensor.  The reference takes the tightest verdict over
    its slabs that hold a non-zero, which is the same thing: a slab is bfloat16-like iff none of its low 16 bits is
    set, and zeros set none."""
    any_value, low16, low13 = fingerprint
    if not any_value or low13:
        return _HALF_ULP["fp32"]
    return _HALF_ULP["fp16"] if low16 else _HALF_ULP["bf16"]


def _candidates(guesses: Sequence[torch.Tensor], active: torch.Tensor, largest: int, odd_only: bool) -> torch.Tensor:
    """Sorted int64 divisors to try (utils.py:1779-1808)."""
    device = active.device
    picked = [g[active] for g in guesses]
    # a guess beyond the range cannot put a divisor into it once it is further than the window away
    centres = torch.cat(picked).clamp(0, largest + 3).round().long().unique()
    if centres.numel() == 0:
        centres = torch.ones(1, dtype=torch.long, device=device)
    window = (centres[:, None] + torch.arange(-2, 3, device=device)).flatten()
    cand = torch.cat([window, torch.tensor([1, largest], device=device)]).unique()
    cand = cand[(cand >= 1) & (cand <= largest)]
    if odd_only:
        cand = cand[cand % 2 == 1]
        if cand.numel() == 0:
            cand = torch.ones(1, dtype=torch.long, device=device)
    return cand


def _score(x: torch.Tensor, absmax: torch.Tensor, cand: torch.Tensor, shift: float, half_ulp: float):
    """[rows, candidates] share of non-zero elements off the candidate's grid and mean distance to it
    (utils.py:1912-1946)."""
    rows, n = x.shape
    counted = x.abs() > _TINY
    population = counted.sum(dim=1, dtype=x.dtype).clamp(min=1)
    steps = (_anchor(absmax, shift)[:, None] / cand.to(x.dtype)[None, :]).clamp(min=_TINY)  # [rows, C]
    noise = _NOISE_ROUNDINGS * half_ulp
    off = x.new_empty((rows, cand.numel()))
    dist = x.new_empty((rows, cand.numel()))
    group = max(1, _SCORE_GROUP_NUMEL // max(1, rows * n))
    for lo in range(0, cand.numel(), group):
        hi = min(cand.numel(), lo + group)
        ratio = x[:, None, :] / steps[:, lo:hi, None]           # the stored magnitude in steps, signed
        code = ratio - shift
        away = (code.round() - code).abs_()
        del code
        miss = (ratio.abs_().mul_(noise) < away) & counted[:, None, :]
        del ratio
        off[:, lo:hi] = miss.sum(dim=2, dtype=torch.float) / population[:, None]
        del miss
        dist[:, lo:hi] = away.mul_(counted[:, None, :]).sum(dim=2) / population[:, None]
        del away
    return off, dist


def _pick(off: torch.Tensor, dist: torch.Tensor, cand: torch.Tensor, active: torch.Tensor):
    """Chosen divisor per block and whether the block is on its grid (utils.py:1948-1963)."""
    in_race = off <= off.amin(dim=1, keepdim=True) + _OFFGRID_SLACK
    best = torch.where(in_race, dist, dist.new_full((), math.inf)).amin(dim=1, keepdim=True)
    good = in_race & (dist <= best * (1.0 + _FIT_SLACK))
    # candidates are ascending: the first good one is the coarsest grid
    col = torch.where(in_race.any(dim=1), good.to(torch.uint8).argmax(dim=1), off.argmin(dim=1))
    on_grid = in_race.any(dim=1) & active & (off.gather(1, col[:, None]).squeeze(1) <= _OFFGRID_LIMIT)
    return cand[col], on_grid


def _codes_plus_shift(x: torch.Tensor, s: torch.Tensor, shift: float, qmin: int, qmax: int) -> torch.Tensor:
    return (x / s[:, None]).sub_(shift).round_().clamp_(qmin, qmax).add_(shift)


def _misfit(x: torch.Tensor, s: torch.Tensor, shift: float, qmin: int, qmax: int) -> torch.Tensor:
    return _codes_plus_shift(x, s, shift, qmin, qmax).mul_(s[:, None]).sub_(x).square_().sum(dim=1)


def _polish(x: torch.Tensor, absmax: torch.Tensor, k: torch.Tensor, shift: float, qmin: int, qmax: int) -> torch.Tensor:
    """Median seed, then codes <-> least-squares scale, the best reconstruction kept per block (utils.py:1966-2022)."""
    first = _anchor(absmax, shift) / k.to(x.dtype)
    level = _codes_plus_shift(x, first, shift, qmin, qmax)
    usable = (level.abs() > _TINY) & (x.abs() > _TINY)
    ratio = (x / torch.where(level.abs() > _TINY, level, level.new_ones(()))).abs_()
    del level
    seed = torch.where(usable, ratio, ratio.new_full((), math.nan)).nanmedian(dim=1).values
    del ratio, usable
    seed = torch.where(torch.isfinite(seed) & (seed > 0), seed, first)

    kept, kept_misfit = seed, _misfit(x, seed, shift, qmin, qmax)
    s = seed
    for _ in range(_POLISH_ROUNDS):
        level = _codes_plus_shift(x, s, shift, qmin, qmax)
        fitted = (x * level).sum(dim=1) / level.square_().sum(dim=1).clamp(min=_TINY)
        del level
        fitted = torch.where(fitted > _TINY, fitted, s)
        misfit = _misfit(x, fitted, shift, qmin, qmax)
        better = misfit < kept_misfit
        kept = torch.where(better, fitted, kept)
        kept_misfit = torch.where(better, misfit, kept_misfit)
        s = fitted
    return kept


@torch.no_grad()
def _decompose_prequantized_tensor(input_qdq: torch.Tensor, qmin: int, qmax: int, scale_shape: Tuple[int, ...],
                                   block_size: Optional[Tuple[int, ...]] = None, zero_point_shift: float = 0.0,
                                   return_input_q: bool = True, _probed: bool = False
                                   ) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
    """``input_qdq -> (input_q, scale)`` with ``input_qdq ~= (input_q + zero_point_shift) * scale`` blockwise, or
    ``_DecompositionError`` (utils.py:2024-2300).  ``input_q`` (float32, the tensor's shape) is None when
    ``return_input_q`` is false; ``scale`` is float32 of shape ``scale_shape``.  ``_probed``: the caller has already
    run the cheap refusal test (step 1) and it passed."""
    if len(scale_shape) > input_qdq.dim():
        raise ValueError("the scale has more dimensions than the tensor")
    if zero_point_shift not in (0.0, 0.5):
        raise ValueError(f"zero_point_shift must be 0.0 (dense grid) or 0.5 (shifted grid), got {zero_point_shift}")
    shift = float(zero_point_shift)
    largest_level = max(abs(qmin), abs(qmax))
    floor = _get_minimum_scale(qmax - qmin)
    blocks = _Blocks(input_qdq, scale_shape, block_size)
    rows = blocks.rows
    device = rows.device

    levels = largest_level + 1
    if not _probed and rows.shape[1] > levels and rows.shape[0] > 0:
        if bool(_too_many_magnitudes(rows, levels)):
            raise _DecompositionError(f"One or more blocks exceed {levels} distinct values")

    per_slab = max(1, _DECOMPOSE_CHUNK_NUMEL // max(rows.shape[1], 1))
    slabs = rows.split(per_slab) if blocks.count > 0 else (rows,)

    survey = [_survey(slab.float(), shift) for slab in slabs]
    absmax = torch.cat([s[0] for s in survey])
    smallest = torch.cat([s[1] for s in survey])
    guesses = [torch.cat([s[2] for s in survey]), torch.cat([s[3] for s in survey])]
    half_ulp = _storage_half_ulp(torch.stack([s[4] for s in survey]).any(dim=0).tolist())
    del survey
    active = torch.isfinite(smallest) & (absmax > 0)
    cand = _candidates(guesses, active, 2 * largest_level + 1 if shift == 0.5 else largest_level, shift == 0.5)
    del guesses

    scales, on_grid, codes = [], [], []
    err2 = torch.zeros((), dtype=torch.float64, device=device)
    norm2 = torch.zeros((), dtype=torch.float64, device=device)
    top_code = torch.zeros((), device=device)
    at = 0
    for slab in slabs:
        x = slab.float()
        sl = slice(at, at + x.shape[0])
        at += x.shape[0]
        off, dist = _score(x, absmax[sl], cand, shift, half_ulp)
        k, fits = _pick(off, dist, cand, active[sl])
        del off, dist
        s = _polish(x, absmax[sl], k, shift, qmin, qmax)
        # a block of zeros has no grid; every other scale keeps the floor the quantizers keep (utils.py:2209-2213)
        s = torch.where(active[sl], s.clamp_min(floor), s.new_full((), floor))
        q = (x / s[:, None]).sub_(shift).round_().clamp_(qmin, qmax)
        back = (q + shift).mul_(s[:, None]).sub_(x)
        err2 += torch.linalg.vector_norm(back).double().square()
        norm2 += torch.linalg.vector_norm(x).double().square()
        del back
        if q.numel():
            top_code = torch.maximum(top_code, q.abs().amax())
        scales.append(s)
        on_grid.append(fits)
        if return_input_q:
            codes.append(q)
        del x, q

    scale = torch.cat(scales)
    matched = (torch.cat(on_grid) & active) | ~active  # a block of zeros reconstructs exactly
    share = matched.float().mean() if blocks.count > 0 else torch.zeros((), device=device)
    relrms = err2.sqrt() / norm2.sqrt().clamp(min=_TINY)
    share, relrms, top_code = torch.stack([share.double(), relrms, top_code.double()]).tolist()
    gate = max(_RELRMS_ROUNDINGS * half_ulp, _RELRMS_FLOOR)
    if not (int(top_code) > 0 and share >= _MIN_MATCHED_BLOCKS and relrms <= gate):
        raise _DecompositionError(f"not QDQ-like: matched={share:.4f}, relRMS={relrms:.2e} (gate={gate:.2e}, "
                                  f"ulp_rel={half_ulp:.2e}), code_absmax={int(top_code)}")

    scale = scale.reshape(tuple(scale_shape))
    if not return_input_q:
        return None, scale
    return blocks.restore(torch.cat(codes)), scale
