"""CPU restatement, in numpy float32, of the reference's lossless decomposition of an already-quantized tensor.

TEST INFRASTRUCTURE ONLY.  Nothing under ``aimet_amd/`` may import this module; only ``tests/`` use it, as the
checker of ``aimet_amd/quantization/_decompose.py``.

Reference followed (``AT`` = TrainingExtensions/torch/src/python/aimet_torch): AT/utils.py:1687-2300
(``_storage_ulp_rel`` :1741, ``_candidate_divisors`` :1779, ``_divisor_estimates`` :1842, ``_select_divisor`` :1883,
``_refine_scale`` :1966, ``_decompose_prequantized_tensor`` :2024).  The whole tensor is one slab here (the reference
works through slabs of 2**24 elements with the same per-block arithmetic); one candidate divisor at a time, as the
reference does.

Pinning: the reference's own tests of this function state their expectations in closed form (the scale and codes a
tensor was built from, a lower bound on the reconstruction SQNR, optimality against the closed-form least-squares
scale, which inputs must be refused and with what message): AT test/python/v2/test_utils.py:411-706 and
v2/nn/test_true_quant.py:2456-2475.  tests/test_decompose_cpu.py runs every one of them against this module.  The
reference's sums are float32 torch reductions whose order differs from numpy's pairwise sums, so scales agree with
the reference's to float32 rounding of those sums (a few 1e-7 relative), not bit for bit; codes of a tensor that is
on a grid agree exactly.
"""

from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np

F = np.float32
EPS = 1e-12

ULP_REL_BF16 = 2.0 ** -8
ULP_REL_FP16 = 2.0 ** -11
ULP_REL_FP32 = 2.0 ** -20
ULP_SAFETY = 3.0
VALID_MARGIN = 0.005
FIT_MARGIN = 0.5
ABS_OFFGRID_CEIL = 0.05
MIN_MATCHED_FRAC = 0.90
RECON_RELRMS_MULT = 5.0
RECON_RELRMS_FLOOR = 1e-3
LS_ITERS = 4


class DecompositionError(RuntimeError):
    pass


def minimum_scale(num_steps: int) -> float:
    """_aimet_common/quantsim.py:538-559"""
    return min(float(np.finfo(np.float32).eps), 0.01 / num_steps)


def block_rows(shape: Sequence[int], scale_shape: Sequence[int], block_size: Optional[Sequence[int]]):
    """utils.py:2070-2096: (split shape, permutation) that turn the tensor into [blocks, elements per block]."""
    n = len(scale_shape)
    bs = list(block_size) if block_size else [-1] * n
    bs = [1 if scale_shape[i] > 1 else -1 for i in range(n - len(bs))] + bs
    tail = list(shape)[len(shape) - n:] if n else []
    bs = [b if b != -1 else tail[i] // scale_shape[i] for i, b in enumerate(bs)]
    full = list(shape[: len(shape) - n]) + bs
    split = []
    for d, b in zip(shape, full):
        split += [d // b, b]
    nd = len(split)
    perm = list(range(0, nd, 2)) + list(range(1, nd, 2))
    return split, perm


def storage_ulp_rel(x: np.ndarray) -> float:
    """utils.py:1741-1776 for float32 values (the caller upcasts first, :2140)."""
    flat = np.ascontiguousarray(x, dtype=F).reshape(-1)
    if not np.any(flat != 0):
        return ULP_REL_FP32
    bits = flat.view(np.int32)
    if not np.any(bits & 0xFFFF):
        return ULP_REL_BF16
    if not np.any(bits & 0x1FFF):
        return ULP_REL_FP16
    return ULP_REL_FP32


def divisor_estimates(x: np.ndarray, absmax: np.ndarray, min_nonzero: np.ndarray, zps: float):
    """utils.py:1842-1880"""
    anchor = (F(2.0) if zps == 0.5 else F(1.0)) * absmax
    k_min = absmax / np.maximum(min_nonzero, F(EPS))
    xs = np.sort(np.abs(x), axis=1)
    gaps = xs[:, 1:] - xs[:, :-1]
    fallback = np.maximum(anchor, F(EPS))
    if gaps.shape[1] == 0:
        min_gap = fallback
    else:
        gaps = np.where(gaps <= F(EPS), F(np.inf), gaps)
        min_gap = gaps.min(axis=1)
        min_gap = np.where(np.isfinite(min_gap), min_gap, fallback)
    with np.errstate(over="ignore"):
        k_gap = anchor / np.maximum(min_gap, F(EPS))
    return k_min.astype(F), k_gap.astype(F)


def candidate_divisors(k_ests, active: np.ndarray, max_k: int, odd_only: bool) -> np.ndarray:
    """utils.py:1779-1808"""
    centres = []
    for k in k_ests:
        if active.any():
            kk = np.rint(k[active].astype(np.float64))
            # the reference converts to int64 unclamped; anything outside [1 - 2, max_k + 2] is dropped below anyway
            kk = kk[np.isfinite(kk) & (np.abs(kk) < 2.0 ** 62)]
            centres.append(kk.astype(np.int64))
    centres = np.unique(np.concatenate(centres)) if centres else np.array([1], dtype=np.int64)
    around = (centres[:, None] + np.arange(-2, 3)[None, :]).reshape(-1)
    cand = np.unique(np.concatenate([around, np.array([1, max_k], dtype=np.int64)]))
    cand = cand[(cand >= 1) & (cand <= max_k)]
    if odd_only:
        cand = cand[cand % 2 == 1]
        if cand.size == 0:
            cand = np.array([1], dtype=np.int64)
    return cand


def select_divisor(x, absmax, min_nonzero, cand, zps: float, ulp_rel: float):
    """utils.py:1883-1963"""
    rows = x.shape[0]
    nonzero = np.abs(x) > F(EPS)
    nnz = np.maximum(nonzero.sum(axis=1).astype(F), F(1))
    active = np.isfinite(min_nonzero) & (absmax > 0)
    anchor = (F(2.0) if zps == 0.5 else F(1.0)) * absmax
    rel_noise = F(ULP_SAFETY * ulp_rel)
    offgrid = np.ones((rows, cand.size), dtype=F)
    meandev = np.ones((rows, cand.size), dtype=F)
    with np.errstate(all="ignore"):
        for j, k in enumerate(cand.tolist()):
            s_k = np.maximum(anchor / F(k), F(EPS))
            r = (x / s_k[:, None]).astype(F)
            shifted = (r - F(zps)).astype(F)
            dev = np.abs(np.rint(shifted) - shifted).astype(F)
            thr = (np.abs(r) * rel_noise).astype(F)
            bad = (thr < dev) & nonzero
            offgrid[:, j] = bad.sum(axis=1).astype(F) / nnz
            meandev[:, j] = (dev * nonzero).astype(F).sum(axis=1, dtype=F) / nnz
        min_off = offgrid.min(axis=1, keepdims=True)
        valid = offgrid <= min_off + F(VALID_MARGIN)
        masked = np.where(valid, meandev, F(np.inf))
        best_fit = masked.min(axis=1, keepdims=True)
        fit_ok = valid & (meandev <= best_fit * F(1.0 + FIT_MARGIN))
    has_valid = valid.any(axis=1)
    smallest_good = fit_ok.argmax(axis=1)
    best_resid = offgrid.argmin(axis=1)
    col = np.where(has_valid, smallest_good, best_resid)
    chosen_off = offgrid[np.arange(rows), col]
    return cand[col], has_valid & active & (chosen_off <= F(ABS_OFFGRID_CEIL))


def _lower_nanmedian(a: np.ndarray) -> np.ndarray:
    """torch.nanmedian: of an even number of values the lower middle one; NaN when there is none."""
    out = np.full(a.shape[0], np.nan, dtype=F)
    for i, row in enumerate(a):
        v = np.sort(row[~np.isnan(row)])
        if v.size:
            out[i] = v[(v.size - 1) // 2]
    return out


def refine_scale(x, k_chosen, zps: float, qmin: int, qmax: int, iters: int = LS_ITERS):
    """utils.py:1966-2022"""
    absmax = np.abs(x).max(axis=1) if x.shape[1] else np.zeros(x.shape[0], dtype=F)
    anchor = (F(2.0) if zps == 0.5 else F(1.0)) * absmax
    with np.errstate(all="ignore"):
        s_anchor = (anchor / k_chosen.astype(F)).astype(F)

        def levels(s):
            r = (x / s[:, None]).astype(F) - F(zps)
            return (np.clip(np.rint(r), F(qmin), F(qmax)) + F(zps)).astype(F)

        def sse(s):
            d = (levels(s) * s[:, None]).astype(F) - x
            return (d * d).astype(F).sum(axis=1, dtype=F)

        denom = levels(s_anchor)
        valid = np.abs(denom) > F(EPS)
        safe = np.where(valid, denom, F(1.0))
        ratio = np.abs(x / safe).astype(F)
        valid &= np.abs(x) > F(EPS)
        ratio = np.where(valid, ratio, F(np.nan))
        s_med = _lower_nanmedian(ratio)
        s_med = np.where(np.isfinite(s_med) & (s_med > 0), s_med, s_anchor).astype(F)

        best_s, best_sse, s = s_med, sse(s_med), s_med
        for _ in range(iters):
            denom = levels(s)
            num = (x * denom).astype(F).sum(axis=1, dtype=F)
            den = np.maximum((denom * denom).astype(F).sum(axis=1, dtype=F), F(EPS))
            s_new = (num / den).astype(F)
            s_new = np.where(s_new > F(EPS), s_new, s)
            sse_new = sse(s_new)
            improve = sse_new < best_sse
            best_s = np.where(improve, s_new, best_s)
            best_sse = np.where(improve, sse_new, best_sse)
            s = s_new
    return best_s.astype(F)


def decompose(input_qdq: np.ndarray, qmin: int, qmax: int, scale_shape: Tuple[int, ...],
              block_size: Optional[Tuple[int, ...]] = None, zps: float = 0.0):
    """utils.py:2024-2300 -> (input_q float32 of the input's shape, scale float32 of scale_shape); the input is the
    tensor already upcast to float32 (exact for float16 / bfloat16 storage)."""
    if len(scale_shape) > input_qdq.ndim:
        raise ValueError
    if zps not in (0.0, 0.5):
        raise ValueError(f"zero_point_shift must be 0.0 (dense grid) or 0.5 (shifted grid), got {zps}")
    max_level = max(abs(qmin), abs(qmax))
    min_scale = F(minimum_scale(qmax - qmin))
    split, perm = block_rows(input_qdq.shape, scale_shape, block_size)
    moved = np.asarray(input_qdq, dtype=F).reshape(split).transpose(perm)
    num_blocks = int(np.prod(split[0::2])) if split else 1
    x = moved.reshape(num_blocks, -1)

    num_levels = max_level + 1
    if x.shape[1] > num_levels:  # :2104-2118
        xs = np.sort(np.abs(x[:64, : num_levels * 2]), axis=1)
        distinct = (xs[:, 1:] != xs[:, :-1]).sum(axis=1) + 1
        if np.any(distinct > num_levels):
            raise DecompositionError(f"One or more blocks exceed {num_levels} distinct values")

    x_abs = np.abs(x)
    absmax = x_abs.max(axis=1) if x.shape[1] else np.zeros(num_blocks, dtype=F)
    min_nonzero = np.where(x_abs <= 0, F(np.inf), x_abs).min(axis=1) if x.shape[1] else np.full(num_blocks, np.inf, F)
    ulp_rel = storage_ulp_rel(x) if np.any(x != 0) else ULP_REL_FP32
    with np.errstate(all="ignore"):
        k_min, k_gap = divisor_estimates(x, absmax, min_nonzero, zps)
    active = np.isfinite(min_nonzero) & (absmax > 0)
    cand = candidate_divisors([k_min, k_gap], active, (2 * max_level + 1) if zps == 0.5 else max_level, zps == 0.5)

    k_chosen, accepted = select_divisor(x, absmax, min_nonzero, cand, zps, ulp_rel)
    scale = refine_scale(x, k_chosen, zps, qmin, qmax)
    scale = np.where(active, np.maximum(scale, min_scale), min_scale).astype(F)
    with np.errstate(all="ignore"):
        codes = np.clip(np.rint((x / scale[:, None]).astype(F) - F(zps)), F(qmin), F(qmax)).astype(F)
        recon = ((codes + F(zps)) * scale[:, None]).astype(F)
    recon_sqerr = float(np.sum((recon - x).astype(np.float64) ** 2))
    x_sqnorm = float(np.sum(x.astype(np.float64) ** 2))
    code_absmax = int(np.abs(codes).max()) if codes.size else 0

    matched = (accepted & active) | ~active
    matched_frac = float(matched.astype(F).mean()) if num_blocks > 0 else 0.0
    recon_relrms = math.sqrt(recon_sqerr) / max(math.sqrt(x_sqnorm), 1e-12)
    recon_gate = max(RECON_RELRMS_MULT * ulp_rel, RECON_RELRMS_FLOOR)
    if not (code_absmax > 0 and matched_frac >= MIN_MATCHED_FRAC and recon_relrms <= recon_gate):
        raise DecompositionError(f"not QDQ-like: matched={matched_frac:.4f}, relRMS={recon_relrms:.2e} "
                                 f"(gate={recon_gate:.2e}, ulp_rel={ulp_rel:.2e}), code_absmax={code_absmax}")

    inv = np.argsort(np.array(perm))
    input_q = codes.reshape(moved.shape).transpose(inv).reshape(input_qdq.shape)
    return input_q, scale.reshape(scale_shape)
