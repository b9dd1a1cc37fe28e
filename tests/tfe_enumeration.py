"""An independent statement of DlQuantization's TF-enhanced encoding search, written from the algorithm's description
(ModelOptimizations/DlQuantization/src/TfEnhancedEncodingAnalyzer.cpp:90-377) as array arithmetic over all candidates
at once -- no loop over candidates or buckets (only the running float sum of the symmetric multipliers is a loop, as
that sum is the definition), nothing shared with oracle/dlq_ref.c or the HIP kernels.  It exists to
pin those two: on probability tables built by hand, the chosen (delta, offset), its position in the candidate list
and the length of that list must agree exactly.

What the description fixes, and where float and double meet (DTYPE = float in the reference):

* range of the statistics: left edge of the first / last bucket with positive probability, widened to hold zero and to
  be at least 0.01 wide; all in float.
* asymmetric candidates: delta_max = float((double(max) - double(min)) / steps); offset_obs = round(min / delta_max);
  the observed range snaps to that grid.  17 deltas f * delta_max, f = 1/16 ... 17/16, times 21 offsets
  trunc(-steps + steps / 20.0 * i) (double arithmetic).  A candidate whose range strictly contains the observed one is
  dropped; otherwise its range is cut to the observed one, dropped if nothing is left, and re-expressed as
  delta = float((double(max') - min') / steps), offset = round(min' / delta).  Last comes (delta_max, offset_obs).
* symmetric candidates: delta_max = float(absmax / (steps / 2.0)), offset = floor(-steps / 2); or, for unsigned
  symmetric statistics starting at zero, delta_max = max / steps with offset 0.  Deltas f * delta_max for f = 1/100,
  2/100, ... accumulated in float while f <= 1.01.
* cost of (delta, offset) over the 1536 buckets with centres c_i = float(float(left_i) + half width): buckets below
  the bucket holding delta * offset pay 3 * p_i * (c_i - c_lo)^2, buckets from the one holding
  delta * (offset + 2^bw - 1) upward pay 3 * p_i * (c_i - c_hi)^2, buckets between pay
  p_i * (c_i - floor(c_i / delta + 1/2) * delta)^2 with the rounding done in float; the sums run in bucket order in
  double.  The first smallest cost wins.
"""

import numpy as np

PDF_SIZE = 1536
F = np.float32
D = np.float64
FLT_MAX = np.finfo(np.float32).max


def _round_half_away(v):
    """C round() on float32 arrays."""
    v = np.asarray(v, dtype=F)
    return (np.sign(v) * np.floor(np.abs(v) + F(0.5))).astype(F)


def stats_range(xleft, pdf):
    pos = np.nonzero(np.asarray(pdf) > 0)[0]
    lo = F(xleft[pos[0]]) if pos.size else F(xleft[0])
    # the downward search stops above bucket 0
    hi = F(xleft[pos[-1]]) if pos.size and pos[-1] > 0 else F(xleft[PDF_SIZE - 1])
    lo = min(lo, F(0))
    hi = max(hi, F(0))
    hi = max(hi, F(lo + F(0.01)))
    return F(lo), F(hi)


def asymmetric_candidates(lo, hi, steps):
    """-> (deltas float32[n], offsets int64[n]) in the reference's order."""
    steps = F(steps)
    delta_max = F((D(hi) - D(lo)) / D(steps))
    off_obs = int(_round_half_away(F(lo) / delta_max))
    lo = max(F(delta_max * F(off_obs)), F(-FLT_MAX))
    hi = min(F(delta_max * F(F(off_obs) + steps)), F(FLT_MAX))
    f = (np.arange(1, 18, dtype=D) / 16).astype(F)                    # exact in float
    off = np.trunc(-D(steps) + D(steps) / 20.0 * np.arange(21, dtype=D)).astype(np.int64)
    delta = (f[:, None] * delta_max).astype(F) * np.ones((1, 21), dtype=F)
    off = np.broadcast_to(off[None, :], delta.shape)
    tmin = np.maximum((delta * off.astype(F)).astype(F), F(-FLT_MAX))
    tmax = np.minimum((delta * (off.astype(F) + steps).astype(F)).astype(F), F(FLT_MAX))
    contains = (tmin < lo) & (tmax > hi)
    tmin = np.maximum(lo, tmin)
    tmax = np.minimum(hi, tmax)
    keep = ~contains & (tmin != tmax)
    with np.errstate(divide="ignore", invalid="ignore"):
        new_delta = ((tmax.astype(D) - tmin.astype(D)) / D(steps)).astype(F)
        new_off = _round_half_away(tmin / new_delta)
    deltas = np.concatenate([new_delta[keep], [delta_max]]).astype(F)   # boolean indexing keeps row-major order
    offsets = np.concatenate([new_off[keep].astype(np.int64), [off_obs]])
    return deltas, offsets


def symmetric_candidates(lo, hi, steps, unsigned_symmetric):
    steps = F(steps)
    if lo == 0 and unsigned_symmetric:
        delta_max = F(F(hi) / steps)
        offset = 0
    else:
        absmax = max(abs(F(hi)), abs(F(lo)))
        delta_max = F(D(absmax) / (D(steps) / 2.0))
        offset = int(np.floor(-steps / F(2)))
    # f += 1.0 / 100 in float, while f <= 1 + 1.0 / 100 compared in double: a running sum that rounds at every step
    fs = []
    f = F(1.0 / 100)
    while D(f) <= 1 + 1.0 / 100:
        fs.append(f)
        f = F(D(f) + 1.0 / 100)
    deltas = (np.array(fs, dtype=F) * delta_max).astype(F)
    return deltas, np.full(deltas.shape, offset, dtype=np.int64)


def costs(xleft, pdf, bw, deltas, offsets, gamma=3.0):
    """float64[n]: quantisation + gamma x saturation cost of every candidate (the reference's gamma is 3)."""
    xleft = np.asarray(xleft, dtype=D)
    pdf = np.asarray(pdf, dtype=D)
    half = (xleft[1] - xleft[0]) / 2
    centres = (xleft.astype(F).astype(D) + half).astype(F)
    deltas = np.asarray(deltas, dtype=F)
    offs = np.asarray(offsets).astype(F)
    step = F(2.0 ** bw - 1)
    vmin = (deltas * offs).astype(F)
    vmax = (deltas * (offs + step).astype(F)).astype(F)
    start = F(xleft[0])
    width = xleft[1] - xleft[0]

    def bucket_of(v):
        q = np.floor((v - start).astype(F).astype(D) / width)
        # a quotient beyond the int range converts to INT_MIN on x86-64, which the clamp then turns into bucket 0
        q = np.where((q >= 2.0 ** 31) | (q < -(2.0 ** 31)) | np.isnan(q), -(2.0 ** 31), q)
        return np.clip(q, 0, PDF_SIZE - 1).astype(np.int64)

    lo_i, hi_i = bucket_of(vmin), bucket_of(vmax)
    i = np.arange(PDF_SIZE)[None, :]
    c64 = centres.astype(D)[None, :]
    below = i < lo_i[:, None]
    above = i >= hi_i[:, None]
    inside = ~below & ~above
    d_lo = c64 - centres[lo_i].astype(D)[:, None]
    d_hi = c64 - centres[hi_i].astype(D)[:, None]
    inv = (F(1) / deltas).astype(F)
    deq = (np.floor((centres[None, :] * inv[:, None]).astype(F) + F(0.5)).astype(F) * deltas[:, None]).astype(F)
    d_q = (centres[None, :] - deq).astype(F).astype(D)
    zero = np.zeros_like(c64 * d_lo)
    # excluded buckets contribute +0, which leaves a non-negative running sum as it is; cumsum adds in bucket order
    sat_lo = np.cumsum(np.where(below, pdf[None, :] * (d_lo * d_lo), zero), axis=1)[:, -1]
    sat_hi = np.cumsum(np.where(above, pdf[None, :] * (d_hi * d_hi), zero), axis=1)[:, -1]
    quant = np.cumsum(np.where(inside, pdf[None, :] * (d_q * d_q), zero), axis=1)[:, -1]
    total = D(F(gamma)) * (sat_lo + sat_hi) + quant
    return np.minimum(total, np.finfo(D).max)


def search(xleft, pdf, bw, symmetric, strict=False, unsigned_symmetric=False, gamma=3.0):
    """-> dict(delta, offset, min, max, index, count, costs)."""
    steps = F(2.0 ** bw - 1)
    lo, hi = stats_range(xleft, pdf)
    if symmetric:
        if strict:
            steps = F(steps - 1)
        deltas, offsets = symmetric_candidates(lo, hi, steps, unsigned_symmetric)
    else:
        deltas, offsets = asymmetric_candidates(lo, hi, steps)
    c = costs(xleft, pdf, bw, deltas, offsets, gamma)
    k = int(np.argmin(c))  # the first of equal minima
    delta, offset = F(deltas[k]), int(offsets[k])
    emin = max(F(delta * F(offset)), F(-FLT_MAX))
    emax = min(F(delta * F(F(offset) + steps)), F(FLT_MAX))
    return {"delta": float(delta), "offset": float(offset), "min": float(emin), "max": float(emax), "index": k,
            "count": int(deltas.size), "costs": c}


def uniform_buckets(first_left, width):
    """Left edges first_left + i * width (exact when both are small multiples of a power of two)."""
    return D(first_left) + np.arange(PDF_SIZE, dtype=D) * D(width)
