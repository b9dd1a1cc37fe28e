"""Formats, reference tables and an exact grid search shared by the float fake-cast tests."""

import bisect
import math
from fractions import Fraction

import torch

# name -> ((exponent bits, mantissa bits, finite, unsigned zero), torch storage dtype or None)
FORMATS = {
    "float16": ((5, 10, False, False), torch.float16),
    "bfloat16": ((8, 7, False, False), torch.bfloat16),
    "float8_e4m3fn": ((4, 3, True, False), torch.float8_e4m3fn),
    "float8_e4m3fnuz": ((4, 3, True, True), torch.float8_e4m3fnuz),
    "float8_e5m2": ((5, 2, False, False), torch.float8_e5m2),
    "float8_e5m2fnuz": ((5, 2, True, True), torch.float8_e5m2fnuz),
    "float4_e2m1fn": ((2, 1, True, False), None),
    "float8_e3m4": ((3, 4, False, False), None),
    "float7_e3m3": ((3, 3, False, False), None),
}

# test_qdq_output_non_standard_dtype (test_float_quantizer.py:166-205)
E2M1_TABLE = (
    [-6.5, -6, -5.5, -5, -4.5, -4, -3.5, -3, -2.5, -2, -1.5, -1, -0.5, 0, 0.5, 1, 1.5, 2, 2.5, 3, 3.5, 4, 4.5, 5, 5.5, 6, 6.5],
    [-6, -6, -6, -4, -4, -4, -4, -3, -2, -2, -1.5, -1, -0.5, 0, 0.5, 1, 1.5, 2, 2, 3, 4, 4, 4, 4, 6, 6, 6],
)


def grid_of(name):
    """Non-negative finite values of the format, increasing; consecutive values alternate in mantissa parity, so an
    even index is an even mantissa.  Storage types are decoded from their bit patterns; the other layouts follow the
    reference's formula: largest value max = (2 - 2^-M) 2^k, bias 2^E - k - 1, smallest binade exponent 1 - bias."""
    (e, m, finite, uz), dtype = FORMATS[name]
    if dtype in (torch.float16, torch.bfloat16):
        bits = torch.arange(0, 1 << 15, dtype=torch.int32).to(torch.int16).view(dtype)
        vals = bits.double()
        return [Fraction(v) for v in vals[torch.isfinite(vals)].tolist()]
    if dtype is not None:
        vals = torch.arange(128, dtype=torch.uint8).view(dtype).double()
        return [Fraction(v) for v in vals[torch.isfinite(vals)].tolist()]
    mx = 6.0 if name == "float4_e2m1fn" else (2 - 2 ** -m) * 2.0 ** ((2 ** e - 1) - (2 ** e - 1) // 2 - 1)
    k = math.floor(math.log2(mx))
    emin = 1 - (2 ** e - k - 1)
    out = [Fraction(i) * Fraction(2) ** (emin - m) for i in range(2 ** m)]  # zero and subnormals
    ex = emin
    while True:
        for i in range(2 ** m):
            v = (Fraction(2 ** m + i) / 2 ** m) * Fraction(2) ** ex
            if v > Fraction(mx):
                return out
            out.append(v)
        ex += 1


def exact_cast(x, scale, grid, unsigned_zero=False, dtype=torch.float32):
    """(x / scale) and (. * scale) as correctly rounded operations of `dtype` (torch CPU); the cast between them by
    exact search.  Saturates at the largest grid value, as the reference's clamp makes it."""
    s = torch.tensor(scale, dtype=torch.float32).to(dtype)
    q = (x.to(dtype) / s)
    out = torch.empty_like(q)
    for i, v in enumerate(q.double().tolist()):
        if math.isnan(v):
            out[i] = float("nan")
            continue
        a = grid[-1] if math.isinf(v) else min(Fraction(abs(v)), grid[-1])
        hi = bisect.bisect_left(grid, a)
        if grid[hi] == a:
            pick = hi
        else:
            lo = hi - 1
            dl, dh = a - grid[lo], grid[hi] - a
            pick = lo if dl < dh else hi if dh < dl else (lo if lo % 2 == 0 else hi)
        r = math.copysign(float(grid[pick]), v)
        if unsigned_zero and r == 0:
            r = 0.0
        out[i] = r
    return out * s
