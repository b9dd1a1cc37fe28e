"""Shared comparison helpers for the parity tests."""

import torch


def assert_same_bits(actual: torch.Tensor, expected: torch.Tensor, what: str = ""):
    """Bit-exact comparison, signs of zero included (any NaN matches any NaN)."""
    a = actual.detach().cpu()
    e = expected.detach().cpu()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    assert a.dtype == e.dtype, f"{what}: dtype {a.dtype} vs {e.dtype}"
    same = ((a == e) & (torch.signbit(a) == torch.signbit(e))) | (a.isnan() & e.isnan())
    if not bool(same.all()):
        bad = (~same).nonzero()
        i = tuple(bad[0].tolist())
        raise AssertionError(
            f"{what}: {bad.shape[0]} of {a.numel()} elements differ; first at {i}: got {a[i].item()!r}, "
            f"expected {e[i].item()!r}"
        )


def assert_close_rel(actual: torch.Tensor, expected: torch.Tensor, rel: float, what: str = "", abs_floor: float = 0.0):
    """|a - e| <= rel * max|e| (+ abs_floor): the bar for order-sensitive floating-point sums.
    Entries where both sides hold the same infinity or both hold NaN count as equal."""
    a = actual.detach().cpu().double()
    e = expected.detach().cpu().double()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    if e.numel() == 0:
        return
    same = (a == e) | (a.isnan() & e.isnan())
    finite = e.isfinite()
    scale = e[finite].abs().max().item() if bool(finite.any()) else 0.0
    diff = torch.where(same, torch.zeros_like(a), (a - e).abs())
    err = diff.max().item()
    assert err <= rel * scale + abs_floor, f"{what}: max abs err {err:.3e} exceeds {rel:.1e} * {scale:.3e}"


def histogram_merge_closed_forms():
    """Two-batch histogram merges whose result is known without running the algorithm (every number below is an exact
    binary fraction).  Each case: (num_bins, first batch, second batch, merged counts, (lo, hi) of the merged range).

    nested    the range doubles, so every old bin lies inside one new bin: the merged histogram is the plain histogram
              of all the data over the new range.
    straddle  new bins of twice the width whose edges cut old bins 0 and 2 in the middle: an old bin of c values gives
              round(c / 2) to the lower new bin (half to even: 3 -> 2, 5 -> 2) and the rest to the upper one.
    """
    import torch

    def rep(pairs):
        return torch.tensor([v for v, n in pairs for _ in range(n)], dtype=torch.float32)

    # old range [0, 1], 8 bins of 1/8: counts 1, 2, 3, 4, 5, 6, 7, 8 (the extremes 0 and 1 are members of bins 0 and 7)
    first = rep([(0.0, 1), (0.1875, 2), (0.3125, 3), (0.4375, 4), (0.5625, 5), (0.6875, 6), (0.8125, 7), (0.9375, 7), (1.0, 1)])
    # new range [0, 2], 8 bins of 1/4
    second = rep([(0.0, 1), (0.125, 2), (0.375, 1), (1.125, 3), (1.375, 2), (1.875, 4), (2.0, 1)])
    nested = (8, first, second, [1 + 2 + 3, 3 + 4 + 1, 5 + 6, 7 + 8, 3, 2, 0, 5], (0.0, 2.0))

    # old range [0, 1], 4 bins of 1/4 with counts 3, 4, 5, 6; new range [-0.375, 1.625], 4 bins of 1/2 with edges
    # -0.375, 0.125, 0.625, 1.125, 1.625
    first = rep([(0.0, 1), (0.0625, 2), (0.3125, 4), (0.5625, 5), (0.8125, 5), (1.0, 1)])
    second = rep([(-0.375, 1), (0.0, 2), (0.5, 1), (1.0, 3), (1.625, 1)])
    old = [2, (3 - 2) + 4 + 2, (5 - 2) + 6, 0]
    new = [1 + 2, 1, 3, 1]
    straddle = (4, first, second, [o + n for o, n in zip(old, new)], (-0.375, 1.625))
    return {"nested": nested, "straddle": straddle}


def nested_range_batches(num_bins: int, seed: int, dtype=None):
    """Three batches whose ranges are [-a, a], [-2a, 2a], [-8a, 8a] for a power of two a, values on a dyadic grid
    fine enough that none lies on a bin edge except the range ends: every old bin then lies inside one bin of the
    next range, no count is ever split, and the merged histogram is -- exactly -- the plain histogram of all the
    data over the last range (with each earlier batch's maximum counted below the edge it sits on).  Returns (batches, expected counts as float32, (lo, hi))."""
    import torch

    g = torch.Generator().manual_seed(seed)
    a = 2.0 ** (seed % 5 - 2)
    batches = []
    for k, width in enumerate((1, 2, 8)):
        n = 3000 + 500 * k
        half = width * a
        # odd multiples of half / (4 * num_bins): never on an edge of any of the three bin grids
        steps = torch.randint(-2 * num_bins, 2 * num_bins, (n,), generator=g) * 2 + 1
        x = steps.to(torch.float32) * (half / (4 * num_bins))
        x[0], x[1] = -half, half
        if dtype is not None:
            x = x.to(dtype)
        batches.append(x)
    lo, hi = -8 * a, 8 * a
    # a batch's maximum is counted in the last bin of its own range (torch.histc closes the range on the right) and
    # stays with that bin's counts from then on, although the value is the left edge of the next bin of a wider grid:
    # for the plain histogram it is therefore taken just below
    inside = [b.to(torch.float32).clone() for b in batches]
    for k, width in enumerate((1, 2)):
        inside[k][1] = width * a * (1 - 1 / (8 * num_bins))
    expected = torch.histc(torch.cat(inside), bins=num_bins, min=lo, max=hi)
    return batches, expected, (lo, hi)
