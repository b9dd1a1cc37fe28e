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
