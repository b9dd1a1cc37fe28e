"""Pins the CPU restatement of aimet_torch's float fake-cast (oracle/torch_ref.py: float_qdq, fake_cast_to_ieee_float)
against the expectations the reference's own tests state (test_float_quantizer.py) and against an exact search over
each format's enumerated grid.  Runs without a GPU."""

import math
from fractions import Fraction

import pytest
import torch

from oracle import torch_ref as O
from tests.float_cases import E2M1_TABLE, FORMATS, exact_cast, grid_of


@pytest.mark.parametrize("name", [n for n, f in FORMATS.items() if f[1] is not None])
def test_standard_dtypes_are_a_cast_and_back(name):
    """test_qdq_output_standard_dtypes (test_float_quantizer.py:44-62): at scale 1 the output equals
    x.to(dtype).float()."""
    fmt, dtype = FORMATS[name]
    x = torch.arange(-200, 200).view(4, 100) / 100
    assert torch.equal(O.float_qdq(x, torch.tensor(1.0), *fmt), x.to(dtype).float())


def test_float4_e2m1fn_table():
    """test_qdq_output_non_standard_dtype (test_float_quantizer.py:160-215)."""
    x, want = torch.tensor(E2M1_TABLE[0]), torch.tensor(E2M1_TABLE[1])
    assert torch.equal(O.float_qdq(x, torch.tensor(1.0), 2, 1, True, False), want)
    assert torch.equal(O.fake_cast_to_ieee_float(x, 6.0, 2, 1, finite=True), want)


@pytest.mark.parametrize("name", list(FORMATS))
def test_against_exact_search_on_the_enumerated_grid(name):
    """Independent of any conversion routine: nearest grid value by exact rational comparison, ties to the even
    mantissa, saturating at the largest value, for awkward scales."""
    fmt, _ = FORMATS[name]
    grid = grid_of(name)
    g = torch.Generator().manual_seed(3)
    mx = float(grid[-1])
    x = torch.randn(3000, generator=g) * torch.exp(torch.rand(3000, generator=g) * 14 - 10) * min(mx, 1e4)
    x[:8] = torch.tensor([0.0, -0.0, mx, -mx, 2 * mx, -2 * mx, float(grid[1]) / 2, -float(grid[1]) / 2])
    for scale in (1.0, 0.37, 3.0):
        got = O.float_qdq(x, torch.tensor(scale), *fmt)
        want = exact_cast(x, scale, grid, unsigned_zero=fmt[3])
        assert torch.equal(got, want)
        assert torch.equal(torch.signbit(got), torch.signbit(want))


def test_formula_based_cast_places_the_smallest_binade_one_below_ieee():
    """fake_cast_to_ieee_float derives its bias from the largest value (fp_quantization.py:177-180); for layouts whose
    top exponent is reserved that bias is one more than IEEE's, so the grid keeps halving one binade further down.
    float8 e3m4 (max 15.5): IEEE's smallest normal would be 2^-2 with subnormal step 2^-6; here the step is 2^-7."""
    x = torch.tensor([2.0 ** -7, 3 * 2.0 ** -8, 2.0 ** -8, 5 * 2.0 ** -8])
    got = O.float_qdq(x, torch.tensor(1.0), 3, 4, False, False)
    assert got.tolist() == [2.0 ** -7, 2 * 2.0 ** -7, 0.0, 2 * 2.0 ** -7]


@pytest.mark.parametrize("name", list(FORMATS))
def test_kernel_format_description_matches_the_enumerated_grid(name):
    """Host logic: the (mantissa bits, smallest normal exponent, largest value) handed to the kernel describe the same
    grid as the enumeration."""
    from aimet_amd.quantization.float._finfo import _finfo

    fmt, dtype = FORMATS[name]
    mbits, emin, mx, overflow_nan, uz = _finfo(*fmt).kernel_format()
    grid = grid_of(name)
    assert mbits == fmt[1] and uz == fmt[3]
    assert grid[-1] == Fraction(mx)
    assert grid[1] == Fraction(2) ** (emin - mbits)          # smallest subnormal
    assert grid[2 ** mbits] == Fraction(2) ** emin           # smallest normal
    if dtype is not None:
        assert overflow_nan == fmt[2]
        assert _finfo.from_torch_dtype(dtype) == fmt and _finfo(*fmt).to_torch_dtype() == dtype
