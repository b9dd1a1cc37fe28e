"""Pins the plain-C restatement of the DlQuantization CPU path (oracle/dlq_ref.c) against the expected outputs of the
reference's own tests and against closed forms.  Runs without a GPU."""

import math

import numpy as np
import pytest
import torch

from tests import dlq_checks as C
from tests.dlq_adapters import QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED, OracleQuantizer
from oracle import dlq as OD


def make(shape, bw, scheme):
    return OracleQuantizer(shape, bw, scheme)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_broadcast_qdq_vectors(dtype):
    C.check_broadcast_qdq(make, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_per_tensor_qdq(dtype):
    C.check_per_tensor_qdq(make, dtype)


def test_minmax_quantizer_vectors():
    C.check_minmax_quantizer(make)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_block_minmax_vectors(dtype):
    C.check_block_minmax(make, dtype)


def test_tfe_all_zero_vector():
    C.check_tfe_all_zero(make)


def test_tfe_reference_bounds():
    C.check_tfe_properties(make)


def test_tfe_search_equals_independent_enumeration():
    C.check_tfe_exact_against_enumeration(make)


def test_tfe_closed_forms():
    C.check_tfe_closed_forms(make)


def test_tfe_saturation_weight_decides():
    C.check_tfe_saturation_weight_decides(make)


def test_pdf_exact_on_binary_fractions():
    C.check_pdf_exact_binary_fractions(make)


def test_percentile_reference_expectations():
    C.check_percentile(make)


def test_fp8_against_torch_cast():
    C.check_fp8_against_torch_cast(make)


def test_fp8_reference_edge_cases():
    C.check_fp8_edge_cases(make)


def test_fp8_reference_tensors():
    C.check_fp8_reference_tensors(make)


def test_fp8_encodings():
    C.check_fp8_encodings(make)


def test_fp8_qtype_is_sticky():
    C.check_fp8_qtype_is_sticky(make)


def test_fp8_format_constants():
    """QuantizationType::Float derives bitwidth, minimum normal exponent and largest value from the layout
    (QuantizationType.hpp:88-135); the published constants of the four OCP / fnuz formats."""
    assert OD.fp8_spec(4, 3, True, False) == (8, 3, -6, 448.0)
    assert OD.fp8_spec(5, 2, False, False) == (8, 2, -14, 57344.0)
    assert OD.fp8_spec(4, 3, True, True) == (8, 3, -7, 240.0)
    assert OD.fp8_spec(5, 2, True, True) == (8, 2, -15, 57344.0)
    for spec, dt in ((OD.FP8_E4M3FN, torch.float8_e4m3fn), (OD.FP8_E5M2, torch.float8_e5m2),
                     (OD.fp8_spec(4, 3, True, True), torch.float8_e4m3fnuz),
                     (OD.fp8_spec(5, 2, True, True), torch.float8_e5m2fnuz)):
        info = torch.finfo(dt)
        assert info.max == spec[3] and info.smallest_normal == 2.0 ** spec[2]


def test_percentile_matches_numpy_quantiles():
    """Closed form: the chosen range brackets the empirical quantiles to within two buckets."""
    x = C.INPUTS["normal_mean2_std2_100k"]
    p = OD.Pdf()
    p.update(x)
    width = p.xleft[1] - p.xleft[0]
    for pct in (99.0, 99.9, 90.0):
        e = p.percentile_encoding(pct, 16, False)
        lo, hi = np.quantile(x.astype(np.float64), [1 - pct / 100, pct / 100])
        assert abs(e[0] - min(lo, 0.0)) <= 2 * width + e[2], (pct, e, lo)
        assert abs(e[1] - max(hi, 0.0)) <= 2 * width + e[2], (pct, e, hi)
    # 100 % keeps the whole observed range
    e = p.percentile_encoding(100.0, 16, False)
    assert e[0] <= x.min() + width and e[1] >= x.max() - width


# ------------------------------------------------------------------------------------------------ closed forms ----
def test_qdq_is_identity_on_grid_points_and_saturates():
    enc = C.tf_encoding(-4.0, 3.96875, 8)  # delta = 1/32: every grid point is exact in float
    grid = enc[0] + np.arange(256) * enc[2]
    y = OD.qdq(grid.astype(np.float32), enc[:4])
    assert np.array_equal(y, grid.astype(np.float32))
    y = OD.qdq(np.array([-100.0, 100.0, np.nan, np.inf, -np.inf], dtype=np.float32), enc[:4])
    assert np.array_equal(y, np.array([enc[0], enc[1], enc[0], enc[1], enc[0]], dtype=np.float32))
    # ties: std::round acts on x/delta - offset, which is positive here (offset = -128), so every tie goes up,
    # unlike rint (ties to even) and unlike rounding x/delta itself away from zero
    y = OD.qdq(np.array([0.5 / 32, 1.5 / 32, -0.5 / 32, -1.5 / 32], dtype=np.float32), enc[:4])
    assert np.array_equal(y, np.array([1 / 32, 2 / 32, 0.0, -1 / 32], dtype=np.float32))


def test_minmax_skips_nan_and_starts_from_float_limits():
    mn, mx = OD.minmax(np.array([np.nan, 1.0, -2.0, np.nan], dtype=np.float32))
    assert (mn, mx) == (-2.0, 1.0)
    mn, mx = OD.minmax(np.array([np.nan], dtype=np.float32))
    assert mn == np.finfo(np.float32).max and mx == -np.finfo(np.float32).max
    mn, mx = OD.minmax(np.array([np.inf, -np.inf], dtype=np.float32))
    assert mn == -np.inf and mx == np.inf


@pytest.mark.parametrize("bw", [2, 4, 8, 16])
def test_computed_encodings_closed_form(bw):
    steps = 2 ** bw - 1
    # asymmetric: a range that is an exact multiple of the step reproduces itself
    e = OD.computed_encodings(bw, -1.0 * 2, 1.0 * (steps - 2), False)
    assert tuple(e) == (-2.0, float(steps - 2), 1.0, -2.0, float(bw))
    # symmetric: delta = max(max / floor(n/2), -min / ceil(n/2)), offset = -ceil(n/2)
    e = OD.computed_encodings(bw, -3.0, 5.0, True)
    pos, neg = steps // 2, steps - steps // 2
    if steps == 3:
        pos = neg
    assert e[2] == max(5.0 / pos, 3.0 / neg) and e[3] == -neg
    assert e[0] == e[2] * e[3] and e[1] == e[2] * (e[3] + steps)
    # strict symmetric: one step fewer, min == -max
    e = OD.computed_encodings(bw, -3.0, 5.0, True, strict=True)
    assert e[0] == -e[1] and e[3] == -((steps - 1) // 2)
    # unsigned symmetric applies only when min >= 0
    e = OD.computed_encodings(bw, 0.0, 5.0, True, unsigned_sym=True)
    assert e[3] == 0 and e[0] == 0 and e[2] == 5.0 / steps
    # degenerate range: the minimum scale keeps delta positive
    e = OD.computed_encodings(bw, 0.0, 0.0, False)
    assert e[2] == min(0.01 / steps, float(np.finfo(np.float32).eps)) and e[3] == 0


def test_zero_point_shift_rules():
    e = OD.computed_encodings(2, -10.0, 10.0, True, zps=0.5)
    assert e[3] == -1.5 and e[2] == 10.0 / 1.5
    for kw in (dict(symmetric=False), dict(symmetric=True, strict=True), dict(symmetric=True, unsigned_sym=True)):
        sym = kw.pop("symmetric")
        mn = 0.0 if kw.get("unsigned_sym") else -10.0
        with pytest.raises(RuntimeError):
            OD.computed_encodings(2, mn, 10.0, sym, zps=0.5, **kw)


def test_pdf_matches_brute_force_histogram():
    rng = np.random.default_rng(0)
    x = rng.normal(0.5, 2.0, 5000).astype(np.float32)
    p = OD.Pdf()
    hist = p.update(x)
    xl = p.xleft
    # range: three times the observed span around its centre, 1536 equal buckets whose left edges are multiples of
    # the bucket size
    mn, mx = np.float32(x.min()), np.float32(x.max())
    center = np.float32((mx + mn) / np.float32(2))
    lo = np.float32(center - np.float32(3) * np.float32(center - mn))
    hi = np.float32(center + np.float32(3) * np.float32(mx - center))
    bucket = (float(hi) - float(lo)) / 1536
    assert np.array_equal(xl, np.floor(float(lo) / bucket + np.arange(1536)) * bucket)
    # counts: every element falls in the bucket whose edges enclose it (up to float rounding at the edges)
    width = xl[1] - xl[0]
    idx = np.floor((x.astype(np.float64) - xl[0]) / width).astype(int)
    brute = np.bincount(idx, minlength=1536)
    assert hist.sum() == x.size
    assert np.abs(hist.astype(int) - brute).sum() <= 4  # an element exactly at an edge may land on either side
    assert np.array_equal(p.pdf, hist / float(x.size))
    # second batch: running average of the per-batch densities; values outside the fixed range are dropped
    x2 = np.concatenate([rng.normal(0.5, 2.0, 3000), [1e6, -1e6, np.nan, np.inf]]).astype(np.float32)
    h2 = p.update(x2)
    assert h2.sum() == 3000
    assert np.array_equal(p.pdf, (hist / float(x.size) * 1 + h2 / float(x2.size)) / 2)
    assert p.meta == (2, 1, 1)


def test_pdf_all_zero_batches_do_not_fix_the_range():
    p = OD.Pdf()
    assert p.update(np.zeros(100, dtype=np.float32)).sum() == 0
    assert p.meta == (0, 0, 1)
    p.update(np.array([0.0, 1.0, 2.0], dtype=np.float32))
    assert p.meta == (1, 1, 1)
    p.reset()
    assert p.meta == (0, 0, 1)  # resetStats leaves _statsUpdated set


def test_tfe_search_agrees_with_exhaustive_numpy_search():
    """Re-derive the candidate costs with vectorised numpy in float64 and check the chosen candidate is a minimiser
    (a different evaluation order, so only near-equality of the minimum cost is required)."""
    x = C.INPUTS["normal_mean2_std2"]
    p = OD.Pdf()
    p.update(x)
    enc, n, best = p.compute_encoding(8, False, with_index=True)
    assert n == 17 * 21 + 1 or n < 17 * 21 + 1
    xl, pdf = p.xleft, p.pdf
    centers = xl + (xl[1] - xl[0]) / 2

    def cost(delta, offset):
        lo, hi = delta * offset, delta * (offset + 255)
        deq = np.clip(np.floor(centers / delta + 0.5) * delta, None, None)
        c = np.where(centers < lo, 3 * (centers - lo) ** 2, np.where(centers > hi, 3 * (centers - hi) ** 2, (centers - deq) ** 2))
        return float((pdf * c).sum())

    chosen = cost(enc[2], enc[3])
    # no encoding of the same family (same delta, neighbouring offsets; neighbouring deltas) is much better
    for d in (enc[2] * 0.9, enc[2], enc[2] * 1.1):
        for o in (enc[3] - 8, enc[3], enc[3] + 8):
            assert chosen <= cost(d, o) * 1.5 + 1e-12
    assert enc[0] == np.float32(np.float32(enc[2]) * np.float32(enc[3]))


def test_block_view_matches_manual_gather():
    x = np.arange(12, dtype=np.float32).reshape(2, 6)
    b = OD.block_view(x, (2, 2))
    assert b.tolist() == [[0, 1, 2], [3, 4, 5], [6, 7, 8], [9, 10, 11]]
    b = OD.block_view(np.arange(24, dtype=np.float32).reshape(2, 3, 2, 2), (3, 1, 1))
    assert b[1].tolist() == [4, 5, 6, 7, 16, 17, 18, 19]
