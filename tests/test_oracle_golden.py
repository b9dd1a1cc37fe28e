"""Pins the CPU oracle (oracle/torch_ref.py) against the vectors the reference's own tests and docstrings hold, and
against facts the mathematics fixes.  Which check pins which oracle function:

    quantize_forward / dequantize_forward / qdq_v2_forward / qdq_v2_backward / quantize_backward
        golden vector sets, block-quantization table, docstring examples, clipped-scale gradient closed form with a
        finite-difference check, block == per-tensor call on the block, STE autograd cross-check
    quantize_backward (scale and offset gradients) / dequantize_backward
        plain autograd of clamp(round_ste(x / s) - o) and of (x + o) * s, float64, four layouts
    percentile_encodings / adjust_min_max
        the reference's percentile cases (exact -990 / 990, one-bin 100 %, constant and zero tensors, 50 %, outliers)
        and hand-derived results that fix the side of the cumulative search and the zero-in-range rule
    qdq_v1                     the installed ATen kernels themselves (library routine) + closed form
    internal_dtype             the dtype table of the reference's test_affine_quantizer.py:1761-1768
    reduce_minmax              torch.amin/amax on explicitly sliced blocks
    minmax_encodings           exact expected min/max of the reference's analyzer tests, zero / constant inputs
    HistObserver               the reference's merge sequences (exact counts and edges), +-inf handling, count conservation,
                               two merges with hand-derived results (nested bins; bins cut in half, rounding half to even)
    sqnr_encodings             uniform-distribution closed form, outlier optimum, brute-force enumeration in Python floats
    sqnr_candidates / _clamp_candidates / sqnr_noise
                               the reference's candidate-grid, noise-estimate (within 1 % of the error measured on
                               the data) and selection cases; gamma scales an all-clipped candidate exactly
    hist_collect               per-slot brute-force counts
    scale_from_minmax / offset_from_minmax / scale_offset_dynamic
                               the reference's low-bitwidth scales (5.25 / 7.0 / 3.5 / 3.0) and hand-worked ranges
    lpbq_scale                 closed form max(1, round(s / gamma)) * gamma
    float_* functions          tests/test_oracle_float.py
"""

import math

import pytest
import torch

from oracle import torch_ref as O
from tests import golden_checks as G
from tests.adapters import OracleImpl

IMPL = OracleImpl()


@pytest.mark.parametrize("name", [n for n in G.vector_set_names() if not n.startswith("bfloat16")])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32], ids=["f16", "f32"])
def test_vector_sets(name, dtype):
    G.check_vector_set(IMPL, name, dtype)


@pytest.mark.parametrize("name", [n for n in G.vector_set_names() if n.startswith("bfloat16")])
def test_vector_sets_bfloat16(name):
    G.check_vector_set(IMPL, name, torch.bfloat16)


def test_block_quant_table():
    G.check_block_quant(IMPL)


def test_docstring_examples():
    G.check_docstring_examples(IMPL)


def test_clipped_scale_gradient():
    G.check_clipped_scale_gradient(IMPL)


def test_minmax_encodings():
    G.check_minmax_encodings(IMPL)


def test_histogram_merges():
    G.check_histogram_merges(IMPL)


def test_sqnr_uniform():
    G.check_sqnr_uniform(IMPL)


def test_sqnr_outlier():
    G.check_sqnr_outlier(IMPL)


def test_sqnr_brute_force():
    G.check_sqnr_brute_force(IMPL)


def test_internal_dtype_table():
    """bf16 stays bf16 up to 4-bit grids, fp16 up to 8-bit, anything wider computes in fp32."""
    table = {
        (torch.bfloat16, 4): torch.bfloat16, (torch.bfloat16, 8): torch.float32, (torch.bfloat16, 16): torch.float32,
        (torch.float16, 4): torch.float16, (torch.float16, 8): torch.float16, (torch.float16, 16): torch.float32,
        (torch.float32, 4): torch.float32, (torch.float32, 16): torch.float32,
    }
    for (dtype, bw), want in table.items():
        assert O.internal_dtype(dtype, 0, 2 ** bw - 1) == want
        assert O.internal_dtype(dtype, -(2 ** (bw - 1)), 2 ** (bw - 1) - 1) == want
    assert O.internal_dtype(torch.float32, 0, 2 ** 32 - 1) == torch.float64
    assert not O.grid_representable(torch.bfloat16, 0, 65535)
    assert O.grid_representable(torch.float16, 0, 2047) and not O.grid_representable(torch.float16, 0, 4097)


def test_aten_arithmetic_closed_form():
    """The ATen fake-quantize kernels compute rint(x * (1/scale)) + zero_point, clamp, subtract, multiply."""
    g = torch.Generator().manual_seed(0)
    for s, off, qmin, qmax in [(0.0123, -7.0, 0, 255), (3.3e-5, -30000.0, 0, 65535), (0.1, 0.0, -128, 127)]:
        x = torch.randn(20000, generator=g) * s * (qmax - qmin) * 0.7
        k = torch.arange(-300, 300).float()
        x = torch.cat([x, (k + 0.5) * s])
        y, mask = O.qdq_v1(x, torch.tensor(s), torch.tensor(off), qmin, qmax)
        inv = torch.tensor(1.0) / torch.tensor(s)
        q = torch.round(x * inv) + (-off)
        expect = (q.clamp(qmin, qmax) - (-off)) * torch.tensor(s)
        assert torch.equal(y, expect)
        assert torch.equal(mask, (q >= qmin) & (q <= qmax))


def test_block_equals_per_tensor_call_on_the_block():
    """Reference: test_backend.py:970-1031."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 4, 6, 12, 9, generator=g)
    scale = torch.rand(1, 4, 9, generator=g) * 0.1 + 0.01
    scale = scale.expand(2, 4, 9).reshape(2, 1, 4, 9)[:, :, :, :].contiguous()
    scale = torch.rand(2, 1, 4, 9, generator=g) * 0.1 + 0.01
    offset = torch.randint(-128, 127, (2, 1, 4, 9), generator=g).float()
    block = [2, 6, 3, 1]
    q = O.quantize_forward(x, scale, offset, 0, 255, block)[0]
    y = O.qdq_v2_forward(x, scale, offset, 0, 255, block).y
    for i in range(2):
        for k in range(4):
            for l in range(9):
                sl = (Ellipsis, slice(2 * i, 2 * i + 2), slice(0, 6), slice(3 * k, 3 * k + 3), slice(l, l + 1))
                s, o = scale[i, 0, k, l], offset[i, 0, k, l]
                assert torch.equal(q[sl], O.quantize_forward(x[sl], s, o, 0, 255)[0])
                assert torch.equal(y[sl], O.qdq_v2_forward(x[sl], s, o, 0, 255).y)


def test_gradients_match_ste_autograd():
    """Reference: test_backend.py:163-210, 715-821 -- gradients equal those of a plain autograd graph with
    straight-through rounding and a clamp that passes gradient on the closed interval."""
    g = torch.Generator().manual_seed(2)
    for shape, sshape, block in [((6, 40), (), None), ((6, 40), (6, 1), None), ((6, 40), (6, 4), (1, 10))]:
        scale = torch.rand(sshape, generator=g) * 0.1 + 0.02
        offset = torch.randint(-200, -50, sshape, generator=g).float()
        qmin, qmax = 0, 255
        # keep away from rounding boundaries so that the straight-through graph is unambiguous
        s_full = scale if block is None else scale.repeat_interleave(10, dim=1)
        o_full = offset if block is None else offset.repeat_interleave(10, dim=1)
        base = torch.randint(-60, 320, shape, generator=g).float() + torch.rand(shape, generator=g) * 0.8 - 0.4
        x = ((base + o_full) * s_full).clone()
        grad = torch.randn(shape, generator=g)
        gx, gs, go = O.qdq_v2_backward(grad, x, scale, offset, qmin, qmax, block)

        xs = x.clone().requires_grad_(True)
        ss = scale.clone().requires_grad_(True)
        os_ = offset.clone().requires_grad_(True)
        sf = ss if block is None else ss.repeat_interleave(10, dim=1)
        of = os_ if block is None else os_.repeat_interleave(10, dim=1)
        t = xs / sf
        r = (t + (torch.round(t) - t).detach()) - of
        inr = (r >= qmin) & (r <= qmax)
        qv = torch.where(inr, r, r.detach().clamp(qmin, qmax))
        ((qv + of) * sf).backward(grad)
        assert torch.allclose(gx, xs.grad, atol=1e-6)
        assert torch.allclose(gs, ss.grad, rtol=1e-4, atol=1e-4)
        assert torch.allclose(go, os_.grad, rtol=1e-4, atol=1e-5)


def test_quantize_and_dequantize_gradients_match_plain_autograd():
    """quantize_backward (all three gradients) and dequantize_backward against plain autograd of the compositions
    the reference's functions differentiate by hand: clamp(round_ste(x / s) - o) and (x + o) * s
    (torch_builtins.py:617-655, 674-701).  float64 so that the only differences are summation order."""
    g = torch.Generator().manual_seed(12)
    for shape, sshape, block in [((6, 40), (), None), ((6, 40), (6, 1), None), ((6, 40), (6, 4), (1, 10)),
                                 ((4, 6, 8), (1, 6, 1), None)]:
        scale = (torch.rand(sshape, generator=g) * 0.1 + 0.02).double()
        offset = torch.randint(-200, -50, sshape, generator=g).double()
        qmin, qmax = 0, 255

        def full(t):
            if block is not None:
                return t.repeat_interleave(10, dim=1)
            return t

        # integer part well inside / outside the grid, fraction away from rounding ties; about a fifth is clipped
        base = torch.randint(-60, 320, shape, generator=g).double() + torch.rand(shape, generator=g).double() * 0.8 - 0.4
        x = ((base + full(offset)) * full(scale)).clone()
        grad = torch.randn(shape, generator=g).double()

        gx, gs, go = O.quantize_backward(grad, x, scale, offset, qmin, qmax, block)
        xs, ss, os_ = (t.clone().requires_grad_(True) for t in (x, scale, offset))
        t = xs / full(ss)
        r = (t + (torch.round(t) - t).detach()) - full(os_)
        torch.clamp(r, qmin, qmax).backward(grad)
        clipped = ((r < qmin) | (r > qmax)).sum().item()
        assert 0 < clipped < x.numel()
        assert torch.allclose(gx, xs.grad, rtol=1e-12, atol=0)
        assert torch.allclose(gs, ss.grad, rtol=1e-10, atol=1e-9)
        assert torch.allclose(go, os_.grad, rtol=1e-10, atol=1e-9)

        codes = torch.randint(qmin, qmax + 1, shape, generator=g).double()
        gx, gs, go = O.dequantize_backward(grad, codes, scale, offset, block)
        cs, ss, os_ = (t.clone().requires_grad_(True) for t in (codes, scale, offset))
        ((cs + full(os_)) * full(ss)).backward(grad)
        assert torch.allclose(gx, cs.grad, rtol=1e-12, atol=0)
        assert torch.allclose(gs, ss.grad, rtol=1e-10, atol=1e-9)
        assert torch.allclose(go, os_.grad, rtol=1e-10, atol=1e-9)


def test_reduce_minmax_against_explicit_slices():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 6, 8, generator=g)
    mn, mx = O.reduce_minmax(x, (6, 1))
    assert torch.equal(mn, x.amin(dim=(0, 2)).view(6, 1)) and torch.equal(mx, x.amax(dim=(0, 2)).view(6, 1))
    mn, mx = O.reduce_minmax(x, (3, 2), (2, 4))
    for i in range(3):
        for j in range(2):
            blk = x[:, 2 * i:2 * i + 2, 4 * j:4 * j + 4]
            assert mn[i, j] == blk.min() and mx[i, j] == blk.max()


def test_histogram_counts_are_conserved_and_finite_only():
    obs = O.HistObserver((1,), 64)
    g = torch.Generator().manual_seed(5)
    total = 0
    for k in range(4):
        x = torch.randn(10000, generator=g) * (k + 1)
        x[:3] = torch.tensor([float("inf"), -float("inf"), float("nan")])
        obs.update(x)
        total += 9999  # everything but the NaN lands in some bin (infinities in the edge bins)
        assert abs(obs.stats[0].histogram.sum().item() - total) <= 2 * (k + 1)  # re-binning rounds per source bin
        assert math.isfinite(obs.stats[0].min.item()) and math.isfinite(obs.stats[0].max.item())


@pytest.mark.parametrize("case", ["nested", "straddle"])
def test_histogram_merge_closed_forms(case):
    from tests.helpers import histogram_merge_closed_forms

    bins, first, second, counts, (lo, hi) = histogram_merge_closed_forms()[case]
    obs = O.HistObserver((1,), bins)
    obs.update(first)
    obs.update(second)
    st = obs.stats[0]
    assert st.histogram.tolist() == [float(c) for c in counts]
    assert st.bin_edges[0].item() == lo and st.bin_edges[-1].item() == hi
    assert st.min.item() == lo and st.max.item() == hi


@pytest.mark.parametrize("seed", range(12))
def test_histogram_merges_conserve_every_count(seed):
    """On arbitrary data the ranges grow by arbitrary factors and most old bins are split between two new ones.  A
    split hands round(share * count) to one bin and the REST to the other, so no merge may gain or lose a single
    count: after every batch the histogram sums to the number of values seen, exactly."""
    g = torch.Generator().manual_seed(100 + seed)
    obs = O.HistObserver((1,), [7, 64, 512][seed % 3])
    total = 0
    for _ in range(5):
        spread = 1 + 3 * torch.rand((), generator=g).item()
        x = torch.randn(10000, generator=g) * spread + torch.rand((), generator=g).item()
        obs.update(x)
        total += x.numel()
        assert obs.stats[0].histogram.double().sum().item() == total


@pytest.mark.parametrize("num_bins", [8, 64, 512])
@pytest.mark.parametrize("seed", range(6))
def test_histogram_merge_of_nested_ranges_is_the_histogram_of_all_the_data(num_bins, seed):
    """Re-binning on data nobody chose by hand: ranges that double and then quadruple keep every old bin inside one
    new bin, so whatever the merge does must add up to torch.histc of all the data over the final range (a wrong
    destination index, a dropped or doubled source bin, or a split where none belongs all break the equality)."""
    from tests.helpers import nested_range_batches

    batches, expected, (lo, hi) = nested_range_batches(num_bins, seed)
    obs = O.HistObserver((1,), num_bins)
    for b in batches:
        obs.update(b)
    st = obs.stats[0]
    assert torch.equal(st.histogram, expected)
    assert st.min.item() == lo and st.max.item() == hi
    assert st.bin_edges[0].item() == lo and st.bin_edges[-1].item() == hi
    assert int(st.histogram.sum()) == sum(b.numel() for b in batches)


def test_lpbq_closed_form():
    """Reference: test_affine_quantizer.py:1426-1474."""
    g = torch.Generator().manual_seed(6)
    raw = torch.rand(4, 6, generator=g) * 0.1 + 0.001
    for bw, dbw in [(4, 8), (4, 16), (3, 5), (6, 6)]:
        scale, pcs = O.lpbq_scale(raw, bw, dbw, (1, 3))
        for i in range(4):
            for j in range(2):
                grp = raw[i, 3 * j:3 * j + 3]
                gamma = grp.max() / 2 ** (dbw - bw)
                expect = torch.maximum(torch.tensor([1.0]), torch.round(grp / gamma)) * gamma
                assert torch.equal(expect, scale[i, 3 * j:3 * j + 3])
                assert pcs[i, j] == gamma


def test_percentile():
    G.check_percentile(IMPL)


def _hist_of(lo, hi, bins=8):
    """Statistics whose observed range is [lo, hi] (two elements)."""
    return O.hist_collect(torch.tensor([float(lo), float(hi)]), (), bins)


def test_sqnr_candidate_grid_structure():
    """The reference's own candidate-grid tests (test_encoding_analyzer.py:1066-1165)."""
    # clamp: (delta, offset) pairs reaching beyond the observed range get a smaller delta, the others keep theirs
    deltas = torch.tensor([[1 / 4, 3 / 4, 5 / 4]])
    offsets = torch.tensor([-255.0, -128.0, 0.0])[None, :]
    should_clamp = torch.tensor([[False, False, False], [True, False, True], [True, True, True]])
    d, o = O._clamp_candidates(torch.tensor([-128.0]), torch.tensor([127.0]), 255, deltas, offsets)
    assert torch.all(torch.where(should_clamp, d < deltas[:, :, None], d == deltas[:, :, None]))
    lo = d * o
    assert torch.all(lo > -128.5) and torch.all(lo + d * 255 < 127.5)
    # asymmetric grid: 5 deltas x 7 offsets on [-128, 127]
    d, o = O.sqnr_candidates(_hist_of(-128, 127), 255, False, 5, 101, 7)
    assert d.shape == (1, 5, 7) and o.shape == (1, 5, 7)
    for v in [1 / 4, 1 / 2, 3 / 4, 1]:
        assert v in d
    for v in [-255, -204, -153, -102, -51, 0, -128]:
        assert v in o
    lo = torch.round(o * d)
    assert torch.all(lo > -128.5) and torch.all(lo + d * 255 < 127.5)
    # symmetric grid: 5 deltas, the single offset -128
    d, o = O.sqnr_candidates(_hist_of(-100, 127.5), 255, True, 17, 5, 21)
    assert d.shape == (1, 5, 1)
    for v in [1 / 4, 1 / 2, 3 / 4, 1]:
        assert v in d
    assert o.numel() == 1 and torch.all(o == -128)


def test_sqnr_noise_estimate_and_selection():
    """test_encoding_analyzer.py:1167-1224: the histogram estimate is within 1 % of the quantization error measured
    on the data itself, and the candidate with the least noise is the one selected."""
    g = torch.Generator().manual_seed(13)
    x = torch.randn(2, 1000, generator=g)
    x[0][0] = 100
    x[0][1] = -50
    stats = O.hist_collect(x, (2, 1), 2048)
    deltas = torch.tensor([0.001, 0.1, 0.5, 1.0])[None, :, None].expand(2, 4, 6)
    offsets = torch.tensor([-255.0, -204, -153, -102, -51, 0]).expand_as(deltas)
    xb = x[:, None, None, :].expand(2, 4, 6, -1)
    db, ob = deltas[:, :, :, None], offsets[:, :, :, None]
    qdq = (torch.clamp(torch.round(xb / db) - ob, 0, 255) + ob) * db
    measured = (xb - qdq).square().sum(dim=-1)
    assert torch.allclose(measured, O.sqnr_noise(stats, deltas, offsets, 255, p=2.0, gamma=1.0), rtol=0.01)
    # a clipped bin costs gamma times as much: with everything clipped the noise scales by exactly gamma
    far = torch.full((2, 1, 1), 1e-4)
    n1 = O.sqnr_noise(stats, far, torch.full((2, 1, 1), 1e6), 255, p=2.0, gamma=1.0)
    n3 = O.sqnr_noise(stats, far, torch.full((2, 1, 1), 1e6), 255, p=2.0, gamma=3.0)
    assert torch.allclose(n3, 3 * n1, rtol=1e-6)

    x = (torch.rand(2, 1000, generator=g) - torch.tensor([[0.5], [0.0]])) * torch.tensor([[1.0], [2.0]])
    stats = O.hist_collect(x, (2, 1), 2048)
    deltas = torch.tensor([1 / 510.0, 1 / 255.0, 2 / 255.0])[None, :, None].expand(2, 3, 3)
    offsets = torch.tensor([-200.0, -128, 0]).expand_as(deltas)
    noise = O.sqnr_noise(stats, deltas, offsets, 255, p=2.0, gamma=1.0)
    idx = noise.flatten(start_dim=1).argmin(dim=1)
    assert torch.equal(deltas.flatten(start_dim=1).gather(1, idx[:, None]), torch.tensor([1 / 255.0, 2 / 255.0]).view(2, 1))
    assert torch.equal(offsets.flatten(start_dim=1).gather(1, idx[:, None]), torch.tensor([-128.0, 0]).view(2, 1))


def test_hist_collect_is_histc_per_slot():
    """hist_collect: each slot is torch.histc over the slot's own range, top edge inclusive
    (encoding_analyzer.py:189-229)."""
    g = torch.Generator().manual_seed(14)
    x = torch.randn(3, 500, generator=g)
    stats = O.hist_collect(x, (3, 1), 16)
    for r, st in enumerate(stats):
        lo, hi = x[r].min(), x[r].max()
        counts = [0] * 16
        for v in x[r].tolist():
            counts[min(int((v - lo.item()) * 16 / (hi.item() - lo.item())), 15)] += 1
        assert st.min == lo and st.max == hi and st.histogram.sum() == 500
        # float32 against double arithmetic may move an element sitting on an edge: none here
        assert st.histogram.tolist() == [float(c) for c in counts]
        assert st.bin_edges[0] == lo and torch.allclose(st.bin_edges[-1], hi)


def test_scale_and_offset_from_a_range():
    """scale_from_minmax / offset_from_minmax / scale_offset_dynamic: the reference's low-bitwidth expectations
    (test_affine_quantizer.py:397-406: scale 5.25 / 7.0 / 3.5 / 3.0 from a calibration on [-10.5, 10.5]) and the
    definitions worked by hand."""
    for bw, symmetric, want in G.VECTORS["low_bw_scales"]["cases"]:
        qmin, qmax = (-(2 ** (bw - 1)), 2 ** (bw - 1) - 1) if symmetric else (0, 2 ** bw - 1)
        lo, hi = O.minmax_encodings(torch.tensor(-10.5), torch.tensor(10.5), qmax - qmin, symmetric)
        assert O.scale_from_minmax(lo, hi, qmin, qmax).item() == want
        s_dyn, o_dyn = O.scale_offset_dynamic(lo, hi, qmin, qmax, symmetric)
        assert s_dyn.item() == want
        off = O.offset_from_minmax(lo, O.scale_from_minmax(lo, hi, qmin, qmax), qmin, qmax, symmetric)
        assert off.item() == o_dyn.item()
        if symmetric:
            assert off.item() == -round((qmin + qmax) / 2) == 0  # round(-0.5) is 0 (ties to even): not +1
    # asymmetric by hand: [-1, 3] on 0..255: scale 4 / 255, offset round(-1 / scale) = round(-63.75) = -64
    s = O.scale_from_minmax(torch.tensor(-1.0), torch.tensor(3.0), 0, 255)
    assert s.item() == (torch.tensor(4.0) / 255).item()
    assert O.offset_from_minmax(torch.tensor(-1.0), s, 0, 255, False).item() == -64.0
    # the offset is clamped to [-qmax, -qmin]: a range that does not hold zero
    s = O.scale_from_minmax(torch.tensor(1.0), torch.tensor(3.0), 0, 255)
    assert O.offset_from_minmax(torch.tensor(1.0), s, 0, 255, False).item() == 0.0
    assert O.offset_from_minmax(torch.tensor(-9.0), s, 0, 255, False).item() == -255.0
    # a reversed or empty range: |.| and the minimum scale
    assert O.scale_from_minmax(torch.tensor(3.0), torch.tensor(-1.0), 0, 255).item() == (torch.tensor(4.0) / 255).item()
    assert O.scale_from_minmax(torch.tensor(0.0), torch.tensor(0.0), 0, 255).item() == O.minimum_scale(255)
    assert O.minimum_scale(255) == min(torch.finfo(torch.float32).eps, 0.01 / 255)


def test_float_dequantize_is_a_product_per_block():
    x = torch.arange(24.0).reshape(4, 6)
    scale = torch.tensor([[0.5, 2.0, 4.0]] * 4)
    want = x * scale.repeat_interleave(2, dim=1)
    assert torch.equal(O.float_dequantize(x, scale, (1, 2)), want)
    assert torch.equal(O.float_dequantize(x, torch.tensor(0.25)), x * 0.25)
