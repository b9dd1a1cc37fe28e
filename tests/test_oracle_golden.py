"""Pins the CPU oracle (oracle/torch_ref.py) against the vectors the reference's own tests and docstrings hold, and
against facts the mathematics fixes.  Which check pins which oracle function:

    quantize_forward / dequantize_forward / qdq_v2_forward / qdq_v2_backward / quantize_backward
        golden vector sets, block-quantization table, docstring examples, clipped-scale gradient closed form with a
        finite-difference check, block == per-tensor call on the block, STE autograd cross-check
    qdq_v1                     the installed ATen kernels themselves (library routine) + closed form
    internal_dtype             the dtype table of the reference's test_affine_quantizer.py:1761-1768
    reduce_minmax              torch.amin/amax on explicitly sliced blocks
    minmax_encodings           exact expected min/max of the reference's analyzer tests, zero / constant inputs
    HistObserver               the reference's merge sequences (exact counts and edges), +-inf handling, count conservation,
                               two merges with hand-derived results (nested bins; bins cut in half, rounding half to even)
    sqnr_encodings             uniform-distribution closed form, outlier optimum, brute-force enumeration in Python floats
    lpbq_scale                 closed form max(1, round(s / gamma)) * gamma
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
