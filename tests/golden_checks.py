"""Checks of the reference-held vectors in tests/golden/reference_vectors.json, written against a small adapter so
that the same assertions pin the CPU oracle (tests/test_oracle_golden.py) and the HIP path (tests/test_golden_gpu.py).

An adapter provides:
    quantize(x, scale, offset, qmin, qmax, block) -> codes
    dequantize(codes, scale, offset, block) -> values
    qdq(x, scale, offset, qmin, qmax, block, zps) -> y
    qdq_backward(g, x, scale, offset, qmin, qmax, block, zps) -> (gx, gscale, goffset)
    quantize_backward(g, x, scale, offset, qmin, qmax, block) -> gx
    minmax_encodings(x, num_steps, symmetric) -> (min, max)           per-tensor min-max analyzer
    hist_observer(num_bins) -> object with update(x) and stat() -> (histogram, bin_edges, min, max) as CPU tensors
    sqnr(x_batches, num_steps, symmetric, **analyzer kwargs) -> (min, max)
    percentile(x_batches, shape, num_bins, percentile, num_steps, symmetric) -> (min, max, histograms, bin_edges)
        histograms / bin_edges: one CPU tensor per slot of the analyzer's statistics
"""

import json
import math
import os

import torch

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.json")
with open(_PATH) as _f:
    VECTORS = json.load(_f)


def _t(v, dtype=torch.float32):
    def conv(e):
        if isinstance(e, list):
            return [conv(i) for i in e]
        if e == "inf":
            return float("inf")
        if e == "-inf":
            return -float("inf")
        return e
    return torch.tensor(conv(v), dtype=dtype)


def vector_set_names():
    return [k for k in VECTORS["qdq_vector_sets"] if not k.startswith("_")]


def check_vector_set(impl, name, dtype):
    vs = VECTORS["qdq_vector_sets"][name]
    x = _t(vs["tensor"], dtype)
    codes = _t(vs["tensor_q"], dtype)
    qdq = _t(vs["tensor_qdq"], dtype)
    clipped = _t(vs["mask"], torch.bool)
    scale = _t(vs["delta"])
    offset = _t(vs["offset"])
    qmin, qmax = vs["qmin"], vs["qmax"]

    q = impl.quantize(x, scale, offset, qmin, qmax, None)
    if dtype == torch.bfloat16:
        # the reference tolerates one code on exact rounding boundaries for bfloat16 (test_backend.py:641-648)
        boundary = (x.float() / scale - offset) % 1 == 0.5
        assert bool(torch.where(boundary, (q.float() - codes.float()).abs() <= 1, q == codes).all())
    else:
        assert torch.equal(q, codes), f"{name}: quantize"
    assert torch.equal(impl.dequantize(codes, scale, offset, None), qdq), f"{name}: dequantize"
    y = impl.qdq(x, scale, offset, qmin, qmax, None, 0.0)
    if dtype != torch.bfloat16:
        assert torch.allclose(y, qdq), f"{name}: quantize-dequantize"
    g = torch.randn(x.shape, generator=torch.Generator().manual_seed(0)).to(dtype)
    gx, _, _ = impl.qdq_backward(g, x, scale, offset, qmin, qmax, None, 0.0)
    assert bool((gx[clipped] == 0).all()), f"{name}: gradient of clipped elements"
    assert torch.equal(gx[~clipped], g[~clipped]), f"{name}: gradient of in-range elements"
    gq = impl.quantize_backward(g, x, scale, offset, qmin, qmax, None)
    assert bool((gq[clipped] == 0).all())
    expect = (g.float() / scale.expand(x.shape) if scale.numel() > 1 else g.float() / scale)
    assert torch.allclose(gq[~clipped].float(), expect[~clipped], rtol=1e-2 if dtype != torch.float32 else 1e-5)


def check_block_quant(impl):
    bq = VECTORS["block_quant"]
    x = _t(bq["input"])
    for case in bq["cases"]:
        scale = _t(case["scale"])
        offset = torch.zeros_like(scale)
        block = case["block_size"]
        q = impl.quantize(x, scale, offset, -128, 127, block)
        assert torch.equal(q, _t(case["codes"])), f"block quant {case}"
        assert torch.allclose(impl.dequantize(q, scale, offset, block), x, atol=1e-6)
        assert torch.allclose(impl.qdq(x, scale, offset, -128, 127, block, 0.0), x, atol=1e-6)


def check_docstring_examples(impl):
    ex = VECTORS["docstring_examples"]
    x = torch.arange(start=-0.3, end=1.3, step=0.05)
    scale, offset = torch.tensor(1 / 15), torch.tensor(0.0)
    assert torch.equal(impl.quantize(x, scale, offset, 0, 15, None), _t(ex["codes"]))
    y = impl.qdq(x, scale, offset, 0, 15, None, 0.0)
    assert torch.allclose(y, _t(ex["qdq_4_decimals"]), atol=5.1e-5)


def check_clipped_scale_gradient(impl):
    spec = VECTORS["clipped_scale_gradient"]
    for lay in spec["layouts"]:
        for inp in spec["inputs"]:
            for zps in spec["zero_point_shifts"]:
                x = torch.full(lay["input_shape"], inp["value"])
                scale = torch.ones(lay["scale_shape"])
                offset = torch.full(lay["scale_shape"], -1.0)
                block = lay["block_size"]
                g = torch.full_like(x, 5.0 * scale.numel() / x.numel())
                expected = inp["bound"] - 1.0 + zps
                y = impl.qdq(x, scale, offset, 0, 3, block, zps)
                torch.testing.assert_close(y, torch.full_like(y, expected))
                gx, gs, go = impl.qdq_backward(g, x, scale, offset, 0, 3, block, zps)
                torch.testing.assert_close(gs, torch.full_like(scale, 5.0 * expected))
                torch.testing.assert_close(gx, torch.zeros_like(x))
                torch.testing.assert_close(go, torch.full_like(offset, 5.0))
                # inputs stay clipped under a small perturbation of the scale: the finite difference is the derivative
                eps = 2 ** -10
                fd = ((impl.qdq(x, scale + eps, offset, 0, 3, block, zps)
                       - impl.qdq(x, scale - eps, offset, 0, 3, block, zps)) * g).sum() / (2 * eps)
                torch.testing.assert_close(gs.sum(), fd)


def _named_input(name):
    if name == "arange(0, 26, 0.5)":
        return torch.arange(start=0, end=26, step=0.5)
    if name == "arange(-2, 10, 1)":
        return torch.arange(start=-2, end=10, step=1, dtype=torch.float)
    if name == "full(3.0)":
        return torch.full((1,), 3.0)
    if name == "pair(-10.5, 10.5)":
        return torch.tensor([-10.5, 10.5])
    if name == "arange(0, 1001)":
        return torch.arange(start=0, end=1001, step=1, dtype=torch.float)
    if name == "zeros()":
        return torch.zeros(())
    if name == "arange(-50, 51)":
        return torch.arange(-50, 51, dtype=torch.float)
    if name == "arange(-50, 51) * 1.5":
        return torch.arange(-50, 51, dtype=torch.float) * 1.5
    raise KeyError(name)


def check_minmax_encodings(impl):
    for c in VECTORS["minmax_encodings"]["cases"]:
        lo, hi = impl.minmax_encodings(_named_input(c["input"]), c["num_steps"], c["symmetric"])
        if c["exact"]:
            assert lo.item() == c["min"] and hi.item() == c["max"], c
        else:
            assert torch.allclose(lo, torch.full_like(lo, c["min"])) and torch.allclose(hi, torch.full_like(hi, c["max"])), c
    # all-zero input: the range is widened to the minimum scale (test_encoding_analyzer.py:251-274)
    ms = min(float(torch.finfo(torch.float32).eps), 0.01 / 255)
    lo, hi = impl.minmax_encodings(torch.zeros(4), 255, False)
    assert torch.allclose(lo, torch.zeros_like(lo)) and torch.allclose(hi, torch.full_like(hi, ms * 255))
    lo, hi = impl.minmax_encodings(torch.zeros(4), 255, True)
    assert torch.allclose(lo, torch.full_like(lo, -ms * 128)) and torch.allclose(hi, torch.full_like(hi, ms * 127))
    # constant non-zero input, symmetric: one more level on the negative side (test_encoding_analyzer.py:240-249)
    lo, hi = impl.minmax_encodings(torch.full((3,), 3.0), 255, True)
    assert torch.allclose(hi, torch.full_like(hi, 3.0)) and torch.allclose(lo, -3.0 - hi / 127)


def check_histogram_merges(impl):
    hm = VECTORS["histogram_merges"]
    dm = hm["during_merging"]
    obs = impl.hist_observer(dm["num_bins"])
    for name in dm["updates"]:
        obs.update(_named_input(name))
    h, e, _, _ = obs.stat()
    assert h.tolist() == dm["histogram"]
    assert e.tolist() == dm["bin_edges"]
    for seq in hm["sequences"]:
        obs = impl.hist_observer(seq["num_bins"])
        for step in seq["steps"]:
            obs.update(_t(step["input"]))
            h, e, mn, mx = obs.stat()
            assert mn.item() == torch.tensor(step["min"], dtype=torch.float32).item(), (seq["name"], step)
            assert mx.item() == torch.tensor(step["max"], dtype=torch.float32).item(), (seq["name"], step)
            assert torch.equal(h, _t(step["histogram"])), (seq["name"], step, h)
            if step["edges_exact"]:
                assert torch.equal(e, _t(step["bin_edges"])), (seq["name"], step)
            else:
                assert torch.allclose(e, _t(step["bin_edges"])), (seq["name"], step)
    inf = hm["inf_inputs"]
    obs = impl.hist_observer(inf["num_bins"])
    prev = None
    for step in inf["steps"]:
        obs.update(_t(step["input"]))
        h, e, mn, mx = obs.stat()
        if "min" in step:
            assert mn.item() == step["min"] and mx.item() == step["max"]
        if "last_bin" in step:
            assert h[-1].item() == step["last_bin"]
        if "first_bin" in step:
            assert h[0].item() == step["first_bin"]
        if "bin_edges" in step:
            assert torch.allclose(e, _t(step["bin_edges"]))
        if "first_bin_delta" in step:
            assert h[0].item() == prev[0].item() + step["first_bin_delta"]
            assert h[-1].item() == prev[-1].item() + step["last_bin_delta"]
        prev = h.clone()


def check_sqnr_uniform(impl):
    n = VECTORS["sqnr"]["uniform"]["num_steps"]
    x = torch.arange(-100, 101) / 100
    delta = torch.tensor(2 / 255.0)
    off = torch.round(-1 / delta)
    lo_ref = off * delta
    hi_ref = lo_ref + 255 * delta
    lo, hi = impl.sqnr([x], n, False, gamma=1)
    assert torch.equal(lo, lo_ref.view((1,)))
    assert torch.equal(hi, hi_ref.view((1,)))


def check_sqnr_outlier(impl):
    """test_encoding_analyzer.py:994-1029: the optimum clips a lone outlier at 3/4 of its value."""
    expected_delta = torch.tensor([0.1])
    outlier = (255 * expected_delta) / 0.75
    n = round(12 * 255 * outlier.item() / expected_delta.item() - 12 * (255 ** 2))
    x = torch.rand((1, n), generator=torch.Generator().manual_seed(0)) * 255 * expected_delta
    lo, hi = impl.sqnr([x, outlier.view(1, 1)], 255, False, gamma=1.0)
    assert torch.allclose(lo, torch.zeros_like(lo))
    assert torch.allclose(hi, expected_delta * 255)


def check_sqnr_brute_force(impl):
    """Independent of the oracle's tensor code: enumerate every candidate with Python floats on a tiny histogram and
    require the implementation's encoding to be (near-)optimal under the documented cost."""
    g = torch.Generator().manual_seed(4)
    x = torch.cat([torch.randn(4000, generator=g), torch.tensor([9.0, -7.5])])
    num_steps, D, O, gamma, B = 15, 9, 7, 3.0, 32
    lo, hi = impl.sqnr([x], num_steps, False, num_bins=B, asymmetric_delta_candidates=D, offset_candidates=O, gamma=gamma)
    delta_sel = (hi.item() - lo.item()) / num_steps
    # histogram with the documented edges
    xmin, xmax = x.min().item(), x.max().item()
    w = (xmax - xmin) / B
    counts = [0] * B
    for v in x.tolist():
        b = min(int((v - xmin) / w), B - 1)
        counts[b] += 1
    mids = [xmin + w / 2 + w * b for b in range(B)]

    def cost(delta, off):
        c = 0.0
        for m, n in zip(mids, counts):
            q = round(m / delta - off)
            clipped = q < 0 or q > num_steps
            q = min(max(q, 0), num_steps)
            e = ((q + off) * delta - m) ** 2 * n
            c += e * gamma if clipped else e
        return c

    lo0, hi0 = min(xmin, 0.0), max(xmax, 0.0)
    dmax = (hi0 - lo0) / num_steps
    obs_off = round(lo0 / dmax)
    obs_min, obs_max = dmax * obs_off, dmax * obs_off + dmax * num_steps
    step = num_steps / (O - 2)
    offs = [round(-num_steps + i * step) for i in range(O - 1)] + [obs_off]
    best = None
    for k in range(1, D + 1):
        d = dmax * k / (D - 1)
        for o in offs:
            tmin = max(obs_min, d * o)
            tmax = min(obs_max, d * o + d * num_steps)
            dd = max((tmax - tmin) / num_steps, 1e-12)
            oo = round(tmin / dd)
            c = cost(dd, oo)
            if best is None or c < best[0]:
                best = (c, dd, oo)
    sel_cost = cost(delta_sel, round(lo.item() / delta_sel))
    assert sel_cost <= best[0] * (1 + 1e-4), (sel_cost, best)


def check_percentile(impl):
    """The percentile analyzer on the cases the reference's tests hold (test_encoding_analyzer.py:556-612, 886-971),
    plus two results derived by hand that fix which side of a tie the cumulative search takes."""
    pv = VECTORS["percentile"]
    for c in pv["exact"]:
        lo, hi, _, _ = impl.percentile([_named_input(c["input"])], (), c["num_bins"], c["percentile"], c["num_steps"],
                                       c["symmetric"])
        assert lo.item() == c["min"] and hi.item() == c["max"], (c, lo, hi)
    for c in pv["close"]:
        lo, hi, _, _ = impl.percentile([_named_input(c["input"])], (), c["num_bins"], c["percentile"], c["num_steps"],
                                       c["symmetric"])
        assert torch.allclose(lo, torch.full_like(lo, c["min"])) and torch.allclose(hi, torch.full_like(hi, c["max"])), c
    for c in pv["quantile_index"]:
        x = _named_input(c["input"])
        if c["input"] == "full(3.0)":
            x = x.reshape(())
        n = c["num_steps"]
        lo_a, hi_a, hists, edges = impl.percentile([x], (), c["num_bins"], c["percentile"], n, False)
        cs = torch.cumsum(hists[0], dim=0)
        value = edges[0][torch.searchsorted(cs, torch.quantile(cs, c["q"]))]
        if c["expect"] == "constant":
            # :556-583: asymmetric (0, v); symmetric (-v - max / (n // 2), v)
            lo_s, hi_s, _, _ = impl.percentile([x], (), c["num_bins"], c["percentile"], n, True)
            assert torch.allclose(lo_a, torch.zeros_like(lo_a)) and torch.allclose(hi_a, torch.full_like(hi_a, value))
            assert torch.allclose(hi_s, torch.full_like(hi_s, value))
            assert torch.allclose(lo_s, torch.full_like(lo_s, -value) - hi_s / (n // 2))
        elif c["expect"] == "zero":
            # :585-612: asymmetric (v, 0); symmetric with n - 1 steps (v, -v)
            lo_s, hi_s, _, _ = impl.percentile([x], (), c["num_bins"], c["percentile"], n - 1, True)
            assert torch.allclose(lo_a, torch.full_like(lo_a, value)) and torch.allclose(hi_a, torch.zeros_like(hi_a))
            assert torch.allclose(lo_s, torch.full_like(lo_s, value)) and torch.allclose(hi_s, torch.full_like(hi_s, -value))
        else:
            # :933-955: symmetric with n - 1 steps gives -+ the middle edge; asymmetric (0, middle edge), exactly
            lo_s, hi_s, _, _ = impl.percentile([x], (), c["num_bins"], c["percentile"], n - 1, True)
            assert lo_s.item() == -value.item() and hi_s.item() == value.item()
            assert lo_a.item() == 0 and hi_a.item() == value.item()
    # :913-931: the 100th percentile is the observed range
    x = torch.randn(10000, generator=torch.Generator().manual_seed(11)) * 2 + 2
    lo, hi, _, _ = impl.percentile([x], (), 3, 100, 254, True)
    assert torch.allclose(lo, -x.abs().max()) and torch.allclose(hi, x.abs().max())
    lo, hi, _, _ = impl.percentile([x], (), 3, 100, 255, False)
    assert torch.allclose(lo, x.min()) and torch.allclose(hi, x.max())
    # :957-971: two outliers above a ramp
    o = pv["outliers"]
    x = torch.arange(start=0, end=101, step=1, dtype=torch.float)
    x[-1] = 1000
    x[-2] = 800
    _, hi, _, _ = impl.percentile([x], tuple(o["shape"]), o["num_bins"], o["percentile"], o["num_steps"], False)
    assert o["max_above"] < hi.item() < o["max_below"]
    # By hand.  Eight values in four bins of width 2 over [0, 8] give counts 2, 2, 2, 2 and cumulative counts 2, 4,
    # 6, 8.  At 50 % both targets are exactly 4.0 = the second cumulative count: the first position whose count is
    # NOT BELOW the target is bin 1, whose left edge is 2.0 (a search for the first count ABOVE it would give 4.0).
    x = torch.tensor([0.0, 1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 8.0])
    lo, hi, hists, edges = impl.percentile([x], (), 4, 50, 255, False)
    assert hists[0].tolist() == [2.0, 2.0, 2.0, 2.0] and edges[0].tolist() == [0.0, 2.0, 4.0, 6.0, 8.0]
    assert lo.item() == 0.0 and hi.item() == 2.0, (lo, hi)
    # Shifted to [-8, 0]: the lower edge survives the "zero in range" rule, the upper one is raised to 0.  At 75 %
    # the targets are 6.0 (upper: bin 2, edge -4) and 2.0 (lower: bin 0, edge -8): (-8, 0).  Symmetric with 254
    # steps: delta = max(0 / 127, 8 / 127), so (-8, 8) up to the rounding of 127 * (8 / 127).
    lo, hi, _, _ = impl.percentile([x - 8.0], (), 4, 75, 255, False)
    assert lo.item() == -8.0 and hi.item() == 0.0, (lo, hi)
    lo, hi, _, _ = impl.percentile([x - 8.0], (), 4, 75, 254, True)
    assert abs(lo.item() + 8.0) < 1e-6 and abs(hi.item() - 8.0) < 1e-6
    # Two slots of one analyzer are independent: slot 0 is the ramp above, slot 1 its mirror image.
    both = torch.stack([x, -x])
    lo, hi, _, _ = impl.percentile([both], (2, 1), 4, 50, 255, False)
    assert lo.flatten().tolist() == [0.0, -4.0] and hi.flatten().tolist() == [2.0, 0.0], (lo, hi)
