"""Parity of the HIP calibration path (histogram observer, SQNR / TF-enhanced search, percentile, min-max encodings)
with the CPU oracle.

Bar: histogram bin counts, bin edges, stored min/max and min-max encodings bit-exact; SQNR-selected candidate index
identical and the selected delta/offset/min/max bit-exact (the candidates are produced by the same fp32 operations);
per-candidate noise sums within 1e-5 relative (fp64 accumulation here, fp32 cascade sums in the reference).
"""

import math

import pytest
import torch

from oracle import torch_ref as O
from tests.helpers import assert_same_bits, assert_close_rel

pytestmark = pytest.mark.gpu


def _laplace_with_outliers(shape, seed, frac=0.001):
    g = torch.Generator().manual_seed(seed)
    u = torch.rand(shape, generator=g) - 0.5
    x = -torch.sign(u) * torch.log1p(-2 * u.abs())
    n = x.numel()
    k = max(1, int(n * frac))
    idx = torch.randperm(n, generator=g)[:k]
    out = (torch.rand(k, generator=g) * 40 + 20) * torch.sign(torch.rand(k, generator=g) - 0.5)
    x.view(-1)[idx] = out
    return x


def _check_hist_lists(got, ref, what):
    assert len(got) == len(ref)
    for s, (a, b) in enumerate(zip(got, ref)):
        assert_same_bits(a.histogram, b.histogram, f"{what}[{s}].histogram")
        assert_same_bits(a.bin_edges, b.bin_edges, f"{what}[{s}].bin_edges")
        assert a.min.dtype == b.min.dtype, f"{what}[{s}].min dtype {a.min.dtype} vs {b.min.dtype}"
        assert_same_bits(a.min, b.min, f"{what}[{s}].min")
        assert_same_bits(a.max, b.max, f"{what}[{s}].max")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("num_bins", [512, 10, 2048, 3])
@pytest.mark.parametrize("growth", [None, 3.0, 1.0])
def test_histogram_stream_single_slot(device, dtype, num_bins, growth):
    """Five batches with drifting ranges (growth, shrink, identical range, clamped growth)."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    obs = _HistogramObserver((1,), num_bins=num_bins, growth_limit=growth)
    ref = O.HistObserver((1,), num_bins, growth)
    g = torch.Generator().manual_seed(11)
    batches = [
        torch.randn(3, 4099, generator=g),
        torch.randn(3, 4099, generator=g) * 2.5 + 1.0,        # wider
        torch.randn(3, 4099, generator=g) * 0.3,              # inside
        torch.randn(3, 4099, generator=g) * 40.0 - 5.0,       # far beyond the growth limit
        torch.cat([torch.randn(3, 4096, generator=g), torch.tensor([[float("inf"), -float("inf"), float("nan")]] * 3)], dim=1),
    ]
    for k, b in enumerate(batches):
        b = b.to(dtype)
        new_ref = ref.update(b)
        new = obs.update(b.to(device))
        _check_hist_lists(new, new_ref, f"batch {k} own statistics")
        _check_hist_lists(obs.get_stats(), ref.stats, f"running statistics after batch {k}")


def _range_whose_last_edge_rounds(num_bins, below: bool, seed):
    """(lo, hi) in float32 such that the last bin edge B * RN((hi - lo) / B) + lo lies below (or above) hi."""
    g = torch.Generator().manual_seed(seed)
    for _ in range(10000):
        lo = (torch.rand((), generator=g) * 4 - 3).float()
        hi = (lo + torch.rand((), generator=g) * 5 + 0.5).float()
        last = torch.tensor(float(num_bins)) * ((hi - lo) / num_bins) + lo
        if (below and last < hi) or (not below and last > hi):
            return lo, hi
    raise AssertionError("no such range found")


@pytest.mark.parametrize("num_bins", [512, 10, 100])
@pytest.mark.parametrize("below", [True, False], ids=["last_edge_below_max", "last_edge_above_max"])
def test_histogram_repeated_batches_and_maxima_at_the_running_maximum(device, num_bins, below):
    """The reference clamps a batch's maximum with the last bin EDGE, which rounding can put below or above the running
    maximum (encoding_analyzer.py:266-270).  Seeing the same tensor again, a batch whose maximum equals the running
    maximum, and one whose maximum lies between the last edge and the running maximum must all leave the running
    statistics as the reference has them."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    lo, hi = _range_whose_last_edge_rounds(num_bins, below, seed=num_bins)
    g = torch.Generator().manual_seed(3)
    n = 3 * 4099
    base = torch.rand(n, generator=g) * (hi - lo) + lo
    base = base.clamp(lo, hi)
    base[17], base[n - 5] = lo, hi
    inside = torch.rand(n, generator=g) * (hi - lo) * 0.5 + lo
    at_max = inside.clone()
    at_max[n // 2] = hi
    just_below = inside.clone()
    just_below[7] = torch.nextafter(hi, lo)  # between the last edge and the maximum when the edge rounds further down
    batches = [base, base, at_max, just_below, inside, base * 1.25, base * 1.25, at_max]
    obs = _HistogramObserver((1,), num_bins=num_bins)
    ref = O.HistObserver((1,), num_bins, None)
    for k, b in enumerate(batches):
        ref.update(b)
        obs.update(b.to(device))
        _check_hist_lists(obs.get_stats(), ref.stats, f"running statistics after batch {k}")


@pytest.mark.parametrize("case", [((4, 1), None, (4, 300)), ((2, 3), (2, 5), (4, 15)), ((3, 1, 1), None, (2, 3, 5, 7)),
                                  ((4, 1), None, (4, 5000)), ((3, 1, 1), None, (2, 3, 64, 64)), ((2, 2), (3, 2048), (6, 4096))],
                         ids=["per_channel", "blockwise", "activation_channels", "long_rows_ragged_tiles",
                              "activation_channels_long_runs", "blockwise_long_runs"])
def test_histogram_several_slots(device, case):
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    shape, block, xshape = case
    obs = _HistogramObserver(shape, num_bins=16, block_size=block)
    ref = O.HistObserver(shape, 16, None, block)
    g = torch.Generator().manual_seed(2)
    for k in range(3):
        x = torch.randn(xshape, generator=g) * (1 + k)
        if x.numel() > 1000:
            x.view(-1)[5], x.view(-1)[77], x.view(-1)[-3] = float("nan"), float("inf"), float("-inf")
            x.view(-1)[100:140] = 0.0
        new_ref = ref.update(x)
        new = obs.update(x.to(device))
        _check_hist_lists(new, new_ref, f"batch {k}")
        _check_hist_lists(obs.get_stats(), ref.stats, f"running {k}")


@pytest.mark.parametrize("case", [((1,), None, (3, 70001)), ((4, 1), None, (4, 5000)), ((2, 3), (2, 5), (4, 15))],
                         ids=["single_slot", "rows", "blockwise"])
def test_histogram_update_with_and_without_the_batch_histogram(device, case):
    """ahq_hist_update with new_hist: both histograms in one pass (what the oracle's update returns and keeps);
    without: only the running one, bit-identical, and the batch's own edges / min / max are still written; without
    those either: the running statistics alone (a single slot is then binned speculatively on the running range)."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    shape, block, xshape = case
    both = _HistogramObserver(shape, num_bins=32, block_size=block)
    only = _HistogramObserver(shape, num_bins=32, block_size=block)
    bare = _HistogramObserver(shape, num_bins=32, block_size=block)  # running statistics only
    ref = O.HistObserver(shape, 32, None, block)
    g = torch.Generator().manual_seed(5)
    for k in range(3):
        x = torch.randn(xshape, generator=g) * (1 + 0.7 * k) + 0.1 * k
        new_ref = ref.update(x)
        xd = x.to(device)
        for obs in (both, only, bare):
            if obs._state is None:
                obs._state = obs._alloc(xd.device)
        h2, e2, mm2 = both._run(xd, both._state, first=(k == 0), batch_hist=True)
        h1, e1, mm1 = only._run(xd, only._state, first=(k == 0), batch_hist=(k == 0))
        assert (h1 is None) == (k > 0)
        h0, e0, mm0 = bare._run(xd, bare._state, first=(k == 0), batch_hist=(k == 0), batch_stats=(k == 0))
        assert (e0 is None) == (k > 0) and (mm0 is None) == (k > 0)
        for key in ("hist", "edges", "minmax", "limits"):
            assert_same_bits(bare._state[key], both._state[key], f"running {key} after batch {k} (running statistics only)")
        for s_, r in enumerate(new_ref):
            assert_same_bits(h2[s_], r.histogram, f"batch {k} slot {s_} own histogram")
            assert_same_bits(e2[s_], r.bin_edges, f"batch {k} slot {s_} own edges")
        assert_same_bits(e1, e2, f"batch {k} own edges")
        assert_same_bits(mm1, mm2, f"batch {k} own min/max")
        for key in ("hist", "edges", "minmax", "limits"):
            assert_same_bits(only._state[key], both._state[key], f"running {key} after batch {k}")
        for s_, r in enumerate(ref.stats):
            assert_same_bits(only._state["hist"][s_], r.histogram, f"running histogram after batch {k} slot {s_}")


@pytest.fixture
def table_binning():
    """Route every eligible 16-bit histogram update through the table kernel, whatever the tensor's size."""
    from aimet_amd import _lib

    lib = _lib.load()
    before = lib.ahq_hist_table_min_numel(0)
    yield
    lib.ahq_hist_table_min_numel(before)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("num_bins", [512, 2048, 7, 5000])
@pytest.mark.parametrize("numel", [8 * 1024 * 37 + 13, 1024 * 8, 1001, 5], ids=lambda n: f"n{n}")
def test_histogram_of_16_bit_tensors_through_the_table(device, table_binning, dtype, num_bins, numel):
    """Running statistics only, one slot, 16-bit elements: the kernel that looks bins up in a 64K-entry table.  Batches
    inside the running range (binned speculatively), beyond it on either side (binned again), with zeros of both signs,
    infinities and NaN, with and without a ragged tail; counts, edges and min/max bit-exact against the oracle, and
    the same with the table switched off."""
    from aimet_amd import _lib
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    table = _HistogramObserver((1,), num_bins=num_bins)
    arith = _HistogramObserver((1,), num_bins=num_bins)
    ref = O.HistObserver((1,), num_bins, None)
    g = torch.Generator().manual_seed(numel + num_bins)
    scales = [(1.0, 0.0), (0.5, 0.1), (3.0, 0.0), (1.0, -9.0), (0.2, 0.0), (1.0, 0.0)]
    lib = _lib.load()
    for k, (s_, shift) in enumerate(scales):
        x = torch.randn(numel, generator=g) * s_ + shift
        if k == 4:
            x = torch.relu(x)
            x[::5] = -0.0
        if k == 5 and numel >= 5:
            x[0], x[1], x[-1] = float("inf"), float("nan"), -float("inf")
        x = x.to(dtype)
        ref.update(x)
        xd = x.to(device)
        for obs, threshold in ((table, 0), (arith, 1 << 62)):
            if obs._state is None:
                obs._state = obs._alloc(xd.device)
            lib.ahq_hist_table_min_numel(threshold)
            obs._run(xd, obs._state, first=(k == 0), batch_hist=False, batch_stats=False)
        lib.ahq_hist_table_min_numel(0)
        for key in ("hist", "edges", "minmax", "limits"):
            assert_same_bits(table._state[key], arith._state[key], f"running {key} after batch {k}")
        r = ref.stats[0]
        assert_same_bits(table._state["hist"][0], r.histogram, f"running histogram after batch {k}")
        assert_same_bits(table._state["edges"][0], r.bin_edges, f"running edges after batch {k}")
        assert table._state["minmax"][0, 0].item() == r.min.float().item()
        assert table._state["minmax"][0, 1].item() == r.max.float().item()


def test_table_threshold_knob(device):
    from aimet_amd import _lib

    lib = _lib.load()
    default = lib.ahq_hist_table_min_numel(-1)
    assert default == 48 << 20
    assert lib.ahq_hist_table_min_numel(123) == default
    assert lib.ahq_hist_table_min_numel(-1) == 123
    assert lib.ahq_hist_table_min_numel(default) == 123


@pytest.mark.parametrize("case", ["nested", "straddle"])
def test_histogram_merge_closed_forms(device, case):
    """The merges whose result is known by hand (tests/helpers.py), on the HIP path."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver
    from tests.helpers import histogram_merge_closed_forms

    bins, first, second, counts, (lo, hi) = histogram_merge_closed_forms()[case]
    obs = _HistogramObserver((1,), num_bins=bins)
    obs.update(first.to(device))
    obs.update(second.to(device))
    st = obs.get_stats()[0]
    assert st.histogram.tolist() == [float(c) for c in counts]
    assert st.bin_edges[0].item() == lo and st.bin_edges[-1].item() == hi
    assert st.min.item() == lo and st.max.item() == hi


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("num_bins", [8, 64, 512])
@pytest.mark.parametrize("seed", range(3))
def test_histogram_merge_of_nested_ranges_is_the_histogram_of_all_the_data(device, num_bins, seed, dtype):
    """The randomized closed form of tests/test_oracle_golden.py on the HIP path (every value of the dyadic grid is
    a bfloat16 value too while num_bins <= 64; beyond that the float32 case alone applies)."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver
    from tests.helpers import nested_range_batches

    if dtype == torch.bfloat16 and num_bins > 64:
        pytest.skip("the grid needs more mantissa bits than bfloat16 has")
    batches, expected, (lo, hi) = nested_range_batches(num_bins, seed, dtype)
    obs = _HistogramObserver((1,), num_bins=num_bins)
    for b in batches:
        obs.update(b.to(device))
    st = obs.get_stats()[0]
    assert torch.equal(st.histogram.cpu().float(), expected)
    assert st.min.item() == lo and st.max.item() == hi
    assert st.bin_edges[0].item() == lo and st.bin_edges[-1].item() == hi


def test_batch_histogram_is_formed_on_first_read(device):
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    obs = _HistogramObserver((1,), num_bins=64)
    ref = O.HistObserver((1,), 64)
    g = torch.Generator().manual_seed(9)
    news = []
    for k in range(3):
        x = torch.randn(2, 9001, generator=g) * (k + 1)
        want = ref.update(x)[0]  # the oracle's first list becomes its running statistics: keep the values, not the list
        news.append((obs.update(x.to(device)), [t.clone() for t in (want.histogram, want.bin_edges, want.min, want.max)]))
    # read in reverse order, after all updates: each list still describes its own batch
    for k in (2, 1, 0):
        got, (w_hist, w_edges, w_min, w_max) = news[k]
        hist, edges, mm, _ = got.stacked()
        assert_same_bits(hist[0], w_hist, f"batch {k} histogram")
        assert_same_bits(edges[0], w_edges, f"batch {k} edges")
        assert_same_bits(got[0].min, w_min, f"batch {k} min")
        assert_same_bits(got[0].max, w_max, f"batch {k} max")


def test_histogram_large_counts_round_like_fp32(device):
    """Running totals above 2^24 are rounded once per batch, as the reference's fp32 accumulation does."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    obs = _HistogramObserver((1,), num_bins=4)
    ref = O.HistObserver((1,), 4)
    n = 9_000_001
    for k in range(3):
        x = torch.zeros(n)
        x[0] = -1.0
        x[1] = 1.0 + k * 1e-3 * 0  # same range every batch
        ref.update(x)
        obs.update(x.to(device))
    _check_hist_lists(obs.get_stats(), ref.stats, "running")
    assert ref.stats[0].histogram.max() > 2 ** 24


@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("cfg", [dict(num_bins=512, asymmetric_delta_candidates=100, offset_candidates=64, gamma=3.0),
                                 dict(num_bins=2048), dict(num_bins=64, gamma=1.0, offset_candidates=300)],
                         ids=["c3_grid", "defaults", "gamma1_many_offsets"])
@pytest.mark.parametrize("num_steps", [255, 15, 65535])
def test_sqnr_search(device, cfg, symmetric, num_steps):
    from aimet_amd.quantization.encoding_analyzer import SqnrEncodingAnalyzer

    an = SqnrEncodingAnalyzer((1,), **cfg)
    ref = O.HistObserver((1,), cfg["num_bins"])
    for k in range(3):
        x = _laplace_with_outliers((64, 1024), seed=k)
        ref.update(x)
        an.update_stats(x.to(device))
    lo, hi = an.compute_encodings(num_steps, symmetric)
    kw = dict(asym_deltas=cfg.get("asymmetric_delta_candidates", 17), sym_deltas=101,
              num_offsets=cfg.get("offset_candidates", 21), gamma=cfg.get("gamma", 3.0))
    d_ref, o_ref = O.sqnr_candidates(ref.stats, num_steps, symmetric, kw["asym_deltas"], kw["sym_deltas"], kw["num_offsets"])
    noise_ref = O.sqnr_noise(ref.stats, d_ref, o_ref, num_steps, 2.0, kw["gamma"])
    lo_ref, hi_ref, bd, bo, bi = O.sqnr_encodings(ref.stats, (1,), num_steps, symmetric, **kw)
    ls = an.last_search
    assert_same_bits(ls["deltas"].expand_as(ls["noise"]), d_ref.expand(noise_ref.shape), "candidate deltas")
    assert_same_bits(ls["offsets"].expand_as(ls["noise"]), o_ref.expand(noise_ref.shape), "candidate offsets")
    assert_close_rel(ls["noise"], noise_ref, 1e-5, "noise")
    assert int(ls["best_index"].item()) == int(bi.item()), "argmin"
    assert_same_bits(lo, lo_ref, "encoding min")
    assert_same_bits(hi, hi_ref, "encoding max")


@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("cfg", [dict(num_bins=512), dict(num_bins=301, gamma=1.0), dict(num_bins=256, p=3.0)],
                         ids=["bins512", "odd_bins_gamma1", "cubic_norm"])
def test_sqnr_search_many_slots(device, cfg, symmetric):
    """Per-channel searches price one candidate per lane; same candidates, noise sums and winners as the oracle.  A slot
    whose winner differs must be a tie of the two noise sums to within the fp32 rounding of the reference's own sums.
    The last ten slots hold values near 2e18: bin centres too large for the division-free quotient, sums that overflow
    and, for the cubic norm, NaN sums."""
    from aimet_amd.quantization.encoding_analyzer import SqnrEncodingAnalyzer, _LpNormEncodingAnalyzer

    S = 300
    p = cfg.get("p", 2.0)
    kw = dict(asym_deltas=17, sym_deltas=101, num_offsets=21, gamma=cfg.get("gamma", 3.0))
    if p == 2.0:
        an = SqnrEncodingAnalyzer((S, 1), num_bins=cfg["num_bins"], gamma=kw["gamma"])
    else:
        an = _LpNormEncodingAnalyzer((S, 1), cfg["num_bins"], p=p, asymmetric_delta_candidates=17,
                                     symmetric_delta_candidates=101, offset_candidates=21, max_parallelism=64,
                                     gamma=kw["gamma"])
    ref = O.HistObserver((S, 1), cfg["num_bins"])
    g = torch.Generator().manual_seed(21)
    scale = torch.logspace(-3, 3, S).reshape(S, 1)
    for k in range(2):
        x = torch.randn(S, 700, generator=g) * scale * (k + 1) + (torch.arange(S).reshape(S, 1) % 5 - 2) * scale
        x[::7] = x[::7].abs()  # one-sided slots
        # bin centres beyond 2^60: these slots take the plain division; squares stay finite, some sums overflow alike
        x[-10:] = 2e18 + torch.randn(10, 700, generator=g) * 1e15
        ref.update(x)
        an.update_stats(x.to(device))
    lo, hi = an.compute_encodings(255, symmetric)
    d_ref, o_ref = O.sqnr_candidates(ref.stats, 255, symmetric, kw["asym_deltas"], kw["sym_deltas"], kw["num_offsets"])
    noise_ref = O.sqnr_noise(ref.stats, d_ref, o_ref, 255, p, kw["gamma"])
    ls = an.last_search
    assert_same_bits(ls["deltas"].expand_as(ls["noise"]), d_ref.expand(noise_ref.shape), "candidate deltas")
    # one-sided slots clamp a candidate minimum of -0 against an observed +0: which zero max() keeps is an accident of
    # torch's vectorised CPU kernel, so zeros are compared without their sign (adding +0 makes them all positive)
    assert_same_bits(ls["offsets"].expand_as(ls["noise"]) + 0.0, o_ref.expand(noise_ref.shape) + 0.0, "candidate offsets")
    got, want = ls["noise"].cpu().double(), noise_ref.double()
    # every term is positive: relative per candidate.  The cubes of the huge slots overflow, and an infinite term times
    # an empty bin makes the sum NaN on both sides; torch.min then returns the first NaN
    close = (got == want) | ((got - want).abs() <= 1e-5 * want.abs()) | (got.isnan() & want.isnan())
    assert bool(close.all()), f"noise: {int((~close).sum())} candidates differ"
    assert bool(want[-10:].isnan().any()) == (p != 2.0) and (p != 2.0 or int(want[-10:].isfinite().sum()) > 0)
    lo_ref, hi_ref, _, _, bi_ref = O.sqnr_encodings(ref.stats, (S, 1), 255, symmetric, p=p, **kw)
    flat_ref = noise_ref.reshape(S, -1)
    bi_ref = bi_ref.reshape(S)
    bi = ls["best_index"].cpu().reshape(S)
    differ = (bi != bi_ref).nonzero().flatten().tolist()
    assert len(differ) <= S // 50, differ
    for s_ in differ:
        a_, b_ = float(flat_ref[s_, bi[s_]]), float(flat_ref[s_, bi_ref[s_]])
        assert abs(a_ - b_) <= 1e-6 * abs(b_), (s_, a_, b_)
    same = torch.ones(S, dtype=torch.bool)
    same[differ] = False
    assert_same_bits(lo.cpu().reshape(S)[same] + 0.0, lo_ref.reshape(S)[same] + 0.0, "encoding min")
    assert_same_bits(hi.cpu().reshape(S)[same], hi_ref.reshape(S)[same], "encoding max")


def test_tf_enhanced_preset_and_per_channel(device):
    from aimet_amd.quantization.encoding_analyzer import TfEnhancedEncodingAnalyzer

    an = TfEnhancedEncodingAnalyzer((4, 1))
    ref = O.HistObserver((4, 1), 512, 3.0)
    g = torch.Generator().manual_seed(9)
    for k in range(3):
        x = torch.randn(4, 5000, generator=g) * torch.tensor([[1.0], [0.1], [10.0], [3.0]]) * (1 + 2 * k)
        ref.update(x)
        an.update_stats(x.to(device))
    for sym in (False, True):
        lo, hi = an.compute_encodings(255, sym)
        lo_ref, hi_ref, _, _, bi = O.sqnr_encodings(ref.stats, (4, 1), 255, sym, asym_deltas=17, sym_deltas=101,
                                                    num_offsets=21, gamma=3.0)
        assert torch.equal(an.last_search["best_index"].cpu(), bi)
        assert_same_bits(lo, lo_ref, "encoding min")
        assert_same_bits(hi, hi_ref, "encoding max")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", [((), None, (37, 129)), ((8, 1), None, (8, 300)), ((4, 4), (1, 32), (4, 128))],
                         ids=["per_tensor", "per_channel", "blockwise"])
@pytest.mark.parametrize("num_steps,symmetric", [(255, False), (255, True), (15, True), (3, True), (65535, False)])
def test_minmax_analyzer(device, case, dtype, num_steps, symmetric):
    from aimet_amd.quantization.encoding_analyzer import MinMaxEncodingAnalyzer

    shape, block, xshape = case
    an = MinMaxEncodingAnalyzer(shape, block)
    g = torch.Generator().manual_seed(5)
    mn_ref = mx_ref = None
    for k in range(3):
        x = (torch.randn(xshape, generator=g) * (k + 1) * 0.5).to(dtype)
        a, b = O.reduce_minmax(x, shape, block)
        mn_ref = a if mn_ref is None else torch.minimum(mn_ref, a)
        mx_ref = b if mx_ref is None else torch.maximum(mx_ref, b)
        st = an.update_stats(x.to(device))
        assert_same_bits(st.min, a, "batch min")
        assert_same_bits(st.max, b, "batch max")
    lo_ref, hi_ref = O.minmax_encodings(mn_ref, mx_ref, num_steps, symmetric)
    lo, hi = an.compute_encodings(num_steps, symmetric)
    assert lo.dtype == dtype
    assert_same_bits(lo, lo_ref, "encoding min")
    assert_same_bits(hi, hi_ref, "encoding max")


def test_minmax_degenerate_ranges(device):
    from aimet_amd.quantization.encoding_analyzer import MinMaxEncodingAnalyzer

    for x in [torch.zeros(100), torch.full((100,), 3.0), torch.full((100,), -2.0), torch.tensor([3.4e38, -3.4e38]),
              torch.tensor([1e-12, -1e-12])]:
        for sym in (False, True):
            an = MinMaxEncodingAnalyzer(())
            an.update_stats(x.to(device))
            lo, hi = an.compute_encodings(255, sym)
            lo_ref, hi_ref = O.minmax_encodings(x.min(), x.max(), 255, sym)
            assert_same_bits(lo, lo_ref, "min")
            assert_same_bits(hi, hi_ref, "max")


@pytest.mark.parametrize("percentile", [100, 99, 80, 50])
@pytest.mark.parametrize("symmetric", [False, True])
def test_percentile_analyzer(device, percentile, symmetric):
    from aimet_amd.quantization.encoding_analyzer import PercentileEncodingAnalyzer

    an = PercentileEncodingAnalyzer((2, 1), num_bins=100, percentile=percentile)
    ref = O.HistObserver((2, 1), 100)
    g = torch.Generator().manual_seed(6)
    for k in range(2):
        x = torch.randn(2, 3000, generator=g) * (k + 1)
        ref.update(x)
        an.update_stats(x.to(device))
    lo, hi = an.compute_encodings(255, symmetric)
    lo_ref, hi_ref = O.percentile_encodings(ref.stats, (2, 1), percentile, 255, symmetric)
    assert_same_bits(lo, lo_ref, "min")
    assert_same_bits(hi, hi_ref, "max")


def test_analyzer_errors(device):
    from aimet_amd.quantization.encoding_analyzer import (MinMaxEncodingAnalyzer, SqnrEncodingAnalyzer,
                                                          PercentileEncodingAnalyzer, TfEnhancedEncodingAnalyzer)
    from aimet_amd.quantization._utils import StatisticsNotFoundError

    for an in [MinMaxEncodingAnalyzer((1,)), SqnrEncodingAnalyzer((1,)), PercentileEncodingAnalyzer((1,)),
               TfEnhancedEncodingAnalyzer((1,))]:
        with pytest.raises(StatisticsNotFoundError):
            an.compute_encodings(255, False)
        an.update_stats(torch.randn(100, device=device))
        with pytest.raises(ValueError):
            an.compute_encodings(0, False)
        an.reset_stats()
        with pytest.raises(StatisticsNotFoundError):
            an.compute_encodings(255, False)
    with pytest.raises(ValueError):
        SqnrEncodingAnalyzer((1,), num_bins=0)
    with pytest.raises(ValueError):
        PercentileEncodingAnalyzer((1,), percentile=40)
    with pytest.raises(RuntimeError):
        SqnrEncodingAnalyzer((1,), histogram_growth_limit=0.5)
    with pytest.raises(RuntimeError):
        SqnrEncodingAnalyzer((3,)).update_stats(torch.randn(4, 4, device=device))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("num_steps", [3, 15, 255, 254, 65535])
@pytest.mark.parametrize("symmetric", [False, True])
def test_minmax_encodings_from_adversarial_statistics(device, dtype, num_steps, symmetric):
    """compute_encodings_from_stats runs as one kernel; feed it statistics directly: degenerate and denormal-narrow
    ranges, all-positive / all-negative ranges, the dtype's extremes, infinities and NaN."""
    from aimet_amd.quantization.encoding_analyzer import MinMaxEncodingAnalyzer, _MinMaxRange

    big = torch.finfo(dtype).max
    tiny = 6e-8 if dtype == torch.float16 else 1e-30
    mn = torch.tensor([0.0, -1.0, 0.5, -3.0, -tiny, 0.0, -big, -big * 0.96, float("-inf"), float("nan"), -2.0, 1e-9,
                       -0.37, -5.0], dtype=torch.float32).to(dtype)
    mx = torch.tensor([0.0, 2.0, 4.0, -1.0, tiny, 1e-8, big, big * 0.96, float("inf"), 1.0, float("nan"), 1e-9,
                       0.21, 5.0], dtype=torch.float32).to(dtype)
    g = torch.Generator().manual_seed(9)
    mn = torch.cat([mn, -(torch.rand(500, generator=g) * 10).to(dtype)])
    mx = torch.cat([mx, (torch.rand(500, generator=g) * 10).to(dtype)])
    lo_ref, hi_ref = O.minmax_encodings(mn, mx, num_steps, symmetric)
    an = MinMaxEncodingAnalyzer((mn.numel(),))
    lo, hi = an.compute_encodings_from_stats(_MinMaxRange(mn.to(device), mx.to(device)), num_steps, symmetric)
    assert lo.dtype == hi.dtype == dtype
    assert hasattr(lo, "_ahq_range_flags"), "the fused kernel did not run"
    assert_same_bits(lo, lo_ref, "encoding min")
    assert_same_bits(hi, hi_ref, "encoding max")
    nonfinite, extreme = (lo._ahq_range_flags != 0).tolist()
    ref_nonfinite = not bool(torch.isfinite(lo_ref.float()).all() and torch.isfinite(hi_ref.float()).all())
    both = torch.stack([lo_ref, hi_ref]).abs()
    ref_extreme = bool(((both - big).abs() <= 1e-8 + 0.05 * big).any())
    assert nonfinite == ref_nonfinite and extreme == ref_extreme


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
def test_histogram_of_rectified_activations(device, dtype):
    """Half of the elements are exact zeros and zero is the batch minimum (the kernel counts zeros in registers and
    lets an estimate of exactly 0 take the fast path); also -0.0, a batch whose zeros sit inside the range, and a
    batch whose minimum is far above zero while the running range still contains it."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    obs = _HistogramObserver((1,), num_bins=512)
    ref = O.HistObserver((1,), 512, None)
    g = torch.Generator().manual_seed(3)
    a = torch.relu(torch.randn(64, 4099, generator=g))
    b = torch.randn(64, 4099, generator=g) * (torch.rand(64, 4099, generator=g) > 0.7)
    b.view(-1)[::7] = -0.0
    c = torch.rand(64, 4099, generator=g) * 2 + 1.5
    for k, x in enumerate((a, b, a * 0.5, c)):
        x = x.to(dtype)
        got = obs.update(x.to(device))
        want = ref.update(x)
        _check_hist_lists(got, want, f"batch {k} own")
        _check_hist_lists(obs.get_stats(), ref.stats, f"batch {k} running")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("shape", [(), (1,)], ids=str)
def test_per_tensor_extrema_kept_as_slots(device, dtype, shape):
    """observe_and_clone() on a single encoding keeps the running extrema as one slot per workgroup
    (ahq_minmax_accumulate) and folds them on demand: the statistics are torch.amin / amax over everything seen, bit
    for bit, whatever the batch sizes (one workgroup, fewer workgroups than slots, all 512), alignment and order; the
    clone is the input."""
    from aimet_amd.quantization.encoding_analyzer import MinMaxEncodingAnalyzer

    g = torch.Generator().manual_seed(21)
    batches = [torch.randn(n, generator=g) * s for n, s in
               ((100, 1.0), (5_000_000, 3.0), (70_001, 9.0), (2048 * 40 + 3, 0.5), (1, 100.0), (1_500_000, 2.0))]
    batches[2] = batches[2][1:]   # contiguous, not 16-byte aligned
    an = MinMaxEncodingAnalyzer(shape)
    lo, hi = None, None
    for i, b in enumerate(batches):
        x = b.to(dtype).to(device)
        if i == 2:
            x = torch.empty(b.numel() + 1, dtype=dtype, device=device)[1:].copy_(b.to(dtype))
            assert x.data_ptr() % 16 != 0
        y = an.observe_and_clone(x)
        assert y.data_ptr() != x.data_ptr() and torch.equal(y, x)
        lo = x.amin() if lo is None else torch.minimum(lo, x.amin())
        hi = x.amax() if hi is None else torch.maximum(hi, x.amax())
        if i in (0, 3, 5):  # reading the statistics in between changes nothing
            st = an.observer.get_stats()
            assert st.min.shape == shape and st.min.dtype == dtype
            assert_same_bits(st.min.reshape(()), lo, f"min after batch {i}")
            assert_same_bits(st.max.reshape(()), hi, f"max after batch {i}")
    assert an.observer._slots_of is not None  # the slots stayed the running statistics throughout
    # update_stats() goes the same way and hands back the batch's own extrema, which fold when they are read
    extra = (torch.randn(1000, generator=g) * 50).to(dtype).to(device)
    own = an.update_stats(extra)
    assert an.observer._slots_of is not None and own.unfolded() is not None
    assert_same_bits(own.min.reshape(()), extra.amin(), "the batch's own min")
    assert_same_bits(own.max.reshape(()), extra.amax(), "the batch's own max")
    assert own.unfolded() is None and own.min.shape == shape
    lo, hi = torch.minimum(lo, extra.amin()), torch.maximum(hi, extra.amax())
    # a view of the running statistics handed out before a batch keeps what it saw
    view = an.observer.get_stats()
    assert view.unfolded() is not None
    more = (torch.randn(3000, generator=g) * 80).to(dtype).to(device)
    an.update_stats(more)
    assert_same_bits(view.min.reshape(()), lo, "view taken before the batch: min")
    assert_same_bits(view.max.reshape(()), hi, "view taken before the batch: max")
    lo, hi = torch.minimum(lo, more.amin()), torch.maximum(hi, more.amax())
    # the other ways of adding statistics take over from the slots and carry on from their content
    last = (torch.randn(500, generator=g) * 200).to(dtype).to(device)
    an.observer.merge_stats(an.observer.collect_stats(last))
    assert an.observer._slots_of is None
    lo, hi = torch.minimum(lo, last.amin()), torch.maximum(hi, last.amax())
    st = an.observer.get_stats()
    assert_same_bits(st.min.reshape(()), lo, "min after merge_stats")
    assert_same_bits(st.max.reshape(()), hi, "max after merge_stats")
    y = an.observe_and_clone(extra * 2)   # statistics exist outside the slots: the running-tensor form continues
    assert an.observer._slots_of is None and torch.equal(y, extra * 2)
    st = an.observer.get_stats()
    assert_same_bits(st.min.reshape(()), torch.minimum(lo, (extra * 2).amin()), "min, running-tensor form")
    # a reset starts the slots afresh (the buffer is reused); NaN is kept like torch.amin / amax keep it
    an.reset_stats()
    buf = an.observer._slots.data_ptr()
    small = torch.tensor([1.0, -2.0, 0.5], dtype=dtype, device=device)
    an.observe_and_clone(small)
    assert an.observer._slots.data_ptr() == buf
    st = an.observer.get_stats()
    assert float(st.min) == -2.0 and float(st.max) == 1.0
    an.observe_and_clone(torch.tensor([3.0, float("nan")], dtype=dtype, device=device))
    an.observe_and_clone(small)
    st = an.observer.get_stats()
    assert torch.isnan(st.min).all() and torch.isnan(st.max).all()
    # a batch of another dtype leaves the slots
    an.reset_stats()
    an.observe_and_clone(small)
    other = torch.float32 if dtype != torch.float32 else torch.float16
    an.observe_and_clone(torch.tensor([7.0, -9.0], dtype=other, device=device))
    assert an.observer._slots_of is None
    st = an.observer.get_stats()
    assert float(st.min) == -9.0 and float(st.max) == 7.0


def test_slot_statistics_through_a_quantizer(device):
    """Pass-through calibration of a per-tensor quantizer over several batches: same range as the batch-by-batch
    form, and compute_encodings() without any observation still leaves the quantizer uninitialized."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    g = torch.Generator().manual_seed(2)
    xs = [(torch.randn(3, 4096, 33, generator=g) * s).to(torch.bfloat16).to(device) for s in (1.0, 4.0, 0.1)]
    q = QuantizeDequantize((), 8, symmetric=False).to(device)
    with torch.no_grad(), q._compute_encodings(passthrough=True):
        for x in xs:
            assert torch.equal(q(x), x)
    ref = QuantizeDequantize((), 8, symmetric=False).to(device)
    with torch.no_grad(), ref.compute_encodings():
        for x in xs:
            ref(x)
    assert_same_bits(q.min, ref.min, "min")
    assert_same_bits(q.max, ref.max, "max")
    fresh = QuantizeDequantize((), 8, symmetric=False).to(device)
    with torch.no_grad(), fresh._compute_encodings(passthrough=True):
        pass
    assert not fresh.is_initialized()


@pytest.mark.parametrize("shape,block", [((6, 1), None), ((6, 4), (1, 8))], ids=["per_channel", "blockwise"])
def test_first_batch_statistics_are_not_changed_by_later_batches(device, shape, block):
    """The first batch's extrema are the running statistics, and the two share their tensors until the running ones
    are written to: what update() returned for the first batch must still be that batch's extrema after the second,
    and the running statistics the fold of both."""
    from aimet_amd.quantization.encoding_analyzer import _MinMaxObserver

    g = torch.Generator().manual_seed(17)
    a = torch.randn(6, 32, generator=g)
    b = torch.randn(6, 32, generator=g) * 3
    obs = _MinMaxObserver(shape, block) if block else _MinMaxObserver(shape)
    first = obs.update(a.to(device))
    want = O.reduce_minmax(a, shape, block)
    assert_same_bits(first.min, want[0].view(shape), "first batch minimum")
    assert_same_bits(obs.get_stats().min, want[0].view(shape), "running minimum after one batch")
    second = obs.update(b.to(device))
    assert_same_bits(first.min, want[0].view(shape), "first batch minimum after the second batch")
    assert_same_bits(first.max, want[1].view(shape), "first batch maximum after the second batch")
    wb = O.reduce_minmax(b, shape, block)
    assert_same_bits(second.min, wb[0].view(shape), "second batch minimum")
    assert_same_bits(obs.get_stats().min, torch.minimum(want[0], wb[0]).view(shape), "running minimum")
    assert_same_bits(obs.get_stats().max, torch.maximum(want[1], wb[1]).view(shape), "running maximum")
