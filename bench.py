#!/usr/bin/env python3
"""Benchmark of the fake-quant hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c1|c2|c3|c4|c5|dlq]

Without --workload every workload runs in this one process and ONE JSON line is printed.  Its top-level fields are
those of c4 (blockwise 4-bit LPBQ quantize-dequantize forward + straight-through backward of a bf16 [14336, 4096]
weight, the largest forward+backward configuration and the only one whose working set exceeds the 256 MB last-level
cache); `configs` holds the records of c1, c2, c3, c5 and dlq (DlQuantization's TF-enhanced stream) in the same form.

A step is one pass of a workload's hot path through the C ABI on tensors already resident in HBM (c4: LPBQ scale
derivation + forward + backward).  The K-step loop is bracketed by device synchronisation and repeated at least seven
times (more until 10 ms have been timed); `ms_per_step` is the median loop divided by K.  `value` = algorithmic bytes
per step / time per step.  Per record: `roofline` for the dominant kernel (HIP events on the launch stream),
`calibration` (min/max statistics of the same tensor), `module_path` (the same step through the drop-in quantizer
module and autograd, allocations included), `cpu_baseline` / `cpu_baseline_1thread` (the CPU oracle, i.e. the
reference's own sequence of torch CPU calls or scalar C loops, on this host) and `parity` against that oracle.
"""

from __future__ import annotations

import argparse
import gc
import json
import math
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "QDQ fwd+bwd GB/s (% of HBM peak); calibration elems/s; vs host-CPU ref"
HBM_PEAK_GBS = 8000.0
COPY_REF_ELEMS = 1 << 26
ROTATION_BYTES = 1 << 31    # tensors a timed loop goes through before it comes back to the first
MIN_REPEATS = 7
MIN_TIMED_SECONDS = 0.010
DEVICE_WARM_SECONDS = 0.100  # untimed steps before the timed loops of a workload, beyond the --warmup steps
# HBM bytes per launch of each workload's dominant kernel(s): rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE averages per
# dispatch, scaled by what the same counters read for _copy_reference() (x2.000 for FETCH_SIZE, x1.000 for WRITE_SIZE);
# the counter summary is profiles/hbm_traffic_pmc__qdq_c1_c2_c4__hist_c3__dlq.txt.  None where no counter run has been
# made.
MEASURED_TRAFFIC_BYTES = {
    ("c1", "qdq_bwd_kernel"): int((200862.2 + 100749.3) * 1024),
    ("c1", "qdq_fwd_kernel"): int((100494.1 + 100398.9) * 1024),
    ("c2", "qdq_bwd_kernel"): int((131570.4 + 65794.4) * 1024),
    ("c2", "qdq_fwd_kernel"): int((65956.2 + 65591.0) * 1024),
    ("c4", "qdq_bwd_kernel"): int((236756.8 + 121856.5) * 1024),
    ("c4", "qdq_fwd_kernel"): int((122033.5 + 114695.3) * 1024),
    ("c4", "qdq_fwd_lpbq_kernel"): int((122082.5 + 118720.7) * 1024),
    # (profiles/hbm_traffic_pmc__per_column_bf16_8192x4096_column_walking_kernels.txt; the backward launch and its
    # finish launch)
    ("cols", "qdq_bwd_kernel"): int((131203.3 + 69632.0 + 4136.5 + 32.0) * 1024),
    ("cols", "qdq_fwd_kernel"): int((65673.6 + 65537.5) * 1024),
    # the timed update (a batch inside the running range): speculative binning pass (read + write) + the launch that
    # folds its extrema and partial histograms into the running state; a batch that moves the range is read a second
    # time (about a quarter of the batches of the c3 stream)
    ("c3", "hist_update"): int((262267.2 + 3216.0 + 3370.9 + 3.5) * 1024),
    ("c3", "hist_update_bf16"): int((131158.4 + 536.0 + 680.9 + 2.0) * 1024),
    ("dlq", "pdf_update"): int((262284.3 + 3072.0 + 3127.6 + 12.0) * 1024),
}
DTYPE_NAME = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}


def _ensure_built():
    from aimet_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from aimet_amd.csrc.build import build

        build(verbose=False)
    return _lib.load()


# -------------------------------------------------------------------------------------------------------- timing --
def _sync():
    torch.cuda.synchronize()


def timed_steps(step, steps, warmup, min_repeats=MIN_REPEATS, min_total=MIN_TIMED_SECONDS, max_repeats=400):
    """Median wall time of a loop of exactly ``steps`` steps, each loop bracketed by a device synchronisation.
    Returns (seconds per loop, repeats)."""
    for _ in range(warmup):
        step()
    # ... and, still untimed, more of the same steps until the device has been busy for DEVICE_WARM_SECONDS: after the
    # idle stretch of a workload's set-up the first tens of milliseconds of launches run below the steady rate (five
    # steps of 0.1 ms are over long before that), and a loop of 20 such steps would be timed inside that ramp
    _sync()
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < DEVICE_WARM_SECONDS:
        for _ in range(max(1, warmup)):
            step()
        _sync()
    loops = []
    total = 0.0
    while len(loops) < min_repeats or (total < min_total and len(loops) < max_repeats):
        _sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        _sync()
        dt = time.perf_counter() - t0
        loops.append(dt)
        total += dt
    return statistics.median(loops), len(loops)


def event_time(fn, reps, repeats=MIN_REPEATS, min_region=2e-3, max_reps=4000):
    """Median over ``repeats`` of the average duration of ``fn`` over back-to-back calls, from HIP events recorded on
    the stream the work is launched on (torch's current stream).  At least ``reps`` calls per timed region, and as many
    as make the region ``min_region`` seconds long: the two event records and the first launch's start-up cost a few
    microseconds per region, which is several per cent of twenty 15-microsecond kernels."""
    fn()
    _sync()

    def region(n):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        _sync()
        return e0.elapsed_time(e1) / n * 1e-3

    pilot = region(reps)
    n = min(max_reps, max(reps, int(math.ceil(min_region / max(pilot, 1e-7)))))
    return statistics.median(region(n) for _ in range(repeats))


def cpu_legs(step, unit_per_step, unit, sample, budget_s=4.0, max_reps=20, one_thread_budget_s=4.0):
    """The CPU oracle timed on this host with torch's default thread count and with one thread.
    ``unit_per_step``: bytes (-> GB/s) or elements (-> elements/s) one call of ``step`` stands for."""

    def leg(budget):
        step()
        t0 = time.perf_counter()
        reps = 0
        while True:
            step()
            reps += 1
            if time.perf_counter() - t0 > budget or reps >= max_reps:
                break
        return (time.perf_counter() - t0) / reps, reps

    def record(dt, reps, cores):
        scale = 1e9 if unit == "GB/s" else 1.0
        return {"value": round(unit_per_step / dt / scale, 3), "unit": unit, "cores": cores, "kind": "port",
                "sample": f"{reps} x {sample} ({dt * 1e3:.1f} ms each)"}

    threads = torch.get_num_threads()
    dt, reps = leg(budget_s)
    all_cores = record(dt, reps, threads)
    torch.set_num_threads(1)
    try:
        t0 = time.perf_counter()
        step()
        first = time.perf_counter() - t0
        if first > one_thread_budget_s:
            one = record(first, 1, 1)
        else:
            dt1, reps1 = leg(one_thread_budget_s)
            one = record(dt1, reps1, 1)
    finally:
        torch.set_num_threads(threads)
    return all_cores, one


def device_ceiling(dev, nbytes=1 << 29, buffers=6):
    """What the memory system gives the simplest possible kernels (ahq_diag_read / ahq_diag_copy: 16-byte loads
    folded into a word, and a copy).  Every launch takes the next of ``buffers`` buffers (3 GiB in all, twelve times the
    last-level cache), so nothing it reads is still cached from its previous turn: the figure is what HBM delivers.
    Best of a few grid sizes, each the median of repeated HIP-event timings.  Also given: the same read kernel going
    over ONE buffer of each min/max workload's size again and again, which is what a benchmark loop over one tensor does
    -- part of such a tensor is served by the last-level cache, the more so with non-temporal loads, which do not
    displace what is resident.  The library's kernels are priced against the published 8 TB/s; this says how much of
    the distance no kernel closes on this device."""
    from aimet_amd import _lib

    lib = _lib.load()
    xs = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(buffers)]
    y = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    out = torch.empty(65536, dtype=torch.int32, device=dev)
    stream = _lib.current_stream(dev)
    turn = [0]

    def next_buffer():
        turn[0] = (turn[0] + 1) % buffers
        return xs[turn[0]].data_ptr()

    def best(fn, moved):
        top = (0.0, 0, 0.0)
        for wgs in (512, 1024, 2048, 4096, 8192):
            t = event_time(lambda: fn(wgs), 12)
            if moved / t / 1e9 > top[0]:
                top = (moved / t / 1e9, wgs, t)
        return {"GBps": round(top[0], 1), "frac_of_peak": round(top[0] / HBM_PEAK_GBS, 4), "workgroups": top[1],
                "us": round(top[2] * 1e6, 2)}

    rec = {
        "read": best(lambda w: lib.ahq_diag_read(next_buffer(), nbytes, w, 0, out.data_ptr(), stream), nbytes),
        "read_nontemporal": best(lambda w: lib.ahq_diag_read(next_buffer(), nbytes, w, 1, out.data_ptr(), stream), nbytes),
        "copy": best(lambda w: lib.ahq_diag_copy(next_buffer(), y.data_ptr(), nbytes, w, stream), 2 * nbytes),
        "bytes_per_launch": nbytes, "buffers_in_rotation": buffers,
    }
    assert torch.equal(xs[turn[0]][:1 << 20], y[:1 << 20]) and torch.equal(xs[turn[0]][-(1 << 20):], y[-(1 << 20):])
    one = xs[0].data_ptr()
    rec["same_buffer_again_and_again"] = {
        name: {"plain": best(lambda w: lib.ahq_diag_read(one, size, w, 0, out.data_ptr(), stream), size),
               "nontemporal": best(lambda w: lib.ahq_diag_read(one, size, w, 1, out.data_ptr(), stream), size),
               "bytes": size}
        for name, size in (("c2_67MB", 4096 * 4096 * 4), ("c1_103MB", 25690112 * 4), ("c4_117MB", 14336 * 4096 * 2))}
    rec["note"] = ("bare streaming kernels of this library (no arithmetic): read = bytes read / time, copy = bytes read "
                   "+ written / time; peak = published 8 TB/s")
    del xs, y
    return rec


def _copy_reference(dev):
    """One plain elementwise pass of known size (256 MiB read, 256 MiB written), outside every timed region: hardware
    counter runs of this script scale FETCH_SIZE / WRITE_SIZE of the kernels below by what they read for this one."""
    src = torch.ones(COPY_REF_ELEMS, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    torch.mul(src, 1.0, out=dst)
    _sync()


def _base_record(value_gbs, steps, warmup, sec_per_step, dtype, config, repeats):
    return {
        "metric": METRIC,
        "value": round(value_gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(sec_per_step * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": config,
        "repeats": repeats,
        "timing": f"median of {repeats} loops of {steps} steps, each loop bracketed by device synchronisation; before "
                  f"them the {warmup} warm-up steps and further untimed steps until the device has been busy for "
                  f"{int(DEVICE_WARM_SECONDS * 1e3)} ms",
        "pct_of_hbm_peak": round(100.0 * value_gbs / HBM_PEAK_GBS, 2),
    }


# ----------------------------------------------------------------------------------------------------- workloads --
def _make_c1():
    g = torch.Generator().manual_seed(0)
    x = torch.relu(torch.randn(32, 64, 112, 112, generator=g))
    g1 = torch.Generator().manual_seed(1)
    grad = torch.randn(x.shape, generator=g1)
    return dict(name="c1_per_tensor_8b_asym_fp32_32x64x112x112", x=x, grad=grad, enc_shape=(), block=None,
                bitwidth=8, symmetric=False, lpbq=False)


def _make_c2():
    g = torch.Generator().manual_seed(0)
    w = torch.randn(4096, 4096, generator=g) * 0.02
    rows = torch.randperm(4096, generator=torch.Generator().manual_seed(1))[:41]
    w[rows] *= 10
    grad = torch.randn(4096, 4096, generator=torch.Generator().manual_seed(2)) * 1e-3
    return dict(name="c2_per_channel_8b_sym_fp32_4096x4096", x=w, grad=grad, enc_shape=(4096, 1), block=None,
                bitwidth=8, symmetric=True, lpbq=False)


def _make_c4():
    g = torch.Generator().manual_seed(0)
    w = (torch.randn(14336, 4096, generator=g) * 0.02).bfloat16()
    grad = torch.randn(14336, 4096, generator=torch.Generator().manual_seed(1)).bfloat16()
    return dict(name="c4_lpbq_blockwise64_4b_sym_bf16_14336x4096", x=w, grad=grad, enc_shape=(14336, 64), block=(1, 64),
                bitwidth=4, symmetric=True, lpbq=True, decompressed_bw=8, grouping=(1, -1))


def _make_cols():
    """Not one of the benchmark configurations: per-channel encodings along the fastest axis, the layout the
    column-walking kernels serve (run with --workload cols; left out of the default run)."""
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(8192, 4096, generator=g) * torch.linspace(0.5, 2.0, 4096)).bfloat16()
    grad = torch.randn(8192, 4096, generator=torch.Generator().manual_seed(1)).bfloat16()
    return dict(name="per_column_8b_sym_bf16_8192x4096", x=x, grad=grad, enc_shape=(1, 4096), block=None,
                bitwidth=8, symmetric=True, lpbq=False)


WORKLOADS = {"c1": _make_c1, "c2": _make_c2, "c4": _make_c4, "cols": _make_cols}


def _grid_limits(w):
    n = 2 ** w["bitwidth"] - 1
    return (-math.ceil(n / 2), math.floor(n / 2), n) if w["symmetric"] else (0, n, n)


def _range_cpu(w):
    """Min/max statistics and the encoding range on the CPU oracle."""
    from oracle import torch_ref as O

    _, _, n = _grid_limits(w)
    mn, mx = O.reduce_minmax(w["x"], w["enc_shape"], w["block"])
    emin, emax = O.minmax_encodings(mn, mx, n, w["symmetric"])
    return mn, mx, emin.float(), emax.float()  # the quantizer's min / max parameters are float32


def _scale_offset_cpu(w, emin, emax):
    """Scale and offset from the encoding range, through the LPBQ requantisation where the workload asks for it."""
    from oracle import torch_ref as O

    qmin, qmax, _ = _grid_limits(w)
    scale = O.scale_from_minmax(emin, emax, qmin, qmax)
    pcs = None
    if w["lpbq"]:
        scale, pcs = O.lpbq_scale(scale, w["bitwidth"], w["decompressed_bw"], w["grouping"])
    offset = O.offset_from_minmax(emin, scale, qmin, qmax, w["symmetric"])
    return scale, offset, pcs


def _make_module(w, dev):
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize, QuantizeDequantize

    if w["lpbq"]:
        q = GroupedBlockQuantizeDequantize(shape=w["enc_shape"], bitwidth=w["bitwidth"], symmetric=True,
                                           decompressed_bw=w["decompressed_bw"], block_size=w["block"],
                                           block_grouping=w["grouping"])
    else:
        q = QuantizeDequantize(w["enc_shape"], w["bitwidth"], w["symmetric"], block_size=w["block"])
    return q.to(dev)


def _host_time_of_module_step(q, xm, grad, reps=60):
    """Python time of QuantizeDequantize.forward and of .backward() with the GPU idle when each starts (device
    synchronised before both): what the interpreter, autograd and the library's host code cost per call, the floor of
    a module-API step however fast the kernels are.  Medians, microseconds."""
    fwd_t, bwd_t = [], []
    for _ in range(reps):
        xm.grad = None
        q.min.grad = None
        q.max.grad = None
        _sync()
        t0 = time.perf_counter()
        out = q(xm)
        t1 = time.perf_counter()
        _sync()
        t2 = time.perf_counter()
        out.backward(grad)
        t3 = time.perf_counter()
        fwd_t.append(t1 - t0)
        bwd_t.append(t3 - t2)
    _sync()
    return {"host_us_forward": round(statistics.median(fwd_t[5:]) * 1e6, 1),
            "host_us_backward": round(statistics.median(bwd_t[5:]) * 1e6, 1)}


def run_qdq_workload(key, steps, warmup, dev, with_cpu_baseline=True, with_cached=True):
    from aimet_amd import _lib
    from aimet_amd.quantization._utils import _get_minimum_scale
    from aimet_amd.quantization.affine.backends import hip
    from oracle import torch_ref as O

    lib = _ensure_built()
    _copy_reference(dev)
    t_start = time.perf_counter()
    w = WORKLOADS[key]()
    qmin, qmax, _ = _grid_limits(w)
    x = w["x"].to(dev)
    grad = w["grad"].to(dev)
    stream = _lib.current_stream(dev)
    code = _lib.DTYPE_CODE[x.dtype]

    # ---- calibration through the drop-in module: min/max statistics -> range, as compute_encodings() does
    q = _make_module(w, dev)
    with torch.no_grad(), q.compute_encodings():
        q(x)
    mn_ref, mx_ref, emin_c, emax_c = _range_cpu(w)
    scale_c, offset_c, pcs_c = _scale_offset_cpu(w, emin_c, emax_c)
    range_exact = bool(torch.equal(q.min.detach().cpu().view(emin_c.shape), emin_c)
                       and torch.equal(q.max.detach().cpu().view(emax_c.shape), emax_c))
    with torch.no_grad():
        enc = q.get_encodings()
    scale = enc.scale.detach().contiguous()
    offset = enc.offset.detach().to(torch.float32).expand(scale.shape).contiguous()
    scale_exact = bool(torch.equal(scale.cpu(), scale_c.view(scale.shape)))

    cd = hip._internal_dtype(x.dtype, qmin, qmax)
    grid = hip._grid(_lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QDQ, x.dtype, cd, qmin, qmax, 0.0)
    _, layout = hip._prepare(x, scale.shape, w["block"])
    gs = torch.empty_like(scale)
    go = torch.empty_like(scale)
    nbytes = lib.ahq_qdq_backward_workspace_bytes(grid, layout, 1)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    # Every timed launch works on the next of `rot` sets of (x, y, grad, gx) at addresses of their own, at least 2 GiB
    # in rotation (eight and more times the 256 MB last-level cache), and the backward pass of a step takes the set
    # half a rotation away from its forward pass: nothing a launch reads was touched by any of the launches before it
    # that the caches could still hold, so bytes / time is what HBM delivered.  Set 0 is the one compared with the
    # oracle; the others hold the same values.
    rot = max(6, -(-ROTATION_BYTES // (4 * x.numel() * x.element_size())))
    rot += rot % 2
    sets = [(x, torch.empty_like(x), grad, torch.empty_like(x))]
    sets += [(x.clone(), torch.empty_like(x), grad.clone(), torch.empty_like(x)) for _ in range(rot - 1)]
    y, gx = sets[0][1], sets[0][3]
    turn = {"fwd": 0, "bwd": rot // 2, "mm": 0, "mod": 0}

    def nxt(which):
        turn[which] = k = (turn[which] + 1) % rot
        return sets[k]

    def fwd_on(t):
        _lib.check(lib.ahq_qdq_forward(grid, layout, t[0].data_ptr(), t[1].data_ptr(), None, scale.data_ptr(),
                                       offset.data_ptr(), None, None, stream), "fwd")

    def bwd_on(t):
        _lib.check(lib.ahq_qdq_backward(grid, layout, t[2].data_ptr(), t[0].data_ptr(), t[3].data_ptr(), gs.data_ptr(),
                                        go.data_ptr(), scale.data_ptr(), offset.data_ptr(), ws.data_ptr(), nbytes,
                                        stream), "bwd")

    def fwd():
        fwd_on(nxt("fwd"))

    def bwd():
        bwd_on(nxt("bwd"))

    derive = None
    if w["lpbq"]:
        # the reference derives the LPBQ scales from min / max on every forward (get_encodings()); so does the step
        group_shape = tuple(d // g if g != -1 else 1 for d, g in zip(w["enc_shape"], w["grouping"]))
        glayout = hip._build_layout(tuple(w["enc_shape"]), tuple(range(len(w["enc_shape"]))), group_shape,
                                    tuple(w["grouping"]))
        pmin, pmax = q.min.detach(), q.max.detach()
        pcs = torch.empty(group_shape, dtype=torch.float32, device=dev)
        mult = 2 ** (w["decompressed_bw"] - w["bitwidth"])
        min_scale = _get_minimum_scale(qmax - qmin)

        def derive():
            _lib.check(lib.ahq_lpbq_scale(_lib.DTYPE_CODE[pmin.dtype], glayout, pmin.data_ptr(), pmax.data_ptr(), qmin,
                                          qmax, min_scale, mult, scale.data_ptr(), pcs.data_ptr(), stream), "lpbq")

    # LPBQ: the scale derivation inside the forward launch (ahq_lpbq_qdq_forward); the separate launches are timed too
    fused = None
    if derive is not None:
        blocks_per_group = q._blocks_per_group()
        if blocks_per_group is not None:
            def fused_on(t):
                _lib.check(lib.ahq_lpbq_qdq_forward(grid, layout, t[0].data_ptr(), t[1].data_ptr(), None,
                                                    _lib.DTYPE_CODE[pmin.dtype], pmin.data_ptr(), pmax.data_ptr(),
                                                    blocks_per_group, min_scale, mult, None, scale.data_ptr(),
                                                    pcs.data_ptr(), stream), "lpbq forward")

            def fused():
                fused_on(nxt("fwd"))

    def step_on(tf, tb):
        if fused is not None:
            fused_on(tf)
        else:
            if derive is not None:
                derive()
            fwd_on(tf)
        bwd_on(tb)

    def step():
        step_on(nxt("fwd"), nxt("bwd"))

    loop_s, repeats = timed_steps(step, steps, warmup)
    sec_per_step = loop_s / steps

    reps = max(steps, 20)
    t_fwd = event_time(fwd, reps)
    t_bwd = event_time(bwd, reps)
    t_derive = event_time(derive, reps) if derive is not None else 0.0
    t_fused = event_time(fused, reps) if fused is not None else 0.0
    # the same launches over ONE set again and again: the tensors then partly come from the last-level cache
    cached = None
    if with_cached:
        c_loop, _ = timed_steps(lambda: step_on(sets[0], sets[0]), steps, warmup)
        tc_fwd = event_time(lambda: (fused_on if fused is not None else fwd_on)(sets[0]), reps)
        tc_bwd = event_time(lambda: bwd_on(sets[0]), reps)
        cached = {"ms_per_step": round(c_loop / steps * 1e3, 5), "fwd_us": round(tc_fwd * 1e6, 2),
                  "bwd_us": round(tc_bwd * 1e6, 2)}
    # every set must hold what set 0 holds (compared with the oracle below)
    _sync()
    for t in sets[1:]:
        fwd_on(t)
        bwd_on(t)
    fwd_on(sets[0])
    bwd_on(sets[0])
    _sync()
    sets_agree = all(torch.equal(t[1], y) and torch.equal(t[3], gx) for t in sets[1:])

    n = x.numel()
    S = x.element_size()
    E = scale.numel()
    bytes_fwd = 2 * S * n + 8 * E
    bytes_bwd = 3 * S * n + 16 * E
    bytes_derive = (12 * E + 4 * pcs.numel()) if derive is not None else 0
    # fused: x, y, min / max of every block read, scale and per-channel scale written (the offset is the constant 0)
    bytes_fused = (2 * S * n + 2 * pmin.element_size() * E + 4 * E + 4 * pcs.numel()) if fused is not None else 0
    bytes_step = (bytes_fused + bytes_bwd) if fused is not None else (bytes_fwd + bytes_bwd + bytes_derive)
    value = bytes_step / sec_per_step / 1e9

    # ---- frozen quantizer (no gradient for scale / offset): the ATen fake-quantize arithmetic, input gradient only
    frozen = None
    if w["block"] is None:
        grid_a = hip._grid(_lib.AHQ_ARITH_ATEN, _lib.AHQ_OP_QDQ, x.dtype, torch.float32, qmin, qmax, 0.0)
        nb_a = lib.ahq_qdq_backward_workspace_bytes(grid_a, layout, 0)
        ws_a = torch.empty(max(nb_a, 16), dtype=torch.uint8, device=dev)

        def fwd_a_on(t):
            _lib.check(lib.ahq_qdq_forward(grid_a, layout, t[0].data_ptr(), t[1].data_ptr(), None, scale.data_ptr(),
                                           offset.data_ptr(), None, None, stream), "fwd aten")

        def bwd_a_on(t):
            _lib.check(lib.ahq_qdq_backward(grid_a, layout, t[2].data_ptr(), t[0].data_ptr(), t[3].data_ptr(), None,
                                            None, scale.data_ptr(), offset.data_ptr(), ws_a.data_ptr(), nb_a, stream),
                       "bwd aten")

        ta_f = event_time(lambda: fwd_a_on(nxt("fwd")), reps)
        ta_b = event_time(lambda: bwd_a_on(nxt("bwd")), reps)
        y_a = torch.empty_like(x)
        fwd_a_on((x, y_a))
        bwd_a_on(sets[0])
        ref_a, mask_a = O.qdq_v1(w["x"], scale_c, offset_c, qmin, qmax)
        frozen = {"arithmetic": "ATen fake-quantize (frozen scale / offset)",
                  "fwd_us": round(ta_f * 1e6, 2), "bwd_us": round(ta_b * 1e6, 2),
                  "GBps": round(5 * S * n / (ta_f + ta_b) / 1e9, 1),
                  "y_bit_exact": bool(torch.equal(y_a.cpu(), ref_a)),
                  "gx_bit_exact": bool(torch.equal(gx.cpu(), torch.where(mask_a, w["grad"], torch.zeros_like(w["grad"]))))}
        del y_a
        fwd_on(sets[0])  # y and gx of the autograd arithmetic again, for the parity check below
        bwd_on(sets[0])

    # ---- min/max calibration of the same tensor (one fused pass for both extrema) + the range it gives
    mm_ws_bytes = lib.ahq_minmax_workspace_bytes(layout)
    mm_ws = torch.empty(max(mm_ws_bytes, 16), dtype=torch.uint8, device=dev)
    mn_out = torch.empty(scale.shape, dtype=x.dtype, device=dev)
    mx_out = torch.empty(scale.shape, dtype=x.dtype, device=dev)

    # the statistics pass reads one tensor: it goes through the inputs and the upstream gradients of all sets in turn
    # (2 * rot tensors of the workload's shape and dtype, 0.8 to 1.4 GB)
    mm_inputs = [t[0] for t in sets] + [t[2] for t in sets]
    mm_turn = [0]

    def mm_next():
        mm_turn[0] = k = (mm_turn[0] + 1) % len(mm_inputs)
        return mm_inputs[k]

    def minmax_on(t):
        _lib.check(lib.ahq_minmax(code, layout, t.data_ptr(), mn_out.data_ptr(), mx_out.data_ptr(), None, None, 0,
                                  mm_ws.data_ptr(), mm_ws_bytes, stream), "minmax")

    an = q.encoding_analyzer

    def calibrate_on(t):
        an.reset_stats()
        an.update_stats(t)
        return an.compute_encodings(qmax - qmin, w["symmetric"])

    t_mm = event_time(lambda: minmax_on(mm_next()), reps)
    t_cal = event_time(lambda: calibrate_on(mm_next()), reps)
    mm_cached = None
    if with_cached:
        mm_cached = {"us": round(event_time(lambda: minmax_on(x), reps) * 1e6, 2),
                     "analyzer_update_plus_compute_encodings_us": round(event_time(lambda: calibrate_on(x), reps) * 1e6, 2)}
    minmax_on(x)
    # a calibration stream only needs the running extrema: per-tensor statistics keep them as one slot per workgroup
    # and skip the launch that folds a batch's partials (ahq_minmax_accumulate); folded once, at the end
    running = None
    if E == 1:
        slots = torch.empty(_lib.MINMAX_SLOTS_BYTES, dtype=torch.uint8, device=dev)
        lib.ahq_minmax_accumulate(code, x.data_ptr(), n_elems := x.numel(), None, slots.data_ptr(), None, 1, stream)

        def accumulate_on(t):
            _lib.check(lib.ahq_minmax_accumulate(code, t.data_ptr(), n_elems, None, slots.data_ptr(), None, 0, stream),
                       "minmax accumulate")

        x_copies = [t[0] for t in sets]  # the running extrema must stay those of x
        acc_turn = [0]

        def accumulate():
            acc_turn[0] = k = (acc_turn[0] + 1) % (2 * rot)
            accumulate_on(x_copies[k % rot] if k < rot else sets[k - rot][1])

        # (the outputs y hold quantize-dequantized x: inside x's range, so they leave the running extrema alone)
        t_acc = event_time(accumulate, reps)
        # what _MinMaxObserver.update() launches per batch: the same with the batch's own extrema left in a second
        # slot array (update_stats() returns them; they are folded when somebody reads them)
        own = torch.empty(_lib.MINMAX_SLOTS_BYTES, dtype=torch.uint8, device=dev)

        def observe():
            acc_turn[0] = k = (acc_turn[0] + 1) % (2 * rot)
            t = x_copies[k % rot] if k < rot else sets[k - rot][1]
            _lib.check(lib.ahq_minmax_accumulate(code, t.data_ptr(), n_elems, None, slots.data_ptr(), own.data_ptr(), 0,
                                                 stream), "minmax accumulate")

        t_obs = event_time(observe, reps)
        b_mn, b_mx = torch.empty_like(mn_out), torch.empty_like(mx_out)
        lib.ahq_minmax_accumulate(code, x.data_ptr(), n_elems, None, slots.data_ptr(), own.data_ptr(), 0, stream)
        _lib.check(lib.ahq_minmax_slots_read(code, own.data_ptr(), b_mn.data_ptr(), b_mx.data_ptr(), stream), "read")
        if with_cached:
            mm_cached["running_us"] = round(event_time(lambda: accumulate_on(x), reps) * 1e6, 2)
        r_mn, r_mx = torch.empty_like(mn_out), torch.empty_like(mx_out)
        _lib.check(lib.ahq_minmax_slots_read(code, slots.data_ptr(), r_mn.data_ptr(), r_mx.data_ptr(), stream), "read")
        running = {"kernel": "ahq_minmax_accumulate (running extrema in per-workgroup slots, no fold launch)",
                   "us": round(t_acc * 1e6, 2), "GBps": round(x.element_size() * n_elems / t_acc / 1e9, 1),
                   "frac_of_hbm_peak": round(x.element_size() * n_elems / t_acc / 1e9 / HBM_PEAK_GBS, 4),
                   "bit_exact": bool(torch.equal(r_mn.cpu(), mn_ref.view(r_mn.shape))
                                     and torch.equal(r_mx.cpu(), mx_ref.view(r_mx.shape))),
                   "with_the_batch_extrema_in_slots_of_their_own": {
                       "what": "the launch of MinMaxEncodingAnalyzer.update_stats() on a per-tensor analyzer",
                       "us": round(t_obs * 1e6, 2),
                       "frac_of_hbm_peak": round(x.element_size() * n_elems / t_obs / 1e9 / HBM_PEAK_GBS, 4),
                       "bit_exact": bool(torch.equal(b_mn.cpu(), mn_ref.view(b_mn.shape))
                                         and torch.equal(b_mx.cpu(), mx_ref.view(b_mx.shape)))}}
    exact_mm = bool(torch.equal(mn_out.cpu(), mn_ref.view(mn_out.shape)) and torch.equal(mx_out.cpu(), mx_ref.view(mx_out.shape)))

    # ---- the same step through the drop-in module: QuantizeDequantize.forward + autograd backward
    xms = [t[0].clone().requires_grad_(True) for t in sets]
    xm = xms[0]

    def module_step_on(k):
        xk = xms[k]
        xk.grad = None
        q.min.grad = None
        q.max.grad = None
        out = q(xk)
        out.backward(sets[(k + rot // 2) % rot][2])

    def module_step():
        turn["mod"] = k = (turn["mod"] + 1) % rot
        module_step_on(k)

    # loops of at least 200 steps: the first steps after a synchronisation wait for autograd's device thread to wake up
    # (about a millisecond), which a loop of twenty 0.1 ms steps would report as half as much again per step
    mod_steps = max(steps, 200)
    mod_loop, mod_repeats = timed_steps(module_step, mod_steps, min(warmup, 5))
    mod_s = mod_loop / mod_steps
    # the same loop with autograd's engine running the backward pass on the calling thread: by default PyTorch hands
    # the backward pass of a GPU tensor to a worker thread and the caller sleeps until it is done, two thread wake-ups
    # per step that cost more than the kernels on most hosts
    with torch.autograd.set_multithreading_enabled(False):
        st_loop, _ = timed_steps(module_step, mod_steps, min(warmup, 5))
    mod_st = st_loop / mod_steps
    mod_cached = None
    if with_cached:
        mc_loop, _ = timed_steps(lambda: module_step_on(0), mod_steps, min(warmup, 5))
        mod_cached = round(mc_loop / mod_steps * 1e3, 5)
    host = _host_time_of_module_step(q, xm, sets[0][2])
    for xk in xms[1:]:
        xk.grad = None
    module_step_on(0)
    _sync()
    mod_gx_exact = None

    # ---- parity against the oracle (same seeded inputs, full size)
    tr = O.qdq_v2_forward(w["x"], scale_c, offset_c, qmin, qmax, w["block"])
    gx_ref, gs_ref, _ = O.qdq_v2_backward(w["grad"], w["x"], scale_c, offset_c, qmin, qmax, w["block"])
    exact_y = bool(torch.equal(y.cpu(), tr.y))
    exact_gx = bool(torch.equal(gx.cpu(), gx_ref))
    mod_gx_exact = bool(torch.equal(xm.grad.cpu(), gx_ref))
    gs_err = float(((gs.cpu().view(gs_ref.shape) - gs_ref).abs().max() / gs_ref.abs().max().clamp_min(1e-30)))
    parity = {"y_bit_exact": exact_y, "gx_bit_exact": exact_gx, "all_sets_in_rotation_agree": bool(sets_agree),
              "gscale_max_rel_err": gs_err,
              "minmax_bit_exact": exact_mm, "encoding_range_bit_exact": range_exact, "scale_bit_exact": scale_exact,
              "module_gx_bit_exact": mod_gx_exact, "sample": "full size"}
    if w["lpbq"]:
        parity["per_channel_scale_bit_exact"] = bool(torch.equal(pcs.cpu(), pcs_c.view(pcs.shape)))
    if fused is not None:
        y.zero_()
        scale.zero_()
        pcs.zero_()
        fused_on(sets[0])
        parity["fused_forward_bit_exact"] = bool(torch.equal(y.cpu(), tr.y) and torch.equal(scale.cpu(), scale_c.view(scale.shape))
                                                 and torch.equal(pcs.cpu(), pcs_c.view(pcs.shape)))

    t_fwd_step, bytes_fwd_step, fwd_name = ((t_fused, bytes_fused, "qdq_fwd_lpbq_kernel") if fused is not None
                                            else (t_fwd, bytes_fwd, "qdq_fwd_kernel"))
    dom = (("qdq_bwd_kernel", t_bwd, bytes_bwd) if t_bwd >= t_fwd_step else (fwd_name, t_fwd_step, bytes_fwd_step))
    # the bytes the step's definition counts: 2 S forward + 3 S backward per element, 8 bytes per encoding
    bytes_step_plain = 5 * S * n + 8 * E
    config = {"workload": w["name"], "elements": n, "encodings": E, "algorithmic_bytes_per_step": bytes_step,
              "algorithmic_bytes_per_step_without_side_outputs": bytes_step_plain,
              "tensor_sets_in_rotation": rot, "bytes_in_rotation": rot * 4 * S * n,
              "arithmetic": "autograd (learnable min/max)", "compute_dtype": str(cd).split(".")[-1],
              "step": ("ahq_lpbq_qdq_forward (block scales derived inside the forward launch) + ahq_qdq_backward"
                       if fused is not None else
                       ("ahq_lpbq_scale + " if derive is not None else "") + "ahq_qdq_forward + ahq_qdq_backward")
                      + " (C ABI, preallocated outputs)"}
    out = _base_record(value, steps, warmup, sec_per_step, DTYPE_NAME[x.dtype], config, repeats)
    kernels = {
        "qdq_fwd_kernel": {"us": round(t_fwd * 1e6, 2), "GBps": round(bytes_fwd / t_fwd / 1e9, 1),
                           "frac_of_hbm_peak": round(bytes_fwd / t_fwd / 1e9 / HBM_PEAK_GBS, 4)},
        "qdq_bwd_kernel": {"us": round(t_bwd * 1e6, 2), "GBps": round(bytes_bwd / t_bwd / 1e9, 1),
                           "frac_of_hbm_peak": round(bytes_bwd / t_bwd / 1e9 / HBM_PEAK_GBS, 4)},
    }
    if derive is not None:
        kernels["lpbq_scale_kernel"] = {"us": round(t_derive * 1e6, 2), "GBps": round(bytes_derive / t_derive / 1e9, 1)}
    if fused is not None:
        kernels["qdq_fwd_lpbq_kernel"] = {"us": round(t_fused * 1e6, 2), "GBps": round(bytes_fused / t_fused / 1e9, 1),
                                          "frac_of_hbm_peak": round(bytes_fused / t_fused / 1e9 / HBM_PEAK_GBS, 4)}
        kernels["qdq_fwd_kernel"]["note"] = kernels["lpbq_scale_kernel"]["note"] = \
            "the two-launch form of the forward pass, not part of the timed step"
    out.update({
        "elements_per_s": round(n / sec_per_step, 1),
        "kernels": kernels,
        "calibration": {"kernel": "ahq_minmax (both extrema in one pass"
                                  + ("; two launches for a single encoding: stream + fold of the partials; the "
                                     "analyzers use the one-launch form under 'running')" if E == 1 else ")"),
                        "us": round(t_mm * 1e6, 2),
                        "GBps": round((S * n + 2 * S * E) / t_mm / 1e9, 1),
                        "elements_per_s": round(n / t_mm, 1),
                        "frac_of_hbm_peak": round((S * n) / t_mm / 1e9 / HBM_PEAK_GBS, 4),
                        "analyzer_update_plus_compute_encodings_us": round(t_cal * 1e6, 2),
                        "analyzer_elements_per_s": round(n / t_cal, 1),
                        "analyzer_frac_of_hbm_peak": round((S * n) / t_cal / 1e9 / HBM_PEAK_GBS, 4),
                        "inputs_in_rotation": len(mm_inputs),
                        **({"same_tensor_again_and_again": mm_cached} if mm_cached is not None else {}),
                        **({"running": running} if running is not None else {})},
        "module_path": {"what": "QuantizeDequantize.forward + .backward() with learnable min/max (allocations, "
                                "autograd and the per-call scale / offset derivation included)",
                        "ms_per_step": round(mod_s * 1e3, 5), "GBps": round(bytes_step / mod_s / 1e9, 1),
                        "frac_of_hbm_peak": round(bytes_step / mod_s / 1e9 / HBM_PEAK_GBS, 4), "repeats": mod_repeats,
                        "steps_per_timed_loop": mod_steps,
                        "autograd_on_the_calling_thread": {
                            "what": "the same loop inside torch.autograd.set_multithreading_enabled(False)",
                            "ms_per_step": round(mod_st * 1e3, 5), "GBps": round(bytes_step / mod_st / 1e9, 1),
                            "frac_of_hbm_peak": round(bytes_step / mod_st / 1e9 / HBM_PEAK_GBS, 4)},
                        **host,
                        **({"same_tensor_again_and_again_ms_per_step": mod_cached} if mod_cached is not None else {})},
        "parity": parity,
        "roofline": {"bound": "hbm", "kernel": dom[0], "achieved": round(dom[2] / dom[1] / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(dom[2] / dom[1] / 1e9 / HBM_PEAK_GBS, 4),
                     "algorithmic_bytes": dom[2], "traffic": MEASURED_TRAFFIC_BYTES.get((key, dom[0])),
                     "memory": f"HBM: every launch takes the next of {rot} tensor sets, {rot * 4 * S * n >> 20} MiB in rotation"},
    })
    out["pct_of_hbm_peak_without_side_outputs"] = round(100.0 * bytes_step_plain / sec_per_step / 1e9 / HBM_PEAK_GBS, 2)
    if cached is not None:
        t_c_dom = cached["bwd_us"] if dom[0] == "qdq_bwd_kernel" else cached["fwd_us"]
        out["roofline"]["cached"] = {
            "what": "the same launches over one tensor set again and again (partly served by the 256 MB last-level cache)",
            "frac": round(dom[2] / (t_c_dom * 1e-6) / 1e9 / HBM_PEAK_GBS, 4), "us": t_c_dom,
            "step_ms": cached["ms_per_step"],
            "step_pct_of_hbm_peak": round(100.0 * bytes_step / (cached["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 2)}
    if frozen is not None:
        out["frozen_quantizer"] = frozen
    if with_cpu_baseline:
        def cpu_step():
            s_c = scale_c
            if w["lpbq"]:
                raw = O.scale_from_minmax(emin_c, emax_c, qmin, qmax)
                s_c, _ = O.lpbq_scale(raw, w["bitwidth"], w["decompressed_bw"], w["grouping"])
            O.qdq_v2_forward(w["x"], s_c, offset_c, qmin, qmax, w["block"])
            O.qdq_v2_backward(w["grad"], w["x"], s_c, offset_c, qmin, qmax, w["block"])

        sample = f"full-size step of {w['name']} with the reference's torch CPU operations"
        out["cpu_baseline"], out["cpu_baseline_1thread"] = cpu_legs(cpu_step, bytes_step, "GB/s", sample)

        def cpu_cal():
            a, b = O.reduce_minmax(w["x"], w["enc_shape"], w["block"])
            O.minmax_encodings(a, b, qmax - qmin, w["symmetric"])

        c_all, c_one = cpu_legs(cpu_cal, n, "elements/s", "min/max calibration of the same tensor", budget_s=2.0,
                                one_thread_budget_s=2.0)
        out["calibration"]["cpu_baseline"] = c_all
        out["calibration"]["cpu_baseline_1thread"] = c_one
    out["bench_seconds"] = round(time.perf_counter() - t_start, 1)
    return out


def _laplace_batch(shape, seed, dev):
    """Laplace(0, 1) with 0.1 % of the elements replaced by +-U(20, 60), generated on the device."""
    g = torch.Generator(device=dev).manual_seed(seed)
    # u = +-0.5 would give an infinite sample; rand() does return 0 a few times in 67 M draws
    u = (torch.rand(shape, generator=g, device=dev) - 0.5).clamp_(-0.4999999, 0.4999999)
    x = -torch.sign(u) * torch.log1p(-2 * u.abs())
    n = x.numel()
    k = n // 1000
    idx = torch.randint(0, n, (k,), generator=g, device=dev)
    out = (torch.rand(k, generator=g, device=dev) * 40 + 20) * torch.sign(torch.rand(k, generator=g, device=dev) - 0.5)
    x.view(-1)[idx] = out
    return x


def run_hist_workload(steps, warmup, dev, with_cpu_baseline=True, batches=16, shape=(8, 2048, 4096)):
    """c3: 16 batches folded into a 512-bin histogram, then the 100 x 64 candidate SQNR search (8-bit asymmetric)."""
    from aimet_amd.quantization.encoding_analyzer import SqnrEncodingAnalyzer
    from oracle import torch_ref as O

    _ensure_built()
    _copy_reference(dev)
    t_start = time.perf_counter()
    xs = [_laplace_batch(shape, b, dev) for b in range(batches)]
    an = SqnrEncodingAnalyzer((1,), num_bins=512, asymmetric_delta_candidates=100, offset_candidates=64, gamma=3.0)

    def step():
        an.reset_stats()
        for x in xs:
            an.update_stats(x)
        return an.compute_encodings(255, False)

    loop_s, repeats = timed_steps(step, steps, warmup)
    wall = loop_s / steps
    lo, hi = step()
    st = an.observer.get_stats()[0]
    hist_gpu, edges_gpu = st.histogram.cpu().clone(), st.bin_edges.cpu().clone()
    best_gpu = int(an.last_search["best_index"].item())

    # one histogram update of a later batch that stays inside the running range (read once), one of a batch that moves
    # it (read twice), and the search alone
    # (the batches are taken in turn, as a calibration stream delivers them: none is found in the last-level cache)
    turn = [0]

    def update_next():
        turn[0] = (turn[0] + 1) % batches
        an.update_stats(xs[turn[0]])

    t_upd = event_time(update_next, 20)
    t_search = event_time(lambda: an.compute_encodings(255, False), 20)
    n_b = xs[0].numel()
    n = n_b * batches
    bytes_step = 8 * n      # the two reads per element of the plain algorithm (range pass + binning pass)
    bytes_read_once = 4 * n_b
    traffic_upd = MEASURED_TRAFFIC_BYTES[("c3", "hist_update")]

    # the same stream in bf16: twice the elements per byte, and an update that holds the range bins them through a
    # table in LDS (hist_bin16_kernel) instead of computing each element's bin.  All 16 batches are folded (one at a
    # time is converted: 16 more resident batches would not fit beside the float32 ones on every box) and the result
    # is compared with the oracle below; the timed updates then go through four resident bf16 batches in turn.
    an16 = SqnrEncodingAnalyzer((1,), num_bins=512, asymmetric_delta_candidates=100, offset_candidates=64, gamma=3.0)
    for x in xs:
        an16.update_stats(x.bfloat16())
    st16 = an16.observer.get_stats()[0]
    hist16_gpu, edges16_gpu = st16.histogram.cpu().clone(), st16.bin_edges.cpu().clone()
    lo16, hi16 = an16.compute_encodings(255, False)
    best16_gpu = int(an16.last_search["best_index"].item())
    xs16 = [x.bfloat16() for x in xs[:4]]
    turn16 = [0]

    def update_next16():
        turn16[0] = (turn16[0] + 1) % len(xs16)
        an16.update_stats(xs16[turn16[0]])

    t_upd16 = event_time(update_next16, 20)
    bf16_stream = {"update_us": round(t_upd16 * 1e6, 2), "GBps_one_read": round(2 * n_b / t_upd16 / 1e9, 1),
                   "frac_of_hbm_peak": round(2 * n_b / t_upd16 / 1e9 / HBM_PEAK_GBS, 4),
                   "elements_per_s": round(n_b / t_upd16, 1), "kernel": "hist_bin16_kernel<SPEC>",
                   "sample": "the first 4 batches rounded to bf16, in turn",
                   "algorithmic_bytes": 2 * n_b, "traffic": MEASURED_TRAFFIC_BYTES.get(("c3", "hist_update_bf16")),
                   "bound": "LDS instruction issue: a table read and an increment per element; bare LDS increments "
                            "alone take 28 us for 67 M elements on this device (16 cycles per wave instruction)"}

    parity = {"sample": "not compared (CPU leg switched off)"}
    cpu_all = cpu_one = None
    if with_cpu_baseline:
        ref16 = O.HistObserver((1,), 512)
        for xb in xs:
            ref16.update(xb.bfloat16().cpu())
        lo16_r, hi16_r, _, _, bi16 = O.sqnr_encodings(ref16.stats, (1,), 255, False, asym_deltas=100, num_offsets=64, gamma=3.0)
        bf16_stream["parity"] = {"hist_bit_exact": bool(torch.equal(hist16_gpu, ref16.stats[0].histogram)),
                                 "edges_bit_exact": bool(torch.equal(edges16_gpu, ref16.stats[0].bin_edges)),
                                 "argmin_identical": bool(best16_gpu == int(bi16.item())),
                                 "encoding_bit_exact": bool(torch.equal(lo16.cpu(), lo16_r) and torch.equal(hi16.cpu(), hi16_r)),
                                 "largest_bin_count": float(hist16_gpu.max()),
                                 "sample": f"all {batches} batches rounded to bf16"}
        del ref16
        # the CPU leg: the whole 16-batch step, one batch on the host at a time; its result is the parity reference
        ref_all = O.HistObserver((1,), 512)
        cpu_dt = 0.0
        for xb in xs:
            xc = xb.cpu()
            t_b = time.perf_counter()
            ref_all.update(xc)
            cpu_dt += time.perf_counter() - t_b
            del xc
        t_b = time.perf_counter()
        lo_r, hi_r, _, _, bi = O.sqnr_encodings(ref_all.stats, (1,), 255, False, asym_deltas=100, num_offsets=64, gamma=3.0)
        cpu_dt += time.perf_counter() - t_b
        threads = torch.get_num_threads()
        cpu_all = {"value": round(n / cpu_dt, 1), "unit": "elements/s", "cores": threads, "kind": "port",
                   "sample": f"all {batches} batches folded + SQNR search with the reference's torch CPU operations "
                             f"({cpu_dt:.2f} s)"}
        parity = {
            "hist_bit_exact": bool(torch.equal(hist_gpu, ref_all.stats[0].histogram)),
            "edges_bit_exact": bool(torch.equal(edges_gpu, ref_all.stats[0].bin_edges)),
            "argmin_identical": bool(best_gpu == int(bi.item())),
            "encoding_bit_exact": bool(torch.equal(lo.cpu(), lo_r) and torch.equal(hi.cpu(), hi_r)),
            "largest_bin_count": float(hist_gpu.max()),
            "sample": f"all {batches} batches",
        }
        # one thread: two batches and the search (bounded)
        torch.set_num_threads(1)
        try:
            ref_1 = O.HistObserver((1,), 512)
            one_dt = 0.0
            for xb in xs[:2]:
                xc = xb.cpu()
                t_b = time.perf_counter()
                ref_1.update(xc)
                one_dt += time.perf_counter() - t_b
                del xc
            t_b = time.perf_counter()
            O.sqnr_encodings(ref_1.stats, (1,), 255, False, asym_deltas=100, num_offsets=64, gamma=3.0)
            t_s1 = time.perf_counter() - t_b
        finally:
            torch.set_num_threads(threads)
        cpu_one = {"value": round(n / (one_dt * batches / 2 + t_s1), 1), "unit": "elements/s", "cores": 1, "kind": "port",
                   "sample": f"2 of {batches} batches folded ({one_dt:.2f} s) + SQNR search ({t_s1:.2f} s), scaled to the "
                             "whole step"}

    config = {"workload": "c3_hist512_sqnr100x64_fp32_16x8x2048x4096", "elements": n,
              "algorithmic_bytes_per_step": bytes_step, "batches": batches,
              "step": "16 x SqnrEncodingAnalyzer.update_stats + compute_encodings (analyzer API over the C ABI)"}
    out = _base_record(bytes_step / wall / 1e9, steps, warmup, wall, "f32", config, repeats)
    out.update({
        "elements_per_s": round(n / wall, 1),
        "kernels": {"hist_update(batch inside the running range)": {"us": round(t_upd * 1e6, 2),
                                                                      "GBps_one_read": round(bytes_read_once / t_upd / 1e9, 1)},
                    "sqnr_search(api)": {"us": round(t_search * 1e6, 2), "candidates": 6400, "bins": 512}},
        "encoding": {"min": float(lo.item()), "max": float(hi.item())},
        "parity": parity,
        "bf16_stream": bf16_stream,
        "roofline": {"bound": "hbm", "kernel": "hist_bin_kernel<SPEC> inside one histogram update (4 launches timed together)",
                     "achieved": round(traffic_upd / t_upd / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(traffic_upd / t_upd / 1e9 / HBM_PEAK_GBS, 4), "algorithmic_bytes": bytes_read_once,
                     "traffic": traffic_upd,
                     "note": "the timed batch lies inside the running range and is read once (speculative binning), so "
                             "achieved / frac are its measured traffic over its time; against the plain algorithm's two "
                             f"reads per element ({2 * bytes_read_once} bytes) the update runs at "
                             f"{round(2 * bytes_read_once / t_upd / 1e9, 1)} GB/s = "
                             f"{round(2 * bytes_read_once / t_upd / 1e9 / HBM_PEAK_GBS, 4)} of peak, and the whole "
                             f"16-batch step at {round(bytes_step / wall / 1e9 / HBM_PEAK_GBS, 4)}"},
    })
    if cpu_all is not None:
        out["cpu_baseline"], out["cpu_baseline_1thread"] = cpu_all, cpu_one
    out["bench_seconds"] = round(time.perf_counter() - t_start, 1)
    del xs, xs16
    return out


def run_dlq_workload(steps, warmup, dev, with_cpu_baseline=True, batches=16, shape=(8, 2048, 4096)):
    """dlq: DlQuantization TF-enhanced calibration of the c3 stream (1536-bucket PDF per batch, then the 17 x 21 + 1
    candidate search for an 8-bit asymmetric encoding) followed by one per-tensor quantize-dequantize of a batch."""
    from aimet_amd import dlq
    from oracle import dlq as OD
    from oracle import torch_ref as O

    _ensure_built()
    _copy_reference(dev)
    t_start = time.perf_counter()
    xs = [_laplace_batch(shape, b, dev) for b in range(batches)]
    q = dlq.BlockTensorQuantizer((), 8, dlq.QUANTIZATION_TF_ENHANCED, device=dev)
    y = torch.empty_like(xs[0])

    def step():
        q.resetEncodingStats()
        for x in xs:
            q.updateStats(x)
        enc = q.computeEncodings(False)
        q.setEncodings(enc)
        q.quantizeDequantize(xs[0], y)
        return enc

    loop_s, repeats = timed_steps(step, steps, warmup)
    wall = loop_s / steps
    enc = step()

    turn = [0]

    def update_next():  # range already fixed: one read of the batch; the batches in turn, as a stream delivers them
        turn[0] = (turn[0] + 1) % batches
        q.updateStats(xs[turn[0]])

    t_upd = event_time(update_next, 20)
    t_qdq = event_time(lambda: q.quantizeDequantize(xs[0], y), 20)
    t_enc = event_time(lambda: q.computeEncodings(False), 5)
    # the FP8 fake-cast of the same batch (E4M3FN, scale = amax / 448 from a min/max calibration), timed beside it
    q8 = dlq.BlockTensorQuantizer((), dlq.QuantizationType.Fp8E4M3FN(), dlq.QUANTIZATION_TF, device=dev)
    q8.updateStats(xs[0])
    enc8 = q8.computeEncodings(False)
    q8.setEncodings(enc8)
    t_fp8 = event_time(lambda: q8.quantizeDequantize(xs[0], y), 20)
    # aimet_torch's float fake-cast of the same batch (float8_e4m3fn, per-tensor scale), also outside the step
    from aimet_amd.quantization.float import float_quantize_dequantize
    from aimet_amd.quantization.float._finfo import _float8_e4m3fn
    fscale = torch.tensor(float(enc8[0].delta), device=dev)
    t_fcast = event_time(lambda: float_quantize_dequantize(xs[0], _float8_e4m3fn, fscale), 20)
    n_b = xs[0].numel()
    n = n_b * batches
    bytes_upd = 4 * n_b
    bytes_qdq = 8 * n_b
    bytes_step = batches * bytes_upd + bytes_qdq

    # parity: the first two batches' integer histograms, then the PDF after all 16 and the chosen encoding, and a
    # bounded sample of the quantize-dequantize, against the C oracle
    q.resetEncodingStats()
    ref = OD.Pdf()
    hist_ok = True
    for b in range(batches):
        xc = xs[b].cpu().numpy()
        if b < 2:
            h = q.updateStats(xs[b], return_histogram=True)
            hr = ref.update(xc)
            hist_ok = hist_ok and bool((h.cpu().numpy().astype("int64")[0] == hr.astype("int64")).all())
        else:
            q.updateStats(xs[b])
            ref.update(xc)
        del xc
    pdf_ok = bool((q._pdf.cpu().numpy()[0] == ref.pdf).all() and (q._xleft.cpu().numpy()[0] == ref.xleft).all())
    enc_gpu = q.computeEncodings(False)[0]
    enc_ref = ref.compute_encoding(8, False)
    enc_ok = tuple(enc_gpu) == tuple(float(v) for v in enc_ref[:4]) + (8,)
    q.setEncodings([enc_gpu])
    sample = xs[0].view(-1)[: 1 << 22]
    y_s = q.quantizeDequantize(sample).cpu().numpy()
    y_ok = bool((y_s.view("int32") == OD.qdq(sample.cpu().numpy(), enc_ref[:4]).view("int32")).all())
    y8 = q8.quantizeDequantize(sample).cpu().numpy()
    fp8_ok = bool((y8.view("int32") == OD.fp8_qdq(sample.cpu().numpy(), enc8[0].delta, OD.FP8_E4M3FN).view("int32")).all())
    yf = float_quantize_dequantize(sample, _float8_e4m3fn, fscale).cpu()
    fcast_ok = bool(torch.equal(yf.view(torch.int32), O.float_qdq(sample.cpu(), fscale.cpu(), 4, 3, True, False).view(torch.int32)))

    config = {"workload": "dlq_tf_enhanced_pdf1536_search17x21_qdq_fp32_16x8x2048x4096", "elements": n,
              "algorithmic_bytes_per_step": bytes_step, "batches": batches,
              "step": "16 x BlockTensorQuantizer.updateStats + computeEncodings + setEncodings + one quantizeDequantize"}
    out = _base_record(bytes_step / wall / 1e9, steps, warmup, wall, "f32", config, repeats)
    out.update({
        "elements_per_s": round(n / wall, 1),
        "kernels": {"pdf_update(range fixed)": {"us": round(t_upd * 1e6, 2), "GBps": round(bytes_upd / t_upd / 1e9, 1)},
                    "dlq_qdq_forward": {"us": round(t_qdq * 1e6, 2), "GBps": round(bytes_qdq / t_qdq / 1e9, 1)},
                    "dlq_fp8_qdq(e4m3fn, not part of the step)": {"us": round(t_fp8 * 1e6, 2),
                                                                  "GBps": round(bytes_qdq / t_fp8 / 1e9, 1)},
                    "float_qdq(float8_e4m3fn, not part of the step)": {"us": round(t_fcast * 1e6, 2),
                                                                       "GBps": round(bytes_qdq / t_fcast / 1e9, 1)},
                    "tfe_search(with host read-back)": {"us": round(t_enc * 1e6, 2), "candidates": 358, "buckets": 1536}},
        "encoding": {"min": enc[0].min, "max": enc[0].max, "delta": enc[0].delta, "offset": enc[0].offset},
        "parity": {"hist_bit_exact": hist_ok, "pdf_bit_exact": pdf_ok, "encoding_bit_exact": bool(enc_ok),
                   "qdq_bit_exact": y_ok, "fp8_qdq_bit_exact": fp8_ok, "float_qdq_bit_exact": fcast_ok,
                   "sample": f"integer histograms of the first 2 batches; PDF and chosen encoding after all {batches}; "
                             "4M-element quantize-dequantize"},
        "roofline": {"bound": "hbm", "kernel": "dlq_pdf_bin_kernel inside one PDF update (timed with the fold-and-finish launch that follows it)",
                     "achieved": round(bytes_upd / t_upd / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(bytes_upd / t_upd / 1e9 / HBM_PEAK_GBS, 4),
                     "algorithmic_bytes": bytes_upd, "traffic": MEASURED_TRAFFIC_BYTES.get(("dlq", "pdf_update"))},
    })
    if with_cpu_baseline:
        # the scalar C restatement of the reference's loops, one thread (the reference's Python binding passes no
        # loop runner, so its CPU path is single-threaded), on a bounded slice of one batch
        m = 1 << 24
        xc = xs[0].view(-1)[:m].cpu().numpy()
        p = OD.Pdf()
        p.update(xc[:1024])
        t0 = time.perf_counter()
        p.update(xc)
        t_pdf = time.perf_counter() - t0
        t0 = time.perf_counter()
        OD.qdq(xc, enc_ref[:4])
        t_q = time.perf_counter() - t0
        t0 = time.perf_counter()
        p.compute_encoding(8, False)
        t_s = time.perf_counter() - t0
        cpu_step = (t_pdf * batches + t_q) * (n_b / m) + t_s
        out["cpu_baseline"] = {"value": round(bytes_step / cpu_step / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"{m} elements of one batch through the scalar C loops (pdf update "
                                         f"{t_pdf * 1e3:.1f} ms, quantize-dequantize {t_q * 1e3:.1f} ms), search "
                                         f"{t_s * 1e3:.2f} ms, scaled to the full step",
                               "elements_per_s": round(n / cpu_step, 1)}
        out["cpu_baseline_1thread"] = out["cpu_baseline"]
    out["bench_seconds"] = round(time.perf_counter() - t_start, 1)
    del xs
    return out


def _model_parity_sweep(model, ids, dev):
    """Every quantizer of the model against the oracle on the tensor it sees: one calibration pass with one batch,
    each quantizer's input reduced on the CPU as it goes by; then the calibrated min / max of all quantizers are
    compared with the oracle's encodings of those statistics."""
    import llama_harness as LH
    from aimet_amd import nn as qnn
    from aimet_amd.quantization.affine import QuantizeDequantize
    from oracle import torch_ref as O

    stats = {}
    hooks = []

    def record(name, q):
        def hook(_mod, args, _out):
            if name in stats:
                return  # a weight quantizer sees its weight again in the forward pass: same tensor
            x = args[0].detach().cpu()
            stats[name] = O.reduce_minmax(x, tuple(q.shape), q.block_size)
        return hook

    quantizers = {n: m for n, m in model.named_modules() if isinstance(m, QuantizeDequantize)}
    weights = {f"{n}.param_quantizers.weight": m.weight for n, m in model.named_modules()
               if isinstance(m, qnn.QuantizedLinear) and m.param_quantizers["weight"] is not None}
    for name, q in quantizers.items():
        if name in weights:
            # no hook: a hooked parameter quantizer is calibrated and called in two steps, and the timed step uses
            # the one-call form; its input is the weight itself
            stats[name] = O.reduce_minmax(weights[name].detach().cpu(), tuple(q.shape), q.block_size)
        else:
            hooks.append(q.register_forward_hook(record(name, q)))
    LH.calibrate(model, [ids])
    for h in hooks:
        h.remove()
    ok = 0
    bad = []
    for name, q in quantizers.items():
        mn, mx = stats[name]
        lo, hi = O.minmax_encodings(mn, mx, q.qmax - q.qmin, q.symmetric)
        same = (torch.equal(q.min.detach().cpu(), lo.view(q.shape).to(torch.float32))
                and torch.equal(q.max.detach().cpu(), hi.view(q.shape).to(torch.float32)))
        ok += int(same)
        if not same:
            bad.append(name)
    return len(quantizers), ok, bad[:5]


def run_model_workload(steps, warmup, dev, with_cpu_baseline=True, batches=8, seq=2048):
    """c5: whole-model calibration (8 batches through compute_encodings) and one quantized forward of the random-init
    bf16 Llama-style decoder; the GEMMs are PyTorch-ROCm's, the quantize-dequantize and min/max kernels are ours."""
    import llama_harness as LH
    from aimet_amd import nn as qnn
    from aimet_amd.quantization.affine import QuantizeDequantize
    from oracle import torch_ref as O

    _ensure_built()
    _copy_reference(dev)
    t_start = time.perf_counter()
    cfg = LH.LlamaConfig()
    model = LH.build(cfg, dev, seed=0)
    nlin = LH.quantize(model)
    ids = LH.calibration_batches(cfg, dev, batches=batches, seq=seq)

    def calibrate():
        LH.calibrate(model, ids)

    def forward():
        with torch.no_grad():
            return model(ids[0])

    def step():
        calibrate()
        return forward()

    # the step is bound by the host interpreter (a few thousand launches): keep the cyclic garbage collector's pauses
    # out of the timed steps
    step()
    gc.collect()
    gc.disable()
    try:
        loop_s, repeats = timed_steps(step, steps, warmup, min_repeats=5)
    finally:
        gc.enable()
    wall = loop_s / steps

    def timed(fn, reps):
        fn()
        _sync()
        t = time.perf_counter()
        for _ in range(reps):
            fn()
        _sync()
        return (time.perf_counter() - t) / reps

    t_cal = timed(calibrate, 2)
    t_fwd = timed(forward, 3)

    # entering and leaving the calibration context (all quantizers of all modules, three library calls) on their own
    def enter_leave():
        with torch.no_grad():
            ctx = qnn.compute_encodings(model)
            _sync()
            t0 = time.perf_counter()
            ctx.__enter__()
            _sync()
            t1 = time.perf_counter()
            model(ids[0])
            _sync()
            t2 = time.perf_counter()
            ctx.__exit__(None, None, None)
            _sync()
            return t1 - t0, time.perf_counter() - t2

    enter_leave()
    t_enter, t_leave = (statistics.median(v) for v in zip(*(enter_leave() for _ in range(3))))

    def inference_forward():
        with torch.no_grad(), qnn.inference_mode(model):
            return timed(lambda: model(ids[0]), 3)

    t_fwd_inf = inference_forward()
    plain = LH.build(cfg, dev, seed=0)
    t_plain = timed(lambda: torch.no_grad()(plain)(ids[0]), 3)
    del plain

    # elements that pass through our kernels per step
    tokens = seq
    wel = LH.weight_elements(cfg)
    act_in = cfg.layers * (4 * cfg.hidden + 2 * cfg.hidden + cfg.ffn) * tokens + cfg.hidden * tokens
    act_out = cfg.layers * (4 * cfg.hidden + 2 * cfg.ffn + cfg.hidden) * tokens + cfg.vocab * tokens
    act = act_in + act_out
    S = 2
    # calibration: weights min/max once + QDQ per batch; activations min/max once per batch (the reference's flow;
    # work that this implementation avoids still counts as algorithmic bytes of the step)
    bytes_cal = wel * S + batches * (wel * 2 * S + act * S)
    bytes_fwd = wel * 2 * S + act * 2 * S
    bytes_step = bytes_cal + bytes_fwd
    elems_step = wel * (1 + batches + 1) + act * (batches + 1)

    # parity: three quantizers of different kinds against the oracle on the tensors they see in one forward
    io = {}
    names = ["blocks.0.attn.q_proj.input_quantizers.0", "blocks.0.mlp.down_proj.param_quantizers.weight",
             "blocks.15.mlp.down_proj.output_quantizers.0"]
    mods = dict(model.named_modules())
    hooks = [mods[n].register_forward_hook(lambda m, a, o, k=n: io.__setitem__(k, (a[0].detach().cpu(), o.detach().cpu())))
             for n in names]
    forward()
    for h in hooks:
        h.remove()
    parity = {}
    for n in names:
        q = mods[n]
        x, y = io[n]
        sc, off = q.get_scale().detach().cpu(), q.get_offset().detach().cpu()
        ref = (O.qdq_v1(x, sc, off, q.qmin, q.qmax)[0] if q.block_size is None
               else O.qdq_v2_forward(x, sc, off, q.qmin, q.qmax, q.block_size).y)
        parity["forward_" + n.split(".")[-3] + "." + n.split(".")[-2]] = bool(
            torch.equal(y.as_subclass(torch.Tensor).view(torch.int16), ref.view(torch.int16)))
    aq_io = io[names[2]]
    wq = mods[names[1]]
    w_cpu = mods["blocks.0.mlp.down_proj"].weight.detach().cpu()
    wq_enc = (wq.get_scale().detach().cpu(), wq.get_offset().detach().cpu())
    aq = mods[names[2]]
    aq_enc = (aq.get_scale().detach().cpu(), aq.get_offset().detach().cpu())
    # every quantizer's calibrated range against the oracle (one pass, one batch); leaves the model calibrated on it
    total, ok, bad = _model_parity_sweep(model, ids[0], dev)
    parity["calibrated_ranges_bit_exact"] = f"{ok} of {total} quantizers"
    parity["all_quantizers_bit_exact"] = bool(ok == total)
    if bad:
        parity["first_mismatches"] = bad
    # the weight a calibration pass multiplies with (quantize-dequantized by the call that calibrated its quantizer)
    with torch.no_grad(), qnn.compute_encodings(model):
        held = mods["blocks.0.mlp.down_proj"].weight.detach().as_subclass(torch.Tensor).cpu()
        model(ids[0])
    ref_w = O.qdq_v2_forward(w_cpu, wq.get_scale().detach().cpu(), wq.get_offset().detach().cpu(), wq.qmin, wq.qmax,
                             wq.block_size).y
    parity["calibration_pass_weight_bit_exact"] = bool(torch.equal(held.view(torch.int16), ref_w.view(torch.int16)))
    parity["sample"] = ("calibrated min/max of every quantizer on its full-size input (1 batch); forward of 3 "
                        "quantizers; the down_proj weight of block 0 as the calibration passes see it")

    config = {"workload": "c5_llama16x2048_ffn8192_w4b64_a16_calib8x2048_plus_forward", "linear_layers": nlin,
              "weight_elements": wel, "activation_elements_per_forward": act,
              "algorithmic_bytes_per_step": bytes_step, "quantizer_elements_per_step": elems_step,
              "step": "nn.compute_encodings over 8 batches + one quantized forward (module API)"}
    out = _base_record(bytes_step / wall / 1e9, steps, warmup, wall, "bf16", config, repeats)
    out.update({
        "elements_per_s": round(elems_step / wall, 1),
        "phases": {"calibration_8_batches_ms": round(t_cal * 1e3, 2),
                   "entering_the_calibration_context_ms": round(t_enter * 1e3, 2),
                   "leaving_the_calibration_context_ms": round(t_leave * 1e3, 2),
                   "quantized_forward_ms": round(t_fwd * 1e3, 2),
                   "quantized_forward_inference_mode_ms": round(t_fwd_inf * 1e3, 2),
                   "unquantized_forward_ms": round(t_plain * 1e3, 2),
                   "linear_tflops_unquantized": round(LH.linear_flops(cfg, tokens) / t_plain / 1e12, 1)},
        "parity": parity,
        "roofline": {"bound": "hbm", "kernel": "qdq_fwd_kernel (weights) inside the quantized forward",
                     "achieved": round(bytes_fwd / t_fwd / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(bytes_fwd / t_fwd / 1e9 / HBM_PEAK_GBS, 4), "algorithmic_bytes": bytes_fwd,
                     "traffic": None,
                     "note": "whole forward including PyTorch GEMMs and attention; the per-kernel figure is in profiles/"},
    })
    if with_cpu_baseline:
        # the reference's CPU path for the same quantizers on a bounded sample: one weight and one activation tensor
        x_act = aq_io[0]

        def cpu_step():
            O.reduce_minmax(w_cpu, tuple(wq.shape), wq.block_size)
            O.qdq_v2_forward(w_cpu, wq_enc[0], wq_enc[1], wq.qmin, wq.qmax, wq.block_size)
            O.reduce_minmax(x_act, ())
            O.qdq_v1(x_act, aq_enc[0], aq_enc[1], aq.qmin, aq.qmax)

        el = 2 * w_cpu.numel() + 2 * x_act.numel()
        sample = ("min/max + quantize-dequantize of one 2048x8192 bf16 weight (block 64, 4 bit) and one 2048x2048 bf16 "
                  "activation (16 bit) with the reference's torch CPU calls; quantizer work only, no GEMMs")
        a, b = cpu_legs(cpu_step, el * (bytes_step / elems_step), "GB/s", sample, budget_s=4.0, max_reps=200)
        out["cpu_baseline"], out["cpu_baseline_1thread"] = a, b
    out["bench_seconds"] = round(time.perf_counter() - t_start, 1)
    del model
    return out


def run_ops_workload(dev):
    """Not one of the benchmark configurations (run with --workload ops; left out of the default run): the public
    operations the driver line does not time -- quantize, dequantize, the ATen-arithmetic quantize-dequantize of frozen
    encodings (per tensor and per channel) and the float fake-cast -- on an [8, 2048, 4096] tensor in the three dtypes,
    every launch on the next of six tensors (HBM figures: one read + one write of the tensor), each checked against
    the oracle on a sample of rows."""
    from aimet_amd.quantization import affine
    from aimet_amd.quantization.float import FloatQuantizeDequantize
    from oracle import torch_ref as O

    _ensure_built()
    t_start = time.perf_counter()
    records = {}
    shape = (8, 2048, 4096)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        g = torch.Generator().manual_seed(0)
        base = torch.randn(shape, generator=g).to(dt)
        xs = [base.to(dev)] + [base.to(dev).clone() for _ in range(5)]
        nbytes = base.numel() * base.element_size()
        turn = [0]

        def nxt():
            turn[0] = (turn[0] + 1) % len(xs)
            return xs[turn[0]]

        s0, o0 = torch.tensor(0.02), torch.tensor(-3.0)
        sc = torch.rand(2048, 1, generator=g) * 0.02 + 0.01
        oc = torch.zeros(2048, 1)
        sd, od, scd, ocd = s0.to(dev), o0.to(dev), sc.to(dev), oc.to(dev)
        codes = affine.quantize(xs[0], sd, od, -128, 127)
        sample = slice(0, 2048, 256)  # rows 0, 256, ... of every batch entry
        cases = {
            "quantize_per_tensor": (lambda: affine.quantize(nxt(), sd, od, -128, 127),
                                    lambda y: torch.equal(y[:, sample].cpu(), O.quantize_forward(base[:, sample], s0, o0, -128, 127)[0])),
            "quantize_per_channel": (lambda: affine.quantize(nxt(), scd, ocd, -128, 127),
                                     lambda y: torch.equal(y[:, sample].cpu(), O.quantize_forward(base[:, sample], sc[sample], oc[sample], -128, 127)[0])),
            "dequantize_per_tensor": (lambda: affine.dequantize(codes, sd, od),
                                      lambda y: torch.equal(y[:, sample].cpu(), O.dequantize_forward(codes[:, sample].cpu(), s0, o0))),
            "qdq_frozen_per_tensor": (lambda: affine.quantize_dequantize(nxt(), sd, od, -128, 127),
                                      lambda y: torch.equal(y[:, sample].cpu(), O.qdq_v1(base[:, sample], s0, o0, -128, 127)[0])),
            "qdq_frozen_per_channel": (lambda: affine.quantize_dequantize(nxt(), scd, ocd, -128, 127),
                                       lambda y: torch.equal(y[:, sample].cpu(), O.qdq_v1(base[:, sample], sc[sample], oc[sample], -128, 127)[0])),
        }
        for name, kw, fmt in (("float_cast_e4m3fn", dict(dtype=torch.float8_e4m3fn), (4, 3, True, False)),
                              ("float_cast_e5m2", dict(dtype=torch.float8_e5m2), (5, 2, False, False)),
                              ("float_cast_e3m4", dict(exponent_bits=3, mantissa_bits=4), (3, 4, False, False))):
            fq = FloatQuantizeDequantize(**kw).to(dev)
            with torch.no_grad(), fq.compute_encodings():
                fq(xs[0])
            with torch.no_grad():
                fscale = fq.get_encodings().scale.detach().cpu()
            cases[name] = ((lambda fq=fq: fq(nxt())),
                           (lambda y, fmt=fmt, fscale=fscale: torch.equal(y[:, sample].as_subclass(torch.Tensor).cpu().view(torch.int16 if dt != torch.float32 else torch.int32),
                                                                          O.float_qdq(base[:, sample], fscale, *fmt).view(torch.int16 if dt != torch.float32 else torch.int32))))
        rec = {}
        with torch.no_grad():
            for name, (fn, check) in cases.items():
                y = fn()
                turn[0] = len(xs) - 1  # the checked call ran on xs[0]
                ok = bool(check(fn().as_subclass(torch.Tensor)))
                t = event_time(fn, 20)
                rec[name] = {"us": round(t * 1e6, 2), "GBps": round(2 * nbytes / t / 1e9, 1),
                             "frac_of_hbm_peak": round(2 * nbytes / t / 1e9 / HBM_PEAK_GBS, 4), "bit_exact_on_sample": ok}
                del y
        records[DTYPE_NAME[dt]] = rec
        del xs, codes
        torch.cuda.empty_cache()
    worst = min(r["frac_of_hbm_peak"] for rec in records.values() for r in rec.values())
    return {"metric": "HBM GB/s of the operations outside the timed step (one read + one write of the tensor)",
            "unit": "GB/s", "config": {"workload": "ops_8x2048x4096_f32_bf16_f16"}, "data": "synthetic",
            "operations": records, "lowest_frac_of_hbm_peak": worst,
            "all_bit_exact_on_sample": all(r["bit_exact_on_sample"] for rec in records.values() for r in rec.values()),
            "bench_seconds": round(time.perf_counter() - t_start, 1)}


RUNNERS = {
    "c1": lambda a, dev, cpu: run_qdq_workload("c1", a.steps, a.warmup, dev, cpu, not a.no_cached),
    "c2": lambda a, dev, cpu: run_qdq_workload("c2", a.steps, a.warmup, dev, cpu, not a.no_cached),
    "c4": lambda a, dev, cpu: run_qdq_workload("c4", a.steps, a.warmup, dev, cpu, not a.no_cached),
    "cols": lambda a, dev, cpu: run_qdq_workload("cols", a.steps, a.warmup, dev, cpu, not a.no_cached),
    "ops": lambda a, dev, cpu: run_ops_workload(dev),
    "c3": lambda a, dev, cpu: run_hist_workload(min(a.steps, 10), min(a.warmup, 2), dev, cpu),
    "dlq": lambda a, dev, cpu: run_dlq_workload(min(a.steps, 10), min(a.warmup, 2), dev, cpu),
    "c5": lambda a, dev, cpu: run_model_workload(min(a.steps, 3), min(a.warmup, 1), dev, cpu),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", choices=["all"] + sorted(RUNNERS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-cached", action="store_true",
                    help="c1 / c2 / c4: leave out the legs that go over one tensor set again and again (the figures "
                         "under 'cached' / 'same_tensor_again_and_again'), so that every launch of a profiled run "
                         "reads from HBM")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives exist on this path); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    cpu = not args.no_cpu_baseline
    t0 = time.perf_counter()
    if args.workload != "all":
        out = RUNNERS[args.workload](args, dev, cpu)
    else:
        out = RUNNERS["c4"](args, dev, cpu)
        torch.cuda.empty_cache()
        configs = {}
        for key in ("c1", "c2", "c3", "dlq", "c5"):
            print(f"[bench] {key} ...", file=sys.stderr, flush=True)
            configs[key] = RUNNERS[key](args, dev, cpu)
            gc.collect()
            torch.cuda.empty_cache()
        out["configs"] = configs
        out["summary"] = {k: {"GBps": r["value"], "pct_of_hbm_peak": r["pct_of_hbm_peak"], "ms_per_step": r["ms_per_step"],
                              "elements_per_s": r["elements_per_s"], "roofline_frac": r["roofline"]["frac"]}
                          for k, r in [("c4", out)] + list(configs.items())}
    if args.workload == "all":
        _ensure_built()
        out["device_ceiling"] = device_ceiling(dev)
    out["host"] = {"cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(),
                   "device": torch.cuda.get_device_name(0)}
    out["bench_total_seconds"] = round(time.perf_counter() - t0, 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
