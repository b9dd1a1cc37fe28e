"""ahq_minmax_static, the entry point that allocates nothing (its scratch is a file-scope device array), against
ahq_minmax with a caller-provided workspace: identical results, bit for bit, through the C ABI, on two calls in a row
of which the second is smaller (the shared scratch keeps the first call's contents)."""

import ctypes

import pytest
import torch

from aimet_amd import _lib
from aimet_amd.quantization.affine.backends.hip import _prepare
from tests.helpers import assert_same_bits

SCRATCH_BYTES = 1 << 20  # AHQ_MINMAX_STATIC_SCRATCH_BYTES


def _both(lib, x, shape, block, finite_only, running=None):
    """(min, max) from ahq_minmax and from ahq_minmax_static on the same tensor."""
    xd, layout = _prepare(x, shape, block)
    code = _lib.DTYPE_CODE[x.dtype]
    stream = _lib.current_stream(x.device)
    out = []
    for static in (False, True):
        mn = torch.full(shape, 123.0, dtype=x.dtype, device=x.device)
        mx = torch.full(shape, -123.0, dtype=x.dtype, device=x.device)
        run = None if running is None else [r.clone() for r in running]
        rp = (None, None) if run is None else (run[0].data_ptr(), run[1].data_ptr())
        if static:
            rc = lib.ahq_minmax_static(code, layout, xd.data_ptr(), mn.data_ptr(), mx.data_ptr(), rp[0], rp[1],
                                       finite_only, stream)
            _lib.check(rc, "ahq_minmax_static")
        else:
            nbytes = lib.ahq_minmax_workspace_bytes(layout)
            ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=x.device)
            rc = lib.ahq_minmax(code, layout, xd.data_ptr(), mn.data_ptr(), mx.data_ptr(), rp[0], rp[1], finite_only,
                                ws.data_ptr(), nbytes, stream)
            _lib.check(rc, "ahq_minmax")
        out.append((mn, mx, run))
    torch.cuda.synchronize()
    return out


CASES = [
    # (first tensor shape, second (smaller) tensor shape, encoding shape of each, block size)
    ("per_tensor", (64, 33000), (7, 4100), (), (), None),              # partials of 516 tiles, then of 8
    ("per_channel_rows", (48, 9000), (16, 5000), (48, 1), (16, 1), None),  # one partial per tile of each row
    ("per_channel_short_rows", (300, 100), (40, 100), (300, 1), (40, 1), None),  # ordered keys + atomics
    ("blockwise", (64, 1024), (8, 256), (64, 16), (8, 4), (1, 64)),     # shuffle reduction, no scratch at all
    ("columns", (700, 512), (90, 256), (512,), (256,), None),           # column walk: a row of partials per row group
    # column walk whose preferred scratch (8 row groups x 16384 x 12 bytes for the 16-bit dtypes) is more than the
    # static array holds: that entry point runs it with the 5 row groups that fit
    ("wide_columns", (600, 16384), (90, 256), (16384,), (256,), None),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("finite_only", [0, 1])
def test_static_scratch_matches_the_workspace_entry_point(device, dtype, case, finite_only):
    _, big, small, big_enc, small_enc, block = case
    lib = _lib.load()
    g = torch.Generator().manual_seed(9)
    for k, (shape, enc) in enumerate(((big, big_enc), (small, small_enc))):
        x = (torch.randn(shape, generator=g) * (3.0 - k)).to(dtype)
        flat = x.view(-1)
        flat[3], flat[-2] = float("inf"), float("-inf")
        if finite_only == 0 and k == 1:
            flat[11] = float("nan")
        xd = x.to(device)
        (mn, mx, _), (smn, smx, _) = _both(lib, xd, enc, block, finite_only)
        assert_same_bits(smn, mn, f"call {k}: minimum")
        assert_same_bits(smx, mx, f"call {k}: maximum")
        # and both agree with torch on the finite part (the entry point it mirrors is itself tested against the oracle)
        if finite_only == 1 and enc == ():
            fin = x[x.isfinite()]
            assert smn.item() == fin.min().item() and smx.item() == fin.max().item()


def test_column_walk_prefers_more_scratch_than_it_needs():
    """Host-side: for per-channel along the fastest axis the workspace query reports the preferred size, the static
    entry point accepts the layout as long as one row of partials fits."""
    lib = _lib.load()
    lay = _lib.make_layout([600, 16384], [600, 1], [0, 1])
    assert lib.ahq_minmax_workspace_bytes(lay) == 8 * 16384 * 12 > SCRATCH_BYTES
    # accepted for its size: the null pointers are what this call is refused for
    assert lib.ahq_minmax_static(_lib.AHQ_BF16, lay, None, None, None, None, None, 0, None) == _lib.AHQ_ERR_INVALID
    cols = SCRATCH_BYTES // 12 + 8
    lay = _lib.make_layout([600, cols], [600, 1], [0, 1])
    assert lib.ahq_minmax_static(_lib.AHQ_BF16, lay, 16, 16, 16, None, None, 0, None) == _lib.AHQ_ERR_WORKSPACE


@pytest.mark.gpu
def test_static_scratch_folds_running_statistics(device):
    lib = _lib.load()
    g = torch.Generator().manual_seed(4)
    x = torch.randn(32, 70000, generator=g).to(device)
    running = (torch.full((), -0.5, device=device), torch.full((), 9.0, device=device))
    (mn, mx, run), (smn, smx, srun) = _both(lib, x, (), None, 0, running)
    assert_same_bits(smn, mn, "minimum")
    assert_same_bits(smx, mx, "maximum")
    assert_same_bits(srun[0], run[0], "running minimum")
    assert_same_bits(srun[1], run[1], "running maximum")
    assert srun[1].item() == 9.0 and srun[0].item() == x.min().item()


def test_static_scratch_rejects_reductions_beyond_its_size():
    """Host-side check, no GPU needed: the plan is pure arithmetic and the refusal comes before any HIP call."""
    lib = _lib.load()
    enc = SCRATCH_BYTES // 12 + 1
    lay = _lib.make_layout([enc, 40], [1, 40], [1, 0])  # per-channel with short rows: 12 bytes per encoding
    assert lib.ahq_minmax_workspace_bytes(lay) > SCRATCH_BYTES
    rc = lib.ahq_minmax_static(_lib.AHQ_F32, lay, 16, 16, 16, None, None, 0, None)
    assert rc == _lib.AHQ_ERR_WORKSPACE
    assert b"static buffer" in lib.ahq_last_error()
    rows = SCRATCH_BYTES // 12 // 3 + 1
    lay = _lib.make_layout([rows, 3 * 4096], [1, 3 * 4096], [1, 0])  # long rows: one partial per tile of each row
    assert lib.ahq_minmax_static(_lib.AHQ_F32, lay, 16, 16, 16, None, None, 0, None) == _lib.AHQ_ERR_WORKSPACE
    # a per-tensor reduction keeps one partial per workgroup of its streaming kernel, 6 KB whatever the size: never
    # refused for its size (the null pointers are what this call is refused for)
    n = 1 << 36
    lay = _lib.make_layout([n], [n], [0])
    assert lib.ahq_minmax_workspace_bytes(lay) == 512 * 12
    assert lib.ahq_minmax_static(_lib.AHQ_F32, lay, None, None, None, None, None, 0, None) == _lib.AHQ_ERR_INVALID


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=lambda c: c[0])
def test_static_scratch_allocates_no_device_memory(device, case):
    """What the entry point exists for: after the first call on the device (which looks the array's address up), calls
    leave the device's free memory and torch's allocator statistics where they were."""
    _, big, _, big_enc, _, block = case
    lib = _lib.load()
    x = torch.randn(big, generator=torch.Generator().manual_seed(5)).to(device)
    _, layout = _prepare(x, big_enc, block)
    mn = torch.empty(big_enc, dtype=x.dtype, device=device)
    mx = torch.empty(big_enc, dtype=x.dtype, device=device)
    stream = _lib.current_stream(device)

    def call():
        return lib.ahq_minmax_static(_lib.DTYPE_CODE[x.dtype], layout, x.data_ptr(), mn.data_ptr(), mx.data_ptr(), None,
                                     None, 0, stream)

    assert call() == 0
    torch.cuda.synchronize()
    free0, allocated0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(20):
        assert call() == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.cuda.memory_allocated() == allocated0 and torch.cuda.memory_reserved() == reserved0


@pytest.mark.gpu
def test_calibrate_forward_backward_replayed_from_a_captured_graph(device):
    """What the static entry point is for: ahq_minmax_static, ahq_range_to_scale_offset, ahq_qdq_forward and
    ahq_qdq_backward (preallocated outputs and workspace) recorded once into a HIP graph and replayed on new contents
    of the same buffers.  Every replay is compared with the eager calls on the same data, with eager work and
    synchronisations of the process between the replays; the first call of the static entry point happens outside
    the capture (it looks its scratch array up)."""
    from aimet_amd.quantization.affine.backends import hip

    lib = _lib.load()
    g0 = torch.Generator().manual_seed(21)
    shape, enc = (256, 4096), (256, 1)
    x = torch.randn(shape, generator=g0).to(device)
    g = torch.randn(shape, generator=g0).to(device)
    y, gx = torch.empty_like(x), torch.empty_like(x)
    mn, mx, scale, gs, go = (torch.empty(enc, device=device) for _ in range(5))
    offset = torch.zeros(enc, device=device)
    xd, layout = hip._prepare(x, enc, None)
    assert xd.data_ptr() == x.data_ptr()
    grid = hip._grid(_lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QDQ, x.dtype, torch.float32, -128, 127, 0.0)
    nbytes = lib.ahq_qdq_backward_workspace_bytes(grid, layout, 1)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device)
    code = _lib.DTYPE_CODE[x.dtype]
    outputs = (mn, mx, scale, y, gx, gs, go)

    def work():
        st = _lib.current_stream(device)
        _lib.check(lib.ahq_minmax_static(code, layout, x.data_ptr(), mn.data_ptr(), mx.data_ptr(), None, None, 0, st),
                   "ahq_minmax_static")
        _lib.check(lib.ahq_range_to_scale_offset(code, mn.data_ptr(), mx.data_ptr(), mn.numel(), -128, 127, 1e-10,
                                                 scale.data_ptr(), None, st), "ahq_range_to_scale_offset")
        _lib.check(lib.ahq_qdq_forward(grid, layout, x.data_ptr(), y.data_ptr(), None, scale.data_ptr(),
                                       offset.data_ptr(), None, None, st), "ahq_qdq_forward")
        _lib.check(lib.ahq_qdq_backward(grid, layout, g.data_ptr(), x.data_ptr(), gx.data_ptr(), gs.data_ptr(),
                                        go.data_ptr(), scale.data_ptr(), offset.data_ptr(), ws.data_ptr(), nbytes, st),
                   "ahq_qdq_backward")

    work()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        work()
    for rep in range(3):
        x.copy_(torch.randn(shape, generator=g0).to(device) * (rep + 1))
        g.copy_(torch.randn(shape, generator=g0).to(device))
        work()
        torch.cuda.synchronize()
        eager = [t.clone() for t in outputs]
        for t in outputs:
            t.fill_(7.0)
        assert float((x * 2).sum()) == float((x * 2).sum())  # eager work and a synchronisation between the replays
        graph.replay()
        torch.cuda.synchronize()
        for name, want, got in zip(("min", "max", "scale", "y", "gx", "gscale", "goffset"), eager, outputs):
            assert_same_bits(got, want, f"replay {rep}: {name}")
