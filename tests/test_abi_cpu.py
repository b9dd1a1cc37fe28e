"""Host-side checks that need no GPU: the shared library loads and exports the C ABI of include/aimet_amd.h, argument
validation answers with error codes before anything is launched, workspace queries and layout planning are pure host
code, and the Python front end keeps the reference's registry / overload / error behaviour."""

import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from aimet_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from aimet_amd.csrc.build import build

        build(verbose=False)
    return _lib.load()


def test_every_declared_symbol_is_exported_and_bound(lib):
    from aimet_amd import _lib

    header = open(os.path.join(ROOT, "include", "aimet_amd.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ahq_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/aimet_amd.h but not exported"
    assert declared == set(_lib.exported_symbols()), "ctypes bindings and header disagree"
    assert lib.ahq_version() >= 1


def test_argument_validation_without_a_gpu(lib):
    from aimet_amd import _lib

    g = _lib.Grid()
    g.arith, g.op, g.io_dtype, g.compute_dtype, g.qmin, g.qmax = _lib.AHQ_ARITH_AUTOGRAD, 0, 0, 0, 0, 255
    lay = _lib.make_layout([16], [16], [0])
    assert lib.ahq_qdq_forward(None, lay, None, None, None, None, None, None, None, None) == 1
    assert b"grid" in lib.ahq_last_error()
    assert lib.ahq_qdq_forward(g, lay, None, None, None, None, None, None, None, None) == 1  # scale is null
    g.qmin, g.qmax = 5, 1
    assert lib.ahq_qdq_forward(g, lay, None, None, None, 1, None, None, None, None) == 1
    assert b"qmin" in lib.ahq_last_error()
    g.qmin, g.qmax, g.compute_dtype = 0, 255, _lib.AHQ_BF16  # fp32 tensors cannot compute in bf16
    assert lib.ahq_qdq_forward(g, lay, None, None, None, 1, None, None, None, None) == 1
    g.compute_dtype, g.zero_point_shift = 0, 0.25
    assert lib.ahq_qdq_forward(g, lay, None, None, None, 1, None, None, None, None) == 1
    g.zero_point_shift = 0.0
    g.arith = _lib.AHQ_ARITH_DLQ
    assert lib.ahq_qdq_backward(g, lay, None, None, None, None, None, 1, None, None, 0, None) == 1
    bad = _lib.make_layout([16], [5], [0])  # block does not divide the dimension
    g.arith = _lib.AHQ_ARITH_AUTOGRAD
    assert lib.ahq_qdq_forward(g, bad, None, None, None, 1, None, None, None, None) == 1
    assert lib.ahq_minmax(7, lay, None, 1, 1, None, None, 0, None, 0, None) == 1
    assert lib.ahq_minmax(0, lay, None, None, None, None, None, 0, None, 0, None) == 1
    assert lib.ahq_hist_update(0, lay, None, None, 1, None, 0, None) == 1
    assert lib.ahq_sqnr_search(None, None, None, None, None, None, None, None, None, None, None) == 1
    # the fused LPBQ forward: validation, then the refusals that send a caller to the two-launch form
    g.arith, g.op, g.io_dtype, g.compute_dtype, g.qmin, g.qmax = _lib.AHQ_ARITH_AUTOGRAD, 0, 0, 0, -8, 7
    blocks = _lib.make_layout([4, 64], [1, 16], [4, 1])   # 4 x 4 blocks of 16 elements

    def fused(grid, layout, group, mult=16):
        return lib.ahq_lpbq_qdq_forward(grid, layout, 1, 1, None, 0, 1, 1, group, 1e-9, mult, None, 1, None, None)

    assert lib.ahq_lpbq_qdq_forward(g, blocks, 1, 1, None, 0, None, 1, 4, 1e-9, 16, None, 1, None, None) == 1  # no min
    assert fused(g, blocks, 0) == 1 and fused(g, blocks, 4, mult=0) == 1
    assert fused(g, blocks, 3) == _lib.AHQ_ERR_UNSUPPORTED        # 16 blocks, groups of 3
    g.compute_dtype = _lib.AHQ_F32
    g.io_dtype = _lib.AHQ_BF16
    assert fused(g, blocks, 4) == _lib.AHQ_ERR_UNSUPPORTED        # arithmetic in float32 on a 16-bit tensor
    g.io_dtype = g.compute_dtype = 0
    g.arith = _lib.AHQ_ARITH_ATEN
    assert fused(g, blocks, 4) == _lib.AHQ_ERR_UNSUPPORTED
    g.arith = _lib.AHQ_ARITH_AUTOGRAD
    repeated = _lib.make_layout([3, 4, 64], [3, 1, 16], [0, 4, 1])
    assert fused(g, repeated, 4) == _lib.AHQ_ERR_UNSUPPORTED      # encodings repeat over the leading dimension
    # calibration and first quantize-dequantize of a parameter in one call
    def calibrate(grid, layout, x=1, y=1, offset=1, ws=1, ws_bytes=1 << 20):
        return lib.ahq_minmax_calibrate_qdq(grid, layout, x, y, 15, 1, 1e-9, 1e-9, 3e38, 1e37, 1, 0, 1, 1, 1e-9, 1,
                                            offset, ws, ws_bytes, None)

    assert calibrate(None, blocks) == 1 and calibrate(g, None) == 1
    assert calibrate(g, blocks, x=None) == 1 and calibrate(g, blocks, y=None) == 1 and calibrate(g, blocks, offset=None) == 1
    g.arith = _lib.AHQ_ARITH_DLQ
    assert calibrate(g, blocks) == 1 and b"arithmetic" in lib.ahq_last_error()
    g.arith, g.op = _lib.AHQ_ARITH_AUTOGRAD, 1
    assert calibrate(g, blocks) == 1
    g.op = 0
    assert calibrate(g, bad) == 1
    assert calibrate(g, blocks, ws=None) == _lib.AHQ_ERR_WORKSPACE
    assert calibrate(g, blocks, ws_bytes=8) == _lib.AHQ_ERR_WORKSPACE
    assert calibrate(g, _lib.make_layout([0, 64], [1, 16], [4, 1])) == 1   # nothing to calibrate on


def test_workspace_queries_and_planning(lib):
    from aimet_amd import _lib

    g = _lib.Grid()
    g.arith, g.op, g.io_dtype, g.compute_dtype, g.qmin, g.qmax = _lib.AHQ_ARITH_AUTOGRAD, 0, 0, 0, -128, 127
    per_tensor = _lib.make_layout([32 * 64 * 112 * 112], [32 * 64 * 112 * 112], [0])
    per_channel = _lib.make_layout([4096, 4096], [1, 4096], [1, 0])
    blockwise = _lib.make_layout([14336, 4096], [1, 64], [64, 1])
    assert lib.ahq_qdq_backward_workspace_bytes(g, per_tensor, 0) == 0
    # per-tensor: one (gscale, goffset) pair of doubles per 16 KiB tile
    tiles = -(-32 * 64 * 112 * 112 // 4096)
    assert lib.ahq_qdq_backward_workspace_bytes(g, per_tensor, 1) >= tiles * 16
    # one tile per row / one wave segment per block: written directly (only the unaligned fallback needs scratch)
    assert lib.ahq_qdq_backward_workspace_bytes(g, per_channel, 1) <= 4096 * 8 * 16
    # per-tensor min/max: one partial triple per workgroup of the streaming kernel, at most 512 whatever the size
    assert lib.ahq_minmax_workspace_bytes(per_tensor) == 512 * 12
    assert lib.ahq_minmax_workspace_bytes(_lib.make_layout([1 << 33], [1 << 33], [0])) == 512 * 12
    assert lib.ahq_hist_update_workspace_bytes(0, per_tensor, 512) > 1024 * 2 * 514 * 4
    assert lib.ahq_qdq_backward_workspace_bytes(g, blockwise, 1) >= 0
    # statistics of every encoding (two aligned arrays) in front of the reduction's own workspace
    assert (lib.ahq_minmax_calibrate_qdq_workspace_bytes(_lib.AHQ_BF16, blockwise)
            >= 2 * 14336 * 64 * 2 + lib.ahq_minmax_workspace_bytes(blockwise))
    assert lib.ahq_minmax_calibrate_qdq_workspace_bytes(0, per_tensor) >= 512 + lib.ahq_minmax_workspace_bytes(per_tensor)
    assert lib.ahq_minmax_calibrate_qdq_workspace_bytes(9, per_tensor) == 0


def test_planning_of_the_column_layouts(lib):
    """Host arithmetic only: one encoding per element of the fastest axis is planned as a column walk with row groups,
    blocks along the leading axis as that many stacked problems, and the scratch follows."""
    from aimet_amd import _lib

    g = _lib.Grid()
    g.arith, g.op, g.io_dtype, g.compute_dtype, g.qmin, g.qmax = _lib.AHQ_ARITH_AUTOGRAD, 0, _lib.AHQ_BF16, _lib.AHQ_BF16, -8, 7
    per_column = _lib.make_layout([8192, 4096], [8192, 1], [0, 1])
    # min/max: about 256 workgroups of 64 lanes x 8 columns (16-bit) -> 8 across, 32 row groups of 12-byte triples;
    # the float32 plan has 16 across and 16 row groups: the larger one is reported
    assert lib.ahq_minmax_workspace_bytes(per_column) == 32 * 4096 * 12
    # backward, 16-bit: four columns per lane -> 16 workgroups across, 1024 / 16 = 64 row groups of double pairs
    assert lib.ahq_qdq_backward_workspace_bytes(g, per_column, 1) == 64 * 4096 * 16
    assert lib.ahq_qdq_backward_workspace_bytes(g, per_column, 0) == 0
    # 64 x 1 blocks: 128 stacked problems of 64 rows; 64 rows are one row group in both passes
    stacked = _lib.make_layout([8192, 4096], [64, 1], [4096, 1])
    assert lib.ahq_minmax_workspace_bytes(stacked) == 128 * 4096 * 12
    assert lib.ahq_qdq_backward_workspace_bytes(g, stacked, 1) == 128 * 4096 * 16
    # the same with a batch axis that has encodings of its own
    batched = _lib.make_layout([5, 70, 512], [1, 70, 1], [512, 0, 1])
    assert lib.ahq_minmax_workspace_bytes(batched) >= 5 * 512 * 12
    # an odd row length: one element per lane, the kernels still apply (scratch per row group and encoding)
    odd = _lib.make_layout([4099, 4099], [4099, 1], [0, 1])
    assert lib.ahq_minmax_workspace_bytes(odd) % (4099 * 12) == 0 and lib.ahq_minmax_workspace_bytes(odd) >= 4099 * 12
    # too few columns for a column walk: one slot per encoding (ordered keys)
    assert lib.ahq_minmax_workspace_bytes(_lib.make_layout([1100, 24], [1100, 1], [0, 1])) == 24 * 12
    # float fake-cast by table: 16-bit tensors of 2^22 elements and more with one encoding
    big, small = _lib.make_layout([1 << 22], [1 << 22], [0]), _lib.make_layout([(1 << 22) - 1], [(1 << 22) - 1], [0])
    assert lib.ahq_float_cast_workspace_bytes(_lib.AHQ_BF16, big) == 131072
    assert lib.ahq_float_cast_workspace_bytes(_lib.AHQ_F16, big) == 131072
    assert lib.ahq_float_cast_workspace_bytes(_lib.AHQ_F32, big) == 0
    assert lib.ahq_float_cast_workspace_bytes(_lib.AHQ_BF16, small) == 0
    assert lib.ahq_float_cast_workspace_bytes(_lib.AHQ_BF16, _lib.make_layout([4096, 4096], [1, 4096], [1, 0])) == 0


def test_backend_registry():
    import aimet_amd.quantization as Q
    from aimet_amd.quantization.affine.backends import hip

    assert Q.get_backend() is hip

    class Dummy:
        quantize = dequantize = quantize_dequantize = staticmethod(lambda *a, **k: "dummy")

    assert Q.add_backend("dummy", Dummy) is None
    assert isinstance(Q.add_backend("dummy", Dummy), RuntimeError)  # returned, not raised
    with Q.set_backend("dummy"):
        assert Q.get_backend() is Dummy
        assert Q.affine.quantize_dequantize(torch.zeros(1), torch.ones(()), torch.zeros(()), 8) == "dummy"
    assert Q.get_backend() is hip
    with pytest.raises(RuntimeError):
        Q.set_backend("no-such-backend")


def test_overload_parsing():
    from aimet_amd.quantization.affine.backends import _parse_args, _derive_qmin_qmax

    assert _parse_args((8,), {}) == (0, 255, None, 0.0)
    assert _parse_args((8, True), {}) == (-128, 127, None, 0.0)
    assert _parse_args((), {"bitwidth": 4, "signed": True, "block_size": (1, 64)}) == (-8, 7, (1, 64), 0.0)
    assert _parse_args((), {"num_steps": 15, "signed": False}) == (0, 15, None, 0.0)
    assert _parse_args((-7, 7), {"zero_point_shift": 0.5}) == (-7, 7, None, 0.5)
    assert _parse_args((0, 255, (2, 2)), {}) == (0, 255, (2, 2), 0.0)
    assert _derive_qmin_qmax(num_steps=3, signed=True) == (-2, 1)
    with pytest.raises(RuntimeError):
        import aimet_amd.quantization as Q
        Q.affine.quantize(torch.zeros(1), torch.ones(()), torch.zeros(()), 8, zero_point_shift=0.5)


def test_cpu_tensors_fail_loudly():
    """There is no CPU or eager-PyTorch fallback: the product path raises on tensors that are not on the GPU."""
    import aimet_amd.quantization as Q
    from aimet_amd.quantization.encoding_analyzer import MinMaxEncodingAnalyzer, SqnrEncodingAnalyzer

    x = torch.randn(4, 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        Q.affine.quantize_dequantize(x, torch.tensor(0.1), torch.tensor(0.0), 8)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        MinMaxEncodingAnalyzer(()).update_stats(x)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        SqnrEncodingAnalyzer(()).update_stats(x)
    # shape errors are reported before the device check, like the reference's validation
    with pytest.raises(RuntimeError, match="cannot be expanded"):
        Q.affine.quantize_dequantize(torch.randn(2, 3, 4, 5), torch.ones(4), torch.zeros(()), 0, 255)


def test_scale_and_offset_are_broadcast_against_each_other_on_the_host():
    """The kernels read scale[e] and offset[e] with one index, so operands of different shapes are expanded to their
    common shape before anything is launched; shapes that do not broadcast are refused."""
    from aimet_amd.quantization.affine.backends import hip as H

    scale, offset = torch.rand(6, 1) + 0.1, torch.tensor(-3.0)
    s2, o2 = H._broadcast_encodings(scale, offset, None)
    assert s2.shape == o2.shape == (6, 1) and bool((o2 == -3.0).all())
    s2, o2 = H._broadcast_encodings(torch.tensor(0.5), torch.zeros(6, 1), None)
    assert s2.shape == o2.shape == (6, 1)
    s2, o2 = H._broadcast_encodings(torch.rand(6, 1), torch.zeros(1, 5), None)
    assert s2.shape == o2.shape == (6, 5)
    with pytest.raises(RuntimeError, match="cannot be broadcast"):
        H._broadcast_encodings(torch.rand(6, 1), torch.zeros(4, 1), None)
    with pytest.raises(RuntimeError, match="cannot be expanded"):
        H._broadcast_encodings(torch.rand(6, 1), torch.zeros(6, 4), (1, 8))
    s2, o2 = H._broadcast_encodings(torch.rand(6, 4), torch.tensor(0.0), (1, 8))
    assert o2.shape == (6, 4)
    # gradients flow back to each operand's own shape through the expansion
    off = torch.zeros((), requires_grad=True)
    _, o2 = H._broadcast_encodings(torch.rand(6, 1), off, None)
    o2.sum().backward()
    assert off.grad.shape == () and float(off.grad) == 6.0


def test_encoding_cache_follows_tracked_writes_and_has_an_invalidate_hook():
    """Scale / offset are cached while no gradient can reach min / max.  Tracked writes (set_range, copy_) are seen
    through the version counter; a write through .data is not and needs invalidate_encoding_cache()."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    q = QuantizeDequantize((), qmin=0, qmax=255, symmetric=False)
    q.set_range(torch.tensor(0.0), torch.tensor(255.0))
    with torch.no_grad():
        assert float(q.get_encodings().scale) == 1.0
        q.set_range(None, torch.tensor(510.0))
        assert float(q.get_encodings().scale) == 2.0
        q.max.copy_(torch.tensor(1020.0))
        assert float(q.get_encodings().scale) == 4.0
        q.max.data.fill_(255.0)  # untracked
        q.invalidate_encoding_cache()
        assert float(q.get_encodings().scale) == 1.0
    # with gradients enabled nothing is cached: the reference's behaviour
    q.max.data.fill_(510.0)
    assert float(q.get_encodings().scale) == 2.0


def test_quantizer_construction_and_bookkeeping_on_cpu():
    from aimet_amd.quantization.affine import QuantizeDequantize, GroupedBlockQuantizeDequantize, Quantize

    q = QuantizeDequantize((3, 1), 8, True)
    assert (q.qmin, q.qmax, q.bitwidth, q.signed, q.symmetric) == (-128, 127, 8, True, True)
    assert not q.is_initialized() and q.get_scale() is None and q.get_encodings() is None
    q.set_range(-torch.ones(3, 1), torch.ones(3, 1))
    assert q.is_initialized()
    assert torch.equal(q.get_offset(), torch.zeros(3, 1))
    q2 = QuantizeDequantize((), qmin=0, qmax=15, symmetric=False)
    assert q2.bitwidth == 4 and not q2.signed
    q2.bitwidth = 8
    assert (q2.qmin, q2.qmax) == (0, 255)
    with pytest.raises(ValueError):
        QuantizeDequantize((), qmin=3, qmax=3, symmetric=False)
    with pytest.raises(ValueError):
        QuantizeDequantize((), 8, True, zero_point_shift=0.3)
    with pytest.raises(RuntimeError):
        Quantize((), 8, True, zero_point_shift=0.5)
    with pytest.raises(RuntimeError):
        GroupedBlockQuantizeDequantize((4, 2), 4, False, 8, None, (1, 8), (1, -1))
    with pytest.raises(RuntimeError):
        GroupedBlockQuantizeDequantize((4, 2), 8, True, 4, None, (1, 8), (1, -1))
    with pytest.raises(TypeError):
        QuantizeDequantize((), 8, True, bogus=1)
    # a group of LPBQ blocks is a run of neighbours in the scale array, or the one-launch forward does not apply
    def per_group(shape, grouping):
        return GroupedBlockQuantizeDequantize(shape, 4, True, 8, None, None, grouping)._blocks_per_group()

    assert per_group((96, 8), (1, -1)) == 8 and per_group((96, 8), (1, 4)) == 4 and per_group((96, 8), (1, 1)) == 1
    assert per_group((10, 64, 1, 1), (1, 64, 1, 1)) == 64 and per_group((4, 6, 8), (1, 3, -1)) == 24
    assert per_group((8, 6), (2, 3)) is None and per_group((64, 10), (64, 1)) is None
    assert per_group((1, 8), (-1, 4)) == 4
    sd = q.state_dict()
    q3 = QuantizeDequantize((3, 1), 8, True)
    q3.load_state_dict(sd)
    assert q3.is_initialized() and torch.equal(q3.max, q.max)
    import copy
    assert copy.deepcopy(q).is_initialized() and not copy.deepcopy(QuantizeDequantize((), 8, True)).is_initialized()


def test_product_never_imports_the_oracle():
    out = subprocess.run(["grep", "-rIl", "--include=*.py", "--include=*.hip", "--include=*.h", "-e", "oracle",
                          os.path.join(ROOT, "aimet_amd")], capture_output=True, text=True).stdout.split()
    assert out == [], f"product files mention the oracle: {out}"
    code = "import sys; import aimet_amd.quantization, aimet_amd.quantization.affine, aimet_amd.quantization.encoding_analyzer; print(any(m.startswith('oracle') for m in sys.modules))"
    res = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True)
    assert res.stdout.strip() == "False", res.stdout + res.stderr


def test_a_quantizer_whose_observer_holds_call_state_can_be_copied_and_pickled():
    """After a pass-through calibration of a per-channel quantizer its observer keeps what the next call reuses
    (layout, workspace, result tensors).  Deep copies and pickles of the quantizer go through that state, so it must
    be plain data: ctypes structures of integers are, a ctypes function pointer is not."""
    import copy
    import pickle

    from aimet_amd import _lib
    from aimet_amd.quantization.affine import QuantizeDequantize

    q = QuantizeDequantize((3, 1), 8, True)
    q.set_range(torch.tensor([[-1.0], [-2.0], [-3.0]]), torch.tensor([[1.0], [2.0], [3.0]]))
    obs = q.encoding_analyzer.observer
    layout = _lib.Layout()
    layout.ndim = 2
    mn, mx = torch.zeros(3, 1), torch.ones(3, 1)
    obs.__dict__["_fast"] = ((torch.Size([3, 8]), torch.float32, torch.device("cpu")), mn, mx, layout,
                             torch.empty(16, dtype=torch.uint8), 16, torch.empty(3, 1), torch.empty(3, 1), 0)
    for twin in (copy.deepcopy(q), pickle.loads(pickle.dumps(q))):
        assert twin.is_initialized() and torch.equal(twin.max, q.max)
        kept = twin.encoding_analyzer.observer.__dict__["_fast"]
        assert kept[3].ndim == 2 and kept[0] == obs.__dict__["_fast"][0]
    # what this guards against
    with pytest.raises(ValueError):
        pickle.dumps(_lib.load().ahq_minmax_copy)


def test_ctypes_structures_have_the_layout_the_header_declares(tmp_path):
    """Every struct of include/aimet_amd.h, compiled by the C compiler, against its ctypes mirror in aimet_amd/_lib.py:
    same size and the same offset for every field (a field added or reordered on one side only would otherwise hand
    the library shifted pointers)."""
    import ctypes
    import os
    import re
    import shutil
    import subprocess

    from aimet_amd import _lib

    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    pairs = {"ahq_layout": _lib.Layout, "ahq_grid": _lib.Grid, "ahq_hist_state": _lib.HistState,
             "ahq_sqnr_params": _lib.SqnrParams, "ahq_dlq_pdf_state": _lib.DlqPdfState,
             "ahq_grid_probe_item": _lib.GridProbeItem, "ahq_calibrate_qdq_item": _lib.CalibrateQdqItem,
             "ahq_slots_finalize_item": _lib.SlotsFinalizeItem}
    header = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "aimet_amd.h")
    declared = set(re.findall(r"^\} (ahq_\w+);", open(header).read(), flags=re.M)) - {"ahq_status", "ahq_arith", "ahq_op"}
    assert declared == set(pairs), "a struct of the header has no ctypes mirror in this test (or the other way round)"
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{header}"', "int main(void) {"]
    for cname, cls in pairs.items():
        lines.append(f'  printf("{cname} size %zu\\n", sizeof({cname}));')
        for field, _ in cls._fields_:
            lines.append(f'  printf("{cname} {field} %zu\\n", offsetof({cname}, {field}));')
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-o", str(exe), str(src)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    seen = {}
    for line in out.splitlines():
        cname, what, value = line.split()
        seen[(cname, what)] = int(value)
    for cname, cls in pairs.items():
        assert seen[(cname, "size")] == ctypes.sizeof(cls), cname
        for field, _ in cls._fields_:
            assert seen[(cname, field)] == getattr(cls, field).offset, f"{cname}.{field}"


def test_argument_validation_of_the_batched_entry_points(lib):
    """ahq_grid_probe_many / ahq_minmax_calibrate_qdq_many / ahq_minmax_slots_finalize_many refuse bad arguments on
    the host, name the failing item and launch nothing (no GPU here)."""
    import ctypes

    from aimet_amd import _lib

    assert lib.ahq_grid_probe_many(None, 0, None, None, None) == 0          # nothing to do
    assert lib.ahq_minmax_calibrate_qdq_many(None, 0, None, None) == 0
    assert lib.ahq_minmax_slots_finalize_many(None, 0, None, None) == 0
    assert lib.ahq_grid_probe_many(None, 2, None, None, None) == 1
    assert lib.ahq_grid_probe_many(None, -1, None, None, None) == 1
    assert lib.ahq_minmax_calibrate_qdq_many(None, 3, None, None) == 1
    assert lib.ahq_minmax_slots_finalize_many(None, 1, None, None) == 1

    probes = (_lib.GridProbeItem * 2)()
    for it in probes:
        it.dtype, it.layout, it.x, it.num_levels = 0, _lib.make_layout([64, 64], [1, 64], [1, 0]), 256, 8
    probes[1].dtype = 9
    verdicts = (ctypes.c_uint8 * 2)()
    assert lib.ahq_grid_probe_many(probes, 2, None, None, None) == 1        # nowhere to put the verdicts
    probes[0].dtype = 9                                                      # the first item fails before any launch
    assert lib.ahq_grid_probe_many(probes, 2, verdicts, None, None) == 1
    assert b"item 0" in lib.ahq_last_error()

    items = (_lib.SlotsFinalizeItem * 2)()
    for it in items:
        it.stat_dtype, it.symmetric, it.slots, it.num_steps = 0, 0, 256, 255
        it.minimum_scale_in_dtype = it.minimum_scale = 1e-9
        it.dtype_max, it.near_max_threshold = 3e38, 1e37
        it.param_dtype, it.param_min, it.param_max = 0, 256, 256
        it.qmin, it.qmax, it.grid_minimum_scale, it.scale, it.offset = 0, 255, 1e-9, 256, 256
    items[0].slots = None
    assert lib.ahq_minmax_slots_finalize_many(items, 2, 256, None) == 1
    assert b"item 0" in lib.ahq_last_error() and b"slots" in lib.ahq_last_error()
    items[0].slots = 258                                                     # not 4-byte aligned
    assert lib.ahq_minmax_slots_finalize_many(items, 2, 256, None) == 1
    items[0].slots, items[0].qmin = 256, 300
    assert lib.ahq_minmax_slots_finalize_many(items, 2, 256, None) == 1 and b"qmax" in lib.ahq_last_error()
    items[0].qmin, items[0].param_dtype = 0, 7
    assert lib.ahq_minmax_slots_finalize_many(items, 2, 256, None) == 1 and b"dtype" in lib.ahq_last_error()
