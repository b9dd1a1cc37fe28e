"""End-to-end parity of the quantizer modules (calibrate -> forward -> backward) with the CPU oracle, plus the
closed-form expectations the reference's own quantizer tests hold
(TrainingExtensions/torch/test/python/v2/quantization/affine/test_affine_quantizer.py)."""

import math
import warnings

import pytest
import torch

from oracle import torch_ref as O
from tests.helpers import assert_same_bits, assert_close_rel

pytestmark = pytest.mark.gpu


class _OracleQdq(torch.autograd.Function):
    """CPU autograd node around the oracle's quantize-dequantize so that torch's CPU autograd can carry gradients on
    to min/max through the same scale/offset expressions the quantizer uses."""

    @staticmethod
    def forward(ctx, x, scale, offset, qmin, qmax, block, zps):
        ctx.args = (qmin, qmax, block, zps)
        ctx.save_for_backward(x, scale, offset)
        return O.qdq_v2_forward(x, scale, offset, qmin, qmax, block, zps).y

    @staticmethod
    def backward(ctx, g):
        x, scale, offset = ctx.saved_tensors
        qmin, qmax, block, zps = ctx.args
        gx, gs, go = O.qdq_v2_backward(g, x, scale, offset, qmin, qmax, block, zps)
        return gx, gs, go, None, None, None, None


class _RoundSTE(torch.autograd.Function):
    @staticmethod
    def forward(ctx, v):
        return torch.round(v)

    @staticmethod
    def backward(ctx, g):
        return g


def _oracle_pipeline(x, grad, shape, qmin, qmax, symmetric, block, zps=0.0):
    """min/max calibration -> parameters -> scale/offset -> QDQ forward/backward, all on the CPU."""
    n = qmax - qmin
    cal_steps = n - 1 if zps == 0.5 else n
    mn, mx = O.reduce_minmax(x, shape, block)
    emin, emax = O.minmax_encodings(mn, mx, cal_steps, symmetric)
    pmin = emin.view(shape).float().clone().requires_grad_(True)
    pmax = emax.view(shape).float().clone().requires_grad_(True)
    ms = O.minimum_scale(n)
    scale = ((pmax - pmin) / n).abs().clamp_min(ms)
    if symmetric:
        offset = torch.full(shape, float(-round((qmin + qmax) / 2)))
    else:
        offset = torch.clamp(_RoundSTE.apply(pmin / scale) - qmin, -qmax, -qmin)
    xr = x.clone().requires_grad_(True)
    y = _OracleQdq.apply(xr, scale, offset, qmin, qmax, block, zps)
    y.backward(grad)
    return dict(min=pmin.detach(), max=pmax.detach(), scale=scale.detach(), offset=offset.detach(), y=y.detach(),
                gx=xr.grad, gmin=pmin.grad, gmax=pmax.grad)


CASES = [
    # name, x shape, dtype, quantizer shape, bitwidth, symmetric, block_size
    ("c1_like", (4, 8, 28, 28), torch.float32, (), 8, False, None),
    ("c2_like", (64, 512), torch.float32, (64, 1), 8, True, None),
    ("blockwise_bf16", (48, 256), torch.bfloat16, (48, 4), 4, True, (1, 64)),
    ("a16_bf16", (2, 64, 128), torch.bfloat16, (), 16, False, None),
    ("per_channel_fp16", (16, 3, 3, 3), torch.float16, (16, 1, 1, 1), 8, True, None),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: c[0])
def test_calibrate_forward_backward(device, case):
    from aimet_amd.quantization.affine import QuantizeDequantize

    _, xshape, dtype, qshape, bw, sym, block = case
    g = torch.Generator().manual_seed(0)
    x = torch.randn(xshape, generator=g)
    if not sym:
        x = torch.relu(x)
    x = x.to(dtype)
    grad = torch.randn(xshape, generator=g).to(dtype)
    n = 2 ** bw - 1
    qmin, qmax = (-math.ceil(n / 2), math.floor(n / 2)) if sym else (0, n)
    ref = _oracle_pipeline(x, grad, qshape, qmin, qmax, sym, block)

    q = QuantizeDequantize(qshape, bw, sym, block_size=block).to(device)
    xd = x.to(device)
    with q.compute_encodings():
        out_dyn = q(xd)
    assert_same_bits(q.min, ref["min"], "calibrated min")
    assert_same_bits(q.max, ref["max"], "calibrated max")
    assert_same_bits(q.get_scale(), ref["scale"], "scale")
    assert_same_bits(q.get_offset(), ref["offset"], "offset")
    xd = xd.clone().requires_grad_(True)
    y = q(xd)
    assert type(y).__name__ == "DequantizedTensor" and y.encoding is not None
    assert_same_bits(y, ref["y"], "forward")
    # inside compute_encodings the output is quantized with the batch's own encodings; those do not require grad,
    # so the reference (and this backend) take the ATen arithmetic wherever it applies
    dyn_ref = None if block is not None else O.qdq_v1(x, ref["scale"], ref["offset"], qmin, qmax)
    dyn_y = ref["y"] if dyn_ref is None else dyn_ref[0]
    assert_same_bits(out_dyn, dyn_y, "dynamic forward")
    y.backward(grad.to(device))
    assert_same_bits(xd.grad, ref["gx"], "input gradient")
    D = O.internal_dtype(dtype, qmin, qmax)
    tol = 1e-5 if D == torch.float32 else float(torch.finfo(D).eps)
    assert_close_rel(q.min.grad, ref["gmin"], tol, "min gradient", abs_floor=1e-30)
    assert_close_rel(q.max.grad, ref["gmax"], tol, "max gradient", abs_floor=1e-30)


def test_frozen_quantizer_takes_aten_arithmetic(device):
    """requires_grad_(False) on the quantizer selects the ATen fake-quantize arithmetic, as in the reference."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    g = torch.Generator().manual_seed(1)
    x = torch.relu(torch.randn(3, 1000, generator=g))
    q = QuantizeDequantize((), 8, False).to(device)
    with q.compute_encodings():
        q(x.to(device))
    scale, offset = q.get_scale().detach().cpu(), q.get_offset().detach().cpu()
    q.requires_grad_(False)
    y = q(x.to(device))
    y_ref, _ = O.qdq_v1(x, scale, offset, 0, 255)
    assert_same_bits(y, y_ref, "frozen forward")
    with torch.no_grad():
        q.requires_grad_(True)
        assert_same_bits(q(x.to(device)), y_ref, "no_grad forward")


@pytest.mark.parametrize("bw,symmetric,expected_scale", [(2, True, 5.25), (2, False, 7.0), (3, True, 3.5), (3, False, 3.0)])
def test_compute_encodings_low_bw(device, bw, symmetric, expected_scale):
    """Reference expectation: test_affine_quantizer.py:397-406."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    qdq = QuantizeDequantize(shape=(), bitwidth=bw, symmetric=symmetric).to(device)
    with qdq.compute_encodings():
        qdq(torch.tensor([-10.5, 10.5], device=device))
    assert qdq.get_scale().item() == expected_scale


@pytest.mark.parametrize("bitwidth,decompressed_bw", [[4, 8], [4, 16], [4, 12], [3, 5], [5, 9], [6, 6]])
def test_gbbq_per_block_sanity(device, bitwidth, decompressed_bw):
    """Reference expectation: test_affine_quantizer.py:1426-1474 -- every LPBQ block scale equals
    max(1, round(scale / gamma)) * gamma with gamma = (largest block scale of the group) / 2^(decompressed_bw - bw)."""
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize, QuantizeDequantize

    g = torch.Generator().manual_seed(0)
    tensor = torch.randn(4, 8, 12, generator=g).to(device)
    gbbq = GroupedBlockQuantizeDequantize(shape=(2, 4, 6), bitwidth=bitwidth, symmetric=True, block_size=(2, 2, 2),
                                          decompressed_bw=decompressed_bw, block_grouping=(2, 2, 3)).to(device)
    qdq = QuantizeDequantize(shape=(2, 4, 6), bitwidth=bitwidth, symmetric=True, block_size=(2, 2, 2)).to(device)
    with gbbq.compute_encodings():
        gbbq(tensor)
    with qdq.compute_encodings():
        qdq(tensor)
    gs, qs = gbbq.get_scale().detach().cpu(), qdq.get_scale().detach().cpu()
    for j in range(2):
        for k in range(2):
            grp_g = gs[0:2, 2 * j:2 * j + 2, 3 * k:3 * k + 3]
            grp_q = qs[0:2, 2 * j:2 * j + 2, 3 * k:3 * k + 3]
            gamma = torch.max(grp_q) / 2 ** (decompressed_bw - bitwidth)
            expect = torch.maximum(torch.tensor([1.0]), torch.round(grp_q / gamma)) * gamma
            assert torch.equal(expect, grp_g)


def test_zero_point_shift_equals_nearest_of_four_levels(device):
    """Reference expectation: test_affine_quantizer.py:2679-2711."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    g = torch.Generator().manual_seed(0)
    for _ in range(10):
        quantizer = QuantizeDequantize(shape=(), bitwidth=2, symmetric=True, zero_point_shift=0.5).to(device)
        t = torch.rand(5, 10, generator=g) * 10.0 - 5
        with quantizer.compute_encodings():
            quantizer(t.to(device))
        scale = torch.max(torch.abs(t)) / 1.5
        assert quantizer.get_scale().item() == scale.item()
        levels = torch.tensor([scale * -1.5, scale * -0.5, scale * 0.5, scale * 1.5])
        nearest = levels[torch.cdist(t.flatten().unsqueeze(1), levels.unsqueeze(1)).argmin(dim=1)].reshape(t.shape)
        assert torch.equal(nearest, quantizer(t.to(device)).detach().cpu())


def test_lpbq_c4_like(device):
    """Blockwise 4-bit weights with 8-bit per-channel scale (LPBQ) on bf16, forward + backward vs the oracle."""
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize

    g = torch.Generator().manual_seed(0)
    w = (torch.randn(96, 512, generator=g) * 0.02).bfloat16()
    grad = torch.randn(96, 512, generator=g).bfloat16()
    q = GroupedBlockQuantizeDequantize(shape=(96, 8), bitwidth=4, symmetric=True, decompressed_bw=8,
                                       block_size=(1, 64), block_grouping=(1, -1)).to(device)
    with q.compute_encodings():
        q(w.to(device))
    mn, mx = O.reduce_minmax(w, (96, 8), (1, 64))
    emin, emax = O.minmax_encodings(mn, mx, 15, True)
    assert_same_bits(q.min, emin.float(), "min")
    assert_same_bits(q.max, emax.float(), "max")
    raw = O.scale_from_minmax(emin, emax, -8, 7)
    scale, pcs = O.lpbq_scale(raw, 4, 8, (1, -1))
    enc = q.get_encodings()
    assert_same_bits(enc.per_channel_scale, pcs, "per-channel scale")
    assert_same_bits(enc.scale, scale, "LPBQ scale")
    mult = enc.per_block_int_scale.detach().cpu()
    assert mult.min() >= 1 and mult.max() <= 16 and torch.equal(mult, mult.round())
    offset = torch.zeros(96, 8)
    wd = w.to(device).requires_grad_(True)
    y = q(wd)
    assert_same_bits(y, O.qdq_v2_forward(w, scale, offset, -8, 7, (1, 64)).y, "forward")
    y.backward(grad.to(device))
    gx_ref, _, _ = O.qdq_v2_backward(grad, w, scale, offset, -8, 7, (1, 64))
    assert_same_bits(wd.grad, gx_ref, "input gradient")
    assert q.min.grad is not None and q.max.grad is not None


@pytest.mark.parametrize("case", [
    ((96, 8), (1, 64), (1, -1), (96, 512)),          # C4's grouping: every row of blocks is one group
    ((40, 12), (1, 16), (1, 4), (40, 192)),          # groups of four neighbouring blocks
    ((10, 64, 1, 1), (1, 8, 1, 1), (1, 64, 1, 1), (10, 512, 1, 1)),  # convolution weight
    ((6, 130), (1, 2), (1, -1), (6, 260)),           # groups longer than a wave
    ((8, 6), (4, 4), (2, 3), (32, 24)),              # groups that are not runs of neighbours: step-by-step form
    ((64, 10), (8, 1), (64, 1), (512, 10)),          # groups down a column: step-by-step form
], ids=["rows", "fours", "conv", "long_groups", "two_dimensional_groups", "column_groups"])
@pytest.mark.parametrize("param_dtype", [torch.float32, torch.bfloat16], ids=["f32_params", "bf16_params"])
def test_lpbq_scale_in_one_launch(device, case, param_dtype):
    """get_encodings() derives the LPBQ scales with one launch (ahq_lpbq_scale), as an autograd node when min / max
    are learned; groupings the library declines run the reference's sequence of torch operations.  All must give the
    oracle's bits."""
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize

    shape, block, grouping, wshape = case
    g = torch.Generator().manual_seed(21)
    w = torch.randn(wshape, generator=g) * 0.05
    w.view(-1)[: w.numel() // 7] *= 30  # uneven block ranges, so the multipliers spread over 1..16
    q = GroupedBlockQuantizeDequantize(shape=shape, bitwidth=4, symmetric=True, decompressed_bw=8, block_size=block,
                                       block_grouping=grouping).to(device)
    with q.compute_encodings():
        q(w.to(device))
    if param_dtype != torch.float32:
        q.to(param_dtype)
    mn, mx = q.min.detach().cpu(), q.max.detach().cpu()
    raw = O.scale_from_minmax(mn.float(), mx.float(), -8, 7)
    scale_ref, pcs_ref = O.lpbq_scale(raw, 4, 8, grouping)
    with torch.no_grad():
        enc = q.get_encodings()
    assert_same_bits(enc.per_channel_scale, pcs_ref, "per-channel scale (one launch)")
    assert_same_bits(enc.scale, scale_ref, "LPBQ scale (one launch)")
    enc_grad = q.get_encodings()  # min / max require gradients
    assert enc_grad.scale.requires_grad
    assert_same_bits(enc_grad.scale, scale_ref, "LPBQ scale (with gradients)")
    fused = type(enc_grad.scale.grad_fn).__name__.startswith("_LpbqScale")
    assert fused == (case[0] not in ((8, 6), (64, 10)))
    mult = enc.per_block_int_scale.detach().cpu()
    assert mult.min() >= 1 and mult.max() <= 16 and torch.equal(mult, mult.round())
    assert mult.unique().numel() > 4


def test_lpbq_scale_propagates_nan(device):
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize

    q = GroupedBlockQuantizeDequantize(shape=(4, 8), bitwidth=4, symmetric=True, decompressed_bw=8, block_size=(1, 16),
                                       block_grouping=(1, -1)).to(device)
    mx = torch.rand(4, 8, generator=torch.Generator().manual_seed(1)) + 0.1
    mx[2, 3] = float("nan")
    q.set_range(-mx.to(device), mx.to(device))
    raw = O.scale_from_minmax(-mx, mx, -8, 7)
    scale_ref, pcs_ref = O.lpbq_scale(raw, 4, 8, (1, -1))
    with torch.no_grad():
        enc = q.get_encodings()
    assert_same_bits(enc.scale, scale_ref, "LPBQ scale")
    assert_same_bits(enc.per_channel_scale, pcs_ref, "per-channel scale")
    assert bool(enc.scale[2].isnan().all()) and not bool(enc.scale[1].isnan().any())


def test_quantize_module_and_state_dict(device):
    from aimet_amd.quantization.affine import Quantize, QuantizeDequantize, Dequantize

    x = torch.randn(8, 32, generator=torch.Generator().manual_seed(3))
    q = Quantize((8, 1), 8, False).to(device)
    with pytest.raises(RuntimeError):
        q(x.to(device))
    with q.compute_encodings():
        q(x.to(device))
    out = q(x.to(device))
    assert type(out).__name__ == "QuantizedTensor"
    codes_ref, _ = O.quantize_forward(x, q.get_scale().detach().cpu(), q.get_offset().detach().cpu(), 0, 255)
    assert_same_bits(out, codes_ref, "codes")
    assert_same_bits(out.dequantize(), O.dequantize_forward(codes_ref, q.get_scale().detach().cpu(),
                                                            q.get_offset().detach().cpu()), "dequantize()")
    # checkpoint round trip keeps values and initialised-ness
    q2 = Quantize((8, 1), 8, False).to(device)
    assert not q2.is_initialized()
    q2.load_state_dict(q.state_dict())
    assert q2.is_initialized()
    assert_same_bits(q2(x.to(device)), codes_ref, "codes after load")
    # frozen parameters are not overwritten
    q2.allow_overwrite(False)
    before = q2.min.detach().clone()
    with q2.compute_encodings():
        q2(10 * x.to(device))
    assert torch.equal(before, q2.min.detach())
    # empty input passes through an uninitialised quantizer
    q3 = QuantizeDequantize((), 8, False).to(device)
    assert q3(torch.empty(0, 3, device=device)).shape == (0, 3)
    with pytest.raises(RuntimeError):
        Dequantize((), 8, False).to(device)(x.to(device))


@torch.no_grad()
@pytest.mark.parametrize("shape,block_size,block_grouping,axis", [
    ((10, 64, 1, 1), (1, 8, 1, 1), (1, 64, 1, 1), 1),
    ((64, 10, 1, 1), (8, 1, 1, 1), (64, 1, 1, 1), 0),
    ((10, 64), (1, 8), (1, 64), 1),
    ((64, 10), (8, 1), (64, 1), 0),
])
@pytest.mark.parametrize("compressed_bw,decompressed_bw", [(4, 8), (8, 16)])
@pytest.mark.parametrize("version", ["2.0.0", "2.1.0", "1.0.0"])
def test_lpbq_encoding_export(device, shape, block_size, block_grouping, axis, compressed_bw, decompressed_bw, version):
    """Parameter table and assertions of the reference's test_lpbq_encoding_schema_2_0_0
    (test_affine_quantizer.py:2443-2535), extended to the other two formats."""
    import numpy as np

    from aimet_amd.quantization import affine
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize

    input_shape = tuple(1 if d == 10 else 64 if d == 64 else 10 for d in shape)
    input_shape = tuple(s * b for s, b in zip(shape, block_size))
    scale = (torch.arange(1, int(np.prod(shape)) + 1).view(shape) * 0.001).to(device)
    qmin, qmax = -(2 ** (decompressed_bw - 1)), 2 ** (decompressed_bw - 1) - 1
    qtzr = GroupedBlockQuantizeDequantize(shape=shape, bitwidth=compressed_bw, symmetric=True,
                                          decompressed_bw=decompressed_bw, block_size=block_size,
                                          block_grouping=block_grouping).to(device)
    qtzr.set_range(scale * qmin, scale * qmax)
    enc = qtzr.get_encodings()._hint_input_shape(input_shape).to_qnn_encoding_dict(version)
    if version == "2.0.0":
        int_scale = torch.tensor(enc["per_block_int_scale"])
        ch_scale = torch.tensor(enc["per_channel_float_scale"])
    elif version == "2.1.0":
        int_scale = torch.tensor(enc["y_scale"]["x"])
        ch_scale = torch.tensor(enc["y_scale"]["x_scale"]).view(qtzr.get_per_channel_scale().shape)
        assert enc["y_scale"]["axis"] in (1 - axis, 1 - axis - len(shape))
    else:
        int_scale = torch.tensor(enc["per_block_int_scale"]).view(shape)
        ch_scale = torch.tensor(enc["scale"]).view(qtzr.get_per_channel_scale().shape)
        assert enc["enc_type"] == "LPBQ" and enc["bw"] == decompressed_bw and enc["compressed_bw"] == compressed_bw
        assert enc["offset"] == [-(2 ** (decompressed_bw - 1))] * ch_scale.numel()
    assert int_scale.min() >= 1 and int_scale.max() <= 2 ** (decompressed_bw - compressed_bw)
    rebuilt = affine.dequantize(int_scale.to(torch.float32).to(device), ch_scale.to(device),
                                torch.zeros_like(ch_scale).to(device), block_size=block_grouping)
    assert torch.allclose(qtzr.get_scale(), rebuilt)
    if version != "1.0.0":
        assert "y_zero_point" not in enc
        assert enc["axis"] in (axis, axis - len(shape))
        assert enc["output_dtype"] == f"int{compressed_bw}"
    assert enc["block_size"] == next(iter(b for b in block_size if b != 1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("grid", [(0, 255, False), (-128, 127, True), (-8, 7, True), (0, 15, False), (0, 65535, False),
                                  (-2 ** 31, 2 ** 31 - 1, False), (3, 11, False)], ids=str)
def test_scale_and_offset_from_a_range_in_one_launch(device, dtype, grid):
    """get_encodings() of a min/max quantizer derives scale and offset with ahq_range_to_scale_offset: bit-exact with
    the reference's step-by-step float32 arithmetic (quantizer.py:319-376) on awkward ranges."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    qmin, qmax, symmetric = grid
    g = torch.Generator().manual_seed(3)
    lo = -torch.rand(4096, generator=g) * torch.logspace(-12, 12, 4096)
    hi = torch.rand(4096, generator=g) * torch.logspace(12, -12, 4096)
    special = torch.tensor([0.0, -0.0, 1.0, -1.0, 1e-30, -1e-30, 3e38, -3e38, float("inf"), -float("inf"), float("nan"),
                            0.1, -0.1, 65504.0, -65504.0, 2.5, -2.5])
    lo = torch.cat([lo, special, special.flip(0), torch.zeros(17), -torch.ones(17)])
    hi = torch.cat([hi, special, special, special, special])
    lo, hi = lo.to(dtype), hi.to(dtype)
    q = QuantizeDequantize((lo.numel(),), qmin=qmin, qmax=qmax, symmetric=symmetric).to(device=device, dtype=dtype)
    with torch.no_grad():
        q.set_range(lo.to(device), hi.to(device))
    with torch.no_grad():
        assert q._fused_scale_offset() is not None
        enc = q.get_encodings()
    scale = O.scale_from_minmax(lo, hi, qmin, qmax)
    offset = O.offset_from_minmax(lo, scale, qmin, qmax, symmetric)
    assert_same_bits(enc.scale, scale, "scale")
    assert_same_bits(enc.offset, offset, "offset")
    # the step-by-step form on the device gives the same answer
    assert_same_bits(q.get_scale(), scale, "get_scale")
    assert_same_bits(q.get_offset(), offset, "get_offset")
    # learned ranges: the same values as one autograd node
    with torch.enable_grad():
        fused = q._fused_scale_offset()
        assert fused[0].grad_fn is not None
        assert_same_bits(fused[0], scale, "scale with grad")
        assert_same_bits(fused[1], offset, "offset with grad")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("grid", [(0, 255, False), (-128, 127, True), (0, 15, False), (0, 65535, False), (3, 11, False),
                                  (-8, 7, False)], ids=str)
def test_learned_range_gradients_in_one_launch(device, dtype, grid):
    """The gradients of min / max through get_scale / _get_offset (quantizer.py:319-376): ahq_range_backward against
    what autograd derives for the reference's composition on the CPU, bit for bit -- ranges below the minimum scale,
    reversed, zero, huge, NaN and infinite included, offsets on and beyond both clamp bounds."""
    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization._utils import ste_round

    qmin, qmax, symmetric = grid
    g = torch.Generator().manual_seed(4)
    n = 4096
    lo = -torch.rand(n, generator=g) * torch.logspace(-10, 10, n)
    hi = torch.rand(n, generator=g) * torch.logspace(10, -10, n)
    lo[::7] = lo[::7].abs()            # positive minima: offsets clamp at -qmax ... -qmin and beyond
    lo[1::11] *= 300.0
    special = torch.tensor([0.0, -0.0, 1.0, -1.0, 1e-30, -1e-30, 3e38, -3e38, float("inf"), -float("inf"), float("nan"),
                            0.1, -0.1, 65504.0, -65504.0, 2.5, -2.5])
    lo = torch.cat([lo, special, special.flip(0), torch.zeros(17), -torch.ones(17)]).to(dtype)
    hi = torch.cat([hi, special, special, special, special]).to(dtype)
    gs = torch.randn(lo.numel(), generator=g) * torch.logspace(-3, 3, lo.numel())
    go = torch.randn(lo.numel(), generator=g)

    # the reference's composition on the CPU, autograd's own backward
    mn_c, mx_c = lo.clone().requires_grad_(True), hi.clone().requires_grad_(True)
    steps = qmax - qmin
    scale_c = ((mx_c.to(torch.float32) - mn_c.to(torch.float32)) / steps).abs().clamp_min_(O.minimum_scale(steps)).to(torch.float32)
    loss = (scale_c * gs).sum()
    if not symmetric:
        offset_c = torch.clamp(ste_round(mn_c / scale_c) - qmin, -qmax, -qmin).to(torch.float32)
        loss = loss + (offset_c * go).sum()
    loss.backward()

    q = QuantizeDequantize((lo.numel(),), qmin=qmin, qmax=qmax, symmetric=symmetric).to(device=device, dtype=dtype)
    with torch.no_grad():
        q.set_range(lo.to(device), hi.to(device))
    enc = q.get_encodings()
    assert enc.scale.grad_fn is not None and type(enc.scale.grad_fn).__name__.startswith("_RangeToScaleOffset")
    assert_same_bits(enc.scale, scale_c, "scale")
    loss = (enc.scale * gs.to(device)).sum()
    if not symmetric:
        assert_same_bits(enc.offset, offset_c, "offset")
        loss = loss + (enc.offset * go.to(device)).sum()
    else:
        assert not enc.offset.requires_grad
    loss.backward()
    assert q.min.grad.dtype == dtype
    assert_same_bits(q.max.grad, mx_c.grad, "gradient of max")
    assert_same_bits(q.min.grad, mn_c.grad, "gradient of min")
    # only one of the two outputs used downstream
    q.min.grad = q.max.grad = None
    q.get_encodings().scale.sum().backward()
    mn_c.grad = mx_c.grad = None
    ((mx_c.to(torch.float32) - mn_c.to(torch.float32)) / steps).abs().clamp_min_(O.minimum_scale(steps)).sum().backward()
    assert_same_bits(q.max.grad, mx_c.grad, "gradient of max, scale only")
    assert_same_bits(q.min.grad, mn_c.grad, "gradient of min, scale only")


@pytest.mark.parametrize("stat_dtype", [torch.float32, torch.float16, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("param_dtype", [torch.float32, torch.bfloat16], ids=["f32_params", "bf16_params"])
@pytest.mark.parametrize("grid", [(0, 255, False, None), (-128, 127, True, None), (-8, 7, True, None),
                                  (0, 65535, False, None), (-2, 1, True, 0.5), (-2, 1, True, None)], ids=str)
def test_end_of_minmax_calibration_in_one_launch(device, monkeypatch, stat_dtype, param_dtype, grid):
    """Leaving compute_encodings() with ahq_minmax_finalize gives the min / max parameters, scale and offset of the
    step-by-step form (analyzer kernel, set_range, get_scale / get_offset) bit for bit, and the oracle's; the
    encodings it leaves in the cache are the ones a later get_encodings() derives afresh."""
    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization.affine.quantizer import AffineQuantizerBase

    qmin, qmax, symmetric, zps = grid
    g = torch.Generator().manual_seed(9)
    rows = 512
    x = torch.randn(rows, 96, generator=g) * torch.logspace(-9, 9, rows).view(-1, 1)
    x[0] = 0.0
    x[1] = 1e-12
    x[2, 0], x[3, 0], x[4, 0] = float("inf"), -float("inf"), float("nan")
    x[5] = x[5].abs()
    x[6] = -x[6].abs()
    x = x.to(stat_dtype).to(device)

    def calibrated(fused: bool):
        q = QuantizeDequantize((rows, 1), qmin=qmin, qmax=qmax, symmetric=symmetric,
                               zero_point_shift=zps).to(device=device, dtype=param_dtype)
        calls = []
        real = AffineQuantizerBase._finalize_from_minmax
        monkeypatch.setattr(AffineQuantizerBase, "_finalize_from_minmax",
                            (lambda self: calls.append(real(self)) or calls[-1]) if fused else (lambda self: False))
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            with torch.no_grad(), q._compute_encodings(passthrough=True):
                q(x)
                q(x * 0.5)
        monkeypatch.undo()
        assert calls == ([True] if fused else [])
        return q

    fast, slow = calibrated(True), calibrated(False)
    assert_same_bits(fast.min, slow.min, "min")
    assert_same_bits(fast.max, slow.max, "max")
    primed = fast.__dict__["_encoding_cache"][1]
    with torch.no_grad():
        assert fast.get_encodings() is primed  # the key it was stored under is the live one
        want = slow.get_encodings()
        assert_same_bits(primed.scale, want.scale, "scale")
        assert_same_bits(primed.offset, want.offset, "offset")
        fast.invalidate_encoding_cache()
        again = fast.get_encodings()
        assert_same_bits(again.scale, primed.scale, "scale derived afresh")
        assert_same_bits(again.offset, primed.offset, "offset derived afresh")
    # the oracle's analyzer on the same statistics
    steps = (qmax - qmin) - (1 if zps else 0)
    mn = torch.minimum(x.amin(dim=1, keepdim=True), (x * 0.5).amin(dim=1, keepdim=True)).cpu()
    mx = torch.maximum(x.amax(dim=1, keepdim=True), (x * 0.5).amax(dim=1, keepdim=True)).cpu()
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        lo, hi = O.minmax_encodings(mn, mx, steps, symmetric)
    # (+ 0.0: which zero the minimum of a row holding both +0 and -0 is depends on the order of the reduction)
    assert_same_bits(fast.min.detach() + 0.0, lo.to(param_dtype) + 0.0, "min against the oracle")
    assert_same_bits(fast.max.detach() + 0.0, hi.to(param_dtype) + 0.0, "max against the oracle")


PARAM_CALIBRATION_CASES = {
    # tensor shape, quantizer shape, block size, (qmin, qmax, symmetric, zero-point shift)
    "blocks_of_64_4bit": ((96, 256), (96, 4), (1, 64), (-8, 7, True, None)),
    "blocks_of_16_shifted_2bit": ((33, 64), (33, 4), (1, 16), (-2, 1, True, 0.5)),
    "per_row_8bit": ((130, 77), (130, 1), None, (-128, 127, True, None)),
    "per_tensor_8bit_asymmetric": ((57, 129), (), None, (0, 255, False, None)),
    "per_tensor_16bit_asymmetric": ((57, 129), (1,), None, (0, 65535, False, None)),
    "blocks_asymmetric": ((64, 128), (64, 2), (1, 64), (0, 15, False, None)),
    "blocks_along_rows": ((128, 40), (4, 40), (32, 1), (-8, 7, True, None)),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("param_dtype", [torch.float32, torch.bfloat16], ids=["f32_params", "bf16_params"])
@pytest.mark.parametrize("case", list(PARAM_CALIBRATION_CASES), ids=str)
def test_parameter_calibration_and_first_quantization_in_one_call(device, case, dtype, param_dtype):
    """_calibrate_and_quantize (ahq_minmax_calibrate_qdq) against the two steps it stands for -- calibrate on the
    parameter, then call the quantizer on it: min / max, scale, offset and the quantize-dequantized parameter bit for
    bit, the encodings left in the cache are the ones the next forward pass uses, and the result against the oracle's
    quantize-dequantize with those encodings."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    xshape, qshape, block, (qmin, qmax, symmetric, zps) = PARAM_CALIBRATION_CASES[case]
    g = torch.Generator().manual_seed(len(case))
    w = (torch.randn(xshape, generator=g) * torch.logspace(-3, 1, xshape[0]).view(-1, 1)).to(dtype)
    w[0, :3] = 0.0
    wd = torch.nn.Parameter(w.to(device))

    def make():
        return QuantizeDequantize(qshape, qmin=qmin, qmax=qmax, symmetric=symmetric, block_size=block,
                                  zero_point_shift=zps).to(device=device, dtype=param_dtype)

    one, two = make(), make()
    with torch.no_grad():
        y1 = one._calibrate_and_quantize(wd)
        assert y1 is not None
        two._calibrate_on(wd)
        y2 = two(wd)
        assert type(y1) is type(y2) and y1.shape == y2.shape and y1.dtype == y2.dtype
        assert_same_bits(one.min, two.min, "min")
        assert_same_bits(one.max, two.max, "max")
        assert_same_bits(y1.as_subclass(torch.Tensor), y2.as_subclass(torch.Tensor), "quantize-dequantized parameter")
        assert_same_bits(y1.encoding.scale, y2.encoding.scale, "scale")
        assert_same_bits(y1.encoding.offset, y2.encoding.offset, "offset")
        assert one.is_initialized() and one.get_encodings() is y1.encoding
        assert one.encoding_analyzer.observer.get_stats().min is None  # nothing is left behind in the analyzer
        again = one(wd)
        assert_same_bits(again.as_subclass(torch.Tensor), y1.as_subclass(torch.Tensor), "next forward pass")
    scale, offset = y1.encoding.scale.cpu(), y1.encoding.offset.cpu()
    if block is None and (len(qshape) == 0 or math.prod(qshape) == 1 or symmetric):
        ref = O.qdq_v1(w, scale, offset, qmin, qmax)[0]
    else:
        ref = O.qdq_v2_forward(w, scale, offset, qmin, qmax, block, zero_point_shift=zps or 0.0).y
    assert_same_bits(y1.as_subclass(torch.Tensor).cpu(), ref, "against the oracle")
    # a second calibration reuses the plan and follows a changed parameter
    with torch.no_grad():
        wd.mul_(0.5)
        y3 = one._calibrate_and_quantize(wd)
        two._calibrate_on(wd)
        assert_same_bits(one.min, two.min, "min after the parameter changed")
        assert_same_bits(y3.as_subclass(torch.Tensor), two(wd).as_subclass(torch.Tensor), "after the parameter changed")


def test_parameter_calibration_in_one_call_steps_aside(device):
    """The cases _calibrate_and_quantize leaves to the two-step form, with nothing touched."""
    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization.encoding_analyzer import SqnrEncodingAnalyzer

    w = torch.randn(32, 64, device=device)

    def untouched(q, x=w, grad=False):
        with torch.set_grad_enabled(grad):
            out = q._calibrate_and_quantize(x)
        return out is None and not q.is_initialized()

    base = dict(bitwidth=4, symmetric=True, block_size=(1, 16))
    assert untouched(QuantizeDequantize((32, 4), **base).to(device), grad=True)
    hooked = QuantizeDequantize((32, 4), **base).to(device)
    hooked.register_forward_hook(lambda m, a, o: None)
    assert untouched(hooked)

    class Mine(QuantizeDequantize):
        pass

    assert untouched(Mine((32, 4), **base).to(device))
    assert untouched(QuantizeDequantize((32, 1), 8, symmetric=False).to(device))  # per row, asymmetric
    sq = QuantizeDequantize((32, 4), encoding_analyzer=SqnrEncodingAnalyzer((32, 4), block_size=(1, 16)), **base)
    assert untouched(sq.to(device))
    frozen = QuantizeDequantize((32, 4), **base).to(device)
    frozen.allow_overwrite(False)
    assert untouched(frozen)
    assert untouched(QuantizeDequantize((32, 4), **base).to(device), x=w.t())          # not contiguous
    assert untouched(QuantizeDequantize((32, 4), **base).to(device), x=w.double())
    assert untouched(QuantizeDequantize((32, 4), **base).to(device), x=w[:, :60].contiguous())  # shape does not fit
    with torch.no_grad():
        assert QuantizeDequantize((32, 4), **base).to(device)._calibrate_and_quantize(w) is not None


@pytest.mark.parametrize("stat_dtype", [torch.float32, torch.float16, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("param_dtype", [torch.float32, torch.bfloat16], ids=["f32_params", "bf16_params"])
@pytest.mark.parametrize("grid", [(0, 255, False), (-128, 127, True), (0, 65535, False), (-2, 1, True)], ids=str)
@pytest.mark.parametrize("special", [None, "nan", "inf", "zeros"])
def test_end_of_a_per_tensor_calibration_straight_from_the_slots(device, monkeypatch, stat_dtype, param_dtype, grid,
                                                                 special):
    """A per-tensor quantizer that observed its batches through observe_and_clone() leaves the calibration with one
    launch that folds the observer's slots itself (ahq_minmax_slots_finalize): same min / max / scale / offset as
    folding first (ahq_minmax_slots_read + ahq_minmax_finalize), the observer's statistics are still there for whoever
    asks, and they are the extrema of everything seen."""
    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization.encoding_analyzer import _MinMaxObserver

    qmin, qmax, symmetric = grid
    g = torch.Generator().manual_seed(17)
    batches = [torch.randn(3, 70001, generator=g) * s_ for s_ in (1.0, 3.0, 0.2)]
    if special == "nan":
        batches[1][2, 5] = float("nan")
    elif special == "inf":
        batches[0][0, 0], batches[2][1, 1] = float("inf"), -float("inf")
    elif special == "zeros":
        batches = [torch.zeros(3, 1000) for _ in range(3)]
    batches = [b.to(stat_dtype).to(device) for b in batches]

    def calibrated(from_slots: bool):
        q = QuantizeDequantize((), qmin=qmin, qmax=qmax, symmetric=symmetric).to(device=device, dtype=param_dtype)
        seen = []
        real = _MinMaxObserver.live_slots
        monkeypatch.setattr(_MinMaxObserver, "live_slots",
                            (lambda self: seen.append(real(self)) or seen[-1]) if from_slots else (lambda self: None))
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            with torch.no_grad(), q._compute_encodings(passthrough=True):
                for b in batches:
                    assert_same_bits(q(b), b, "pass-through copy")
        monkeypatch.undo()
        assert (len(seen) == 1 and seen[0] is not None) if from_slots else not seen
        return q

    fast, slow = calibrated(True), calibrated(False)
    assert_same_bits(fast.min, slow.min, "min")
    assert_same_bits(fast.max, slow.max, "max")
    with torch.no_grad():
        assert_same_bits(fast.get_encodings().scale, slow.get_encodings().scale, "scale")
        assert_same_bits(fast.get_encodings().offset, slow.get_encodings().offset, "offset")
    stats = fast.encoding_analyzer.observer.get_stats()
    everything = torch.cat([b.flatten() for b in batches])
    assert_same_bits(stats.min, everything.amin(), "the observer's minimum, read afterwards")
    assert_same_bits(stats.max, everything.amax(), "the observer's maximum, read afterwards")


STEADY_CASES = {
    "per_tensor_asymmetric": ((3, 64, 96), (), None, dict(bitwidth=16, symmetric=False)),
    "per_tensor_symmetric": ((3, 64, 96), (1,), None, dict(bitwidth=8, symmetric=True)),
    "per_row_symmetric": ((48, 200), (48, 1), None, dict(bitwidth=8, symmetric=True)),
    "per_row_asymmetric": ((48, 200), (48, 1), None, dict(bitwidth=8, symmetric=False)),   # offsets known to be in the grid
    "blocks_4bit": ((48, 256), (48, 4), (1, 64), dict(bitwidth=4, symmetric=True)),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", list(STEADY_CASES), ids=str)
def test_repeated_forward_without_gradients_reuses_the_previous_call(device, monkeypatch, case, dtype):
    """From the third identical call on, a forward pass without gradients is the library call alone
    (_forward_steady): same bits as the step-by-step form; a changed range, another shape, a strided input or a
    wanted gradient go back to it; copies of the quantizer work."""
    import copy

    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization.affine import quantizer as Q

    xshape, qshape, block, kw = STEADY_CASES[case]
    g = torch.Generator().manual_seed(21)
    x = (torch.randn(xshape, generator=g) * 3).to(dtype).to(device)
    q = QuantizeDequantize(qshape, block_size=block, **kw).to(device)
    with torch.no_grad(), q.compute_encodings():
        q(x)
    planned = True
    q.__dict__.pop("_forward_seen", None)  # (the calibration pass has already shown the shape once)
    calls = []
    real = Q.quantize_dequantize
    monkeypatch.setattr(Q, "quantize_dequantize", lambda *a, **k: calls.append(1) or real(*a, **k))
    with torch.no_grad():
        first, second, third = q(x), q(x), q(x)
        assert len(calls) == (2 if planned else 3)
        assert ("_forward_plan" in q.__dict__) == planned
        assert type(third) is type(first) and third.encoding is first.encoding
        assert_same_bits(second.as_subclass(torch.Tensor), first.as_subclass(torch.Tensor), "second call")
        assert_same_bits(third.as_subclass(torch.Tensor), first.as_subclass(torch.Tensor), "third call")
        other = torch.randn(xshape, generator=g).to(dtype).to(device)
        want = real(other, first.encoding.scale, first.encoding.offset, q.qmin, q.qmax, block_size=q.block_size)
        assert_same_bits(q(other).as_subclass(torch.Tensor), want, "other values, same shape")
        n = len(calls)
        # a strided input of the same shape, and another shape: the step-by-step form
        strided = torch.empty(xshape[:-1] + (2 * xshape[-1],), dtype=dtype, device=device)[..., ::2].copy_(x)
        assert_same_bits(q(strided).as_subclass(torch.Tensor), first.as_subclass(torch.Tensor), "strided input")
        assert len(calls) == n + 1
        if block is None and len(qshape) < 2:
            q(x[:2])
            assert len(calls) == n + 2
        # a new range is followed
        q.set_range(q.min * 0.5, q.max * 0.5)
        n = len(calls)
        moved = q(x)
        assert len(calls) == n + 1
        fresh = QuantizeDequantize(qshape, block_size=block, **kw).to(device)
        fresh.set_range(q.min, q.max)
        assert_same_bits(moved.as_subclass(torch.Tensor), fresh(x).as_subclass(torch.Tensor), "after set_range")
        q(x)
        clone = copy.deepcopy(q)
        assert_same_bits(clone(x).as_subclass(torch.Tensor), moved.as_subclass(torch.Tensor), "deep copy")
        assert_same_bits(q(x).as_subclass(torch.Tensor), moved.as_subclass(torch.Tensor), "steady again")
        # grid and layout outlive new encodings (a calibration between two forward passes)
        for passthrough in (True, False):
            with q._compute_encodings(passthrough=passthrough):
                q(x * 4)
            n = len(calls)
            wider = q(x)
            assert len(calls) == (n if planned else n + 1)
        fresh = QuantizeDequantize(qshape, block_size=block, **kw).to(device)
        fresh.set_range(q.min, q.max)
        assert_same_bits(wider.as_subclass(torch.Tensor), fresh(x).as_subclass(torch.Tensor), "new range, old plan")
        # precomputed encodings (inference mode) go the same way
        n = len(calls)
        with q._precompute_encodings(dtype=torch.float32):
            held = q(x)
            assert held.encoding is q.get_encodings()
        assert len(calls) == (n if planned else n + 1)
        assert_same_bits(held.as_subclass(torch.Tensor), wider.as_subclass(torch.Tensor), "precomputed encodings")
        assert wider.encoding is q.get_encodings() and wider.encoding is not moved.encoding
    # gradients wanted: the autograd forms
    xg = x.clone().requires_grad_(True)
    out = q(xg)
    assert out.requires_grad
    out.sum().backward()
    assert xg.grad is not None


@pytest.mark.parametrize("qshape,block", [((16, 1), None), ((16, 4), (1, 8)), ((), None)])
def test_copy_and_pickle_after_passthrough_calibration(device, qshape, block):
    """A quantizer (and so a whole model) is deep-copied and pickled after calibration: the observer's kept call state
    must survive both, and the twins must go on working."""
    import copy
    import pickle

    from aimet_amd.quantization.affine import QuantizeDequantize

    g = torch.Generator().manual_seed(21)
    x = torch.randn(16, 32, generator=g).to(device)
    q = QuantizeDequantize(qshape, 8, True, block_size=block).to(device)
    with q._compute_encodings(passthrough=True):
        for k in range(3):  # the third call is the one that reuses the kept state
            out = q(x * (k + 1))
            assert_same_bits(out, x * (k + 1), "pass-through")
    want = q(x).as_subclass(torch.Tensor)
    for twin in (copy.deepcopy(q), pickle.loads(pickle.dumps(q))):
        assert twin.is_initialized()
        assert_same_bits(twin(x).as_subclass(torch.Tensor), want, "twin forward")
        with twin._compute_encodings(passthrough=True):
            for k in range(3):
                twin(x * (k + 4))
        assert_same_bits(twin.max, q.max * 2, "twin calibrates on its own")
    assert_same_bits(q(x).as_subclass(torch.Tensor), want, "original untouched")


def test_range_warnings_of_the_fused_calibration_end(device):
    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization.encoding_analyzer import deferred_range_warnings

    def run(value, deferred):
        q = QuantizeDequantize((), 8, symmetric=False).to(device)
        x = torch.full((64,), value, device=device)
        with torch.no_grad():
            if deferred:
                with deferred_range_warnings():
                    with q._compute_encodings(passthrough=True):
                        q(x)
            else:
                with q._compute_encodings(passthrough=True):
                    q(x)

    for deferred in (False, True):
        with pytest.warns(UserWarning, match="Infinite or NaN"):
            run(float("nan"), deferred)  # an infinite statistic is clamped to the largest finite value first
        with pytest.warns(UserWarning, match="Extreme values"):
            run(3.3e38, deferred)
        with warnings.catch_warnings():
            warnings.simplefilter("error")
            run(1.0, deferred)


def test_lpbq_training_step_with_the_fused_scale_node(device):
    """A training step of an LPBQ quantizer with learned ranges: with the block scales from the one-launch autograd
    node (_LpbqScale) output and input gradient equal those of the step-by-step composition bit for bit, and the
    min / max gradients agree to the tolerance of the per-group sums (double precision against float32)."""
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize

    g = torch.Generator().manual_seed(8)
    w = (torch.randn(96, 512, generator=g) * 0.02).bfloat16().to(device)
    grad = torch.randn(96, 512, generator=g).bfloat16().to(device)

    def run(fused: bool):
        q = GroupedBlockQuantizeDequantize(shape=(96, 8), bitwidth=4, symmetric=True, decompressed_bw=8,
                                           block_size=(1, 64), block_grouping=(1, -1)).to(device)
        with q.compute_encodings():
            q(w)
        if not fused:
            q.__dict__["_lpbq_unsupported"] = ((96, 8), (1, -1))  # what a grouping the library declines leaves behind
        name = type(q.get_encodings().scale.grad_fn).__name__
        assert name.startswith("_LpbqScale") == fused
        wd = w.clone().requires_grad_(True)
        y = q(wd)
        y.backward(grad)
        return y.detach(), wd.grad, q.min.grad, q.max.grad

    a, b = run(True), run(False)
    assert_same_bits(a[0], b[0], "output")
    assert_same_bits(a[1], b[1], "input gradient")
    assert_close_rel(a[2], b[2], 1e-5, "gradient of min", abs_floor=1e-30)
    assert_close_rel(a[3], b[3], 1e-5, "gradient of max", abs_floor=1e-30)
    assert float(a[2].abs().sum()) > 0 and float(a[3].abs().sum()) > 0


class _OracleScaleQdq(torch.autograd.Function):
    """The reference's quantize-dequantize with its hand-written backward (torch_builtins.py:727-831), on the CPU."""

    @staticmethod
    def forward(ctx, x, scale, qmin, qmax, block):
        ctx.save_for_backward(x, scale)
        ctx.args = (qmin, qmax, block)
        return O.qdq_v2_forward(x.detach(), scale.detach(), torch.zeros_like(scale), qmin, qmax, block).y

    @staticmethod
    def backward(ctx, g):
        x, scale = ctx.saved_tensors
        qmin, qmax, block = ctx.args
        gx, gs, _ = O.qdq_v2_backward(g, x.detach(), scale.detach(), torch.zeros_like(scale), qmin, qmax, block)
        return gx, gs.view(scale.shape), None, None, None


@pytest.mark.parametrize("case", [
    ((96, 8), (1, -1), 16),           # C4's grouping
    ((40, 12), (1, 4), 16),           # groups of four neighbouring blocks
    ((6, 130), (1, -1), 256),         # groups longer than a wave, 8 extra bits
    ((10, 64, 1, 1), (1, 64, 1, 1), 16),
], ids=["rows", "fours", "long_groups", "conv"])
@pytest.mark.parametrize("param_dtype", [torch.float32, torch.bfloat16], ids=["f32_params", "bf16_params"])
def test_lpbq_learned_range_gradients_in_one_launch(device, case, param_dtype):
    """ahq_lpbq_scale_backward against the CPU: autograd through get_scale, torch.amax and the division, and the
    reference's own backward formulas for the quantize-dequantize of the block scales.  The per-group sum is taken
    in double precision here and in float32 there: 1e-5 relative, as for every scale gradient; ties for the group
    maximum, ranges below the minimum scale and reversed ranges included."""
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize
    from aimet_amd.quantization.affine import quantizer as Q

    shape, grouping, mult = case
    bw = 4
    dbw = bw + {16: 4, 256: 8}[mult]
    g = torch.Generator().manual_seed(13)
    hi = (torch.rand(shape, generator=g) * 0.1 + 1e-3)
    hi.view(-1)[::5] *= 7.0
    hi.view(-1)[3] = 0.0                      # below the minimum scale
    lo = -hi * (8.0 / 7.0)
    lo.view(-1)[7], hi.view(-1)[7] = hi.view(-1)[7].clone(), lo.view(-1)[7].clone()   # reversed range
    flat = hi.view(shape[0], -1)
    flat[1, 1] = flat[1].max()                # two members attain the group maximum
    lo.view(shape[0], -1)[1, 1] = -flat[1, 1] * (8.0 / 7.0)
    j = int(flat[1].argmax())
    lo.view(shape[0], -1)[1, j] = -flat[1, j] * (8.0 / 7.0)
    lo, hi = lo.to(param_dtype), hi.to(param_dtype)
    up = torch.randn(shape, generator=g)

    # CPU: the reference's composition
    mn_c, mx_c = lo.clone().requires_grad_(True), hi.clone().requires_grad_(True)
    raw = ((mx_c.to(torch.float32) - mn_c.to(torch.float32)) / 15).abs().clamp_min_(O.minimum_scale(15))
    pcs_shape = [d // gsz if gsz != -1 else 1 for d, gsz in zip(shape, grouping)]
    cg = O.concrete_block_size(shape, pcs_shape, grouping)
    resh = raw.reshape(*O.interleave(pcs_shape, cg))
    pcs = torch.amax(resh, dim=tuple(range(1, resh.dim(), 2))) / mult
    snapped = _OracleScaleQdq.apply(raw, pcs, 1, mult, grouping)
    (snapped * up).sum().backward()

    q = GroupedBlockQuantizeDequantize(shape=shape, bitwidth=bw, symmetric=True, decompressed_bw=dbw,
                                       block_size=None if len(shape) != 2 else None, block_grouping=grouping)
    q = q.to(device=device, dtype=param_dtype)
    with torch.no_grad():
        q.min.copy_(lo.to(device))
        q.max.copy_(hi.to(device))
    scale = q.get_encodings().scale
    assert type(scale.grad_fn).__name__.startswith("_LpbqScale")
    assert_same_bits(scale, snapped, "LPBQ scale")
    (scale * up.to(device)).sum().backward()
    tol = 1e-5 if param_dtype == torch.float32 else float(torch.finfo(param_dtype).eps)
    assert_close_rel(q.max.grad, mx_c.grad, tol, "gradient of max", abs_floor=1e-30)
    assert_close_rel(q.min.grad, mn_c.grad, tol, "gradient of min", abs_floor=1e-30)
    # and the step-by-step composition on the device gives the same gradients to the same tolerance
    q.min.grad = q.max.grad = None
    q.__dict__["_lpbq_unsupported"] = (tuple(shape), tuple(grouping))
    scale2 = q.get_encodings().scale
    assert not type(scale2.grad_fn).__name__.startswith("_LpbqScale")
    (scale2 * up.to(device)).sum().backward()
    assert_close_rel(q.max.grad, mx_c.grad, tol, "gradient of max, step by step", abs_floor=1e-30)


LPBQ_FORWARD_CASES = [
    # (quantizer shape, block size, block grouping, weight shape)
    ((96, 8), (1, 64), (1, -1), (96, 512)),       # a group is a row of blocks
    ((6, 24), (1, 64), (1, -1), (6, 1536)),       # tiles end inside a group
    ((16, 32), (1, 16), (1, 4), (16, 512)),       # four neighbouring blocks to a group
    ((5, 3), (1, 2), (1, -1), (5, 6)),            # blocks shorter than a vector
    ((8, 6), (4, 4), (2, 3), (32, 24)),           # blocks along two dimensions: two launches
    ((64, 10), (8, 1), (64, 1), (512, 10)),       # groups down a column: two launches
]


@pytest.mark.parametrize("case", LPBQ_FORWARD_CASES, ids=["rows", "split_groups", "fours", "short_blocks",
                                                            "two_dimensional", "column_groups"])
@pytest.mark.parametrize("dtype,param_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                               (torch.float16, torch.float32), (torch.bfloat16, torch.float32)],
                         ids=["f32", "bf16", "f16_f32params", "bf16_f32params"])
def test_lpbq_forward_in_one_launch(device, case, dtype, param_dtype):
    """Without gradients the LPBQ forward pass is one launch (ahq_lpbq_qdq_forward: block scales from min / max,
    snapped to the group's multiples, quantize-dequantize).  Output, block scales and per-channel scales must be the
    oracle's bits, and equal to what the two-launch form (get_encodings(), then quantize_dequantize) gives."""
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize
    from aimet_amd.quantization.affine import quantize_dequantize

    shape, block, grouping, wshape = case
    g = torch.Generator().manual_seed(33)
    w = torch.randn(wshape, generator=g) * 0.05
    w.view(-1)[: w.numel() // 7] *= 30
    q = GroupedBlockQuantizeDequantize(shape=shape, bitwidth=4, symmetric=True, decompressed_bw=8, block_size=block,
                                       block_grouping=grouping).to(device)
    with q.compute_encodings():
        q(w.to(device))
    q.to(param_dtype)
    x = (torch.randn(wshape, generator=g) * 0.08).to(dtype)
    x.view(-1)[-1] = 1e30
    x.view(-1)[0] = float("nan")
    mn, mx = q.min.detach().cpu(), q.max.detach().cpu()
    raw = O.scale_from_minmax(mn.float(), mx.float(), -8, 7)
    scale_ref, pcs_ref = O.lpbq_scale(raw, 4, 8, grouping)
    y_ref = O.qdq_v2_forward(x, scale_ref, torch.zeros_like(scale_ref), -8, 7, block_size=block).y
    with torch.no_grad():
        out = q(x.to(device))
        enc = q.get_encodings()
        two = quantize_dequantize(x.to(device), enc.scale, enc.offset, -8, 7, block_size=block)
    assert type(out).__name__ == "DequantizedTensor" and out.dtype == dtype
    assert_same_bits(out.encoding.scale, scale_ref, "block scales written by the forward launch")
    assert_same_bits(out.encoding.per_channel_scale, pcs_ref, "per-channel scales written by the forward launch")
    assert_same_bits(out.as_subclass(torch.Tensor), y_ref, "output against the oracle")
    assert_same_bits(out.as_subclass(torch.Tensor), two.as_subclass(torch.Tensor), "output against the two-launch form")
    fused = q.__dict__.get("_lpbq_forward_unsupported") is None and q._blocks_per_group() is not None
    assert fused == (case[0] not in ((8, 6), (64, 10)))
    codes = out.quantize()
    assert float(codes.as_subclass(torch.Tensor)[~x.isnan().to(device)].abs().max()) <= 8


def test_lpbq_forward_misaligned_and_refused_layouts(device):
    """ahq_lpbq_qdq_forward on a tensor that is not 16-byte aligned (scalar loads), and its refusals: encodings that
    repeat over a leading dimension, a block count that is no multiple of the group, arithmetic in float32 on a
    16-bit tensor."""
    from aimet_amd import _lib
    from aimet_amd.quantization.affine.backends import hip
    from aimet_amd.quantization._utils import _get_minimum_scale

    lib = _lib.load()
    g = torch.Generator().manual_seed(5)
    base = (torch.randn(16 * 256 + 1, generator=g) * 0.1).to(device)
    x = base[1:].view(16, 256)
    mx = (torch.rand(16, 4, generator=g) + 0.05).to(device)
    mn = -mx
    raw = O.scale_from_minmax(mn.cpu(), mx.cpu(), -8, 7)
    scale_ref, pcs_ref = O.lpbq_scale(raw, 4, 8, (1, -1))
    y_ref = O.qdq_v2_forward(x.cpu(), scale_ref, torch.zeros_like(scale_ref), -8, 7, block_size=(1, 64)).y

    def call(xx, enc_shape, block, group, cd=None, mn_=mn, mx_=mx):
        xd, layout = hip._prepare(xx, enc_shape, block)
        grid = hip._grid(_lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QDQ, xd.dtype, cd or xd.dtype, -8, 7, 0.0)
        y = torch.empty_like(xd)
        scale = torch.empty(enc_shape, dtype=torch.float32, device=device)
        pcs = torch.empty(max(1, scale.numel() // group), dtype=torch.float32, device=device)
        status = lib.ahq_lpbq_qdq_forward(grid, layout, xd.data_ptr(), y.data_ptr(), None, _lib.DTYPE_CODE[mn_.dtype],
                                          mn_.data_ptr(), mx_.data_ptr(), group, _get_minimum_scale(15), 16, None,
                                          scale.data_ptr(), pcs.data_ptr(), _lib.current_stream(device))
        return status, y, scale, pcs

    status, y, scale, pcs = call(x, (16, 4), (1, 64), 4)
    assert status == _lib.AHQ_OK
    assert_same_bits(scale, scale_ref, "scales")
    assert_same_bits(pcs.view(16, 1), pcs_ref, "per-channel scales")
    assert_same_bits(y, y_ref, "output of the scalar-load path")
    x3 = torch.randn(3, 16, 256, generator=g).to(device)
    assert call(x3, (16, 4), (1, 64), 4)[0] == _lib.AHQ_ERR_UNSUPPORTED       # encodings repeat over the leading dimension
    assert call(x.contiguous(), (16, 4), (1, 64), 3)[0] == _lib.AHQ_ERR_UNSUPPORTED   # 64 blocks, groups of 3
    xb = x.contiguous().bfloat16()
    assert call(xb, (16, 4), (1, 64), 4, cd=torch.float32)[0] == _lib.AHQ_ERR_UNSUPPORTED
    assert call(xb, (16, 4), (1, 64), 4)[0] == _lib.AHQ_OK


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("case", [
    ((37, 129), (), None, 8, False),
    ((64, 512), (64, 1), None, 8, True),
    ((32, 256), (32, 4), (1, 64), 4, True),
    ((4, 6, 10, 10), (6, 1, 1), None, 8, False),
    ((16, 64), (16, 1), None, 16, False),
], ids=["per_tensor", "per_channel", "blockwise", "activation_channels", "sixteen_bit"])
def test_forward_with_learned_ranges_as_one_autograd_node(device, monkeypatch, dtype, case):
    """With learned min / max, QuantizeDequantize.forward is one autograd node (_QdqFromRange: scale / offset
    derivation and quantize-dequantize forward, their two backward launches behind it).  Output, input gradient and
    the gradients of min / max must equal, bit for bit, what the two-node form gives -- get_encodings() followed by
    the backend's quantize_dequantize -- also when the loss uses the scale and offset of the encoding the output
    carries."""
    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization.affine.quantizer import QuantizeDequantize as QdqClass

    shape, enc_shape, block, bitwidth, symmetric = case
    g = torch.Generator().manual_seed(17)
    x = (torch.randn(shape, generator=g) * 0.7).to(dtype)
    grad = torch.randn(shape, generator=g).to(dtype)
    q = QuantizeDequantize(enc_shape, bitwidth, symmetric, block_size=block).to(device)
    with q.compute_encodings():
        q(x.to(device) * 0.5)          # narrower ranges than the data: clipped elements carry the range gradients
    w = torch.randn(enc_shape, generator=g).to(device)

    def run(through_encoding):
        xd = x.to(device).requires_grad_(True)
        q.min.grad = q.max.grad = None
        out = q(xd)
        loss = (out.as_subclass(torch.Tensor).float() * grad.to(device).float()).sum()
        if through_encoding:
            loss = loss + (out.encoding.scale * w).sum()
            if not symmetric:
                loss = loss + (out.encoding.offset * w).sum() * 1e-3
        loss.backward()
        return (out.detach().as_subclass(torch.Tensor).clone(), xd.grad.clone(), q.min.grad.clone(), q.max.grad.clone(),
                type(out.encoding.scale.grad_fn).__name__)

    for through_encoding in (False, True):
        one = run(through_encoding)
        assert one[4].startswith("_QdqFromRange")
        with monkeypatch.context() as m:
            m.setattr(QdqClass, "_forward_from_range", lambda self, input: None)
            two = run(through_encoding)
        assert not two[4].startswith("_QdqFromRange")
        for a, b, what in zip(one[:4], two[:4], ("output", "input gradient", "gradient of min", "gradient of max")):
            assert_same_bits(a, b, f"{what} (loss through the encoding: {through_encoding})")
        assert float(one[2].abs().sum()) > 0 and float(one[3].abs().sum()) > 0


@pytest.mark.parametrize("dtype,param_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                               (torch.bfloat16, torch.float32)], ids=["f32", "bf16", "bf16_f32params"])
@pytest.mark.parametrize("case", LPBQ_FORWARD_CASES[:4], ids=["rows", "split_groups", "fours", "short_blocks"])
def test_lpbq_forward_with_gradients_as_one_autograd_node(device, monkeypatch, case, dtype, param_dtype):
    """With gradients wanted the LPBQ forward pass is one autograd node (_LpbqQdqFromRange: ahq_lpbq_qdq_forward, then
    ahq_qdq_backward and ahq_lpbq_scale_backward).  Output, input gradient and the gradients of min / max must equal,
    bit for bit, what the two-node form gives (_LpbqScale, then the backend's quantize_dequantize), also when the loss
    uses the scales of the encoding the output carries."""
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize
    from aimet_amd.quantization.affine.quantizer import GroupedBlockQuantizeDequantize as Cls

    shape, block, grouping, wshape = case
    g = torch.Generator().manual_seed(29)
    w = torch.randn(wshape, generator=g) * 0.05
    w.view(-1)[: w.numel() // 7] *= 30
    q = GroupedBlockQuantizeDequantize(shape=shape, bitwidth=4, symmetric=True, decompressed_bw=8, block_size=block,
                                       block_grouping=grouping).to(device)
    with q.compute_encodings():
        q(w.to(device) * 0.6)
    q.to(param_dtype)
    x = w.to(dtype)
    grad = torch.randn(wshape, generator=g).to(dtype)
    ws = torch.randn(shape, generator=g).to(device)

    def run(through_encoding):
        xd = x.to(device).requires_grad_(True)
        q.min.grad = q.max.grad = None
        out = q(xd)
        loss = (out.as_subclass(torch.Tensor).float() * grad.to(device).float()).sum()
        if through_encoding:
            loss = loss + (out.encoding.scale * ws).sum() + out.encoding.per_channel_scale.sum()
        loss.backward()
        return (out.detach().as_subclass(torch.Tensor).clone(), xd.grad.clone(), q.min.grad.clone(), q.max.grad.clone(),
                type(out.encoding.scale.grad_fn).__name__)

    for through_encoding in (False, True):
        one = run(through_encoding)
        assert one[4].startswith("_LpbqQdqFromRange")
        with monkeypatch.context() as m:
            m.setattr(Cls, "_fused_forward", lambda self, input: None)
            two = run(through_encoding)
        assert two[4].startswith("_LpbqScale")
        for a, b, what in zip(one[:4], two[:4], ("output", "input gradient", "gradient of min", "gradient of max")):
            assert_same_bits(a, b, f"{what} (loss through the encoding: {through_encoding})")
        assert float(one[2].abs().sum()) > 0 and float(one[3].abs().sum()) > 0


# ------------------------------------------------------- quantizers that hold their encoding as scale / offset --
@pytest.mark.parametrize("case", CASES, ids=lambda c: c[0])
def test_scale_offset_parametrisation_forward_backward(device, case):
    """A quantizer reparametrized to (scale, offset) computes what it computed before (same scale, same offset, hence
    the same bits out and the same input gradient), and its gradients reach scale and offset themselves: those are the
    oracle's scale and offset gradients (offset through the straight-through rounding, i.e. unchanged)."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    _, xshape, dtype, qshape, bw, sym, block = case
    g = torch.Generator().manual_seed(5)
    x = torch.randn(xshape, generator=g)
    if not sym:
        x = torch.relu(x)
    x = x.to(dtype)
    grad = torch.randn(xshape, generator=g).to(dtype)
    n = 2 ** bw - 1
    qmin, qmax = (-math.ceil(n / 2), math.floor(n / 2)) if sym else (0, n)

    q = QuantizeDequantize(qshape, bw, sym, block_size=block).to(device)
    xd = x.to(device)
    with q.compute_encodings():
        q(xd)
    scale, offset = q.get_scale().detach().clone(), q.get_offset().detach().clone()
    with torch.no_grad():
        y_min_max = q(xd).clone()
    y_learning = q(xd).detach().clone()  # learned encodings take the composed arithmetic: other bits in 16-bit types
    q._reparametrize_to_scale_offset()
    assert q._is_scale_offset_quantizer() and q.is_initialized() and q.scale.device == xd.device
    assert_same_bits(q.get_scale(), scale, "scale after reparametrizing")
    assert_same_bits(q.get_offset(), offset, "offset after reparametrizing")
    with torch.no_grad():
        assert_same_bits(q(xd), y_min_max, "forward without gradients")

    xg = xd.clone().requires_grad_(True)
    y = q(xg)
    assert type(y).__name__ == "DequantizedTensor"
    assert_same_bits(y, y_learning, "forward with gradients")
    y.backward(grad.to(device))
    sc, of = scale.cpu(), offset.cpu()
    ref_y = O.qdq_v2_forward(x, sc, of, qmin, qmax, block, 0.0).y
    assert_same_bits(y, ref_y, "forward against the oracle")
    gx, gs, go = O.qdq_v2_backward(grad, x, sc, of, qmin, qmax, block, 0.0)
    assert_same_bits(xg.grad, gx, "input gradient")
    D = O.internal_dtype(dtype, qmin, qmax)
    # float32: up to 25088 signed terms per encoding, summed in two different orders and cancelling to a few percent
    # of their absolute sum -- 4e-5 of the result is a few units in the last place of that absolute sum
    tol = 4e-5 if D == torch.float32 else float(torch.finfo(D).eps)
    assert_close_rel(q.scale.grad, gs.view(qshape), tol, "scale gradient", abs_floor=1e-30)
    if sym:
        assert q.offset is None
    else:
        assert_close_rel(q.offset.grad, go.view(qshape), tol, "offset gradient", abs_floor=1e-30)

    # calibrating again goes through set_range(): the same encodings as a min/max quantizer finds
    fresh = QuantizeDequantize(qshape, bw, sym, block_size=block).to(device)
    fresh._reparametrize_to_scale_offset()
    with fresh.compute_encodings():
        fresh(xd)
    assert_same_bits(fresh.get_scale(), scale, "scale of a calibrated scale/offset quantizer")
    assert_same_bits(fresh.get_offset(), offset, "offset of a calibrated scale/offset quantizer")
    q._reparametrize_to_min_max()
    with torch.no_grad():
        assert_same_bits(q(xd), y_min_max, "forward after reparametrizing back")


@pytest.mark.parametrize("params", ["min_max", "scale_offset"])
def test_import_signed_flag(device, params):
    """Reference expectation: test_affine_quantizer.py:1592-1627."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    symmetric_quantizer = QuantizeDequantize((1,), 8, symmetric=True).to(device)
    asymmetric_quantizer = QuantizeDequantize((1,), 8, symmetric=False).to(device)
    if params == "scale_offset":
        symmetric_quantizer._reparametrize_to_scale_offset()
        asymmetric_quantizer._reparametrize_to_scale_offset()
    assert symmetric_quantizer.signed
    g = torch.Generator().manual_seed(0)
    with symmetric_quantizer.compute_encodings():
        symmetric_quantizer(torch.randn(10, generator=g).to(device))
    asymmetric_quantizer.set_legacy_encodings(symmetric_quantizer.get_legacy_encodings())
    assert asymmetric_quantizer.signed and asymmetric_quantizer.symmetric
    x = torch.randn(10, generator=g).to(device)
    assert_same_bits(asymmetric_quantizer(x), symmetric_quantizer(x), "the same encodings after the import")

    asymmetric_quantizer = QuantizeDequantize((), 8, symmetric=False).to(device)
    if params == "scale_offset":
        asymmetric_quantizer._reparametrize_to_scale_offset()
    with asymmetric_quantizer.compute_encodings():
        asymmetric_quantizer(torch.randn(10, generator=g).to(device))
    symmetric_quantizer.set_legacy_encodings(asymmetric_quantizer.get_legacy_encodings())
    assert not symmetric_quantizer.signed and not symmetric_quantizer.symmetric


def test_grouped_block_quantizer_held_as_scale_offset(device):
    from aimet_amd.quantization.affine import GroupedBlockQuantizeDequantize

    g = torch.Generator().manual_seed(3)
    w = torch.randn(16, 256, generator=g).to(device)
    q = GroupedBlockQuantizeDequantize((16, 8), 4, True, 8, block_size=(1, 32), block_grouping=(1, 8)).to(device)
    with q.compute_encodings():
        q(w)
    scale, per_channel = q.get_scale().clone(), q.get_per_channel_scale().clone()
    with torch.no_grad():
        y = q(w).clone()
    q._reparametrize_to_scale_offset()
    assert_same_bits(q.get_scale(), scale, "snapped block scales")
    assert_same_bits(q.get_per_channel_scale(), per_channel, "per-channel scales")
    with torch.no_grad():
        assert_same_bits(q(w), y, "forward without gradients")
    wg = w.clone().requires_grad_(True)
    out = q(wg)
    assert_same_bits(out, y, "forward with gradients")
    out.sum().backward()
    assert q.scale.grad is not None and torch.isfinite(q.scale.grad).all()


def test_model_calibration_with_a_scale_offset_parameter_quantizer(device):
    """The batched calibration of a whole model leaves a quantizer held as scale / offset to the generic route; its
    encodings come out as those of its min/max twin."""
    import copy as _copy

    import aimet_amd.nn as qnn
    from aimet_amd.quantization.affine import QuantizeDequantize

    torch.manual_seed(0)

    def build():
        lin = qnn.QuantizedLinear(64, 32, bias=False).to(device)
        lin.param_quantizers["weight"] = QuantizeDequantize((32, 1), 8, True).to(device)
        lin.input_quantizers[0] = QuantizeDequantize((), 8, False).to(device)
        lin.output_quantizers[0] = QuantizeDequantize((), 8, False).to(device)
        return lin

    a = build()
    b = _copy.deepcopy(a)
    for qz in (b.param_quantizers["weight"], b.input_quantizers[0]):
        qz._reparametrize_to_scale_offset()
    x = torch.randn(8, 64, device=device)
    for m in (a, b):
        with qnn.compute_encodings(m):
            m(x)
    for qa, qb in ((a.param_quantizers["weight"], b.param_quantizers["weight"]),
                   (a.input_quantizers[0], b.input_quantizers[0]), (a.output_quantizers[0], b.output_quantizers[0])):
        assert qb.is_initialized()
        assert_same_bits(qb.get_scale(), qa.get_scale(), "scale")
        assert_same_bits(qb.get_offset(), qa.get_offset(), "offset")
    assert b.param_quantizers["weight"]._is_scale_offset_quantizer()
    with torch.no_grad():
        assert_same_bits(b(x), a(x), "layer output")


@pytest.mark.parametrize("symmetric", [True, False])
def test_quantize_held_as_scale_offset(device, symmetric):
    """Quantize (integer codes out) with its encoding held as scale / offset: the codes, the dequantized values and
    the gradients of scale and offset are those of the oracle at the same scale and offset."""
    from aimet_amd.quantization.affine import Quantize

    g = torch.Generator().manual_seed(8)
    x = torch.randn(12, 40, generator=g)
    if not symmetric:
        x = torch.relu(x)
    grad = torch.randn(12, 40, generator=g)
    q = Quantize((12, 1), 8, symmetric).to(device)
    with q.compute_encodings():
        q(x.to(device))
    scale, offset = q.get_scale().detach().cpu(), q.get_offset().detach().cpu()
    q._reparametrize_to_scale_offset()
    xd = x.to(device).requires_grad_(True)
    out = q(xd)
    assert type(out).__name__ == "QuantizedTensor"
    qmin, qmax = (-128, 127) if symmetric else (0, 255)
    codes = torch.clamp(torch.round(x / scale) - offset, qmin, qmax)  # torch_builtins.py:588-632 on the CPU
    assert_same_bits(out, codes, "codes")
    assert_same_bits(out.dequantize(), (codes + offset) * scale, "dequantized codes")
    out.backward(grad.to(device))
    # plain autograd of clamp(round_ste(x / s) - o, qmin, qmax)
    s = scale.clone().requires_grad_(True)
    o = offset.clone().requires_grad_(True)
    xr = x.clone().requires_grad_(True)
    t = xr / s
    ref = torch.clamp(t + (torch.round(t) - t).detach() - o, qmin, qmax)
    ref.backward(grad)
    assert_same_bits(xd.grad, xr.grad, "input gradient")
    assert_close_rel(q.scale.grad, s.grad, 1e-5, "scale gradient", abs_floor=1e-30)
    if not symmetric:
        assert_close_rel(q.offset.grad, o.grad, 1e-5, "offset gradient", abs_floor=1e-30)


def test_blockwise_encoding_read_as_a_grouped_one(device):
    """GroupedBlockEncoding._from_affine_encoding (encoding.py:686-735): block scales that ARE integer multiples of a
    per-channel scale convert (with the same scales, the grouping along the block axis and twice the bitwidth);
    scales that are not, asymmetric and per-channel encodings are refused."""
    from aimet_amd.quantization.affine import AffineEncoding, GroupedBlockEncoding

    per_channel = torch.tensor([[0.01], [0.02], [0.04]], device=device)
    multipliers = torch.tensor([[16.0, 3.0, 7.0, 1.0], [16.0, 16.0, 2.0, 9.0], [5.0, 16.0, 11.0, 4.0]], device=device)
    scale = per_channel * multipliers  # 4-bit grid, 8-bit expansion: multipliers 1..16, the largest one is 16
    enc = AffineEncoding(scale, torch.zeros_like(scale), -8, 7, True, (1, 32))._hint_input_shape((3, 128))
    lpbq = GroupedBlockEncoding._from_affine_encoding(enc)
    assert isinstance(lpbq, GroupedBlockEncoding)
    assert lpbq.block_grouping == (1, 4) and lpbq.decompressed_bw == 8 and lpbq.bitwidth == 4
    assert torch.allclose(lpbq.scale, scale) and torch.allclose(lpbq.per_channel_scale, per_channel)
    assert torch.equal(lpbq.per_block_int_scale.float(), multipliers)
    assert GroupedBlockEncoding._from_affine_encoding(lpbq) is lpbq
    exported = lpbq.to_qnn_encoding_dict("2.0.0")
    assert exported["per_block_int_scale"] == multipliers.int().tolist()

    off_grid = AffineEncoding(scale * torch.tensor([[1.0, 1.03, 1.0, 1.0]], device=device), torch.zeros_like(scale), -8, 7,
                              True, (1, 32))._hint_input_shape((3, 128))
    with pytest.raises(ValueError, match="Failed to interpret"):
        GroupedBlockEncoding._from_affine_encoding(off_grid)
    with pytest.raises(ValueError, match="blockwise"):
        GroupedBlockEncoding._from_affine_encoding(AffineEncoding(per_channel, torch.zeros_like(per_channel), -8, 7, True))
    with pytest.raises(ValueError, match="symmetric"):
        GroupedBlockEncoding._from_affine_encoding(
            AffineEncoding(scale, torch.full_like(scale, -3.0), 0, 15, False, (1, 32))._hint_input_shape((3, 128)))
    with pytest.raises(ValueError, match="Only AffineEncoding"):
        GroupedBlockEncoding._from_affine_encoding(object())


def test_asymmetric_per_channel_forward_needs_no_device_read(device):
    """The offsets an asymmetric min/max quantizer derives are clamped into the grid, and say so: the backend takes the
    ATen arithmetic for a no-grad forward without reading them back (a synchronisation per forward otherwise).  The
    result is what the reference's fast path gives, bit for bit; offsets of unknown origin are still read."""
    from aimet_amd.quantization.affine import QuantizeDequantize
    from aimet_amd.quantization.affine.backends import hip

    g = torch.Generator().manual_seed(5)
    x = (torch.randn(4, 64, 96, generator=g) * 2 + 0.7)
    q = QuantizeDequantize((64, 1), 8, symmetric=False).to(device)
    with q.compute_encodings():
        q(x.to(device))
    with torch.no_grad():
        enc = q.get_encodings()
    assert getattr(enc.offset, "_ahq_in_grid", None) == (q.qmin, q.qmax)
    reads = []
    real = hip._offsets_fit_grid  # pylint: disable=protected-access

    def counting(offset, qmin, qmax):
        reads.append(getattr(offset, "_ahq_in_grid", None) is None and getattr(offset, "_ahq_constant", None) is None)
        return real(offset, qmin, qmax)

    hip._offsets_fit_grid = counting  # pylint: disable=protected-access
    try:
        with torch.no_grad():
            y = q(x.to(device))
            y2 = q(x.to(device))
            y3 = q(x.to(device))
    finally:
        hip._offsets_fit_grid = real  # pylint: disable=protected-access
    assert not any(reads), "an offset derived from min / max was read back from the device"
    ref = O.qdq_v1(x, enc.scale.detach().cpu(), enc.offset.detach().cpu(), q.qmin, q.qmax)
    assert ref is not None
    for out in (y, y2, y3):
        assert_same_bits(out.as_subclass(torch.Tensor), ref[0], "no-grad forward")
    # a plain tensor of offsets is still checked by reading it -- once per version of its contents
    off = enc.offset.detach().clone()
    assert getattr(off, "_ahq_in_grid", None) is None
    assert real(off, q.qmin, q.qmax) is True
    assert real(off - 1000.0, q.qmin, q.qmax) is False
    assert off._ahq_fit_checked[1] is True  # pylint: disable=protected-access
    off.sub_(1000.0)  # a tracked write: the kept answer no longer applies
    assert real(off, q.qmin, q.qmax) is False
    off.add_(1000.0)
    assert real(off, q.qmin, q.qmax) is True
