"""Parity of the HIP quantize / dequantize / quantize-dequantize kernels with the CPU oracle.

Bar: outputs and input gradients bit-exact; scale/offset gradients (order-sensitive sums) within 1e-5 relative in
fp32 arithmetic and within one unit in the last place of the compute dtype for 16-bit arithmetic.
"""

import math

import pytest
import torch

from oracle import torch_ref as O
from tests.helpers import assert_same_bits, assert_close_rel

pytestmark = pytest.mark.gpu

# (tensor shape, encoding shape, block_size)
LAYOUTS = [
    ((37, 129), (), None),                 # per-tensor, ragged tail
    ((4, 8, 16, 16), (1,), None),          # per-tensor, shape (1,)
    ((1024, 1030), (), None),              # per-tensor, many tiles (last-workgroup reduction)
    ((64, 4096), (64, 1), None),           # per-channel, one tile per row
    ((16, 5000), (16, 1), None),           # per-channel, two tiles per row
    ((8, 100), (8, 1), None),              # per-channel, rows shorter than a tile (atomic reduction)
    ((8, 128), (8, 1), None),              # per-channel, power-of-two run inside a wave
    ((4, 6, 10, 10), (6, 1, 1), None),     # activation per-channel (I > 1)
    ((2, 3, 64, 64), (3, 1, 1), None),     # activation per-channel, long runs
    ((32, 256), (32, 4), (1, 64)),         # blockwise along the input dimension
    ((3, 32, 256), (32, 4), (1, 64)),      # blockwise with a leading broadcast dimension
    ((8, 16), (2, 4), (4, 4)),             # two-dimensional blocks (generic walk)
    ((10, 12), (12,), None),               # per-channel on the fastest axis
    ((6, 10), (6, 1), None),               # run length not a multiple of the vector width
    ((5, 7, 64), (5, 1, 2), (1, -1, -1)),  # wildcard block sizes
    ((70, 256), (256,), None),             # run length 1 over whole vectors: column-walking kernels
    ((1100, 264), (1, 264), None),         # same, many rows per workgroup, lanes without columns
    ((1100, 24), (1, 24), None),           # too few columns for them: tiled kernel
    ((3, 40, 1536), (1536,), None),        # same, several groups of 64 lanes across
    ((300, 24), (300, 1), None),           # whole runs per workgroup, one thread adds a run
    ((37, 5, 48), (5, 1), None),           # whole runs per workgroup, each encoding met 37 times
    ((12, 4096), (12, 1), None),           # runs of half a tile and less (16-bit): one wave adds a run
    ((301, 203), (1, 203), None),          # run length 1, rows no multiple of a vector: one element per lane
    ((192, 256), (3, 256), (64, 1)),       # blocks along the leading axis, run length 1: stacked column problems
    ((5, 70, 512), (5, 1, 512), None),     # the same from a batch axis with encodings of its own
]

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _grid(bitwidth, symmetric):
    n = 2 ** bitwidth - 1
    if symmetric:
        return -math.ceil(n / 2), math.floor(n / 2)
    return 0, n


def _make_case(shape, enc_shape, dtype, qmin, qmax, symmetric, seed):
    g = torch.Generator().manual_seed(seed)
    scale = (torch.rand(enc_shape, generator=g) * 0.05 + 0.002).to(torch.float32)
    if symmetric:
        offset = torch.full(enc_shape, float(-round((qmin + qmax) / 2)))
    else:
        offset = torch.randint(-qmax, -qmin + 1, enc_shape, generator=g).to(torch.float32)
    span = float(qmax - qmin)
    x = torch.randn(shape, generator=g) * 0.04 * span * 0.4
    flat = x.flatten()
    # exact half-way points and a few far outliers
    k = torch.arange(min(flat.numel() // 3, 600), dtype=torch.float32)
    flat[: k.numel()] = (k - k.numel() // 2 + 0.5) * 0.01
    if flat.numel() > 8:
        flat[-1] = 1e30
        flat[-2] = -1e30
        flat[-3] = 0.0
    x = flat.view(shape).to(dtype)
    grad = torch.randn(shape, generator=g).to(dtype)
    return x, scale, offset, grad


def _tol(compute_dtype):
    if compute_dtype == torch.float32:
        return 1e-5
    return float(torch.finfo(compute_dtype).eps)  # one unit in the last place of the rounded sum


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("layout", LAYOUTS, ids=lambda l: "x".join(map(str, l[0])) + "_" + "x".join(map(str, l[1])))
@pytest.mark.parametrize("bitwidth,symmetric", [(4, True), (8, False), (8, True), (16, False)])
def test_quantize_dequantize_learnable(device, layout, dtype, bitwidth, symmetric):
    """Composed autograd arithmetic (scale/offset require grad): forward, gx, gscale, goffset."""
    from aimet_amd.quantization import affine

    shape, enc_shape, block = layout
    qmin, qmax = _grid(bitwidth, symmetric)
    x, scale, offset, grad = _make_case(shape, enc_shape, dtype, qmin, qmax, symmetric, seed=bitwidth * 7 + len(shape))

    tr = O.qdq_v2_forward(x, scale, offset, qmin, qmax, block)
    gx_ref, gs_ref, go_ref = O.qdq_v2_backward(grad, x, scale, offset, qmin, qmax, block)

    xd = x.to(device).requires_grad_(True)
    sd = scale.to(device).requires_grad_(True)
    od = offset.to(device).requires_grad_(True)
    y = affine.quantize_dequantize(xd, sd, od, qmin, qmax, block_size=block)
    assert y.dtype == dtype and y.shape == x.shape
    assert_same_bits(y, tr.y, "output")
    y.backward(grad.to(device))
    assert_same_bits(xd.grad, gx_ref, "input gradient")
    tol = _tol(tr.dtype)
    assert_close_rel(sd.grad, gs_ref, tol, "scale gradient", abs_floor=1e-30)
    assert_close_rel(od.grad, go_ref, tol, "offset gradient", abs_floor=1e-30)


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("layout", [l for l in LAYOUTS if l[2] is None],
                         ids=lambda l: "x".join(map(str, l[0])) + "_" + "x".join(map(str, l[1])))
@pytest.mark.parametrize("bitwidth,symmetric", [(4, False), (8, False), (8, True), (16, False)])
def test_quantize_dequantize_frozen(device, layout, dtype, bitwidth, symmetric):
    """Frozen encodings take the ATen fake-quantize arithmetic where the reference does."""
    from aimet_amd.quantization import affine

    shape, enc_shape, _ = layout
    qmin, qmax = _grid(bitwidth, symmetric)
    x, scale, offset, grad = _make_case(shape, enc_shape, dtype, qmin, qmax, symmetric, seed=bitwidth * 11 + 3)
    # the ATen kernels have undefined behaviour for inf * inv_scale: keep the outliers finite after scaling
    xf = x.float()
    x = torch.where(xf.abs() > 1e20, torch.sign(xf) * 1e4, xf).to(dtype)

    ref = O.qdq_v1(x, scale, offset, qmin, qmax)
    if ref is None:
        # the reference leaves the ATen path (encodings along more than one axis, ...): its own autograd function,
        # whose input gradient is where(mask, grad, 0) -- a masked-out negative gradient becomes +0, not -0
        tr = O.qdq_v2_forward(x, scale, offset, qmin, qmax)
        y_ref, gx_ref = tr.y, torch.where(tr.mask, grad, 0).to(dtype)
    else:
        y_ref, gx_ref = ref[0], (grad * ref[1]).to(dtype)

    xd = x.to(device).requires_grad_(True)
    y = affine.quantize_dequantize(xd, scale.to(device), offset.to(device), qmin, qmax)
    assert_same_bits(y, y_ref, "output")
    y.backward(grad.to(device))
    assert_same_bits(xd.grad, gx_ref, "input gradient")


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("layout", LAYOUTS[:1] + LAYOUTS[3:4] + LAYOUTS[9:12],
                         ids=lambda l: "x".join(map(str, l[0])) + "_" + "x".join(map(str, l[1])))
def test_zero_point_shift(device, layout, dtype):
    """zero_point_shift = 0.5 (symmetric 4-bit) including the gradient correction of the scale term."""
    from aimet_amd.quantization import affine

    shape, enc_shape, block = layout
    qmin, qmax = -8, 7
    x, scale, offset, grad = _make_case(shape, enc_shape, dtype, qmin, qmax, True, seed=5)
    tr = O.qdq_v2_forward(x, scale, offset, qmin, qmax, block, 0.5)
    gx_ref, gs_ref, go_ref = O.qdq_v2_backward(grad, x, scale, offset, qmin, qmax, block, 0.5)
    xd = x.to(device).requires_grad_(True)
    sd = scale.to(device).requires_grad_(True)
    od = offset.to(device).requires_grad_(True)
    y = affine.quantize_dequantize(xd, sd, od, qmin, qmax, block_size=block, zero_point_shift=0.5)
    assert_same_bits(y, tr.y, "output")
    y.backward(grad.to(device))
    assert_same_bits(xd.grad, gx_ref, "input gradient")
    assert_close_rel(sd.grad, gs_ref, _tol(tr.dtype), "scale gradient", abs_floor=1e-30)
    assert_close_rel(od.grad, go_ref, _tol(tr.dtype), "offset gradient", abs_floor=1e-30)


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("layout", LAYOUTS[:1] + LAYOUTS[3:4] + LAYOUTS[7:8] + LAYOUTS[9:10] + LAYOUTS[11:12],
                         ids=lambda l: "x".join(map(str, l[0])) + "_" + "x".join(map(str, l[1])))
@pytest.mark.parametrize("bitwidth,symmetric", [(4, True), (8, False)])
def test_quantize_and_dequantize(device, layout, dtype, bitwidth, symmetric):
    from aimet_amd.quantization import affine

    shape, enc_shape, block = layout
    qmin, qmax = _grid(bitwidth, symmetric)
    x, scale, offset, grad = _make_case(shape, enc_shape, dtype, qmin, qmax, symmetric, seed=17)

    q_ref, _ = O.quantize_forward(x, scale, offset, qmin, qmax, block)
    gx_ref, gs_ref, go_ref = O.quantize_backward(grad, x, scale, offset, qmin, qmax, block)
    D = O.internal_dtype(dtype, qmin, qmax)
    xd = x.to(device).requires_grad_(True)
    sd = scale.to(device).requires_grad_(True)
    od = offset.to(device).requires_grad_(True)
    q = affine.quantize(xd, sd, od, qmin, qmax, block_size=block)
    assert_same_bits(q, q_ref, "codes")
    q.backward(grad.to(device))
    assert_same_bits(xd.grad, gx_ref, "quantize input gradient")
    # the scale gradient multiplies two quotients: outliers make it huge, compare relative to its own magnitude
    assert_close_rel(sd.grad, gs_ref, max(_tol(D), 1e-5), "quantize scale gradient", abs_floor=1e-30)
    assert_close_rel(od.grad, go_ref, max(_tol(D), 1e-5), "quantize offset gradient", abs_floor=1e-30)

    # dequantize the codes again
    codes = q_ref
    dq_ref = O.dequantize_forward(codes, scale, offset, block)
    gx2, gs2, go2 = O.dequantize_backward(grad, codes, scale, offset, block)
    cd = codes.to(device).requires_grad_(True)
    sd2 = scale.to(device).requires_grad_(True)
    od2 = offset.to(device).requires_grad_(True)
    dq = affine.dequantize(cd, sd2, od2, block_size=block)
    assert_same_bits(dq, dq_ref, "dequantized")
    dq.backward(grad.to(device))
    assert_same_bits(cd.grad, gx2, "dequantize input gradient")
    assert_close_rel(sd2.grad, gs2, max(_tol(dtype), 1e-5), "dequantize scale gradient", abs_floor=1e-30)
    assert_close_rel(od2.grad, go2, max(_tol(dtype), 1e-5), "dequantize offset gradient", abs_floor=1e-30)


def test_non_finite_inputs(device):
    """NaN propagates, +-inf saturates (composed arithmetic); gradients of NaN inputs are zero."""
    from aimet_amd.quantization import affine

    x = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.3, -0.0, 1e-45, -1e-45, 3.4e38])
    scale = torch.tensor(0.01)
    offset = torch.tensor(-128.0)
    grad = torch.ones_like(x)
    tr = O.qdq_v2_forward(x, scale, offset, 0, 255)
    gx_ref, gs_ref, go_ref = O.qdq_v2_backward(grad, x, scale, offset, 0, 255)
    xd = x.to(device).requires_grad_(True)
    sd = scale.to(device).requires_grad_(True)
    od = offset.to(device).requires_grad_(True)
    y = affine.quantize_dequantize(xd, sd, od, 0, 255)
    assert_same_bits(y, tr.y, "output")
    y.backward(grad.to(device))
    assert_same_bits(xd.grad, gx_ref, "input gradient")


@pytest.mark.parametrize("memory_format", [torch.channels_last, torch.channels_last_3d])
def test_memory_format_is_preserved(device, memory_format):
    """Dense non-contiguous inputs keep their memory format (reference: test_backend.py:410-448)."""
    from aimet_amd.quantization import affine

    shape = (2, 3, 4, 5) if memory_format == torch.channels_last else (2, 3, 4, 5, 2)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(shape, generator=g)
    scale = torch.rand(3, *([1] * (len(shape) - 2)), generator=g) * 0.05 + 0.01
    offset = torch.randint(-255, 1, scale.shape, generator=g).float()
    tr = O.qdq_v2_forward(x, scale, offset, 0, 255)
    xd = x.to(device).to(memory_format=memory_format)
    sd = scale.to(device).requires_grad_(True)
    y = affine.quantize_dequantize(xd, sd, offset.to(device), 0, 255)
    assert y.is_contiguous(memory_format=memory_format)
    assert_same_bits(y, tr.y, "output")
    q = affine.quantize(xd, scale.to(device), offset.to(device), 0, 255)
    assert q.is_contiguous(memory_format=memory_format)
    assert_same_bits(q, O.quantize_forward(x, scale, offset, 0, 255)[0], "codes")


def test_non_dense_and_misaligned_inputs(device):
    from aimet_amd.quantization import affine

    g = torch.Generator().manual_seed(4)
    base = torch.randn(64, 130, generator=g)
    scale = torch.tensor(0.02)
    offset = torch.tensor(-100.0)
    bd = base.to(device)
    # strided view (not dense) and a view whose storage offset breaks 16-byte alignment
    for cpu_view, dev_view in [(base[:, ::2], bd[:, ::2]), (base.flatten()[1:], bd.flatten()[1:])]:
        tr = O.qdq_v2_forward(cpu_view, scale, offset, 0, 255)
        sd = scale.to(device).requires_grad_(True)
        y = affine.quantize_dequantize(dev_view, sd, offset.to(device), 0, 255)
        assert_same_bits(y, tr.y, "output")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_column_kernels_with_encodings_off_16_byte_alignment(device, dtype):
    """Per-channel encodings along the fastest axis are read as 16-byte vectors when their arrays allow it and one
    float at a time when a view starts in the middle of such a vector: both must give the same bits, forward and
    backward."""
    from aimet_amd.quantization import affine

    g = torch.Generator().manual_seed(11)
    x = (torch.randn(300, 256, generator=g) * 3).to(dtype).to(device)
    grad = torch.randn(300, 256, generator=g).to(dtype).to(device)
    sbuf = (torch.rand(257, generator=g) * 0.04 + 0.01).to(device)
    obuf = torch.randint(-3, 4, (257,), generator=g).float().to(device)
    results = []
    for off_view in (False, True):
        if off_view:
            s, o = sbuf[1:], obuf[1:]
            assert s.data_ptr() % 16 == 4 and s.is_contiguous()
        else:
            s, o = sbuf[1:].clone(), obuf[1:].clone()
            assert s.data_ptr() % 16 == 0
        s = s.detach().requires_grad_(True)
        o = o.detach().requires_grad_(True)
        xi = x.clone().requires_grad_(True)
        y = affine.quantize_dequantize(xi, s, o, -8, 7)
        y.backward(grad)
        results.append((y.detach(), xi.grad, s.grad, o.grad))
    for name, a, b in zip(("output", "input gradient", "scale gradient", "offset gradient"), *results):
        assert_same_bits(b, a, name)


def test_errors(device):
    from aimet_amd.quantization import affine

    x = torch.randn(2, 3, 4, 5, device=device)
    off = torch.zeros((), device=device)
    for bad in [(4,), (2,), (3, 1), (2, 1, 1)]:
        s = torch.rand(bad, device=device) + 0.1
        with pytest.raises(RuntimeError):
            affine.quantize_dequantize(x, s, off, 0, 255)
        with pytest.raises(RuntimeError):
            affine.quantize(x, s, off, 0, 255)
        with pytest.raises(RuntimeError):
            affine.dequantize(x, s, off)
    s = torch.tensor(0.1, device=device)
    with pytest.raises(RuntimeError):  # mixed devices
        affine.quantize_dequantize(x, s.cpu(), off, 0, 255)
    with pytest.raises(RuntimeError):  # CPU tensors have no path here
        affine.quantize_dequantize(x.cpu(), s.cpu(), off.cpu(), 0, 255)
    with pytest.raises(RuntimeError):  # qmin > qmax
        affine.quantize_dequantize(x, s, off, 5, 1)
    with pytest.raises(RuntimeError):  # bf16 cannot hold a 16-bit grid
        affine.quantize(x.bfloat16(), s, off, 0, 65535)
    with pytest.raises(RuntimeError):  # block size that does not tile the tensor
        affine.quantize_dequantize(x, torch.ones(4, 2, device=device), torch.zeros(4, 2, device=device), 0, 255,
                                   block_size=(1, 3))
    # empty tensors pass through
    e = torch.empty(0, 4, device=device)
    assert affine.quantize_dequantize(e, s, off, 0, 255).shape == (0, 4)


# ------------------------------------------------------------------------------------- division without dividing --
def _awkward_scales(n, seed):
    """Scales whose reciprocal rounds badly or whose quotients hit rounding ties: all-ones and near-one significands,
    powers of two, thirds, plus log-uniform random values."""
    g = torch.Generator().manual_seed(seed)
    s = torch.exp(torch.rand(n, generator=g) * 16 - 10)
    special = torch.tensor([1.0, 2.0 ** -7, 3.0, 1.0 / 3.0, 0.1, 1.9999999, 1.0000001, 0.99999994, 5e-5, 7.0 / 127,
                            0.0078125 * 1.9999999, 1e-10, 123456.7])
    s[: special.numel()] = special
    return s.to(torch.float32)


@pytest.mark.parametrize("op", ["quantize", "qdq"])
def test_division_free_quotients_are_correctly_rounded_fp32(device, op):
    """The kernels replace x / scale by two fused residual corrections of x * (1 / scale); the integer codes (ties
    included) must still be those of the true division.  16-bit grid so that codes spread over many values."""
    C, K = 2048, 4096
    scale = _awkward_scales(C, 5).reshape(C, 1)
    g = torch.Generator().manual_seed(6)
    k = torch.randint(-30000, 30000, (C, K), generator=g).float()
    # elements at and next to the rounding ties (k + 0.5) * scale, and ordinary random values
    x = (k + 0.5) * scale
    x[:, 1::4] = torch.nextafter(x[:, 1::4], torch.full_like(x[:, 1::4], float("inf")))
    x[:, 2::4] = torch.nextafter(x[:, 2::4], torch.full_like(x[:, 2::4], float("-inf")))
    x[:, 3::4] = torch.randn(C, K // 4, generator=g) * scale * 9000
    offset = torch.zeros(C, 1)
    qmin, qmax = -32768, 32767
    xd, sd, od = x.to(device), scale.to(device), offset.to(device)
    from aimet_amd.quantization import affine
    if op == "quantize":
        got = affine.quantize(xd, sd, od, qmin, qmax).cpu()
        ref = O.quantize_forward(x, scale, offset, qmin, qmax)[0]
    else:
        sd.requires_grad_(True)  # keeps the true-division (autograd) arithmetic
        got = affine.quantize_dequantize(xd, sd, od, qmin, qmax).detach().cpu()
        ref = O.qdq_v2_forward(x, scale, offset, qmin, qmax).y
    assert_same_bits(got, ref)


@pytest.mark.parametrize("dtype,qmin,qmax", [(torch.bfloat16, -8, 7), (torch.float16, -128, 127), (torch.float16, 0, 15)])
def test_division_free_quotients_16bit_exhaustive(device, dtype, qmin, qmax):
    """Every finite 16-bit value against a set of scales of the same dtype, in that dtype's arithmetic."""
    allv = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(dtype)
    allv = allv[torch.isfinite(allv.float())]
    scales = _awkward_scales(256, 7)
    if dtype == torch.float16:
        scales = scales.clamp(6.2e-5, 6e4)
    scales = scales.to(dtype).float().reshape(-1, 1)
    x = allv.reshape(1, -1).repeat(scales.shape[0], 1).contiguous()
    offset = torch.zeros_like(scales)
    from aimet_amd.quantization import affine
    sd = scales.to(device).requires_grad_(True)
    got = affine.quantize_dequantize(x.to(device), sd, offset.to(device), qmin, qmax).detach().cpu()
    ref = O.qdq_v2_forward(x, scales, offset, qmin, qmax).y
    assert ref.dtype == dtype
    assert_same_bits(got, ref)


def test_huge_inputs_and_scales_take_the_general_division(device):
    from aimet_amd.quantization import affine
    x = torch.tensor([[1e30, -3e38, float("inf"), 1.0, -2.5, 3e19, 0.0, float("-inf")] * 64] * 4)
    x[1] = x[1] * 1e-30
    scale = torch.tensor([[1e25], [1e-30], [0.5], [2e18]])
    offset = torch.zeros(4, 1)
    sd = scale.to(device).requires_grad_(True)
    got = affine.quantize_dequantize(x.to(device), sd, offset.to(device), -128, 127).detach().cpu()
    ref = O.qdq_v2_forward(x, scale, offset, -128, 127).y
    assert_same_bits(got, ref)


# (compute dtype, tensor dtype, qmin, qmax, offsets): grids and offsets on both sides of the limits up to which the
# kernels may work on rint(x / scale) directly (integer offset; bounds, offset and shifted bounds at most 255 in
# bfloat16, 2047 in float16, 2^24 - 1 in float32 arithmetic); rows that do not qualify take the step-by-step form
_SHORTCUT_CASES = [
    (torch.bfloat16, torch.bfloat16, 0, 255, [0.0, -100.0, -255.0, -254.0, 1.0, 0.5, -128.5, 37.0]),
    (torch.bfloat16, torch.bfloat16, -128, 127, [-128.0, -127.0, 127.0, 128.0, 0.0, 0.25, 300.0, -300.0]),
    (torch.bfloat16, torch.bfloat16, -256, 255, [0.0, 1.0, -1.0, 16.0]),
    (torch.bfloat16, torch.bfloat16, -8, 7, [0.0, 247.0, 248.0, 249.0, -247.0, -248.0, 0.75, -8.0]),
    (torch.float16, torch.float16, 0, 2047, [0.0, -2047.0, -1000.0, 1.0, -0.5, 3.0, -2046.0, 0.125]),
    (torch.float16, torch.float16, -1024, 1023, [0.0, 1024.0, 1025.0, -1023.0, -1024.0, 512.5, 7.0, -7.0]),
    (torch.float32, torch.bfloat16, -32768, 32767, [0.0, -32768.0, 0.5, 123.0, 16777215.0, 16744448.0, -16777216.0, 8.0]),
    (torch.float32, torch.float32, 0, 65535, [0.0, -65535.0, 0.5, 16711680.0, 16711681.0, -0.25, 77.0, -16777215.0]),
]


@pytest.mark.parametrize("case", _SHORTCUT_CASES, ids=lambda c: f"{str(c[0])[6:]}_{str(c[1])[6:]}_{c[2]}_{c[3]}")
def test_small_integer_grid_shortcut_limits(device, monkeypatch, case):
    """Outputs, masks-as-gradients and parameter gradients with the arithmetic dtype forced, at codes one and two
    steps either side of both grid ends, at rounding ties, far outside, and with NaN / infinities in some rows."""
    from aimet_amd import _lib
    from aimet_amd.quantization.affine.backends import hip as H

    cd, dtype, qmin, qmax, offsets = case
    monkeypatch.setattr(O, "internal_dtype", lambda *a: cd)
    R, K = len(offsets), 4096
    g = torch.Generator().manual_seed(R * 31 + qmax)
    scale = (torch.rand(R, 1, generator=g) * 0.05 + 0.002).to(cd).float()
    offset = torch.tensor(offsets).reshape(R, 1)
    off_cd = offset.to(cd).float()
    lo, hi = off_cd + qmin, off_cd + qmax
    # codes around both ends of each row's grid, ties and near-ties, ordinary values, far outliers
    j = torch.arange(K).reshape(1, K)
    around = torch.where(j % 2 == 0, lo, hi) + ((j // 2) % 9 - 4).float()
    frac = torch.tensor([0.0, 0.5, -0.5, 0.25, 0.499, -0.499, 0.75, 0.0])[(j // 18) % 8]
    t = around + frac
    t[:, K // 2:] = (torch.rand(R, K - K // 2, generator=g) - 0.5) * (hi - lo + 40) + (hi + lo) / 2
    x = t * scale
    x[:, -1], x[:, -2], x[:, -3] = 1e30, -1e30, 0.0
    x[1, 5], x[1, 6], x[2, 7] = float("nan"), float("inf"), float("-inf")
    x = x.to(dtype)
    grad = torch.randn(R, K, generator=g).to(dtype)

    tr = O.qdq_v2_forward(x, scale, offset, qmin, qmax)
    gx_ref, gs_ref, go_ref = O.qdq_v2_backward(grad, x, scale, offset, qmin, qmax)
    assert tr.dtype == cd

    xd = x.to(device).requires_grad_(True)
    sd = scale.to(device).requires_grad_(True)
    od = offset.to(device).requires_grad_(True)
    y = H._apply(xd, sd, od, _lib.AHQ_ARITH_AUTOGRAD, _lib.AHQ_OP_QDQ, cd, qmin, qmax, None, 0.0)
    assert_same_bits(y, tr.y, "output")
    y.backward(grad.to(device))
    assert_same_bits(xd.grad, gx_ref, "input gradient")
    tol = _tol(cd)
    finite_rows = torch.tensor([r not in (1, 2) for r in range(R)])  # NaN / inf rows: the sums are NaN on both sides
    assert_close_rel(sd.grad[finite_rows], gs_ref[finite_rows], tol, "scale gradient", abs_floor=1e-30)
    assert_close_rel(od.grad[finite_rows], go_ref[finite_rows], tol, "offset gradient", abs_floor=1e-30)
    assert bool((sd.grad[~finite_rows].cpu().isnan() == gs_ref[~finite_rows].isnan()).all())


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
def test_quantize_keeps_the_sign_of_a_zero_code(device, dtype):
    """With a zero offset, inputs in [-scale / 2, -0] have the code -0.0 in the reference (round(-0.2) - 0); the
    division-free quotient must not lose the sign of an input that is exactly -0."""
    from aimet_amd.quantization import affine

    x = torch.tensor([-0.0, 0.0, -0.01, 0.01, -1e-30, 1e-30, -0.6, 0.6] * 40, dtype=torch.float32).to(dtype)
    scale, offset = torch.tensor(1.0), torch.tensor(0.0)
    codes_ref, _ = O.quantize_forward(x, scale, offset, -2, 1)
    codes = affine.quantize(x.to(device), scale.to(device), offset.to(device), -2, 1)
    assert_same_bits(codes.as_subclass(torch.Tensor), codes_ref, "codes")
    assert torch.signbit(codes_ref[0]) and not torch.signbit(codes_ref[1])


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", ["scalar_offset", "scalar_scale", "row_offset_column_scale"])
def test_offset_and_scale_of_different_shapes_broadcast(device, dtype, case):
    """The reference's elementwise arithmetic broadcasts scale and offset against each other
    (torch_builtins.py:727-773); a 0-dim offset next to a (C, 1) scale, and the reverse, must give the oracle's result
    and gradients of each operand's own shape."""
    from aimet_amd.quantization import affine

    g = torch.Generator().manual_seed(31)
    C, K = 24, 320
    x = (torch.randn(C, K, generator=g) * 2).to(dtype)
    grad = torch.randn(C, K, generator=g).to(dtype)
    if case == "scalar_offset":
        scale = torch.rand(C, 1, generator=g) * 0.05 + 0.01
        offset = torch.tensor(-37.0)
    elif case == "scalar_scale":
        scale = torch.tensor(0.03)
        offset = torch.randint(-200, -20, (C, 1), generator=g).float()
    else:
        scale = torch.rand(C, 1, generator=g) * 0.05 + 0.01
        offset = torch.randint(-200, -20, (1, K), generator=g).float()
    tr = O.qdq_v2_forward(x, scale, offset, 0, 255)
    gx_ref, gs_ref, go_ref = O.qdq_v2_backward(grad, x, scale, offset, 0, 255)
    xd = x.to(device).requires_grad_(True)
    sd = scale.to(device).requires_grad_(True)
    od = offset.to(device).requires_grad_(True)
    y = affine.quantize_dequantize(xd, sd, od, 0, 255)
    assert_same_bits(y.as_subclass(torch.Tensor), tr.y, "output")
    y.backward(grad.to(device))
    assert_same_bits(xd.grad, gx_ref, "input gradient")
    assert sd.grad.shape == scale.shape and od.grad.shape == offset.shape
    tol = max(4 * _tol(tr.dtype), 1e-5)  # the 16-bit oracle rounds its partial sums
    assert_close_rel(sd.grad, gs_ref.reshape(scale.shape), tol, "scale gradient", abs_floor=1e-30)
    assert_close_rel(od.grad, go_ref.reshape(offset.shape), tol, "offset gradient", abs_floor=1e-30)
    # without gradients the same operands go through the same broadcast
    with torch.no_grad():
        y2 = affine.quantize_dequantize(x.to(device), scale.to(device), offset.to(device), 0, 255)
    assert_same_bits(y2.as_subclass(torch.Tensor), tr.y, "output without gradients")
    q = affine.quantize(x.float().to(device), scale.to(device), offset.to(device), 0, 255)
    assert_same_bits(q.as_subclass(torch.Tensor), O.quantize_forward(x.float(), scale, offset, 0, 255)[0], "codes")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("layout", [
    ((8, 100), (8, 1), None, True),               # runs shorter than a tile
    ((256, 4096), (256, 1), None, True),          # runs of a quarter / an eighth of a tile
    ((300, 24), (300, 1), None, True),            # runs of a few vectors: one thread adds a run
    ((4, 6, 10, 10), (6, 1, 1), None, True),      # short runs, each encoding met several times
    ((37, 5, 48), (5, 1), None, True),
    ((1100, 264), (1, 264), None, True),          # column-walking kernel, several row groups
    ((3, 40, 1536), (1536,), None, True),
    ((640, 256), (2, 256), (320, 1), True),       # stacked column problems (blocks along the leading axis)
    ((700, 203), (1, 203), None, True),           # column-walking kernel, one element per lane (odd row length)
    ((1100, 24), (1, 24), None, False),           # run length 1 without the column kernel: atomics
    ((8, 16), (2, 4), (4, 4), False),             # generic walk: atomics
], ids=lambda l: "x".join(map(str, l[0])) + "_" + "x".join(map(str, l[1])))
def test_parameter_gradients_repeat(device, layout, dtype):
    """Scale / offset gradients are float32 terms added in double precision and rounded once.  On every layout of the
    flat [outer, encoding, run] form the order of the additions is fixed by the layout (whole runs per workgroup,
    lanes and waves combined in a fixed pattern, per-run or per-row-group partial sums added up by a second launch),
    so repeated runs agree bit for bit.  Two kinds of layout still add with 64-bit floating-point atomics, in an
    order that varies between runs: blocks along several dimensions (the generic walk) and runs of a single element
    that the column kernel does not take.  There two runs differ by about 1e-16 of the sum of magnitudes before the
    final rounding: they must agree to one unit in the last place of the compute dtype."""
    from aimet_amd.quantization import affine

    shape, enc_shape, block, ordered = layout
    x, scale, offset, grad = _make_case(shape, enc_shape, dtype, -128, 127, True, seed=11)
    xd, gd = x.to(device), grad.to(device)
    # other work in between changes which workgroups finish first
    noise = torch.randn(1 << 20, device=device)
    runs = []
    for i in range(5):
        sd = scale.to(device).requires_grad_(True)
        od = offset.to(device).requires_grad_(True)
        if i % 2:
            noise.mul_(1.0001)
        affine.quantize_dequantize(xd, sd, od, -128, 127, block_size=block).backward(gd)
        runs.append((sd.grad.clone(), od.grad.clone()))
    ulp = float(torch.finfo(torch.float32 if dtype == torch.float32 else dtype).eps)
    for gs, go in runs[1:]:
        if ordered:
            assert_same_bits(gs, runs[0][0], "scale gradient of a repeated run")
            assert_same_bits(go, runs[0][1], "offset gradient of a repeated run")
        else:
            assert_close_rel(gs, runs[0][0], ulp, "scale gradient of a repeated run", abs_floor=1e-30)
            assert_close_rel(go, runs[0][1], ulp, "offset gradient of a repeated run", abs_floor=1e-30)
