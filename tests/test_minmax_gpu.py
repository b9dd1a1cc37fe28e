"""Parity of the fused min/max reduction with torch.amin/amax applied the way the reference's reduce() applies them."""

import pytest
import torch

from oracle import torch_ref as O
from tests.helpers import assert_same_bits

pytestmark = pytest.mark.gpu

CASES = [
    ((37, 129), (), None),
    ((1024, 1030), (1,), None),
    ((64, 4096), (64, 1), None),
    ((16, 5000), (16, 1), None),
    ((8, 100), (8, 1), None),
    ((8, 128), (8, 1), None),
    ((4, 6, 10, 10), (6, 1, 1), None),
    ((4, 6, 10, 10), (1, 6, 1, 1), None),
    ((2, 3, 64, 64), (3, 1, 1), None),
    ((32, 256), (32, 4), (1, 64)),
    ((3, 32, 256), (32, 4), (1, 64)),
    ((8, 16), (2, 4), (4, 4)),
    ((10, 12), (12,), None),
    ((6, 10), (6, 1), None),
    ((5, 7, 64), (5, 1, 2), (1, -1, -1)),
    ((3, 5), (3, 5), None),
    ((200, 2056), (2056,), None),          # one encoding per element of the fastest axis: lanes walk down columns
    ((3, 70, 512), (512,), None),          # the same with several slabs of rows and leading dimensions folded in
    ((301, 203), (203,), None),            # rows no multiple of a vector: the column walk with one element per lane
    ((192, 256), (3, 256), (64, 1)),       # blocks along the leading axis, run length 1: stacked column problems
    ((5, 300, 512), (5, 1, 512), None),    # the same from a batch axis with encodings of its own, several row groups
    ((256, 256), (2, 2), (128, 128)),      # two-dimensional blocks wider than a wave (generic walk, wave pre-reduction)
    ((96, 100), (3, 4), (32, 25)),         # two-dimensional blocks narrower than a wave
    ((32, 512, 14, 14), (512, 1, 1), None),  # short runs, many per tile (LDS table of the tile's runs)
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(map(str, c[0])) + "_" + "x".join(map(str, c[1])))
def test_min_max(device, case, dtype):
    from aimet_amd.quantization._stats import reduce_min_max

    shape, enc_shape, block = case
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(shape, generator=g) * 3).to(dtype)
    mn_ref, mx_ref = O.reduce_minmax(x, enc_shape, block)
    mn, mx = reduce_min_max(x.to(device), enc_shape, block)
    assert mn.dtype == dtype
    assert_same_bits(mn, mn_ref, "min")
    assert_same_bits(mx, mx_ref, "max")

    # running update == torch.minimum / torch.maximum with the previous statistics
    x2 = (torch.randn(shape, generator=g) * 2 + 0.5).to(dtype)
    mn2_ref, mx2_ref = O.reduce_minmax(x2, enc_shape, block)
    b_mn, b_mx = reduce_min_max(x2.to(device), enc_shape, block, running=(mn, mx))
    assert_same_bits(b_mn, mn2_ref, "batch min")
    assert_same_bits(b_mx, mx2_ref, "batch max")
    assert_same_bits(mn, torch.minimum(mn_ref, mn2_ref), "running min")
    assert_same_bits(mx, torch.maximum(mx_ref, mx2_ref), "running max")


def test_nan_and_inf(device):
    from aimet_amd.quantization._stats import reduce_min_max

    x = torch.randn(8, 300)
    x[1, 5] = float("nan")
    x[2, 7] = float("inf")
    x[3, 9] = -float("inf")
    x[4, :] = float("inf")
    for shape in [(), (8, 1)]:
        mn_ref, mx_ref = O.reduce_minmax(x, shape)
        mn, mx = reduce_min_max(x.to(device), shape)
        assert_same_bits(mn, mn_ref, "min with NaN")
        assert_same_bits(mx, mx_ref, "max with NaN")
        # finite-only variant: the histogram observer's range (encoding_analyzer.py:213-219), per slice
        if shape == ():
            fin = x.isfinite()
            lo = torch.where(fin, x, float("inf")).min()
            hi = torch.where(fin, x, -float("inf")).max()
        else:
            fin = x.isfinite()
            lo = torch.where(fin, x, float("inf")).amin(dim=1, keepdim=True)
            hi = torch.where(fin, x, -float("inf")).amax(dim=1, keepdim=True)
        mnf, mxf = reduce_min_max(x.to(device), shape, finite_only=True)
        assert_same_bits(mnf, lo, "finite min")
        assert_same_bits(mxf, hi, "finite max")


def test_errors(device):
    from aimet_amd.quantization._stats import reduce_min_max

    x = torch.randn(4, 6, device=device)
    with pytest.raises(RuntimeError):
        reduce_min_max(x, (5, 1))
    with pytest.raises(RuntimeError):
        reduce_min_max(x.cpu(), ())
    with pytest.raises(RuntimeError):
        reduce_min_max(torch.empty(0, 3, device=device), ())


@pytest.mark.parametrize("case", [((64, 520), (520,), None), ((256, 256), (2, 2), (128, 128)), ((32, 64, 7, 7), (64, 1, 1), None)],
                         ids=["columns", "blocks_2d", "short_runs"])
def test_nan_and_inf_in_the_aggregating_paths(device, case):
    """NaN wins, infinities count, and the finite-only variant skips both, on the layouts that pre-aggregate in LDS,
    across a wave, or down columns before they touch the global keys."""
    from aimet_amd.quantization._stats import reduce_min_max

    shape, enc_shape, block = case
    g = torch.Generator().manual_seed(5)
    x = torch.randn(shape, generator=g)
    f = x.view(-1)
    f[3], f[1000], f[2001], f[-1] = float("nan"), float("inf"), float("-inf"), float("nan")
    mn_ref, mx_ref = O.reduce_minmax(x, enc_shape, block)
    mn, mx = reduce_min_max(x.to(device), enc_shape, block)
    assert_same_bits(mn, mn_ref, "min")
    assert_same_bits(mx, mx_ref, "max")
    fin = torch.where(x.isfinite(), x, torch.zeros_like(x))  # the test data has finite values on both sides of zero
    lo_ref, hi_ref = O.reduce_minmax(torch.where(x.isfinite(), x, torch.full_like(x, 1e30)), enc_shape, block)[0], \
        O.reduce_minmax(torch.where(x.isfinite(), x, torch.full_like(x, -1e30)), enc_shape, block)[1]
    lo, hi = reduce_min_max(x.to(device), enc_shape, block, finite_only=True)
    assert_same_bits(lo, lo_ref, "finite min")
    assert_same_bits(hi, hi_ref, "finite max")
    del fin


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
@pytest.mark.parametrize("case", [((37, 129), (), None), ((3, 1024, 1027), (1,), None), ((5,), (), None),
                                  ((64, 4096), (64, 1), None), ((200, 2056), (2056,), None)],
                         ids=lambda c: "x".join(map(str, c[0])) + "_" + "x".join(map(str, c[1])))
def test_min_max_with_copy(device, case, dtype):
    """ahq_minmax_copy: the statistics of ahq_minmax and a bit-identical copy of the tensor (NaN payloads and signs of
    zero included), with and without running statistics; layouts with several encodings copy separately."""
    from aimet_amd.quantization._stats import reduce_min_max

    shape, enc_shape, block = case
    g = torch.Generator().manual_seed(sum(shape) + 1)
    x = (torch.randn(shape, generator=g) * 3).to(dtype)
    x.view(-1)[0] = -0.0
    xd = x.to(device)
    mn_ref, mx_ref = reduce_min_max(xd, enc_shape, block)
    out = torch.full_like(xd, 7.0)
    mn, mx = reduce_min_max(xd, enc_shape, block, copy_to=out)
    assert_same_bits(mn, mn_ref.cpu(), "min")
    assert_same_bits(mx, mx_ref.cpu(), "max")
    assert_same_bits(out, x, "copy")
    x2 = (torch.randn(shape, generator=g) * 2 + 0.5).to(dtype)
    if x2.numel() > 3:
        x2.view(-1)[2] = float("nan")
    out2 = torch.empty_like(xd)
    reduce_min_max(x2.to(device), enc_shape, block, running=(mn, mx), copy_to=out2)
    rm, rx = mn_ref.clone(), mx_ref.clone()
    reduce_min_max(x2.to(device), enc_shape, block, running=(rm, rx))
    assert_same_bits(mn, rm.cpu(), "running min")
    assert_same_bits(mx, rx.cpu(), "running max")
    assert out2.view(torch.int16 if dtype != torch.float32 else torch.int32).cpu().equal(
        x2.view(torch.int16 if dtype != torch.float32 else torch.int32)), "copy of a tensor holding NaN"


def test_passthrough_calibration_returns_a_clone(device):
    """Whole-model calibration observes and passes the input on as a new tensor with the same values."""
    from aimet_amd.quantization.affine import QuantizeDequantize

    q = QuantizeDequantize((), 8, False).to(device)
    x = torch.randn(3, 1000, device=device, dtype=torch.bfloat16)
    with torch.no_grad(), q._compute_encodings(passthrough=True):
        y = q(x)
        y2 = q(x.t())  # not contiguous: the step-by-step form
    assert y.data_ptr() != x.data_ptr() and torch.equal(y, x)
    assert torch.equal(y2, x.t()) and y2.stride() == x.t().clone().stride()
    assert float(q.min.detach()) <= float(x.float().min()) and float(q.max.detach()) >= float(x.float().max())
    xg = x.float().requires_grad_(True)
    with q._compute_encodings(passthrough=True):
        yg = q(xg)
    yg.sum().backward()
    assert torch.equal(xg.grad, torch.ones_like(xg))
