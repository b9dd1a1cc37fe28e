"""The cases the reference's own tests hold for its lossless decomposition of an already-quantized tensor
(TrainingExtensions/torch/test/python/v2/test_utils.py:411-706), each stated by its inputs and by what the reference's
test expects of the outputs -- the scale and codes the tensor was built from, an SQNR bound, least-squares optimality,
a refusal and its message.  ``decompose(x, qmin, qmax, scale_shape, block_size=None, zero_point_shift=0.0)`` is the
implementation under test (the numpy restatement or the device path, see tests/decompose_adapters.py); it takes and
returns CPU torch tensors and raises ``error`` for a refusal."""

import itertools

import pytest
import torch


def _dequantize(q, scale, block_size):
    """q * scale blockwise; scale of shape S applies to blocks of the trailing len(S) dimensions."""
    shape = tuple(scale.shape)
    if not shape:
        return q * scale
    bs = block_size or tuple(d // s for d, s in zip(q.shape[q.dim() - len(shape):], shape))
    split = []
    for s, b in zip(shape, bs):
        split += [s, b]
    lead = q.shape[: q.dim() - len(shape)]
    view = scale.reshape(*[v for s in shape for v in (s, 1)])
    return (q.reshape(*lead, *split) * view).reshape(q.shape)


AXES = [(None, None), (0, None), (1, None), (0, 1), (1, 0)]
SCALES = [1e-0, 1e-1, 1e-2, 1e-3, 1e-4, 1e-5, 1e-6]


def grid_patches(bitwidth):
    qmin, qmax = -(2 ** (bitwidth - 1)), 2 ** (bitwidth - 1)
    for lo in range(qmin, qmax):
        for hi in range(qmax, lo, -1):
            yield [1, *range(lo, hi + 1, 2)]


def check_lossless_grid(decompose, bitwidth, scale, channel_axis, block_axis, patches=None):
    """test_decomposition (:427-481): every sub-range of the grid, per tensor / per channel / per block."""
    qmin, qmax = -(2 ** (bitwidth - 1)), 2 ** (bitwidth - 1)
    scale = torch.tensor(scale)
    for patch in (patches if patches is not None else grid_patches(bitwidth)):
        n = len(patch)
        if channel_axis is None:
            scale_shape, block_size = (), None
        elif block_axis is None:
            scale_shape = (6, 1) if channel_axis == 0 else (1, 2 * n)
            block_size = None
        elif channel_axis == 0:
            scale_shape, block_size = (6, 2), (1, n)
        else:
            scale_shape, block_size = (2, 2 * n), (3, 1)
        q = torch.tensor([patch * 2] * 6, dtype=torch.float32)
        x = _dequantize(q, scale.repeat(scale_shape), block_size)
        got_q, got_scale = decompose(x, qmin, qmax, scale_shape, block_size)
        assert got_scale.shape == scale_shape
        assert got_q.shape == q.shape
        assert torch.allclose(x, _dequantize(got_q, got_scale, block_size)), (patch, scale_shape)
        assert torch.all((qmin <= got_q) & (got_q <= qmax))


def _channels_on_a_grid(bitwidth, elements, storage=None, seed=0):
    g = torch.Generator().manual_seed(seed)
    qmin, qmax = -(2 ** (bitwidth - 1)), 2 ** (bitwidth - 1)
    true_scale = torch.rand(8, 1, generator=g) * 0.4 + 0.05
    codes = torch.randint(qmin, qmax + 1, (8, elements), generator=g).float()
    codes[:, 0] = qmax
    codes[:, 1] = 1
    x = codes * true_scale
    if storage is not None:
        x = x.to(storage).float()
    return x, qmin, qmax


def _sqnr_db(x, recon):
    return 10 * torch.log10((x ** 2).mean() / ((x - recon) ** 2).mean())


def check_storage_rounding(decompose, storage):
    """test_decomposition_storage_rounding (:484-516)."""
    x, qmin, qmax = _channels_on_a_grid(4, 2048, storage)
    q, scale = decompose(x, qmin, qmax, (8, 1))
    assert scale.shape == (8, 1)
    assert torch.all((qmin <= q) & (q <= qmax))
    assert _sqnr_db(x, q * scale) > 40


def check_native_low_precision(decompose, storage, bitwidth):
    """test_decomposition_native_low_precision_input (:519-551): scale, codes and product all in the narrow dtype."""
    g = torch.Generator().manual_seed(0)
    qmin, qmax = -(2 ** (bitwidth - 1)), 2 ** (bitwidth - 1)
    true_scale = (torch.rand(8, 1, generator=g) * 0.4 + 0.05).to(storage)
    codes = torch.randint(qmin, qmax + 1, (8, 2048), generator=g).to(storage)
    codes[:, 0] = qmax
    codes[:, 1] = 1
    x = codes * true_scale
    q, scale = decompose(x, qmin, qmax, (8, 1))
    assert torch.all((qmin <= q) & (q <= qmax))
    assert _sqnr_db(x.float(), (q * scale.to(q.dtype)).float()) > 40


def check_least_squares_optimal(decompose, bitwidth):
    """test_decomposition_scale_is_least_squares_optimal (:554-583)."""
    x, qmin, qmax = _channels_on_a_grid(bitwidth, 4096, torch.bfloat16)
    q, scale = decompose(x, qmin, qmax, (8, 1))
    ls = (x * q).sum(dim=1, keepdim=True) / (q ** 2).sum(dim=1, keepdim=True).clamp(min=1e-12)
    assert ((q * scale - x) ** 2).sum() <= ((q * ls - x) ** 2).sum() * (1 + 1e-4)


def check_refuses_unquantized(decompose, error):
    """test_decomposition_rejects_unquantized_tensor (:586-594) and the message of the early exit (:597-618)."""
    g = torch.Generator().manual_seed(0)
    with pytest.raises(error):
        decompose(torch.randn(8, 2048, generator=g).bfloat16().float(), -8, 8, (8, 1))
    with pytest.raises(error, match=r"One or more blocks exceed \d+ distinct values"):
        decompose(torch.randn(8, 2048, generator=g), -8, 8, (8, 1))


def check_refused_after_the_search(decompose, error):
    """Past the early exit (few distinct magnitudes) but on no grid: values from a set of four magnitudes whose ratios
    are irrational, so no integer divisor fits; the refusal has to come from the block / tensor gates."""
    g = torch.Generator().manual_seed(1)
    values = torch.tensor([1.0, 2.0 ** 0.5, 3.0 ** 0.5, 7.0 ** 0.5])
    x = values[torch.randint(0, 4, (16, 512), generator=g)] * (torch.randint(0, 2, (16, 512), generator=g) * 2.0 - 1)
    with pytest.raises(error, match="not QDQ-like"):
        decompose(x, -8, 7, (16, 1))


def check_near_constant_channel(decompose, absmax):
    """test_decomposition_recovers_near_constant_channel (:621-645)."""
    pattern = torch.tensor([absmax - 2, absmax - 1, absmax], dtype=torch.float32)
    w = pattern.repeat(8, 129 // 3 + 1)[:, :129].contiguous()
    q, scale = decompose(w, -128, 127, (8, 1))
    assert torch.allclose(scale, torch.ones_like(scale))
    assert torch.allclose(q * scale, w)


def check_single_level_grid(decompose):
    """test_decomposition_keeps_genuine_single_level_grid (:648-664)."""
    scale = torch.tensor([[0.05], [0.10], [0.20]])
    q, got = decompose(torch.ones(3, 64) * scale, -8, 7, (3, 1))
    assert torch.allclose(got, scale)
    assert torch.all(q == 1.0)


def check_single_element_blocks(decompose):
    """test_decomposition_single_element_blocks (:667-682)."""
    q, scale = decompose(torch.tensor([[5.0], [3.0], [100.0], [0.0]]), -128, 127, (4, 1))
    assert torch.allclose(scale.flatten()[:3], torch.tensor([5.0, 3.0, 100.0]))
    assert torch.allclose(q.flatten()[:3].abs(), torch.ones(3))


def shifted_and_blocked_input(zero_point_shift, qmin, qmax, block_size, seed=0):
    """The tensor of test_decomposition_chunked_matches_unchunked (:685-706): 37 x 64, one all-zero row, bfloat16
    storage, optionally blocks of 16 and the half-integer grid."""
    g = torch.Generator().manual_seed(seed)
    rows, cols = 37, 64
    nb = cols // block_size[1] if block_size else 1
    codes = torch.randint(qmin, qmax + 1, (rows, cols), generator=g).float()
    codes[5] = 0
    scale = torch.rand(rows, nb, 1, generator=g) * 0.1 + 1e-3
    x = ((codes.view(rows, nb, -1) + zero_point_shift) * scale).view(rows, cols)
    x[5] = 0
    return x.bfloat16().float(), codes, scale.view(rows, nb), (rows, nb)


SHIFTED_CASES = list(itertools.product([(0.0, -8, 7), (0.5, -2, 1)], [None, (1, 16)]))


def check_shifted_and_blocked(decompose, grid, block_size):
    """The same tensors, checked against what they were built from: codes exactly (wherever the block is not all
    zero), scales to bfloat16 rounding."""
    zps, qmin, qmax = grid
    x, codes, scale, scale_shape = shifted_and_blocked_input(zps, qmin, qmax, block_size)
    q, got = decompose(x, qmin, qmax, scale_shape, block_size, zps)
    live = torch.ones(37, dtype=torch.bool)
    live[5] = False
    recon = _dequantize(q + zps, got, block_size)
    assert _sqnr_db(x[live], recon[live]) > 40
    # a block's scale is identifiable only up to the common factor of its codes (+ shift); with 16+ random codes of
    # a 2- or 4-bit grid per block the factor is 1 in all of these blocks
    assert torch.equal(q[live], codes[live])
    assert torch.allclose(got[live], scale[live], rtol=2.0 ** -8)
