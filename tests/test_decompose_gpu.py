"""The recovery of an already-quantized tensor's grid (aimet_amd/quantization/_decompose.py) on the GPU: the
reference's own cases (tests/decompose_checks.py) and agreement with the numpy restatement (oracle/decompose.py)."""

import pytest
import torch

from tests import decompose_checks as C
from tests.decompose_adapters import oracle_decompose, product_decompose
from aimet_amd.quantization import _decompose as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def decompose(device):
    return product_decompose(device)


@pytest.mark.parametrize("channel_axis, block_axis", C.AXES)
@pytest.mark.parametrize("scale", [1e-0, 1e-3, 1e-6])
@pytest.mark.parametrize("bitwidth", [2, 4])
def test_lossless_on_sub_ranges_of_the_grid(decompose, bitwidth, scale, channel_axis, block_axis):
    # every sub-range runs on the CPU (tests/test_decompose_cpu.py); here every fifth, to keep the run short
    patches = list(C.grid_patches(bitwidth))[::5]
    C.check_lossless_grid(decompose, bitwidth, scale, channel_axis, block_axis, patches)


@pytest.mark.parametrize("storage", [torch.bfloat16, torch.float16])
def test_storage_rounding_and_narrow_dtypes(decompose, storage):
    C.check_storage_rounding(decompose, storage)
    for bw in (2, 4):
        C.check_native_low_precision(decompose, storage, bw)


def test_least_squares_refusals_and_special_blocks(decompose):
    for bw in (2, 4):
        C.check_least_squares_optimal(decompose, bw)
    C.check_refuses_unquantized(decompose, P._DecompositionError)
    C.check_refused_after_the_search(decompose, P._DecompositionError)
    for absmax in (127, 100):
        C.check_near_constant_channel(decompose, absmax)
    C.check_single_level_grid(decompose)
    C.check_single_element_blocks(decompose)


@pytest.mark.parametrize("grid, block_size", C.SHIFTED_CASES)
def test_half_integer_grid_and_blocks_equal_the_oracle(decompose, grid, block_size):
    C.check_shifted_and_blocked(decompose, grid, block_size)
    zps, qmin, qmax = grid
    x, _, _, scale_shape = C.shifted_and_blocked_input(zps, qmin, qmax, block_size, seed=3)
    want_q, want_s = oracle_decompose(x, qmin, qmax, scale_shape, block_size, zps)
    got_q, got_s = decompose(x, qmin, qmax, scale_shape, block_size, zps)
    assert torch.equal(got_q, want_q)
    torch.testing.assert_close(got_s, want_s, rtol=4e-6, atol=0)  # float32 sums in a different order


@pytest.mark.parametrize("storage", [None, torch.float16, torch.bfloat16])
def test_int8_channels_equal_the_oracle(decompose, storage):
    g = torch.Generator().manual_seed(5)
    codes = torch.randint(-128, 128, (24, 700), generator=g).float()
    codes[3] = 0
    codes[4] = codes[4].clamp(-3, 3) * 40
    x = codes * (torch.rand(24, 1, generator=g) * 0.02 + 1e-4)
    if storage is not None:
        x = x.to(storage).float()
    want_q, want_s = oracle_decompose(x, -128, 127, (24, 1))
    got_q, got_s = decompose(x, -128, 127, (24, 1))
    assert torch.equal(got_q, want_q)
    torch.testing.assert_close(got_s, want_s, rtol=4e-6, atol=0)


def test_slabs_do_not_change_the_result_and_bound_the_memory(device, monkeypatch):
    """test_decomposition_chunked_matches_unchunked / test_decomposition_peak_memory_bounded
    (test_utils.py:685-751), the latter at a quarter of its size: the working set follows the slab, not the tensor."""
    rows, cols = 8192, 2048
    g = torch.Generator(device=device).manual_seed(0)
    codes = torch.randint(-8, 8, (rows, cols), device=device, dtype=torch.int8, generator=g)
    scale = torch.rand(rows, 1, device=device, generator=g) * 0.01 + 1e-3
    weight = (codes.float() * scale).bfloat16()
    del codes
    monkeypatch.setattr(P, "_DECOMPOSE_CHUNK_NUMEL", 2 ** 22)
    monkeypatch.setattr(P, "_SCORE_GROUP_NUMEL", 2 ** 22)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    _, got = P._decompose_prequantized_tensor(weight, -8, 7, scale_shape=(rows, 1), return_input_q=False)
    overhead = torch.cuda.max_memory_allocated() - before
    assert overhead <= weight.numel() * weight.element_size() * 4
    torch.testing.assert_close(got, scale, rtol=2.0 ** -8, atol=0)
    monkeypatch.setattr(P, "_DECOMPOSE_CHUNK_NUMEL", 2 ** 20)
    _, again = P._decompose_prequantized_tensor(weight, -8, 7, scale_shape=(rows, 1), return_input_q=False)
    # the device's row reductions may split a row differently for a different number of rows
    torch.testing.assert_close(again, got, rtol=1e-6, atol=0)
