"""DlQuantization rows on the GPU: the HIP path against the reference's own expected outputs (shared checks) and,
bit for bit, against the plain-C oracle on seeded inputs.  Everything goes through the C ABI (aimet_amd.dlq)."""

import numpy as np
import pytest
import torch

from oracle import dlq as OD
from tests import dlq_checks as C
from tests.dlq_adapters import (QUANTIZATION_PERCENTILE, QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED, HipQuantizer,
                                OracleQuantizer)

pytestmark = pytest.mark.gpu

TFE_MODES = [(False, False, False), (True, False, False), (True, True, False), (True, False, True)]


@pytest.fixture()
def make(device):
    return lambda shape, bw, scheme: HipQuantizer(shape, bw, scheme, device)


# ------------------------------------------------------------------------------ the reference's expected outputs --
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_broadcast_qdq_vectors(make, dtype):
    C.check_broadcast_qdq(make, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_per_tensor_qdq(make, dtype):
    C.check_per_tensor_qdq(make, dtype)


def test_minmax_quantizer_vectors(make):
    C.check_minmax_quantizer(make)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_block_minmax_vectors(make, dtype):
    C.check_block_minmax(make, dtype)


def test_tfe_all_zero_vector(make):
    C.check_tfe_all_zero(make)


def test_tfe_reference_bounds(make):
    C.check_tfe_properties(make)


def test_percentile_reference_expectations(make):
    C.check_percentile(make)


# ------------------------------------------------------- exact pins: independent enumeration and closed forms --------
def test_tfe_search_equals_independent_enumeration(make):
    C.check_tfe_exact_against_enumeration(make)


def test_tfe_closed_forms(make):
    C.check_tfe_closed_forms(make)


def test_tfe_saturation_weight_decides(make):
    C.check_tfe_saturation_weight_decides(make)


def test_pdf_exact_on_binary_fractions(make):
    C.check_pdf_exact_binary_fractions(make)


@pytest.mark.parametrize("slots", [5, 24])
def test_tfe_search_of_several_hand_built_tables_at_once(device, slots):
    """The same pins with several slots in one call: up to 16 slots are priced with one wave per candidate, more with
    one lane per candidate; every slot must pick what the independent enumeration picks for its table."""
    from tests import tfe_enumeration as T

    tables = list(C.hand_built_pdfs().values())
    xl = T.uniform_buckets(-32.0, 1.0 / 16)
    one = np.zeros(1536)
    one[512 + 255] = 1.0
    tables.append((xl, one))
    xls = np.stack([tables[s % len(tables)][0] for s in range(slots)])
    pdfs = np.stack([tables[s % len(tables)][1] for s in range(slots)])
    for sym, strict, uns in TFE_MODES:
        q = HipQuantizer((slots, 1), 8, QUANTIZATION_TF_ENHANCED, device)
        q.setStrictSymmetric(strict)
        q.setUnsignedSymmetric(uns)
        q.load_pdf(xls, pdfs)
        encs = q.computeEncodings(sym)
        for s in range(slots):
            want = T.search(xls[s], pdfs[s], 8, sym, strict, uns)
            assert tuple(q.last_best[s]) == (want["index"], want["count"]), (s, sym, strict, uns)
            assert tuple(encs[s]) == (want["min"], want["max"], want["delta"], want["offset"], 8), (s, sym, strict, uns)


# ------------------------------------------------------------------------------------- bit-exact against the oracle --
def _data(shape, seed, dtype=torch.float32, special=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * 3 + 0.25
    if special and x.numel() >= 16:
        f = x.view(-1)
        f[1] = float("nan")
        f[5] = float("inf")
        f[7] = float("-inf")
        f[11] = 1e30
        f[13] = 0.0
    return x.to(dtype)


QDQ_CASES = [
    ((1000,), ()),
    ((4099,), ()),
    ((64, 256), (64, 1)),
    ((64, 256), (1, 256)),
    ((48, 512), (48, 8)),
    ((2, 6, 10, 12), (2, 3, 1, 4)),
    ((4, 2, 3), (2, 3)),
    ((3, 5, 7), (5, 1)),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape,enc_shape", QDQ_CASES)
def test_qdq_bit_exact(device, dtype, shape, enc_shape):
    x = _data(shape, 3, dtype)
    E = int(np.prod(enc_shape)) if enc_shape else 1
    g = torch.Generator().manual_seed(4)
    encs = []
    for e in range(E):
        lo = -float(torch.rand((), generator=g)) * 8 - 0.1
        hi = float(torch.rand((), generator=g)) * 8 + 0.1
        bw = [4, 8, 16][e % 3]
        encs.append(tuple(OD.computed_encodings(bw, lo, hi, e % 2 == 1)))
    a = OracleQuantizer(enc_shape, 8, QUANTIZATION_TF)
    b = HipQuantizer(enc_shape, 8, QUANTIZATION_TF, device)
    a.setEncodings(encs)
    b.setEncodings(encs)
    ya, yb = a.quantizeDequantize(x), b.quantizeDequantize(x)
    assert ya.dtype == yb.dtype == dtype and ya.shape == yb.shape
    assert torch.equal(ya.view(torch.int16 if dtype != torch.float32 else torch.int32),
                       yb.view(torch.int16 if dtype != torch.float32 else torch.int32))


def test_qdq_requires_encodings_and_matching_length(device):
    q = HipQuantizer((4,), 8, QUANTIZATION_TF, device)
    with pytest.raises(RuntimeError, match="before computing encodings"):
        q.quantizeDequantize(torch.zeros(8, 4))
    with pytest.raises(RuntimeError, match="did not match"):
        q.setEncodings([(0.0, 1.0, 1 / 255, 0.0, 8)])
    q = HipQuantizer((3,), 8, QUANTIZATION_TF, device)
    q.setEncodings([(0.0, 1.0, 1 / 255, 0.0, 8)] * 3)
    with pytest.raises(RuntimeError, match="broadcastable"):
        q.quantizeDequantize(torch.zeros(8, 4))


MM_CASES = [((4099,), ()), ((64, 256), (64, 1)), ((48, 512), (48, 8)), ((2, 6, 10, 12), (2, 3, 1, 4)), ((3, 5, 7), (5, 1))]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape,enc_shape", MM_CASES)
def test_minmax_stats_and_encodings_bit_exact(device, dtype, shape, enc_shape):
    a = OracleQuantizer(enc_shape, 8, QUANTIZATION_TF)
    b = HipQuantizer(enc_shape, 8, QUANTIZATION_TF, device)
    for seed in (1, 2, 3):
        x = _data(shape, seed, dtype)
        if dtype != torch.float32:
            x = torch.nan_to_num(x, posinf=6e4, neginf=-6e4)  # keep infinities out of the encodings for 16-bit ranges
        a.updateStats(x)
        b.updateStats(x)
        sa, sb = a.stats(), b.stats()
        assert np.array_equal(sa[0], sb[0]) and np.array_equal(sa[1], sb[1])
    for bw in (2, 4, 8, 16):
        a.bitwidth = bw
        b.q.bitwidth = bw
        for sym, strict, uns in ((False, False, False), (True, False, False), (True, True, False), (True, False, True)):
            for q in (a, b):
                q.setStrictSymmetric(strict)
                q.setUnsignedSymmetric(uns)
            ea, eb = a.computeEncodings(sym), b.computeEncodings(sym)
            assert np.array_equal(np.array(ea), np.array(eb)), (bw, sym, strict, uns)


def test_minmax_all_nan_block_keeps_float_limits(device):
    x = torch.full((2, 8), float("nan"))
    x[1] = torch.arange(8.0)
    a = OracleQuantizer((2, 1), 8, QUANTIZATION_TF)
    b = HipQuantizer((2, 1), 8, QUANTIZATION_TF, device)
    a.updateStats(x)
    b.updateStats(x)
    assert np.array_equal(a.stats()[0], b.stats()[0]) and np.array_equal(a.stats()[1], b.stats()[1])
    assert b.stats()[0][0] == np.finfo(np.float32).max and b.stats()[1][0] == -np.finfo(np.float32).max


def _same_pdf(a, b):
    xa, pa, ma = a.stats()
    xb, pb, mb = b.stats()
    assert np.array_equal(ma, mb), (ma, mb)
    assert np.array_equal(xa, xb)
    assert np.array_equal(pa, pb)


PDF_CASES = [((6000,), ()), ((70001,), ()), ((1 << 20,), ()), ((8, 4096), (8, 1)), ((6, 2, 512), (3, 2, 1)), ((4, 2, 3), (2, 3)),
             ((5, 1001), (5, 1)), ((3, 300), (3, 1))]  # one run per slot, ragged and vector-aligned


@pytest.mark.parametrize("shape,enc_shape", PDF_CASES)
def test_pdf_update_bit_exact(device, shape, enc_shape):
    a = OracleQuantizer(enc_shape, 8, QUANTIZATION_TF_ENHANCED)
    b = HipQuantizer(enc_shape, 8, QUANTIZATION_TF_ENHANCED, device)
    for seed in (1, 2, 3, 4):
        x = _data(shape, seed) * (1.0 if seed < 3 else 2.5)  # later batches reach past the fixed range
        ha = a.updateStats(x, return_histogram=True)
        hb = b.updateStats(x, return_histogram=True)
        assert torch.equal(ha, hb), (seed, (ha != hb).sum())
        _same_pdf(a, b)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_pdf_update_16bit_inputs(device, dtype):
    a = OracleQuantizer((), 8, QUANTIZATION_TF_ENHANCED)
    b = HipQuantizer((), 8, QUANTIZATION_TF_ENHANCED, device)
    for seed in (1, 2):
        x = torch.nan_to_num(_data((33000,), seed, dtype), posinf=6e4, neginf=-6e4)
        assert torch.equal(a.updateStats(x, True), b.updateStats(x, True))
        _same_pdf(a, b)


def test_pdf_zero_and_empty_batches(device):
    a = OracleQuantizer((2, 1), 8, QUANTIZATION_TF_ENHANCED)
    b = HipQuantizer((2, 1), 8, QUANTIZATION_TF_ENHANCED, device)
    z = torch.zeros(2, 100)
    for q in (a, b):
        q.updateStats(z)
    _same_pdf(a, b)
    ea, eb = a.computeEncodings(False), b.computeEncodings(False)
    assert np.array_equal(np.array(ea), np.array(eb))
    x = z.clone()
    x[1] = torch.linspace(-1, 3, 100)  # block 0 still all zero: stays uninitialised while block 1 gets its range
    for q in (a, b):
        q.updateStats(x)
    _same_pdf(a, b)
    assert b.stats()[2][:, 1].tolist() == [0, 1]
    x[0] = torch.linspace(-2, 0.5, 100)
    for q in (a, b):
        q.updateStats(x)
    _same_pdf(a, b)
    for sym in (False, True):
        assert np.array_equal(np.array(a.computeEncodings(sym)), np.array(b.computeEncodings(sym)))
    for q in (a, b):
        q.resetEncodingStats()
    _same_pdf(a, b)


def test_empty_tensors_do_not_broadcast(device):
    # a zero-sized dimension is neither equal to nor a multiple of the encoding dimension (tensor_utils.cpp:28-58)
    for shape, t in (((), torch.zeros(0)), ((2, 1), torch.zeros(2, 0))):
        for scheme in (QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED):
            for q in (OracleQuantizer(shape, 8, scheme), HipQuantizer(shape, 8, scheme, device)):
                with pytest.raises(RuntimeError, match="broadcastable"):
                    q.updateStats(t)


def test_pdf_per_channel_rows_with_an_all_zero_row(device):
    """One run per slot (a workgroup per row): a row of zeros stays uninitialised while its neighbours collect."""
    a = OracleQuantizer((3, 1), 8, QUANTIZATION_TF_ENHANCED)
    b = HipQuantizer((3, 1), 8, QUANTIZATION_TF_ENHANCED, device)
    g = torch.Generator().manual_seed(4)
    for k in range(3):
        x = torch.randn(3, 2048, generator=g) * (1 + k)
        if k < 2:
            x[1] = 0.0
        for q in (a, b):
            q.updateStats(x)
        _same_pdf(a, b)
    ea, eb = a.computeEncodings(False), b.computeEncodings(False)
    assert np.array_equal(np.array(ea), np.array(eb))


def test_pdf_update_of_an_empty_tensor_through_the_c_abi(device):
    """UpdatePdf returns at once for cnt == 0 (math_functions.cpp:240-243): only the updated flag changes."""
    from aimet_amd import _lib

    lib = _lib.load()
    xl = torch.zeros(1, 1536, dtype=torch.float64, device=device)
    pdf = torch.zeros_like(xl)
    meta = torch.zeros(1, 4, dtype=torch.int32, device=device)
    st = _lib.DlqPdfState()
    st.num_slots, st.xleft, st.pdf, st.meta = 1, xl.data_ptr(), pdf.data_ptr(), meta.data_ptr()
    lay = _lib.make_layout([0], [1], [0])
    _lib.check(lib.ahq_dlq_pdf_update(_lib.AHQ_F32, lay, None, st, 1, None, None, 0, _lib.current_stream(device)), "update")
    assert meta.cpu().tolist() == [[0, 0, 1, 0]] and float(pdf.abs().sum()) == 0.0



@pytest.mark.parametrize("bw", [4, 8, 16])
@pytest.mark.parametrize("kind", ["normal", "positive", "laplace_outliers", "two_values"])
def test_tfe_encodings_bit_exact(device, kind, bw):
    g = torch.Generator().manual_seed(11)
    if kind == "normal":
        batches = [torch.randn(50000, generator=g) * 2 + 2 for _ in range(3)]
    elif kind == "positive":
        batches = [torch.randn(50000, generator=g).abs() * 1.5 for _ in range(2)]
    elif kind == "laplace_outliers":
        u = torch.rand(100000, generator=g) - 0.5
        x = -torch.sign(u) * torch.log1p(-2 * u.abs())
        x[::1000] = 40.0
        batches = [x, x * 0.5]
    else:
        batches = [torch.tensor([0.0, 1.0] * 500)]
    a = OracleQuantizer((), bw, QUANTIZATION_TF_ENHANCED)
    b = HipQuantizer((), bw, QUANTIZATION_TF_ENHANCED, device)
    for x in batches:
        a.updateStats(x)
        b.updateStats(x)
    _same_pdf(a, b)
    for sym, strict, uns in TFE_MODES:
        for q in (a, b):
            q.setStrictSymmetric(strict)
            q.setUnsignedSymmetric(uns)
        ea, eb = a.computeEncodings(sym), b.computeEncodings(sym)
        assert np.array_equal(np.array(ea), np.array(eb)), (sym, strict, uns, ea, eb)
        assert a.last_best == b.last_best, (sym, strict, uns, a.last_best, b.last_best)


@pytest.mark.parametrize("shape,enc_shape", [((6, 2, 512), (3, 2, 1)), ((48, 2, 256), (24, 2, 1))])
def test_tfe_encodings_per_block(device, shape, enc_shape):
    """6 slots are searched with one wave per candidate, 48 with one lane per candidate."""
    x = _data(shape, 5, special=False)
    a = OracleQuantizer(enc_shape, 8, QUANTIZATION_TF_ENHANCED)
    b = HipQuantizer(enc_shape, 8, QUANTIZATION_TF_ENHANCED, device)
    for q in (a, b):
        q.updateStats(x)
        q.updateStats(x * 0.5 + 1)
    for sym in (False, True):
        ea, eb = a.computeEncodings(sym), b.computeEncodings(sym)
        assert np.array_equal(np.array(ea), np.array(eb))
        assert a.last_best == b.last_best


def test_end_to_end_tf_enhanced_then_qdq(device):
    x = torch.from_numpy(C.INPUTS["normal_mean2_std2"].copy())
    a = OracleQuantizer((), 8, QUANTIZATION_TF_ENHANCED)
    b = HipQuantizer((), 8, QUANTIZATION_TF_ENHANCED, device)
    for q in (a, b):
        q.updateStats(x)
        q.setEncodings(q.computeEncodings(False))
    assert torch.equal(a.quantizeDequantize(x), b.quantizeDequantize(x))


@pytest.mark.parametrize("percentile", [100.0, 99.9999, 99.9, 99.0, 90.0, 50.0])
@pytest.mark.parametrize("enc_shape,shape", [((), (100000,)), ((4, 1), (4, 30000))])
def test_percentile_encodings_bit_exact(device, percentile, enc_shape, shape):
    g = torch.Generator().manual_seed(21)
    a = OracleQuantizer(enc_shape, 8, QUANTIZATION_PERCENTILE)
    b = HipQuantizer(enc_shape, 8, QUANTIZATION_PERCENTILE, device)
    for q in (a, b):
        q.setPercentileValue(percentile)
    for k in range(3):
        x = torch.randn(shape, generator=g) * (1.0 + k) + 0.5
        x.view(-1)[::997] = 25.0  # a thin tail of outliers for the percentile to cut
        a.updateStats(x)
        b.updateStats(x)
    _same_pdf(a, b)
    for bw in (4, 8, 16):
        a.bitwidth = bw
        b.q.bitwidth = bw
        for sym, strict, uns in TFE_MODES:
            for q in (a, b):
                q.setStrictSymmetric(strict)
                q.setUnsignedSymmetric(uns)
            ea, eb = a.computeEncodings(sym), b.computeEncodings(sym)
            assert np.array_equal(np.array(ea), np.array(eb)), (bw, sym, strict, uns, ea, eb)


def test_percentile_value_only_exists_for_the_percentile_scheme(device):
    q = HipQuantizer((), 8, QUANTIZATION_TF_ENHANCED, device)
    with pytest.raises(RuntimeError):
        q.setPercentileValue(90.0)
    q = HipQuantizer((), 8, QUANTIZATION_PERCENTILE, device)
    q.setPercentileValue(90.0)
    assert q.q.getPercentileValue() == 90.0


# ---------------------------------------------------------------------------------------------------- FP8 fake-cast --
def test_fp8_against_torch_cast(make):
    C.check_fp8_against_torch_cast(make)


def test_fp8_reference_edge_cases(make):
    C.check_fp8_edge_cases(make)


def test_fp8_reference_tensors(make):
    C.check_fp8_reference_tensors(make)


def test_fp8_encodings(make):
    C.check_fp8_encodings(make)


def test_fp8_qtype_is_sticky(make):
    C.check_fp8_qtype_is_sticky(make)


@pytest.mark.parametrize("fmt", ["e4m3fn", "e5m2"])
@pytest.mark.parametrize("shape,enc_shape", [((1 << 20,), ()), ((1031,), ()), ((64, 3, 40, 9), (1, 3, 1, 1)),
                                             ((256, 4096), (256, 64)), ((37, 130), (37, 1))])
def test_fp8_qdq_bit_exact(device, fmt, shape, enc_shape):
    """Magnitudes from far below the smallest subnormal to beyond saturation, scales of every size (tiny and huge ones
    take the general division), NaN and infinities: identical bits to the plain-C restatement."""
    layout = C.FP8_FORMATS[fmt][0]
    g = torch.Generator().manual_seed(len(shape) * 131 + len(enc_shape))
    x = torch.randn(shape, generator=g) * torch.exp(torch.rand(shape, generator=g) * 40 - 30)
    f = x.view(-1)
    f[1], f[5], f[7], f[11] = float("nan"), float("inf"), float("-inf"), -0.0
    E = int(np.prod(enc_shape)) if enc_shape else 1
    scales = torch.exp(torch.rand(E, generator=g, dtype=torch.float64) * 20 - 14).tolist()
    if E >= 4:
        scales[0], scales[1], scales[2], scales[3] = 1e-30, 3e25, 1.0, 2.0 ** -70
    encs = [(-s, s, s, 0.0, 8) for s in scales]
    hip, ora = HipQuantizer(enc_shape, layout, QUANTIZATION_TF, device), OracleQuantizer(enc_shape, layout, QUANTIZATION_TF)
    hip.setEncodings(encs)
    ora.setEncodings(encs)
    C._same_floats(hip.quantizeDequantize(x).numpy(), ora.quantizeDequantize(x).numpy())


def test_fp8_c_abi_rejects_bad_arguments(device):
    from aimet_amd import _lib
    from aimet_amd.quantization.affine.backends import hip as H

    lib = _lib.load()
    x = torch.randn(64, device=device)
    s = torch.ones(1, device=device)
    _, layout = H._prepare(x, (), None)
    st = _lib.current_stream(x.device)
    args = (x.data_ptr(), x.data_ptr(), s.data_ptr())
    assert lib.ahq_dlq_fp8_qdq(_lib.DTYPE_CODE[torch.float16], layout, *args, 3, -6, 448.0, st) == _lib.AHQ_ERR_UNSUPPORTED
    assert b"float tensors only" in lib.ahq_last_error()
    assert lib.ahq_dlq_fp8_qdq(_lib.DTYPE_CODE[torch.float32], layout, *args, 3, -6, 0.0, st) == _lib.AHQ_ERR_INVALID
    assert lib.ahq_dlq_fp8_qdq(_lib.DTYPE_CODE[torch.float32], layout, *args, 24, -6, 448.0, st) == _lib.AHQ_ERR_INVALID
    assert lib.ahq_dlq_fp8_qdq(_lib.DTYPE_CODE[torch.float32], layout, x.data_ptr(), x.data_ptr(), None, 3, -6, 448.0,
                               st) == _lib.AHQ_ERR_INVALID
    # in place is allowed, like every element-wise entry point
    y = x.clone()
    assert lib.ahq_dlq_fp8_qdq(_lib.DTYPE_CODE[torch.float32], layout, y.data_ptr(), y.data_ptr(), s.data_ptr(), 3, -6,
                               448.0, st) == _lib.AHQ_OK
    assert torch.equal(y.cpu(), x.cpu().to(torch.float8_e4m3fn).float())
