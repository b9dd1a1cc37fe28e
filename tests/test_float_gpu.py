"""aimet_torch's float fake-cast on the GPU: the kernel against the CPU restatement bit for bit (signs of zero
included), and the quantizer against the scenarios of the reference's own tests
(TrainingExtensions/torch/test/python/v2/quantization/float/test_float_quantizer.py)."""

import itertools
import warnings

import pytest
import torch

from oracle import torch_ref as O
from tests.float_cases import E2M1_TABLE, FORMATS
from tests.helpers import assert_same_bits

pytestmark = pytest.mark.gpu


def _fq():
    from aimet_amd.quantization import float as F
    return F


def _finfo(name):
    from aimet_amd.quantization.float._finfo import _finfo as FI
    return FI(*FORMATS[name][0])


def _data(shape, dtype, seed, span):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * torch.exp(torch.rand(shape, generator=g) * 16 - 12) * span
    f = x.view(-1)
    f[0], f[1], f[2], f[3], f[4] = float("nan"), float("inf"), float("-inf"), -0.0, 0.0
    f[5], f[6] = 1e-42, -1e-42
    return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("fmt", [(3, 9, False, False), (5, 9, False, False), (4, 6, False, False), (5, 3, False, False),
                                 (2, 6, False, False), (6, 4, False, False), (2, 1, False, False)], ids=str)
@pytest.mark.parametrize("scale", [1.0, 0.7451069355010986, 29.658720016479492])
def test_every_16bit_value_through_a_format_without_a_storage_type(device, fmt, dtype, scale):
    """Formats that torch has no dtype for go through the reference's logarithm formula, whose steps round to the
    tensor's dtype: next to the top of a binade and at a clamp bound that the dtype rounds upward that is not the
    exact cast.  Every bit pattern of the tensor dtype, against the CPU restatement."""
    from aimet_amd.quantization.float._finfo import _finfo as FI

    x = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(dtype)
    sc = torch.tensor(scale)
    mx = O.float_max(*fmt)
    if mx > torch.finfo(dtype).max:
        with pytest.raises(RuntimeError, match="without overflow"):
            _fq().float_quantize_dequantize(x.to(device), FI(*fmt), sc.to(device))
        return
    want = O.float_qdq(x, sc, *fmt)
    got = _fq().float_quantize_dequantize(x.to(device), FI(*fmt), sc.to(device))
    assert_same_bits(got, want, str(fmt))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("name", list(FORMATS))
@pytest.mark.parametrize("scale", [1.0, 0.7451069355010986, 2.0 ** -70])
def test_large_16bit_tensors_go_through_a_table_with_the_same_bits(device, name, dtype, scale):
    """A 16-bit tensor with one encoding and at least 2^22 elements is cast through a table of the cast's value for
    every bit pattern.  Every pattern, repeated until the tensor is large enough (plus a ragged tail), against the
    per-element arithmetic on a tensor below the threshold and against the CPU restatement; quantize as well."""
    from aimet_amd import _lib
    from aimet_amd.quantization.affine.backends.hip import _prepare

    fmt, _ = FORMATS[name]
    fi = _finfo(name)
    if O.float_max(*fmt) > torch.finfo(dtype).max:
        pytest.skip("the format's largest value does not fit the tensor's dtype")
    pats = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(dtype)
    big = torch.cat([pats.repeat(65), pats[:4099]]).to(device)          # 4 264 003 elements: table
    assert _lib.load().ahq_float_cast_workspace_bytes(_lib.DTYPE_CODE[dtype], _prepare(big, (), None)[1]) == 131072
    assert _lib.load().ahq_float_cast_workspace_bytes(_lib.DTYPE_CODE[dtype], _prepare(pats.to(device), (), None)[1]) == 0
    sc = torch.tensor(scale, device=device)
    small = _fq().float_quantize_dequantize(pats.to(device), fi, sc)      # 65 536 elements: per-element arithmetic
    got = _fq().float_quantize_dequantize(big, fi, sc)
    assert_same_bits(got[:65536], small, f"{name}: first copy of the patterns")
    assert_same_bits(got[64 * 65536:65 * 65536], small, f"{name}: last whole copy")
    assert_same_bits(got[65 * 65536:], small[:4099], f"{name}: tail")
    assert_same_bits(small, O.float_qdq(pats, torch.tensor(scale), *fmt), f"{name}: against the restatement")
    from aimet_amd.quantization.float.quantizer import float_quantize
    q_small = float_quantize(pats.to(device), fi, sc)
    q_big = float_quantize(big, fi, sc)
    assert_same_bits(q_big[:65536], q_small, f"{name}: quantize")
    assert_same_bits(q_big[65 * 65536:], q_small[:4099], f"{name}: quantize, tail")
    # per-channel scales, a float32 tensor and a tensor off 16-byte alignment keep the per-element arithmetic
    off = torch.cat([big[:1], big])[1:]
    assert off.data_ptr() % 16 != 0
    assert_same_bits(_fq().float_quantize_dequantize(off, fi, sc)[:65536], small, f"{name}: unaligned tensor")


# ------------------------------------------------------------------------------------- kernel against the oracle --
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("name", list(FORMATS))
@pytest.mark.parametrize("shape,scale_shape,block", [((4099,), (), None), ((64, 515), (64, 1), None),
                                                     ((32, 256), (32, 4), (1, 64)), ((3, 16, 64), (16, 1), None)])
def test_kernel_matches_the_restatement(device, name, dtype, shape, scale_shape, block):
    fmt, _ = FORMATS[name]
    mx = O.float_max(*fmt)
    x = _data(shape, dtype, seed=len(name) * 7 + len(shape), span=min(mx, 3e4))
    g = torch.Generator().manual_seed(17)
    scale = torch.exp(torch.rand(scale_shape, generator=g) * 6 - 4)
    if scale.numel() >= 4:
        scale.view(-1)[0], scale.view(-1)[1] = 1.0, 2.0 ** -70   # the second one leaves the division-free range
    if mx > torch.finfo(torch.result_type(x, scale)).max:
        # bfloat16's range does not fit a float16 computation: torch refuses the clamp bound, and so do we
        with pytest.raises(RuntimeError, match="without overflow"):
            O.float_qdq(x, scale, *fmt, block_size=block)
        with pytest.raises(RuntimeError, match="without overflow"):
            _fq().float_quantize_dequantize(x.to(device), _finfo(name), scale.to(device), block)
        return
    want = O.float_qdq(x, scale, *fmt, block_size=block)
    got = _fq().float_quantize_dequantize(x.to(device), _finfo(name), scale.to(device), block)
    assert got.dtype == want.dtype  # torch's promotion of (x, scale): a float32 tensor scale widens 16-bit inputs
    assert_same_bits(got, want, name)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("name", list(FORMATS))
@pytest.mark.parametrize("shape,scale_shape,block", [((4099,), (), None), ((64, 515), (64, 1), None),
                                                     ((32, 256), (32, 4), (1, 64))])
def test_encoding_quantize_and_dequantize_match_the_restatement(device, name, dtype, shape, scale_shape, block):
    """FloatEncoding.quantize / dequantize / quantize_dequantize (float/encoding.py:140-178) bit for bit, and
    dequantize(quantize(x)) is quantize_dequantize(x)."""
    from aimet_amd.quantization.float.encoding import FloatEncoding

    fmt, _ = FORMATS[name]
    mx = O.float_max(*fmt)
    x = _data(shape, dtype, seed=len(name) * 5 + len(shape), span=min(mx, 3e4))
    g = torch.Generator().manual_seed(23)
    scale = torch.exp(torch.rand(scale_shape, generator=g) * 6 - 4)
    enc = FloatEncoding(fmt[1], fmt[0], fmt[2], fmt[3], scale.to(device), block)
    if mx > torch.finfo(torch.result_type(x, scale)).max:
        with pytest.raises(RuntimeError, match="without overflow"):
            enc.quantize(x.to(device))
        return
    want_q = O.float_quantize(x, scale, *fmt, block_size=block)
    got_q = enc.quantize(x.to(device))
    assert got_q.dtype == want_q.dtype
    assert_same_bits(got_q, want_q, name)
    want = O.float_dequantize(want_q, scale, block)
    got = enc.dequantize(got_q)
    assert_same_bits(got, want, name)
    assert_same_bits(enc.quantize_dequantize(x.to(device)), want, name)


def test_bfloat16_tensor_cast_to_float16_overflows_like_the_conversion(device):
    """The clamp bound 65504 becomes 65536 in bfloat16 (a Python scalar against a bfloat16 tensor), so the largest
    inputs convert to infinity."""
    x = torch.tensor([65280.0, 65536.0, 1e6, -1e6, 60000.0, 65400.0]).to(torch.bfloat16)
    want = O.float_qdq(x, torch.tensor(1.0), 5, 10, False, False)
    got = _fq().float_quantize_dequantize(x.to(device), _finfo("float16"), torch.tensor(1.0, device=device))
    assert_same_bits(got, want)
    assert torch.isinf(want[1]) and torch.isinf(want[2])


def test_input_gradient(device):
    """What autograd derives for the reference's composition: 1 inside the clamp (bounds included), 0 outside, for
    formats with a storage type; zero everywhere for the logarithm-based cast."""
    x = torch.tensor([0.3, -1.7, 500.0, -449.0, 448.0, 2.0, 896.0, 897.0])
    scale = torch.tensor(2.0)
    xr = x.clone().requires_grad_(True)
    O.float_qdq(xr, scale, 4, 3, True, False).backward(torch.arange(1.0, 9.0))
    xd = x.to(device).requires_grad_(True)
    _fq().float_quantize_dequantize(xd, _finfo("float8_e4m3fn"), scale.to(device)).backward(torch.arange(1.0, 9.0, device=device))
    assert_same_bits(xd.grad, xr.grad)
    assert xr.grad.tolist() == [1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 0.0]
    xr = x.clone().requires_grad_(True)
    O.float_qdq(xr, scale, 3, 4, False, False).backward(torch.ones(8))
    xd = x.to(device).requires_grad_(True)
    _fq().float_quantize_dequantize(xd, _finfo("float8_e3m4"), scale.to(device)).backward(torch.ones(8, device=device))
    assert_same_bits(xd.grad, xr.grad)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("name", [n for n, f in FORMATS.items() if f[1] is not None])
@pytest.mark.parametrize("shape,scale_shape,block", [((4099,), (), None), ((64, 515), (64, 1), None),
                                                     ((32, 256), (32, 4), (1, 64)), ((300, 256), (1, 256), None)])
def test_input_gradient_is_what_autograd_derives_for_the_composition(device, name, dtype, shape, scale_shape, block):
    """The backward of .to(storage type).to(dtype) converts the gradient to the storage type and back, so the
    reference's input gradient lies on the simulated format's grid: g * scale, rounded to the format, masked by the
    clamp, divided by the scale.  Arbitrary gradients (not representable in the format, huge, infinite, NaN) against
    autograd through the CPU restatement, bit for bit."""
    fmt, _ = FORMATS[name]
    mx = O.float_max(*fmt)
    x = _data(shape, dtype, seed=len(name) * 3 + len(shape), span=min(mx, 3e4))
    g = torch.Generator().manual_seed(31)
    scale = torch.exp(torch.rand(scale_shape, generator=g) * 6 - 4)
    grad = _data(shape, dtype, seed=77, span=min(mx, 3e4) * 4)
    if mx > torch.finfo(torch.result_type(x, scale)).max:
        pytest.skip("the format's largest value does not fit the computation's dtype")
    xr = x.clone().requires_grad_(True)
    y = O.float_qdq(xr, scale, *fmt, block_size=block)
    y.backward(grad.to(y.dtype))
    xd = x.to(device).requires_grad_(True)
    yd = _fq().float_quantize_dequantize(xd, _finfo(name), scale.to(device), block)
    yd.backward(grad.to(device).to(yd.dtype))
    assert xd.grad.dtype == xr.grad.dtype
    assert_same_bits(xd.grad, xr.grad, f"{name}: input gradient")


# ------------------------------------------------------------------------- the reference's quantizer scenarios --
@pytest.fixture()
def x(device):
    return (torch.arange(-200, 200).view(4, 100) / 100).to(device)


@torch.no_grad()
@pytest.mark.parametrize("name", [n for n, f in FORMATS.items() if f[1] is not None])
def test_qdq_output_standard_dtypes(x, name):
    from aimet_amd.quantization.tensor import DequantizedTensor
    F = _fq()
    (e, m, finite, uz), dtype = FORMATS[name]
    qdq = F.FloatQuantizeDequantize(dtype=dtype).to(x.device)
    assert torch.equal(qdq(x).cpu(), x.cpu().to(dtype).float())
    q1 = F.FloatQuantizeDequantize(dtype=dtype).to(x.device)
    q2 = F.FloatQuantizeDequantize(e, m, finite, uz).to(x.device)
    assert q1._finfo == q2._finfo
    assert (q1.encoding_analyzer is None) == (q1.bitwidth >= 16)
    assert (q2.encoding_analyzer is None) == (q2.bitwidth >= 16)
    o1, o2 = q1(x), q2(x)
    assert torch.equal(o1, o2)
    assert isinstance(o1, DequantizedTensor) and isinstance(o2, DequantizedTensor)
    assert o1.encoding._finfo == o2.encoding._finfo == q1._finfo
    assert o1.dequantize() is o1
    with q1.compute_encodings(), q2.compute_encodings():
        _ = q1(x)
        _ = q2(x)
    p1, p2 = q1(x), q2(x)
    assert torch.equal(p1, p2)
    if q1.bitwidth < 16:
        assert not torch.isclose(o1, p1).all()   # maxval moved from the format's maximum to the observed one
    else:
        assert torch.equal(o1, p1)
    assert p1.encoding.producer is q1 and p2.encoding.producer is q2


@pytest.mark.parametrize("finite,unsigned_zero", [(True, True), (True, False), (False, True)])
def test_special_floats_sanity(device, finite, unsigned_zero):
    F = _fq()
    with pytest.raises(RuntimeError):
        F.FloatQuantizeDequantize(3, 3, finite=finite, unsigned_zero=unsigned_zero)
    qdq = F.FloatQuantizeDequantize(3, 3, finite=False, unsigned_zero=False).to(device)
    qdq._finfo = type(qdq._finfo)(qdq.exponent_bits, qdq.mantissa_bits, finite, unsigned_zero)
    with pytest.raises(RuntimeError):
        qdq(torch.randn(10, device=device))


@torch.no_grad()
def test_qdq_output_non_standard_dtype(device):
    qdq = _fq().FloatQuantizeDequantize(exponent_bits=2, mantissa_bits=1, finite=True, unsigned_zero=False).to(device)
    xt, want = torch.tensor(E2M1_TABLE[0]), torch.tensor(E2M1_TABLE[1])
    assert torch.equal(qdq(xt.to(device)).cpu(), want)


@torch.no_grad()
@pytest.mark.parametrize("dtype", [torch.float8_e5m2, torch.float8_e4m3fn, torch.float8_e5m2fnuz, torch.float8_e4m3fnuz],
                         ids=lambda d: str(d)[6:])
@pytest.mark.parametrize("shape,block_size", [[(100,), None], [(10, 1), None], [(10, 2), (1, 50)], [(2, 2), (5, 50)]])
def test_qdq_compute_encodings(device, dtype, shape, block_size):
    """test_float_quantizer.py:218-280: after calibration every block is fake-cast with largest value = its observed
    absolute maximum."""
    tiny, fmax = torch.finfo(dtype).tiny, torch.finfo(dtype).max
    for xs in (torch.arange(-2, 2, 0.004) * fmax, torch.arange(-0.5, 0.5, 0.001) * fmax):
        xs = xs.view(10, 100)
        qdq = _fq().FloatQuantizeDequantize(dtype=dtype, shape=shape, block_size=block_size).to(device)
        with qdq.compute_encodings():
            _ = qdq(xs.to(device))
        out = qdq(xs.to(device)).cpu()
        scale = qdq.get_scale().cpu().unsqueeze(0)
        if block_size:
            b0, b1 = block_size
        else:
            b0, b1 = xs.shape[-2] // scale.shape[-2], xs.shape[-1] // scale.shape[-1]
        for i, j in itertools.product(range(scale.shape[-2]), range(scale.shape[-1])):
            blk = xs[i * b0:(i + 1) * b0, j * b1:(j + 1) * b1]
            s = scale[..., i, j]
            assert torch.allclose(s, blk.abs().amax() / fmax)
            want = (blk / s).clamp(-fmax, fmax).to(dtype).to(xs.dtype) * s
            assert torch.allclose(out[i * b0:(i + 1) * b0, j * b1:(j + 1) * b1], want, atol=tiny)


def test_allow_overwrite(x):
    q = _fq().FloatQuantizeDequantize(3, 4, shape=(1, 100)).to(x.device)
    with q.compute_encodings():
        q(x)
    q_max = q.maxval.detach().clone()
    q.allow_overwrite(False)
    assert not q.is_overwrite_allowed("maxval")
    with q.compute_encodings():
        q(x * 2)
    assert torch.equal(q_max, q.maxval)
    q.allow_overwrite(True)
    assert q.is_overwrite_allowed("maxval")
    with q.compute_encodings():
        q(x * 2)
    assert torch.equal(q.maxval, q_max * 2)


def test_save_and_load_state_dict(device):
    F = _fq()
    a = F.FloatQuantizeDequantize(dtype=torch.float8_e5m2).to(device)
    b = F.FloatQuantizeDequantize(dtype=torch.float8_e4m3fn, shape=(20, 20), block_size=(5, 5)).to(device)
    dummy = torch.randn(100, 100, generator=torch.Generator().manual_seed(0)).to(device)
    with a.compute_encodings(), b.compute_encodings():
        _ = a(dummy)
        _ = b(dummy)
    assert not torch.allclose(a(dummy), b(dummy))
    a.load_state_dict(b.state_dict())
    assert a._finfo == b._finfo == (4, 3, True, False)
    assert a.shape == b.shape == (20, 20)
    assert a.block_size == b.block_size == (5, 5)
    assert torch.equal(a(dummy), b(dummy))


def test_extreme_values_warning(device):
    from aimet_amd.quantization.encoding_analyzer import MinMaxEncodingAnalyzer
    big = torch.finfo(torch.float16).max
    dummy = torch.arange(start=0, end=big, dtype=torch.float16).to(device)
    qdq = _fq().FloatQuantizeDequantize(dtype=torch.float16, encoding_analyzer=MinMaxEncodingAnalyzer((1,))).to(device)
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        with qdq.compute_encodings():
            qdq(dummy)
        assert len(w) == 1
        assert issubclass(w[-1].category, UserWarning)
        assert "Extreme values" in str(w[-1].message)


def test_default_args_and_non_float_inputs(device):
    F = _fq()
    with pytest.raises(ValueError):
        F.FloatQuantizeDequantize()
    with pytest.raises(ValueError):
        F.FloatQuantizeDequantize(5, 10, dtype=torch.float16)
    qdq = F.FloatQuantizeDequantize(dtype=torch.float16).to(device)
    for dt in (torch.bool, torch.int32):
        t = torch.ones(4, dtype=dt, device=device)
        assert qdq(t) is t


def test_empty_input(device):
    qdq = _fq().FloatQuantizeDequantize(dtype=torch.float8_e4m3fn).to(device)
    out = qdq(torch.empty(0, 16, device=device))
    assert out.shape == (0, 16)
    with qdq.compute_encodings():
        qdq(torch.empty(0, 16, device=device))   # not observed: statistics stay empty, maxval untouched
    assert torch.equal(qdq.maxval.cpu(), torch.tensor(448.0))


def test_from_encodings_round_trip(x):
    F = _fq()
    q = F.FloatQuantizeDequantize(dtype=torch.float8_e4m3fn, shape=(4, 1)).to(x.device)
    with q.compute_encodings():
        q(x)
    enc = q.get_encodings()
    assert enc.mapping == "float" and enc.bitwidth == 8 and enc.granularity == "perchannel"
    q2 = F.FloatQuantizeDequantize.from_encodings(enc)
    assert torch.allclose(q2.maxval, q.maxval)
    assert torch.equal(q2(x), q(x))
    assert enc.to(torch.float16).scale.dtype == torch.float16
    with pytest.raises(RuntimeError):
        enc.to(torch.int32)
