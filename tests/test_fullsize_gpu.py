"""The kernels at the full sizes of the benchmark configurations, where the CPU oracle would take too long for a unit
test: properties that do not depend on size (idempotence, consistency between the three operations, linearity of the
backward pass in the upstream gradient, additivity of counts, agreement of a strided sample with the oracle)."""

import pytest
import torch

from oracle import torch_ref as O
from tests.helpers import assert_same_bits

pytestmark = pytest.mark.gpu


def _affine():
    from aimet_amd.quantization import affine
    return affine


# (name, tensor shape, dtype, encoding shape, block size, qmin, qmax, symmetric)
CONFIGS = [
    ("c1", (32, 64, 112, 112), torch.float32, (), None, 0, 255, False),
    ("c2", (4096, 4096), torch.float32, (4096, 1), None, -128, 127, True),
    ("c4", (14336, 4096), torch.bfloat16, (14336, 64), (1, 64), -8, 7, True),
]


def _make(name, shape, dtype, enc_shape, block, qmin, qmax, symmetric, device):
    g = torch.Generator(device=device).manual_seed(0)
    if name == "c1":
        x = torch.relu(torch.randn(shape, generator=g, device=device))
    else:
        x = torch.randn(shape, generator=g, device=device) * 0.02
    x = x.to(dtype)
    from aimet_amd.quantization._stats import reduce_min_max
    mn, mx = reduce_min_max(x, enc_shape, block)
    mn, mx = mn.float(), mx.float()
    if symmetric:
        amax = torch.maximum(mn.abs(), mx.abs()).clamp_min(1e-8)
        scale = amax / qmax
        offset = torch.zeros_like(scale)
    else:
        scale = ((mx - mn) / (qmax - qmin)).clamp_min(1e-8)
        offset = torch.round(mn / scale) - qmin
    grad = torch.randn(shape, generator=g, device=device).to(dtype)
    return x, scale, offset, grad


@pytest.mark.parametrize("cfg", CONFIGS, ids=lambda c: c[0])
def test_qdq_properties_at_full_size(device, cfg):
    A = _affine()
    name, shape, dtype, enc_shape, block, qmin, qmax, symmetric = cfg
    x, scale, offset, grad = _make(*cfg, device)
    s_req = scale.clone().requires_grad_(True)   # learnable scale: the composed (true-division) arithmetic
    y = A.quantize_dequantize(x, s_req, offset, qmin, qmax, block_size=block).detach()
    # idempotence: a tensor that is already on the grid maps to itself
    y2 = A.quantize_dequantize(y, s_req, offset, qmin, qmax, block_size=block).detach()
    assert torch.equal(y.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       y2.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    # the three operations agree: dequantize(quantize(x)) is quantize_dequantize(x), codes are integers on the grid
    codes = A.quantize(x, s_req, offset, qmin, qmax, block_size=block).detach()
    c = codes.as_subclass(torch.Tensor).float()
    assert bool(((c >= qmin) & (c <= qmax) & (c == c.round())).all())
    dq = A.dequantize(codes.as_subclass(torch.Tensor), s_req.detach(), offset, block_size=block)
    assert torch.equal(dq.as_subclass(torch.Tensor), y.as_subclass(torch.Tensor))
    # a strided sample against the oracle (elementwise operation: rows can be checked on their own)
    rows = slice(0, shape[0], max(1, shape[0] // 16))
    sub_scale = scale if scale.dim() == 0 else scale[rows]
    sub_off = offset if offset.dim() == 0 else offset[rows]
    ref = O.qdq_v2_forward(x[rows].cpu(), sub_scale.cpu(), sub_off.cpu(), qmin, qmax, block)
    assert_same_bits(y[rows].as_subclass(torch.Tensor), ref.y, f"{name} sample")


@pytest.mark.parametrize("cfg", CONFIGS, ids=lambda c: c[0])
def test_backward_is_linear_in_the_upstream_gradient(device, cfg):
    """gx, gscale and goffset of 2g are exactly twice those of g (a power of two commutes with every rounding), gx is
    g or 0, and a strided sample of gx matches the oracle."""
    A = _affine()
    name, shape, dtype, enc_shape, block, qmin, qmax, symmetric = cfg
    x, scale, offset, grad = _make(*cfg, device)

    def run(g):
        xd = x.clone().requires_grad_(True)
        sd = scale.clone().requires_grad_(True)
        od = offset.clone().requires_grad_(True)
        A.quantize_dequantize(xd, sd, od, qmin, qmax, block_size=block).backward(g)
        return xd.grad, sd.grad, od.grad

    gx1, gs1, go1 = run(grad)
    gx2, gs2, go2 = run(grad * 2)
    assert torch.equal(gx2.float(), gx1.float() * 2)
    assert torch.equal(gs2, gs1 * 2) and torch.equal(go2, go1 * 2)
    assert bool(((gx1 == grad) | (gx1 == 0)).all())
    rows = slice(0, shape[0], max(1, shape[0] // 16))
    sub_scale = scale if scale.dim() == 0 else scale[rows]
    sub_off = offset if offset.dim() == 0 else offset[rows]
    gx_ref, _, _ = O.qdq_v2_backward(grad[rows].cpu(), x[rows].cpu(), sub_scale.cpu(), sub_off.cpu(), qmin, qmax, block)
    assert_same_bits(gx1[rows], gx_ref, f"{name} gx sample")


@pytest.mark.parametrize("cfg", CONFIGS, ids=lambda c: c[0])
def test_minmax_at_full_size(device, cfg):
    """Against torch's own reductions on the device, and: the extrema of the whole are the extrema of its halves."""
    from aimet_amd.quantization._stats import reduce_min_max
    name, shape, dtype, enc_shape, block, *_ = cfg
    x = _make(*cfg, device)[0]
    mn, mx = reduce_min_max(x, enc_shape, block)
    if enc_shape == ():
        assert mn == x.amin() and mx == x.amax()
        h = shape[0] // 2
        a, b = reduce_min_max(x[:h], (), None), reduce_min_max(x[h:], (), None)
        assert mn == torch.minimum(a[0], b[0]) and mx == torch.maximum(a[1], b[1])
    elif block is None:
        assert torch.equal(mn, x.amin(dim=1, keepdim=True)) and torch.equal(mx, x.amax(dim=1, keepdim=True))
    else:
        v = x.view(shape[0], enc_shape[1], block[1])
        assert torch.equal(mn, v.amin(dim=2)) and torch.equal(mx, v.amax(dim=2))


def test_histogram_counts_are_additive_at_full_size(device):
    """One batch of the calibration stream ([8, 2048, 4096] float32): every finite element is counted once; feeding
    the same batch again leaves the range alone and doubles every count; a second, narrower batch only adds."""
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    g = torch.Generator(device=device).manual_seed(1)
    u = (torch.rand((8, 2048, 4096), generator=g, device=device) - 0.5).clamp_(-0.4999999, 0.4999999)
    x = -torch.sign(u) * torch.log1p(-2 * u.abs())
    del u
    obs = _HistogramObserver((1,), num_bins=512)
    first = obs.update(x)[0]
    n = x.numel()
    assert float(first.histogram.double().sum()) == n
    assert first.min == x.amin() and first.max == x.amax()
    h1 = obs.get_stats()[0].histogram.clone()
    obs.update(x)
    h2 = obs.get_stats()[0].histogram
    assert torch.equal(h2, h1 * 2)
    obs.update(x * 0.5)
    h3 = obs.get_stats()[0].histogram
    assert float(h3.double().sum()) == 3 * n
    assert bool((h3 >= h2).all())
    # the batch's own histogram against torch.histc on the device (same formula, counts below 2^24 are exact)
    lo, hi = float(first.min), float(first.max)
    assert torch.equal(first.histogram.view(-1), torch.histc(x, 512, lo, hi))


def _laplace_with_outliers(shape, seed, device):
    """One batch of the calibration stream: Laplace(0, 1), 0.1 % of the elements replaced by +-U(20, 60)."""
    g = torch.Generator(device=device).manual_seed(seed)
    u = (torch.rand(shape, generator=g, device=device) - 0.5).clamp_(-0.4999999, 0.4999999)
    x = -torch.sign(u) * torch.log1p(-2 * u.abs())
    n = x.numel()
    k = n // 1000
    idx = torch.randint(0, n, (k,), generator=g, device=device)
    out = (torch.rand(k, generator=g, device=device) * 40 + 20) * torch.sign(torch.rand(k, generator=g, device=device) - 0.5)
    x.view(-1)[idx] = out
    return x


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_histogram_stream_and_candidate_search_at_the_benchmark_shape(device, dtype):
    """Four batches of [8, 2048, 4096] through SqnrEncodingAnalyzer(512 bins, 100 x 64 candidates, 8-bit asymmetric)
    against the oracle on the same batches: running counts (the fullest bin passes 2^24 with the third batch, from
    where float32 counts round), edges, range, the candidate chosen and the encoding, bit for bit.  bf16: the same
    through the table-binning kernel."""
    from aimet_amd.quantization.encoding_analyzer import SqnrEncodingAnalyzer

    an = SqnrEncodingAnalyzer((1,), num_bins=512, asymmetric_delta_candidates=100, offset_candidates=64, gamma=3.0)
    ref = O.HistObserver((1,), 512)
    for b in range(4):
        x = _laplace_with_outliers((8, 2048, 4096), b, device).to(dtype)
        an.update_stats(x)
        ref.update(x.cpu())
        del x
    st, st_ref = an.observer.get_stats()[0], ref.stats[0]
    assert float(st_ref.histogram.max()) > 2 ** 24
    assert_same_bits(st.histogram, st_ref.histogram, "running counts")
    assert_same_bits(st.bin_edges, st_ref.bin_edges, "bin edges")
    assert_same_bits(st.min, st_ref.min, "min")
    assert_same_bits(st.max, st_ref.max, "max")
    lo, hi = an.compute_encodings(255, False)
    lo_r, hi_r, _, _, best = O.sqnr_encodings(ref.stats, (1,), 255, False, asym_deltas=100, num_offsets=64, gamma=3.0)
    assert int(an.last_search["best_index"].item()) == int(best.item())
    assert_same_bits(lo, lo_r, "encoding min")
    assert_same_bits(hi, hi_r, "encoding max")


def test_decoder_layer_at_the_benchmark_shape(device):
    """One decoder layer of the whole-model configuration (hidden 2048, FFN 8192, 32 heads, sequence 2048, bf16;
    W4 blocks of 64, A16 per tensor at every Linear input and output; a small vocabulary keeps the CPU side short):
    two calibration batches through aimet_amd.nn.compute_encodings, then a quantized forward.  Every quantizer's
    calibrated range, scale and offset, and its output in the quantized forward, against the oracle on the very
    tensors it saw."""
    import llama_harness as LH
    from aimet_amd import nn as qnn
    from aimet_amd.quantization.affine import QuantizeDequantize

    cfg = LH.LlamaConfig(layers=1, hidden=2048, ffn=8192, heads=32, vocab=4096)
    model = LH.build(cfg, device, seed=0)
    assert LH.quantize(model) == 8
    quantizers = {n: m for n, m in model.named_modules() if isinstance(m, QuantizeDequantize)}
    weights = {f"{n}.param_quantizers.weight": m.weight for n, m in model.named_modules()
               if isinstance(m, qnn.QuantizedLinear)}
    assert len(quantizers) == 24 and len(weights) == 8
    stats = {}

    def observe(name, q):
        def hook(_mod, args, _out):
            a, b = O.reduce_minmax(args[0].detach().cpu(), tuple(q.shape), q.block_size)
            if name in stats:
                a, b = torch.minimum(a, stats[name][0]), torch.maximum(b, stats[name][1])
            stats[name] = (a, b)
        return hook

    hooks = [q.register_forward_hook(observe(n, q)) for n, q in quantizers.items() if n not in weights]
    batches = LH.calibration_batches(cfg, device, batches=2, seq=2048)
    LH.calibrate(model, batches)
    for h in hooks:
        h.remove()
    for name, w in weights.items():  # (no hook on these: they take the one-call form, on the weight itself)
        q = quantizers[name]
        stats[name] = O.reduce_minmax(w.detach().cpu(), tuple(q.shape), q.block_size)
    for name, q in quantizers.items():
        lo, hi = O.minmax_encodings(*stats[name], q.qmax - q.qmin, q.symmetric)
        assert_same_bits(q.min.detach(), lo.view(q.shape).to(torch.float32), f"{name}: min")
        assert_same_bits(q.max.detach(), hi.view(q.shape).to(torch.float32), f"{name}: max")
        scale = O.scale_from_minmax(q.min.detach().cpu(), q.max.detach().cpu(), q.qmin, q.qmax)
        assert_same_bits(q.get_scale().detach(), scale, f"{name}: scale")
        assert_same_bits(q.get_offset().detach(),
                         O.offset_from_minmax(q.min.detach().cpu(), scale, q.qmin, q.qmax, q.symmetric), f"{name}: offset")
    io = {}
    hooks = [q.register_forward_hook(lambda _m, args, out, key=n: io.__setitem__(key, (args[0].detach().cpu(),
                                                                                        out.detach().cpu())))
             for n, q in quantizers.items()]
    with torch.no_grad():
        logits = model(batches[0])
    for h in hooks:
        h.remove()
    assert torch.isfinite(logits.float()).all() and len(io) == 24
    for name, q in quantizers.items():
        x, y = io[name]
        scale, offset = q.get_scale().detach().cpu(), q.get_offset().detach().cpu()
        if q.block_size is None:
            want = O.qdq_v1(x, scale, offset, q.qmin, q.qmax)[0]   # no gradients: the ATen fake-quantize arithmetic
        else:
            want = O.qdq_v2_forward(x, scale, offset, q.qmin, q.qmax, q.block_size).y
        assert_same_bits(y.as_subclass(torch.Tensor), want, f"{name}: forward")


def test_tf_enhanced_pdf_at_the_benchmark_shape(device):
    """DlQuantization's TF-enhanced statistics on batches of the calibration stream ([8, 2048, 4096] float32), by
    properties that do not need a CPU pass over 67 M elements: the first batch fixes the range and every one of its
    elements is counted; the integer histogram of a batch equals torch.histc over the same buckets on the device; the
    same batch fed twice leaves the probabilities where they were (a running average of equal terms); a batch scaled
    down by two only moves probability towards the middle; the search returns an encoding inside the range."""
    from aimet_amd import dlq

    x = _laplace_with_outliers((8, 2048, 4096), 3, device)
    n = x.numel()
    q = dlq.BlockTensorQuantizer((), 8, dlq.QUANTIZATION_TF_ENHANCED, device=device)
    h1 = q.updateStats(x, return_histogram=True).view(-1)
    assert int(h1.sum()) == n  # the range is the first batch's own: nothing falls outside it
    left = q._xleft.view(-1).clone()
    pdf1 = q._pdf.view(-1).clone()
    width = float(left[1] - left[0])
    lo = float(left[0])
    hi = lo + width * dlq.PDF_SIZE
    assert lo <= float(x.amin()) and float(x.amax()) <= hi
    # same buckets by an independent route: floor((x - lo) / width) in float64 on the device, away from bucket edges
    pos = (x.double().view(-1) - lo) / width
    clear = (pos - pos.round()).abs() > 1e-4
    want = torch.bincount(pos[clear].floor().long().clamp_(0, dlq.PDF_SIZE - 1), minlength=dlq.PDF_SIZE)
    unclear = int((~clear).sum())
    assert int((h1.long() - want).abs().sum()) <= 2 * unclear and unclear < n // 1000
    assert torch.allclose(pdf1, h1.double() / n, rtol=0, atol=1e-15)
    h2 = q.updateStats(x, return_histogram=True).view(-1)
    assert torch.equal(h2, h1)
    assert torch.allclose(q._pdf.view(-1), pdf1, rtol=0, atol=1e-15)
    q.updateStats(x * 0.5)
    pdf3 = q._pdf.view(-1)
    assert abs(float(pdf3.sum()) - 1.0) < 1e-9
    mid = dlq.PDF_SIZE // 2
    assert float(pdf3[mid - 200:mid + 200].sum()) > float(pdf1[mid - 200:mid + 200].sum())
    encs = q.computeEncodings(False)
    (enc,) = encs
    e_min, e_max = float(enc[0]), float(enc[1])
    assert lo - width <= e_min < 0.0 < e_max <= hi + width
    q.setEncodings(encs)
    y = q.quantizeDequantize(x)
    assert float(y.amin()) >= e_min - 1e-3 and float(y.amax()) <= e_max + 1e-3
    assert float((y - x).abs()[(x > e_min) & (x < e_max)].max()) <= (e_max - e_min) / 255 * 0.5001


def test_tensors_of_more_than_two_to_the_31_elements(device):
    """A 288 GB device holds tensors whose element index does not fit 32 bits.  One bfloat16 tensor of 2^31 + 98760
    elements (4.3 GB): min/max finds values planted past the 2^31st element and in the last one; the forward and the
    input gradient of chunks at the start, across the 2^31 boundary and at the end equal those chunks computed alone;
    the offset gradient counts the clipped elements; per-row statistics and encodings on a [65537, 32768] view of the
    same memory; the histogram counts every element."""
    from aimet_amd.quantization import affine
    from aimet_amd.quantization._stats import reduce_min_max
    from aimet_amd.quantization.encoding_analyzer import _HistogramObserver

    free, _ = torch.cuda.mem_get_info()
    if free < 40 << 30:
        pytest.skip("needs 40 GB of free device memory")
    n = (1 << 31) + 8 * 12345
    g = torch.Generator(device=device).manual_seed(0)
    x = torch.empty(n, dtype=torch.bfloat16, device=device)
    step = 1 << 28
    for i in range(0, n, step):
        x[i:i + step] = torch.randn(min(step, n - i), generator=g, device=device).to(torch.bfloat16)
    x[(1 << 31) + 5] = 300.0
    x[n - 1] = -400.0
    mn, mx = reduce_min_max(x, ())
    assert float(mn) == -400.0 and float(mx) == 300.0

    scale = torch.tensor(0.05, device=device)
    offset = torch.tensor(-128.0, device=device)
    with torch.no_grad():
        y = affine.quantize_dequantize(x, scale, offset, 0, 255)
    m = 1 << 20
    starts = (0, (1 << 31) - m // 2, n - m)
    for lo in starts:
        with torch.no_grad():
            part = affine.quantize_dequantize(x[lo:lo + m].clone(), scale, offset, 0, 255)
        assert torch.equal(part.view(torch.int16), y[lo:lo + m].view(torch.int16)), lo
    del y

    xg = x.requires_grad_(True)
    s = scale.clone().requires_grad_(True)
    o = offset.clone().requires_grad_(True)
    out = affine.quantize_dequantize(xg, s, o, 0, 255)
    out.backward(torch.ones(1, dtype=torch.bfloat16, device=device).expand(n))
    del out
    x = x.detach()
    clipped = 0
    for lo in range(0, n, step):
        q = (x[lo:lo + step].float() / 0.05).round() + 128
        clipped += int(((q < 0) | (q > 255)).sum())
    for lo in starts:
        q = (x[lo:lo + m].float() / 0.05).round() + 128
        assert torch.equal(xg.grad[lo:lo + m], ((q >= 0) & (q <= 255)).to(torch.bfloat16)), lo
    assert clipped >= 2 and abs(float(o.grad) - 0.05 * clipped) <= 1e-3 * 0.05 * clipped  # a clipped element adds scale
    del xg

    rows, cols = 65537, 32768
    xr = x[:rows * cols].view(rows, cols)
    mn, mx = reduce_min_max(xr, (rows, 1))
    for r in (0, 12345, rows - 1):
        assert float(mn[r]) == float(xr[r].amin()) and float(mx[r]) == float(xr[r].amax()), r
    sc = (mx.float() - mn.float()).clamp_min(1e-3) / 255
    of = torch.round(mn.float() / sc)
    with torch.no_grad():
        yr = affine.quantize_dequantize(xr, sc, of, 0, 255)
        for r in (0, 40000, rows - 1):
            part = affine.quantize_dequantize(xr[r:r + 1].clone(), sc[r:r + 1], of[r:r + 1], 0, 255)
            assert torch.equal(part.view(torch.int16), yr[r:r + 1].view(torch.int16)), r
    del yr

    obs = _HistogramObserver((1,), num_bins=512)
    first = obs.update(x)[0]
    assert float(first.min) == -400.0 and float(first.max) == 300.0
    assert abs(float(first.histogram.double().sum()) - n) <= n * 1e-6  # float32 counts: every bin rounds once


# (name, tensor shape, dtype, encoding shape, block size): one encoding per element of the fastest axis, which the
# column-walking kernels serve -- 16-byte vectors per lane, stacked problems (blocks along the leading axis), and one
# element per lane where the rows are no multiple of a vector
COLUMN_CONFIGS = [
    ("per_column_bf16", (8192, 4096), torch.bfloat16, (1, 4096), None),
    ("blocks_64x1_bf16", (8192, 4096), torch.bfloat16, (128, 4096), (64, 1)),
    ("per_column_odd_fp32", (4099, 4099), torch.float32, (1, 4099), None),
]


@pytest.mark.parametrize("cfg", COLUMN_CONFIGS, ids=lambda c: c[0])
def test_column_layouts_at_full_size(device, cfg):
    """Min/max against torch's reductions; forward output and input gradient of a sample of rows, and scale / offset
    gradients of a sample of columns (a column's sums involve no other column), against the oracle."""
    from aimet_amd.quantization._stats import reduce_min_max
    from tests.helpers import assert_close_rel

    A = _affine()
    name, shape, dtype, enc_shape, block = cfg
    qmin, qmax = -128, 127
    g = torch.Generator(device=device).manual_seed(3)
    x = (torch.randn(shape, generator=g, device=device) * torch.linspace(0.5, 2.0, shape[1], device=device)).to(dtype)
    grad = torch.randn(shape, generator=g, device=device).to(dtype)
    groups = enc_shape[0]                       # 1, or the number of blocks along the leading axis
    rows_per_group = shape[0] // groups
    xv = x.view(groups, rows_per_group, shape[1])

    mn, mx = reduce_min_max(x, enc_shape, block)
    assert torch.equal(mn, xv.amin(dim=1)) and torch.equal(mx, xv.amax(dim=1))

    # encodings that clip a few per cent of the values, so that every gradient term occurs
    scale = (torch.maximum(mn.float().abs(), mx.float().abs()) / qmax * 0.6).clamp_min(1e-6)
    offset = torch.zeros_like(scale)
    xd = x.clone().requires_grad_(True)
    sd = scale.clone().requires_grad_(True)
    od = offset.clone().requires_grad_(True)
    y = A.quantize_dequantize(xd, sd, od, qmin, qmax, block_size=block)
    y.backward(grad)

    # rows: a few whole groups, or every 85th row (elementwise results)
    if groups > 1:
        gsel = sorted({0, groups // 2, groups - 1})
        rsel = torch.cat([torch.arange(i * rows_per_group, (i + 1) * rows_per_group) for i in gsel])
        sub_scale, sub_off, sub_block = scale[gsel].cpu(), offset[gsel].cpu(), block
    else:
        rsel = torch.arange(0, shape[0], max(1, shape[0] // 96))
        sub_scale, sub_off, sub_block = scale.cpu(), offset.cpu(), None
    ref = O.qdq_v2_forward(x[rsel].cpu(), sub_scale, sub_off, qmin, qmax, sub_block)
    assert_same_bits(y.detach()[rsel].as_subclass(torch.Tensor), ref.y, f"{name}: output, sample of rows")
    gx_ref, _, _ = O.qdq_v2_backward(grad[rsel].cpu(), x[rsel].cpu(), sub_scale, sub_off, qmin, qmax, sub_block)
    assert_same_bits(xd.grad[rsel], gx_ref, f"{name}: input gradient, sample of rows")

    # columns: all rows of 48 columns spread over the width, with their own encodings
    csel = torch.arange(0, shape[1], max(1, shape[1] // 48))[:48]
    _, gs_ref, go_ref = O.qdq_v2_backward(grad[:, csel].cpu(), x[:, csel].cpu(), scale[:, csel].cpu(), offset[:, csel].cpu(),
                                          qmin, qmax, block)
    assert bool((xd.grad == 0).any()) and bool((od.grad != 0).any())
    assert_close_rel(sd.grad[:, csel], gs_ref, 4e-5, f"{name}: scale gradient, sample of columns")
    assert_close_rel(od.grad[:, csel], go_ref, 4e-5, f"{name}: offset gradient, sample of columns")
