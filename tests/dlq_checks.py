"""Checks against the expected outputs of DlQuantization's own tests (tests/golden/dlq_vectors.json, dlq_inputs.npz).
`make(shape, bitwidth, scheme)` returns an object with the BlockTensorQuantizer interface of tests/dlq_adapters.py; the
same checks run on the CPU oracle (pinning it) and on the HIP path."""

import json
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
V = json.load(open(os.path.join(HERE, "golden", "dlq_vectors.json")))
INPUTS = np.load(os.path.join(HERE, "golden", "dlq_inputs.npz"))
TF, TFE, PCT = 0, 1, 3


def _t(v, dtype=torch.float32):
    return torch.tensor(v, dtype=torch.float32).to(dtype)


def tf_encoding(mn, mx, bw):
    """getTfEncoding of the reference's test library (test_quantization_lib.hpp:162-176)."""
    steps = int(2 ** bw - 1)
    delta = (mx - mn) / float(steps)
    offset = math.copysign(math.floor(abs(mn / delta) + 0.5), mn / delta)  # C round(): half away from zero
    emin = delta * offset
    emax = delta * steps + emin
    if abs(emin) < 1e-10:
        emin = 0.0
    if abs(emax) < 1e-10:
        emax = 0.0
    return emin, emax, delta, offset, bw


def tf_symmetric_encoding(mx, bw):
    """getTfSymmetricEncoding (test_quantization_lib.hpp:178-189)."""
    half_steps = int(2 ** bw - 2)
    pos = half_steps // 2
    delta = mx / pos
    offset = -float(math.ceil(half_steps // 2))
    return offset * delta, delta * pos, delta, offset, bw


def _ulps(a, b):
    if a == b:
        return 0
    ia = np.array([a], dtype=np.float64).view(np.int64)[0]
    ib = np.array([b], dtype=np.float64).view(np.int64)[0]
    if (ia < 0) != (ib < 0):
        return 1 << 62
    return abs(int(ia) - int(ib))


def assert_encodings_double_eq(got, want):
    """compareEncodings: gtest's 4-ulp double equality on min, max, delta, offset; exact bw."""
    for name, g, w in zip(("min", "max", "delta", "offset"), got[:4], want[:4]):
        assert _ulps(float(g), float(w)) <= 4, f"{name}: {g!r} vs {w!r}"
    assert int(got[4]) == int(want[4])


def check_broadcast_qdq(make, dtype):
    for case in V["broadcast_qdq"]["cases"]:
        q = make(case["encoding_shape"], 8, TF)
        q.setEncodings([(mn, mx, d, o, 8) for mn, mx, d, o in zip(case["min"], case["max"], case["delta"], case["offset"])])
        x = _t(case["input"], dtype).reshape(case["input_shape"])
        y = q.quantizeDequantize(x)
        want = _t(case["expected"], dtype).reshape(case["input_shape"])
        assert y.dtype == dtype
        assert torch.equal(y.float(), want.float()), (case["input_shape"], y.flatten().tolist(), want.flatten().tolist())


def check_per_tensor_qdq(make, dtype):
    c = V["per_tensor_qdq"]
    mn, mx = np.float32(c["min"]), np.float32(c["max"])
    delta = np.float32(c["delta_num"] / c["delta_den"])
    offset = np.float32(mn / delta)
    q = make((), 8, TF)
    q.setEncodings([(float(mn), float(mx), float(delta), float(offset), 8)])
    x = _t(c["input"], dtype).reshape(6, 1)
    y = q.quantizeDequantize(x)
    for xi, yi in zip(x.flatten().float().tolist(), y.flatten().float().tolist()):
        clipped = np.float32(max(min(np.float32(xi), mx), mn))
        r = np.float32(clipped / delta - offset)
        r = np.float32(math.copysign(math.floor(abs(float(r)) + 0.5), float(r)))  # std::round
        expected = float(_t([float(np.float32((r + offset) * delta))], dtype).float())
        assert abs(yi - expected) <= 0.001, (xi, yi, expected)
    # 16-bit results stay close to the fp32 result of the same encoding (TestQuantizeDequantizeFp16 / BFloat16)
    h = c["half_case"]
    enc = tf_encoding(h["enc_min"], h["enc_max"], h["bw"])
    q = make((), 8, TF)
    q.setEncodings([enc])
    ref = q.quantizeDequantize(_t(h["input"], torch.float32))
    got = q.quantizeDequantize(_t(h["input"], dtype))
    tol = {torch.float32: 0.0, torch.float16: 0.01, torch.bfloat16: 0.04}[dtype]
    assert (got.float() - ref).abs().max().item() <= tol


def _named(name):
    if name == "iota24":
        return torch.arange(24, dtype=torch.float32)
    if name == "ramp60":
        return torch.arange(60, dtype=torch.float32) * 0.5 - 15
    raise KeyError(name)


def check_minmax_quantizer(make):
    m = V["minmax_quantizer"]
    c = m["per_channel_params"]
    q = make(c["quantizer_shape"], 8, TF)
    q.updateStats(_named(c["input"]).reshape(c["tensor_shape"]))
    encs = q.computeEncodings(False)
    assert len(encs) == 3
    for e, (lo, hi) in zip(encs, c["expected_tf_encoding_min_max"]):
        assert_encodings_double_eq(e, tf_encoding(lo, hi, 8))

    for key in ("asymmetric", "strict_symmetric"):
        c = m[key]
        q = make(c["quantizer_shape"], 8, TF)
        q.setStrictSymmetric(c["strict"])
        q.setUnsignedSymmetric(False)
        x = _named(c["input"]).reshape(c["tensor_shape"])
        q.updateStats(x)
        assert not q.isEncodingValid
        encs = q.computeEncodings(c["symmetric"])
        q.setEncodings(encs)
        assert q.isEncodingValid
        if key == "asymmetric":
            want = [tf_encoding(lo, hi, 8) for lo, hi in c["expected_tf_encoding_min_max"]]
        else:
            want = [tf_symmetric_encoding(mx, 8) for mx in c["expected_tf_symmetric_max"]]
        assert len(encs) == len(want)
        for e, w in zip(encs, want):
            assert_encodings_double_eq(e, w)
        y = q.quantizeDequantize(x).flatten()
        exp = torch.tensor(c["expected_output"])
        # the expected values are printed with six significant digits
        assert (y - exp).abs().max().item() <= c["tolerance"] + 5e-5 * 15 / 10, (y - exp).abs().max().item()
        assert (y - x.flatten()).abs().max().item() <= 0.06


def check_block_minmax(make, dtype):
    b = V["block_minmax"]
    c = b["symmetric"]
    q = make(c["quantizer_shape"], c["bw"], TF)
    x = _t(c["input"], dtype).reshape(c["tensor_shape"])
    q.updateStats(x)
    encs = q.computeEncodings(True)
    q.setEncodings(encs)
    xr = x.float().flatten().tolist()
    # per (row, 3-column block): expected max after the dtype cast; block 2 holds -10*128/127 so its max is 10
    exp_max = [float(_t([v], dtype).float()) for v in c["expected_max"]]
    if dtype != torch.float32:
        exp_max[2] = abs(xr[6]) * 127.0 / 128.0
    for e, m in zip(encs, exp_max):
        assert abs(e[1] - m) <= 0.001 + (0.02 if dtype != torch.float32 else 0), (e, m)
        assert abs(e[0] + e[1] + e[2]) <= 0.001
        assert e[3] == c["expected_offset"]
        assert abs(e[2] - e[1] / 127) <= 0.001
    y = q.quantizeDequantize(x).float().flatten().tolist()
    for i, (xi, yi) in enumerate(zip(xr, y)):
        mn, mx, delta, offset = (np.float32(v) for v in encs[i // 3][:4])
        clipped = np.float32(max(min(np.float32(xi), mx), mn))
        r = np.float32(clipped / delta - offset)
        r = np.float32(math.copysign(math.floor(abs(float(r)) + 0.5), float(r)))
        expected = float(_t([float(np.float32((r + offset) * delta))], dtype).float())
        assert abs(yi - expected) <= 0.001, (i, xi, yi, expected)

    c = b["asymmetric"]
    q = make(c["quantizer_shape"], c["bw"], TF)
    q.updateStats(_t(c["input"], dtype).reshape(c["tensor_shape"]))
    encs = q.computeEncodings(False)
    for e, mx, mn in zip(encs, c["expected_max"], c["expected_min"]):
        assert abs(e[1] - mx) <= e[2] + 0.02 and abs(e[0] - mn) <= e[2] + 0.02
        assert abs(e[2] - (e[1] - e[0]) / 255) <= 0.001
        assert abs(e[3] - e[0] / e[2]) <= 0.001

    c = b["zero_point_shift"]
    q = make(c["quantizer_shape"], c["bw"], TF)
    q.setZeroPointShift(c["shift"])
    q.updateStats(_t(c["input"], dtype).reshape(c["tensor_shape"]))
    encs = q.computeEncodings(True)
    for e, mx, mn in zip(encs, c["expected_max"], c["expected_min"]):
        assert abs(e[1] - mx) <= e[2] and abs(e[0] - mn) <= e[2]
        assert abs(e[2] - (e[1] - e[0]) / 3) <= 0.001
        assert e[3] == c["expected_offset"]
    for sym, strict in ((False, False), (True, True)):
        q.setStrictSymmetric(strict)
        try:
            q.computeEncodings(sym)
        except RuntimeError:
            pass
        else:
            raise AssertionError("zero-point shift must be rejected outside plain symmetric mode")
    q.setStrictSymmetric(False)

    c = b["zero_point_shift_qdq"]
    q = make(c["quantizer_shape"], c["bw"], TF)
    q.setZeroPointShift(c["shift"])
    x = _t(c["input"], dtype).reshape(c["tensor_shape"])
    q.updateStats(x)
    encs = q.computeEncodings(True)
    q.setEncodings(encs)
    for e, mx in zip(encs, c["expected_max"]):
        assert abs(e[1] - mx) <= 0.001 and abs(e[0] + e[1]) <= 0.001 and e[3] == -1.5
    y = q.quantizeDequantize(x).float().flatten()
    assert (y - _t(c["expected_output"], dtype).float()).abs().max().item() <= c["tolerance"]


def check_tfe_all_zero(make):
    c = V["tf_enhanced"]["all_zero"]
    q = make((), c["bw"], TFE)
    q.updateStats(torch.zeros(c["count"]))
    (e,) = q.computeEncodings(False)
    assert abs(e[0] - c["expected_min"]) <= c["tolerance"] and abs(e[1] - c["expected_max"]) <= c["tolerance"]
    assert e[3] == c["expected_offset"] and e[4] == c["bw"]
    # a quantizer that never saw data returns the all-zero failure encoding
    q = make((), c["bw"], TFE)
    try:
        q.computeEncodings(False)
    except RuntimeError:
        pass
    else:
        raise AssertionError("computeEncodings before updateStats must throw")


def check_tfe_properties(make):
    """Bounds the reference asserts for its normal-distributed inputs and constant tensors."""
    d22 = torch.from_numpy(INPUTS["normal_mean2_std2"].copy())
    dm21 = torch.from_numpy(INPUTS["normal_meanm2_std1"].copy())
    # Asymmetric (TestTfEnhancedEncodingAnalyzer.cpp:57-96): covers between 2 and 6 standard deviations
    q = make((), 8, TFE)
    q.updateStats(d22)
    (e,) = q.computeEncodings(False)
    assert 2 - 12 < e[0] < 2 - 4 and 2 + 4 < e[1] < 2 + 12
    # SanityTestTfEnhancedPerTensorQdqCpu (TestTensorQuantizer.cpp:103-140)
    lo, hi = min(0.0, float(d22.min())), max(0.0, float(d22.max()))
    bucket = 3 * (hi - lo) / 1536
    assert abs(e[2] - (hi - lo) / 255) <= 2 * bucket / 255
    assert abs(e[0] - lo) <= bucket + 0.5 * e[2] and abs(e[1] - hi) <= bucket + 0.5 * e[2]
    assert e[4] == 8 and e[2] > 0 and e[3] <= 0
    q.setEncodings([e])
    y = q.quantizeDequantize(torch.full((6000,), 5.0))
    assert y[0].item() != 5.0 and abs(y[0].item() - 5.0) <= 0.5 * e[2]
    # constant tensors (AllSameValuesAsymmetric, :98-131)
    q = make((), 8, TFE)
    q.updateStats(torch.full((6000,), 4.0))
    (e,) = q.computeEncodings(False)
    assert e[0] <= 0 and e[1] >= 3.5
    q = make((), 8, TFE)
    q.updateStats(torch.full((6000,), -5.0))
    (e,) = q.computeEncodings(False)
    assert e[0] <= -4.5 and e[1] >= 0
    # Symmetric / StrictSymmetric (:155-228)
    amax = float(dm21.abs().max())
    for strict, steps, off in ((False, 255, -128), (True, 254, -127)):
        q = make((), 8, TFE)
        q.setStrictSymmetric(strict)
        q.updateStats(dm21)
        (e,) = q.computeEncodings(True)
        assert e[0] > -amax and e[1] < amax
        assert np.float32(e[2]) == np.float32((e[1] - e[0]) / steps) or abs(e[2] - (e[1] - e[0]) / steps) <= 4e-7 * abs(e[2])
        assert abs(e[3] - e[0] / e[2]) <= 4e-7 * abs(e[3])
        assert e[3] == off and e[4] == 8
        if strict:
            assert e[0] == -e[1]
    # SymmetricUnsigned (:230-280): values clipped at zero
    clipped = dm21.clamp_min(0.0)
    q = make((), 8, TFE)
    q.setUnsignedSymmetric(True)
    q.updateStats(clipped)
    (e,) = q.computeEncodings(True)
    amax = float(clipped.abs().max())
    assert e[0] == 0 and abs(e[1] - amax) <= 0.015 + 3 * (2 * amax) / 1536
    assert abs(e[2] - (e[1] - e[0]) / 255) <= 4e-7 * abs(e[2])
    # EncodingAnalyzerWrapper TfEnhancedMode (TestEncodingAnalyzerWrapper.cpp:99-144)
    c = V["tf_enhanced"]["wrapper"]
    q = make((), c["bw"], TFE)
    q.updateStats(_t(c["input"]).reshape(c["tensor_shape"]))
    _, pdf, _ = q.stats()
    assert abs(pdf.sum() - 1.0) <= 0.001
    (e,) = q.computeEncodings(False)
    assert abs(e[1] - c["expected_max"]) <= c["tolerance"] and abs(e[0] - c["expected_min"]) <= c["tolerance"]
    assert abs(e[3] - e[0] / e[2]) <= 0.001
    q.setZeroPointShift(0.5)
    try:
        q.computeEncodings(True)
    except RuntimeError:
        pass
    else:
        raise AssertionError("TF-enhanced must reject a zero-point shift")


def check_percentile(make):
    """test/TestPercentileEncodingAnalyzer.cpp:21-296: the reference's bounds and exact expectations."""
    d100k = torch.from_numpy(INPUTS["normal_mean2_std2_100k"].copy())
    dm21 = torch.from_numpy(INPUTS["normal_meanm2_std1"].copy())
    # Asymmetric, 99.9999 %, 100000 samples of N(2, 2): between 2 and 6 standard deviations each side
    q = make((), 8, PCT)
    q.setPercentileValue(99.9999)
    q.updateStats(d100k)
    (e,) = q.computeEncodings(False)
    assert 2 - 12 < e[0] < 2 - 4 and 2 + 4 < e[1] < 2 + 12
    amax = float(dm21.abs().max())
    for strict, steps, off in ((False, 255, -128), (True, 254, -127)):
        q = make((), 8, PCT)
        q.setPercentileValue(99.9)
        q.setStrictSymmetric(strict)
        q.updateStats(dm21)
        (e,) = q.computeEncodings(True)
        assert e[0] > -amax and e[1] < amax
        assert abs(e[2] - (e[1] - e[0]) / steps) <= 4e-7 * abs(e[2])
        assert abs(e[3] - e[0] / e[2]) <= 4e-7 * abs(e[3])
        assert e[3] == off and e[4] == 8
        if strict:
            assert e[0] == -e[1]
    # SymmetricUnsigned, 99.9999 %
    clipped = dm21.clamp_min(0.0)
    q = make((), 8, PCT)
    q.setPercentileValue(99.9999)
    q.setUnsignedSymmetric(True)
    q.updateStats(clipped)
    (e,) = q.computeEncodings(True)
    assert e[0] == 0 and abs(e[1] - float(clipped.max())) <= 0.015
    assert abs(e[2] - (e[1] - e[0]) / 255) <= 4e-7 * abs(e[2])
    # percentile 100: the full observed range
    q = make((), 8, PCT)
    q.setPercentileValue(100)
    q.updateStats(dm21)
    (e,) = q.computeEncodings(True)
    assert e[1] < amax + 1536 and e[3] == -128 and e[4] == 8
    assert abs(e[2] - (e[1] - e[0]) / 255) <= 4e-7 * abs(e[2])
    # constant tensors
    q = make((), 8, PCT)
    q.setPercentileValue(99.9999)
    q.updateStats(torch.full((6000,), 4.0))
    (e,) = q.computeEncodings(False)
    assert e[0] <= 0 and e[1] >= 3.99006
    q = make((), 8, PCT)
    q.setPercentileValue(99.9999)
    q.updateStats(torch.full((6000,), -5.0))
    (e,) = q.computeEncodings(False)
    assert e[0] <= -4.99992 and e[1] >= 0
    # all zeros
    q = make((), 8, PCT)
    q.setPercentileValue(99.9999)
    q.updateStats(torch.zeros(6000))
    (e,) = q.computeEncodings(False)
    assert abs(e[0] + 1.00392) <= 1e-4 and abs(e[1] - 0.996078) <= 1e-4 and e[3] == -128 and e[4] == 8
