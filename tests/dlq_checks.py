"""Checks against the expected outputs of DlQuantization's own tests (tests/golden/dlq_vectors.json, dlq_inputs.npz).
`make(shape, bitwidth, scheme)` returns an object with the BlockTensorQuantizer interface of tests/dlq_adapters.py; the
same checks run on the CPU oracle (pinning it) and on the HIP path."""

import bisect
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest
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


# ------------------------------------------------------------------ exact pins of the TF-enhanced statistics and search --
def hand_built_pdfs():
    """Probability tables whose candidate costs lie far apart: name -> (left edges, probabilities).  Bucket edges are
    multiples of a power of two, so every left edge and centre is exact."""
    from tests import tfe_enumeration as T

    out = {}
    xl = T.uniform_buckets(-12.0, 1.0 / 64)
    pdf = np.zeros(1536)
    pdf[640], pdf[992] = 0.7, 0.3                      # mass at the centres of two buckets: -2 and 3.5
    out["two_centres"] = (xl, pdf)
    pdf = np.zeros(1536)
    pdf[600], pdf[840], pdf[1100] = 0.25, 0.5, 0.25    # three centres
    out["three_centres"] = (xl, pdf)
    pdf = np.zeros(1536)
    pdf[768:1025] = np.arange(257)                     # one-sided ramp from 0 to 4
    out["ramp"] = (xl, pdf / pdf.sum())
    pdf = np.zeros(1536)
    pdf[768:832] = 0.999 / 64                          # a block on [0, 1] and a lone outlier at 9
    pdf[768 + 9 * 64] = 0.001
    out["lone_outlier"] = (xl, pdf)
    return out


def _assert_search_equals_enumeration(q, xleft, pdf, bw, symmetric, strict=False, unsigned=False, what=""):
    from tests import tfe_enumeration as T

    q.load_pdf(xleft, pdf)
    (e,) = q.computeEncodings(symmetric)
    best, count = q.last_best[0]
    want = T.search(xleft, pdf, bw, symmetric, strict, unsigned)
    assert count == want["count"], f"{what}: {count} candidates, the enumeration has {want['count']}"
    assert best == want["index"], f"{what}: candidate {best} chosen, the enumeration picks {want['index']}"
    got = (e[0], e[1], e[2], e[3], e[4])
    assert got == (want["min"], want["max"], want["delta"], want["offset"], bw), f"{what}: {got} vs {want}"
    return want


def check_tfe_exact_against_enumeration(make):
    """The chosen (delta, offset), its index and the number of candidates against tests/tfe_enumeration.py, an
    independent array-arithmetic statement of TfEnhancedEncodingAnalyzer.cpp:90-377: on the hand-built tables (whose
    best and second-best costs are far apart, or tie exactly) and on the statistics of the reference tests' inputs."""
    tables = dict(hand_built_pdfs())
    for name in ("normal_mean2_std2", "normal_meanm2_std1"):
        q = make((), 8, TFE)
        q.updateStats(torch.from_numpy(INPUTS[name].copy()))
        xl, pdf, _ = q.stats()
        tables[name] = (xl[0].copy(), pdf[0].copy())
    for name, (xl, pdf) in tables.items():
        for bw in (8, 4, 2, 16):
            for symmetric, strict, unsigned in ((False, False, False), (True, False, False), (True, True, False),
                                                (True, False, True)):
                q = make((), bw, TFE)
                q.setStrictSymmetric(strict)
                q.setUnsignedSymmetric(unsigned)
                want = _assert_search_equals_enumeration(q, xl, pdf, bw, symmetric, strict, unsigned,
                                                         f"{name} bw={bw} sym={symmetric} strict={strict} unsigned={unsigned}")
                if name in ("two_centres", "three_centres", "ramp", "lone_outlier") and bw == 8:
                    c = np.sort(want["costs"])
                    # far apart (no rounding can swap them) or the very same candidate twice (the first one wins)
                    assert c[1] == c[0] or (c[1] - c[0]) > 1e-6 * c[1], name


def check_tfe_closed_forms(make):
    """Two searches whose answer follows by hand.

    All mass in the one bucket [255/16, 256/16) of a table with buckets of 1/16 starting at -32, 8 bits, asymmetric:
    the observed range is [0, 255/16], so delta_max = 1/16 and the grid k/16 holds the range exactly.  A candidate
    whose largest value falls into the mass's own bucket costs nothing (the bucket saturates onto its own centre);
    every candidate with a smaller range costs something.  In the reference's order -- 17 multipliers f = 1/16 ..
    17/16 times 21 offsets, dropping for f <= 1 only the offset -255 (empty after the clamp to the observed range) --
    the first such candidate is f = 16/16 with offset 0: position 15 * 20 + 19 = 319.  The same (1/16, 0) comes again
    from f = 17/16 (cut back to the observed range) and as the appended observed candidate: the FIRST of equal costs
    has to win.  For f = 17/16 the offsets -255 (empty) and -12 (strictly contains the observed range) are dropped:
    16 * 20 + 19 + 1 = 340 candidates.

    Same table, symmetric: delta_max = (255/16) / 127.5 = 1/8, offset -128, multipliers are the running float sum
    0.01, 0.02, ...: 100 of them stay below 1 (the float sum of 100 x 0.01 is 0.99999934), the 101st (1.0099993) is
    still <= 1.01, a 102nd is not: 101 candidates.  Only the last one reaches past the mass's bucket (127 * 1.01 / 8 >
    255/16), so the mass is quantised (error < delta / 2) instead of saturated onto a centre two buckets away at three
    times the cost: the last candidate wins."""
    from tests import tfe_enumeration as T

    xl = T.uniform_buckets(-32.0, 1.0 / 16)
    pdf = np.zeros(1536)
    pdf[512 + 255] = 1.0
    q = make((), 8, TFE)
    q.load_pdf(xl, pdf)
    (e,) = q.computeEncodings(False)
    assert tuple(e) == (0.0, 255.0 / 16, 1.0 / 16, 0.0, 8)
    assert tuple(q.last_best[0]) == (319, 340)
    q = make((), 8, TFE)
    q.load_pdf(xl, pdf)
    (e,) = q.computeEncodings(True)
    f = np.float32(0.01)
    for _ in range(100):
        f = np.float32(np.float64(f) + 0.01)
    delta = np.float32(f * np.float32(0.125))
    assert tuple(q.last_best[0]) == (100, 101)
    assert (e[2], e[3]) == (float(delta), -128.0)
    assert (e[0], e[1]) == (float(np.float32(delta * np.float32(-128))), float(np.float32(delta * np.float32(127))))


def check_tfe_saturation_weight_decides(make):
    """Tables on which the factor 3 on the saturation cost decides the winner: a heavy mass near zero and a light one
    far out, on a coarse grid.  With the factor the search keeps a wider range than it would without; the enumeration
    run with a factor of 1 confirms that the two answers differ, so a dropped or wrong factor cannot pass."""
    from tests import tfe_enumeration as T

    xl = T.uniform_buckets(-32.0, 1.0 / 16)
    for bw, light, far in ((4, 0.05, 900), (2, 0.02, 900), (3, 0.1, 900)):
        pdf = np.zeros(1536)
        pdf[512 + 40], pdf[far] = 1.0 - light, light
        q = make((), bw, TFE)
        want = _assert_search_equals_enumeration(q, xl, pdf, bw, False, what=f"bw={bw}")
        unweighted = T.search(xl, pdf, bw, False, gamma=1.0)
        assert unweighted["delta"] < want["delta"] and unweighted["index"] != want["index"]


def check_pdf_exact_binary_fractions(make):
    """Statistics of inputs that sit on exact binary fractions strictly inside their buckets: no rounding anywhere, so
    the counts must equal a brute-force count with no slack, and the running average of three unequal batches is what
    a hand calculation gives.

    First batch spans [-1, 1]: the range becomes three times that around the centre 0, [-3, 3], in 1536 buckets of
    1/256 whose left edges are (i - 768) / 256."""
    k1 = np.concatenate([np.arange(-256, 256), np.arange(-256, 256, 2)])
    x1 = np.concatenate([(k1 + 0.5) / 256, [-1.0, 1.0]]).astype(np.float32)       # 770 values; -1 and 1 fix the range
    k2 = np.concatenate([np.arange(-700, 700, 7), np.arange(0, 64), np.arange(0, 64)])
    x2 = np.concatenate([(k2 + 0.25) / 256, [5.0, -5.0, 3.0, np.nan, np.inf]]).astype(np.float32)  # the last five fall outside
    k3 = np.arange(-768, 768, 3)
    x3 = ((k3 + 0.75) / 256).astype(np.float32)
    q = make((), 8, TFE)
    hists = [q.updateStats(torch.from_numpy(x.copy()), return_histogram=True)[0].numpy().astype(np.int64) for x in (x1, x2, x3)]
    xl, pdf, meta = q.stats()
    assert np.array_equal(xl[0], (np.arange(1536) - 768) / 256.0)
    brute1 = np.bincount(k1 + 768, minlength=1536)
    brute1[768 - 256] += 1          # -1.0 is the left edge of its bucket
    brute1[768 + 256] += 1          # 1.0 likewise
    brute2 = np.bincount(k2 + 768, minlength=1536)  # 5, -5, 3 (= the right end of the range), NaN and inf are dropped
    brute3 = np.bincount(k3 + 768, minlength=1536)
    for h, b, x in zip(hists, (brute1, brute2, brute3), (x1, x2, x3)):
        assert np.array_equal(h, b)
    assert hists[1].sum() == x2.size - 5
    # running average by hand: ((p1 * 0 + p1) / 1 -> p1; (p1 * 1 + p2) / 2; (that * 2 + p3) / 3), p = counts / batch size
    p1, p2, p3 = brute1 / float(x1.size), brute2 / float(x2.size), brute3 / float(x3.size)
    expect = (((p1 * 1 + p2) / 2) * 2 + p3) / 3
    assert np.array_equal(pdf[0], expect)
    assert tuple(meta[0][:3]) == (3, 1, 1)


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


# ------------------------------------------------------------------------------------------------ FP8 fake-cast ----
# Formats as the adapters take them: (exponent bits, mantissa bits, finite, unsigned zero); torch's storage type of the
# same format serves as an independent decoder of the 256 bit patterns.
FP8_FORMATS = {
    "e4m3fn": ((4, 3, True, False), torch.float8_e4m3fn, 448.0, 3, -6),
    "e5m2": ((5, 2, False, False), torch.float8_e5m2, 57344.0, 2, -14),
}


def fp8_grid(f8dtype):
    """The non-negative finite values of the format in increasing order; index == bit pattern."""
    vals = torch.arange(128, dtype=torch.uint8).view(f8dtype).float()
    vals = vals[torch.isfinite(vals)]
    assert torch.all(vals[1:] > vals[:-1])
    return [Fraction(v) for v in vals.tolist()]


def fp8_brute(x, scale, f8dtype):
    """x / scale and the product with scale in correctly rounded float arithmetic (numpy float32); the cast itself by
    exact search on the enumerated grid, ties to the even bit pattern, saturating."""
    grid = fp8_grid(f8dtype)
    s = np.float32(scale)
    with np.errstate(all="ignore"):
        q = (np.asarray(x, dtype=np.float32) / s).astype(np.float32)
    out = np.empty(q.shape, dtype=np.float32)
    for i, v in enumerate(q.tolist()):
        if math.isnan(v):
            out[i] = np.nan
            continue
        a = grid[-1] if math.isinf(v) else min(Fraction(abs(v)), grid[-1])
        hi = bisect.bisect_left(grid, a)
        if grid[hi] == a:
            pick = hi
        else:
            lo = hi - 1
            dl, dh = a - grid[lo], grid[hi] - a
            pick = lo if dl < dh else hi if dh < dl else (lo if lo % 2 == 0 else hi)
        out[i] = np.float32(math.copysign(float(grid[pick]), v)) * s
    return out


def _fp8_encoding(scale, max_value):
    return (-max_value * scale, max_value * scale, scale, 0.0, 8)


def _same_floats(got, want):
    """Bit-for-bit, signs of zero included; NaN matches NaN."""
    got, want = np.asarray(got, dtype=np.float32).ravel(), np.asarray(want, dtype=np.float32).ravel()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32)), \
        [(i, g, w) for i, (g, w) in enumerate(zip(got, want)) if g != w][:8]


def check_fp8_against_torch_cast(make):
    """Scale 1: inside the finite range the fake-cast is exactly torch's conversion to the storage type and back."""
    rng = np.random.default_rng(11)
    for fmt, f8, max_value, _, _ in FP8_FORMATS.values():
        q = make((), fmt, TF)
        q.setEncodings([_fp8_encoding(1.0, max_value)])
        grid = np.array([float(g) for g in fp8_grid(f8)], dtype=np.float32)
        mids = (grid[1:] + grid[:-1]) / 2  # exact ties
        near = np.concatenate([np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(np.inf))])
        rnd = (rng.standard_normal(20000) * np.exp(rng.uniform(-12, math.log(max_value), 20000))).astype(np.float32)
        tiny = np.array([0.0, 1e-45, 1e-30, float(grid[1]) / 2, float(grid[1]) / 4], dtype=np.float32)
        x = np.concatenate([grid, mids, near, rnd, tiny])
        x = np.concatenate([x, -x])
        x = x[np.abs(x) <= max_value]
        y = q.quantizeDequantize(torch.from_numpy(x)).numpy()
        want = torch.from_numpy(x).to(f8).float().numpy()
        _same_floats(y, want)


def check_fp8_edge_cases(make):
    """The inputs of Fp8QdqCpuGpuBitExactAtEdgeCases (TestTensorQuantizer.cpp:439-510) at its scale 0.3f, against the
    exact search on the enumerated grid; plus saturation and the sign of zero spelled out."""
    for fmt, f8, max_value, mbits, emin in FP8_FORMATS.values():
        f = np.float32
        scale = f(0.3)
        mx = f(max_value)
        step1, sub = f(2.0 ** -mbits), f(2.0 ** (emin - mbits))
        x = np.array([-np.inf, f(-2) * mx * scale, -mx * scale, -(f(1) + f(1.5) * step1) * scale,
                      -(f(1) + f(0.5) * step1) * scale, f(-0.5) * sub * scale, -0.0, 0.0, f(0.5) * sub * scale,
                      (f(1) + f(0.5) * step1) * scale, (f(1) + f(1.5) * step1) * scale, mx * scale, f(2) * mx * scale,
                      np.inf, np.nan], dtype=np.float32)
        q = make((), fmt, TF)
        q.setEncodings([_fp8_encoding(float(scale), max_value)])
        y = q.quantizeDequantize(torch.from_numpy(x)).numpy()
        _same_floats(y, fp8_brute(x, scale, f8))
        assert y[0] == y[1] == -mx * scale and y[-2] == y[-3] == mx * scale
        assert np.signbit(y[6]) and not np.signbit(y[7]) and y[6] == 0 and y[7] == 0
        assert np.isnan(y[-1])


def check_fp8_reference_tensors(make):
    """The tensors and encodings of Fp8PerTensorQdq... / Fp8PerChannelQdq... / their E5M2 twins
    (TestTensorQuantizer.cpp:302-437) against the exact search."""
    data4 = INPUTS["normal_mean2_std2"]
    data1 = np.arange(24, dtype=np.float32).reshape(2, 3, 2, 2)
    for fmt, f8, max_value, _, _ in FP8_FORMATS.values():
        q = make((), fmt, TF)
        q.setEncodings([_fp8_encoding(0.5, max_value)])
        _same_floats(q.quantizeDequantize(torch.from_numpy(data4)).numpy(), fp8_brute(data4, 0.5, f8))
        q = make((1, 3, 1, 1), fmt, TF)
        q.setEncodings([_fp8_encoding(0.25 * (c + 1), max_value) for c in range(3)])
        y = q.quantizeDequantize(torch.from_numpy(data1)).numpy()
        for c in range(3):
            _same_floats(y[:, c], fp8_brute(data1[:, c].ravel(), 0.25 * (c + 1), f8))
        # scales that are not powers of two, blocks along two axes
        x = (np.random.default_rng(5).standard_normal((4, 6, 8)) * 37).astype(np.float32)
        q = make((2, 1, 4), fmt, TF)
        scales = [0.013 * (k + 1) for k in range(8)]
        q.setEncodings([_fp8_encoding(s, max_value) for s in scales])
        y = q.quantizeDequantize(torch.from_numpy(x)).numpy()
        for k in range(8):
            i, j = divmod(k, 4)
            blk = (slice(2 * i, 2 * i + 2), slice(None), slice(2 * j, 2 * j + 2))
            _same_floats(y[blk], fp8_brute(x[blk].ravel(), scales[k], f8))


def check_fp8_encodings(make):
    """TensorQuantizer.cpp:182-224: scale = amax / maxValue from the raw observed extrema under the min/max scheme
    (the example in the reference's comment: observed 7.25 must not become 7.307), from the analyzer's range
    otherwise; delta carries the scale, offset is 0, bw 8, min/max = -/+ scale * maxValue."""
    fmt, _, max_value, _, _ = FP8_FORMATS["e4m3fn"]
    x = torch.tensor([[-7.25, 1.0, 0.5, 3.0], [0.25, 2.0, 5.5, -1.0]])
    q = make((), fmt, TF)
    q.updateStats(x)
    (e,) = q.computeEncodings(False)
    assert e[2] == 7.25 / max_value and e[3] == 0.0 and e[4] == 8
    assert e[0] == -(7.25 / max_value) * max_value and e[1] == (7.25 / max_value) * max_value
    # per block, E5M2
    fmt5, _, max5, _, _ = FP8_FORMATS["e5m2"]
    q = make((2, 1), fmt5, TF)
    q.updateStats(x)
    encs = q.computeEncodings(True)
    assert [e[2] for e in encs] == [7.25 / max5, 5.5 / max5]
    # all-zero statistics: the observed amax is 0, the analyzer's widened range (MIN_RANGE 0.01) decides
    q = make((), fmt, TF)
    q.updateStats(torch.zeros(16))
    (e,) = q.computeEncodings(False)
    twin = make((), 8, TF)
    twin.updateStats(torch.zeros(16))
    (t,) = twin.computeEncodings(False)
    assert e[2] == max(abs(t[0]), abs(t[1])) / max_value > 0
    # histogram schemes keep no raw extrema: the scale follows the searched range
    data = torch.from_numpy(INPUTS["normal_mean2_std2"])
    for scheme in (TFE, PCT):
        q, twin = make((), fmt, scheme), make((), 8, scheme)
        for z in (q, twin):
            z.updateStats(data)
        (e,), (t,) = q.computeEncodings(False), twin.computeEncodings(False)
        assert e[2] == max(abs(t[0]), abs(t[1])) / max_value and e[3] == 0.0 and e[4] == 8
    # end to end: calibrate, set, quantize; every output is on the scaled grid and the largest magnitude survives
    q = make((), fmt, TF)
    q.updateStats(data)
    encs = q.computeEncodings(False)
    q.setEncodings(encs)
    y = q.quantizeDequantize(data).numpy()
    amax = np.abs(data.numpy()).max()
    assert np.abs(y).max() == np.float32(np.float32(448.0) * np.float32(encs[0][2]))
    assert abs(float(np.abs(y).max()) - float(amax)) <= 1e-6 * float(amax)


def check_fp8_qtype_is_sticky(make):
    """SetEncodingsDoesNotChangeFp8QuantizationType (TestTensorQuantizer.cpp:74-90): the legacy bitwidth field follows
    the encodings, the quantization type does not; and 16-bit tensors are refused."""
    fmt, f8, max_value, _, _ = FP8_FORMATS["e4m3fn"]
    q = make((), fmt, TF)
    q.setEncodings([(-448.0, 448.0, 1.0, 0.0, 4)])
    x = torch.tensor([0.3, 1.06, -17.4, 500.0])
    _same_floats(q.quantizeDequantize(x).numpy(), fp8_brute(x.numpy(), 1.0, f8))
    with pytest.raises(RuntimeError, match="float tensors only"):
        q.quantizeDequantize(x.half())
