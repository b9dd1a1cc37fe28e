"""The C++ BlockTensorQuantizer facade (include/aimet_amd_dlq.hpp): a small C++ program built against the library runs
the reference's test scenarios on the GPU and prints JSON; every number is compared with the CPU oracle."""

import json
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import dlq_checks as C
from tests.dlq_adapters import FP8_E4M3FN, FP8_E5M2, QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED, OracleQuantizer

pytestmark = pytest.mark.gpu

from oracle import dlq as OD

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "dlq_facade_test.bin")


def test_facade_program_matches_the_oracle(device):
    assert os.path.exists(BIN), f"{BIN} is missing: run __graft_entry__.build()"
    res = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    out = json.loads(res.stdout)
    assert out["throws_before_stats"] is True
    _check_reference_caller(out)
    _check_free_functions(out)

    x = torch.from_numpy(C.INPUTS["normal_mean2_std2"].copy())
    a = OracleQuantizer((), 8, QUANTIZATION_TF_ENHANCED)
    a.updateStats(x)
    a.updateStats(x[:3000])
    asym, sym = a.computeEncodings(False), a.computeEncodings(True)
    assert np.array_equal(np.array(out["tfe_asymmetric"]), np.array(asym))
    assert np.array_equal(np.array(out["tfe_symmetric"]), np.array(sym))
    a.setEncodings(asym)
    y = a.quantizeDequantize(x)[:64]
    assert np.array_equal(np.array(out["tfe_qdq_head"], dtype=np.float32), y.numpy())
    assert out["tfe_hist_buckets"] == 1536

    ramp = (torch.arange(60, dtype=torch.float32) * 0.5 - 15).reshape(1, 4, 5, 3)
    b = OracleQuantizer((3,), 8, QUANTIZATION_TF)
    b.updateStats(ramp)
    encs = b.computeEncodings(False)
    assert np.array_equal(np.array(out["tf_per_channel"]), np.array(encs))
    b.setEncodings(encs)
    assert np.array_equal(np.array(out["tf_per_channel_qdq"], dtype=np.float32), b.quantizeDequantize(ramp).flatten().numpy())
    for e, (lo, hi) in zip(out["tf_per_channel"], C.V["minmax_quantizer"]["asymmetric"]["expected_tf_encoding_min_max"]):
        C.assert_encodings_double_eq(e, C.tf_encoding(lo, hi, 8))

    s = OracleQuantizer((1, 1, 5, 1), 8, QUANTIZATION_TF)
    s.setStrictSymmetric(True)
    s.updateStats(ramp)
    assert np.array_equal(np.array(out["tf_strict_symmetric"]), np.array(s.computeEncodings(True)))

    f = OracleQuantizer((3,), FP8_E4M3FN, QUANTIZATION_TF)
    f.updateStats(ramp)
    encs = f.computeEncodings(False)
    assert np.array_equal(np.array(out["fp8_e4m3_per_channel"]), np.array(encs))
    f.setEncodings(encs)
    assert np.array_equal(np.array(out["fp8_e4m3_per_channel_qdq"], dtype=np.float32), f.quantizeDequantize(ramp).flatten().numpy())
    g = OracleQuantizer((), FP8_E5M2, QUANTIZATION_TF)
    g.setEncodings([(-57344.0 * 0.3, 57344.0 * 0.3, 0.3, 0.0, 4)])
    assert np.array_equal(np.array(out["fp8_e5m2_qdq_head"], dtype=np.float32), g.quantizeDequantize(x)[:256].numpy())
    assert out["fp8_sticky"] == [1, 8, 4]


def _check_reference_caller(out):
    """modeSpecificActionTensorQuantizer (the reference's ONNX Runtime op, typed out in the C++ program) in its four
    modes, with an allocator and a loop runner, on float, half and bfloat16 tensors."""
    x = torch.from_numpy(C.INPUTS["normal_mean2_std2"].copy())
    a = OracleQuantizer((), 8, QUANTIZATION_TF_ENHANCED)
    a.resetEncodingStats()
    a.updateStats(x)
    enc = a.computeEncodings(False)
    assert np.array_equal(np.array(out["op_oneshot_encodings"]), np.array(enc))
    a.setEncodings(enc)
    assert np.array_equal(np.array(out["op_oneshot_qdq_head"], dtype=np.float32), a.quantizeDequantize(x)[:64].numpy())
    assert out["op_update_passes_through"] is True and out["op_pass_through"] is True
    a.updateStats(x)
    a.updateStats(x[:3000])
    enc = a.computeEncodings(True)
    assert np.array_equal(np.array(out["op_after_updates_symmetric"]), np.array(enc))
    a.setEncodings(enc)
    assert np.array_equal(np.array(out["op_qdq_head"], dtype=np.float32), a.quantizeDequantize(x)[:64].numpy())
    # every allocateRaw of the caller's allocator is matched by a deleteRaw, and the allocator was really used; the loop
    # runner has nothing to run on the device
    assert out["allocator"][0] == out["allocator"][1] and out["allocator"][0] >= 3 and out["allocator"][2] == 1
    assert out["allocator_balanced"] is True and out["runner_calls"] == 0

    ramp = (torch.arange(60, dtype=torch.float32) * 0.5 - 15).reshape(1, 4, 5, 3)
    h = OracleQuantizer((3,), 8, QUANTIZATION_TF)
    h.updateStats(ramp.half())
    enc = h.computeEncodings(False)
    assert np.array_equal(np.array(out["half_tf_per_channel"]), np.array(enc))
    h.setEncodings(enc)
    assert np.array_equal(np.array(out["half_tf_per_channel_qdq"], dtype=np.float32),
                          h.quantizeDequantize(ramp.half()).float().flatten().numpy())
    xb = x.bfloat16()
    b = OracleQuantizer((), 8, QUANTIZATION_TF_ENHANCED)
    b.updateStats(xb)
    enc = b.computeEncodings(False)
    assert np.array_equal(np.array(out["bf16_tfe"]), np.array(enc))
    b.setEncodings(enc)
    assert np.array_equal(np.array(out["bf16_tfe_qdq_head"], dtype=np.float32), b.quantizeDequantize(xb)[:64].float().numpy())
    t = OracleQuantizer((), 8, QUANTIZATION_TF)
    t.updateStats(xb[:3000])
    t.updateStats(xb[3000:])
    assert np.array_equal(np.array(out["bf16_tf_two_batches"]), np.array(t.computeEncodings(False)))


def _check_free_functions(out):
    """quantizeDequantize<T>, quantizeDequantizeBroadcast<T>, quantizeDequantizeFp8[Broadcast] and
    getBlockEncodingAnalyzerInstance<float>."""
    x = C.INPUTS["normal_mean2_std2"]
    assert np.array_equal(np.array(out["free_qdq_head"], dtype=np.float32), OD.qdq(x, (-5.0, 7.75, 0.05, -100.0))[:64])
    assert out["cpu_mode_throws"] is True
    ramp = (np.arange(60, dtype=np.float32) * 0.5 - 15).reshape(1, 4, 5, 3)
    encs = [(-15.0, 14.0, 29.0 / 255, -132.0), (-3.0, 3.0, 6.0 / 255, -128.0), (0.0, 10.0, 10.0 / 255, 0.0)]
    assert np.array_equal(np.array(out["free_broadcast_qdq"], dtype=np.float32), OD.qdq_broadcast(ramp, (3,), encs).flatten())
    assert np.array_equal(np.array(out["free_fp8_qdq"], dtype=np.float32), OD.fp8_qdq(ramp.flatten(), 0.07, OD.FP8_E4M3FN))
    assert np.array_equal(np.array(out["free_fp8_broadcast_qdq"], dtype=np.float32),
                          OD.fp8_qdq_broadcast(ramp, (3,), [0.01, 0.05, 0.25], OD.FP8_E4M3FN).flatten())
    s = OracleQuantizer((1, 1, 5, 1), 8, QUANTIZATION_TF)
    s.setStrictSymmetric(True)
    s.updateStats(torch.from_numpy(ramp))
    assert np.array_equal(np.array(out["factory_minmax_strict_symmetric"]), np.array(s.computeEncodings(True)))
    mn, mx = s.stats()
    assert np.array_equal(np.array(out["factory_observed"]), np.stack([mn, mx], axis=1).astype(np.float64))
