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

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "dlq_facade_test.bin")


def test_facade_program_matches_the_oracle(device):
    assert os.path.exists(BIN), f"{BIN} is missing: run __graft_entry__.build()"
    res = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    out = json.loads(res.stdout)
    assert out["throws_before_stats"] is True

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
