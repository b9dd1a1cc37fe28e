"""A seeded slice of a random sweep over tensor shapes, encoding shapes, block sizes, dtypes and grids: quantize-dequantize
forward and backward through the backend against the CPU oracle.  Outputs and input gradients bit for bit; scale and
offset gradients within a tolerance that knows about cancelling sums (both sides add float32 terms, in different
orders)."""

import math
import random

import pytest
import torch

from oracle import torch_ref as O
from tests.helpers import assert_same_bits, assert_close_rel

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 5, 8, 16, 24, 33, 64, 100, 128, 257, 512, 1000]


def _draw(rng: random.Random):
    """(tensor shape, encoding shape, block size or None, dtype, symmetric) of one case."""
    nd = rng.choice([1, 2, 2, 3, 3, 4])
    shape = [rng.choice(SIZES) for _ in range(nd)]
    while math.prod(shape) > 1_500_000:
        k = rng.randrange(nd)
        shape[k] = max(1, shape[k] // 2)
    k = rng.randint(0, nd)
    enc, block = [], []
    for d in shape[nd - k:]:
        choice = rng.random()
        if choice < 0.4:
            enc.append(1)
            block.append(-1)
        elif choice < 0.75:
            enc.append(d)
            block.append(1)
        else:
            b = rng.choice([b for b in range(1, d + 1) if d % b == 0])
            enc.append(d // b)
            block.append(b)
    blocked = any(e not in (1, d) for e, d in zip(enc, shape[nd - k:])) or rng.random() < 0.2
    bs = tuple(block) if (blocked and k > 0) else None
    if bs is None:
        enc = [e if e in (1, d) else d for e, d in zip(enc, shape[nd - k:])]
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    return shape, enc, bs, dtype, rng.random() < 0.5


@pytest.mark.parametrize("seed", range(8))
def test_random_layouts_forward_and_backward(device, seed):
    from aimet_amd.quantization import affine

    rng = random.Random(1000 + seed)
    done = 0
    for it in range(40):
        shape, enc, bs, dtype, sym = _draw(rng)
        per_enc = math.prod(shape) / max(1, math.prod(enc))
        if dtype != torch.float32 and per_enc > 20000:
            continue  # the oracle's own 16-bit sums round partial sums away at that length
        qmin, qmax = (-128, 127) if sym else (0, 255)
        g = torch.Generator().manual_seed(seed * 1000 + it)
        x = (torch.randn(shape, generator=g) * 1.2).to(dtype)
        gr = torch.randn(shape, generator=g).to(dtype)
        scale = torch.rand(enc, generator=g) * 0.05 + 0.005
        offset = torch.full(enc, 0.0) if sym else torch.randint(-200, -50, enc, generator=g).float()
        try:
            tr = O.qdq_v2_forward(x, scale, offset, qmin, qmax, bs)
            gx_ref, gs_ref, go_ref = O.qdq_v2_backward(gr, x, scale, offset, qmin, qmax, bs)
        except RuntimeError:
            continue  # a combination the reference refuses as well
        desc = f"seed {seed} case {it}: shape {shape} encodings {enc} block {bs} {dtype} symmetric {sym}"
        xd = x.to(device).requires_grad_(True)
        sd = scale.to(device).requires_grad_(True)
        od = offset.to(device).requires_grad_(True)
        y = affine.quantize_dequantize(xd, sd, od, qmin, qmax, block_size=bs)
        y.backward(gr.to(device))
        assert_same_bits(y, tr.y, desc + ": output")
        assert_same_bits(xd.grad, gx_ref, desc + ": input gradient")
        if tr.dtype == torch.float32:
            tol = 2e-4
            # sums that cancel: a few float32 units of the largest term a sum can hold
            floor = 64 * 6e-8 * float(gr.float().abs().max()) * (qmax - qmin) * max(1.0, float(scale.max()))
        else:
            tol = float(torch.finfo(tr.dtype).eps) * (1 if per_enc <= 1000 else 64)
            floor = 1e-30
        assert_close_rel(sd.grad, gs_ref, tol, desc + ": scale gradient", abs_floor=floor)
        assert_close_rel(od.grad, go_ref, tol, desc + ": offset gradient", abs_floor=floor)
        done += 1
    assert done >= 20
