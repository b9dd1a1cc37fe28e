"""The numpy restatement (oracle/decompose.py) and the device path (aimet_amd/quantization/_decompose.py) behind one
call signature, so the same checks (tests/decompose_checks.py) run against both.  CPU torch tensors in and out."""

import torch

from oracle import decompose as OD


def oracle_decompose(x, qmin, qmax, scale_shape, block_size=None, zero_point_shift=0.0):
    q, scale = OD.decompose(x.detach().float().cpu().numpy(), qmin, qmax, tuple(scale_shape), block_size,
                            zero_point_shift)
    return torch.from_numpy(q.copy()), torch.from_numpy(scale.copy())


def product_decompose(device):
    from aimet_amd.quantization._decompose import _decompose_prequantized_tensor

    def run(x, qmin, qmax, scale_shape, block_size=None, zero_point_shift=0.0):
        q, scale = _decompose_prequantized_tensor(x.to(device), qmin, qmax, tuple(scale_shape), block_size,
                                                  zero_point_shift)
        assert q.device.type == torch.device(device).type and scale.device.type == torch.device(device).type
        return q.cpu(), scale.cpu()

    return run
