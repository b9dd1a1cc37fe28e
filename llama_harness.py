"""A random-init bf16 Llama-style decoder and its quantization set-up, used by bench.py and the whole-model tests.

Only the quantize-dequantize and calibration kernels under test are this repository's; the GEMMs, attention, norms and
rotary embedding below are plain PyTorch-ROCm calls (fused RMS norm, rotary tables formed once per sequence length).
The quantization layout is the one of the benchmark configuration: 4-bit symmetric blockwise weights (block 64 along
the input dimension) and 16-bit asymmetric per-tensor quantize-dequantize at the input and output of every nn.Linear.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
from torch import nn
from torch.nn import functional as F

from aimet_amd import nn as qnn
from aimet_amd.quantization.affine import QuantizeDequantize


@dataclass
class LlamaConfig:
    layers: int = 16
    hidden: int = 2048
    ffn: int = 8192
    heads: int = 32
    vocab: int = 32000
    rope_theta: float = 10000.0
    eps: float = 1e-5


class RMSNorm(nn.Module):
    def __init__(self, dim, eps):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        return F.rms_norm(x, self.weight.shape, self.weight, self.eps)  # one fused kernel, statistics in float32


def rotary_tables(seq: int, head_dim: int, theta: float, device, dtype):
    """cos / sin of the rotary angles, [1, 1, seq, head_dim] in the model's dtype, the two halves of the last axis
    alike: a function of the sequence length only, so a model forms them once and every layer uses them."""
    half = head_dim // 2
    freqs = 1.0 / (theta ** (torch.arange(0, half, device=device, dtype=torch.float32) / half))
    ang = torch.arange(seq, device=device, dtype=torch.float32)[:, None] * freqs[None, :]
    ang = torch.cat([ang, ang], dim=-1)
    return ang.cos()[None, None].to(dtype), ang.sin()[None, None].to(dtype)


def rotary(x, cos, sin):
    # x: [B, H, T, D]; x * cos + rotate_half(x) * sin
    half = x.shape[-1] // 2
    return x * cos + torch.cat([-x[..., half:], x[..., :half]], dim=-1) * sin


class Attention(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        h = cfg.hidden
        self.q_proj = nn.Linear(h, h, bias=False)
        self.k_proj = nn.Linear(h, h, bias=False)
        self.v_proj = nn.Linear(h, h, bias=False)
        self.o_proj = nn.Linear(h, h, bias=False)

    def forward(self, x, rope):
        B, T, C = x.shape
        H = self.cfg.heads
        q = self.q_proj(x).view(B, T, H, C // H).transpose(1, 2)
        k = self.k_proj(x).view(B, T, H, C // H).transpose(1, 2)
        v = self.v_proj(x).view(B, T, H, C // H).transpose(1, 2)
        q, k = rotary(q, *rope), rotary(k, *rope)
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return self.o_proj(y.transpose(1, 2).reshape(B, T, C))


class MLP(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.gate_proj = nn.Linear(cfg.hidden, cfg.ffn, bias=False)
        self.up_proj = nn.Linear(cfg.hidden, cfg.ffn, bias=False)
        self.down_proj = nn.Linear(cfg.ffn, cfg.hidden, bias=False)

    def forward(self, x):
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


class Block(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.input_norm = RMSNorm(cfg.hidden, cfg.eps)
        self.attn = Attention(cfg)
        self.post_norm = RMSNorm(cfg.hidden, cfg.eps)
        self.mlp = MLP(cfg)

    def forward(self, x, rope):
        x = x + self.attn(self.input_norm(x), rope)
        return x + self.mlp(self.post_norm(x))


class Llama(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        self.embed = nn.Embedding(cfg.vocab, cfg.hidden)
        self.blocks = nn.ModuleList([Block(cfg) for _ in range(cfg.layers)])
        self.norm = RMSNorm(cfg.hidden, cfg.eps)
        self.lm_head = nn.Linear(cfg.hidden, cfg.vocab, bias=False)
        self._rope = {}

    def rope(self, seq: int, like: torch.Tensor):
        key = (seq, like.device, like.dtype)
        if key not in self._rope:
            self._rope[key] = rotary_tables(seq, self.cfg.hidden // self.cfg.heads, self.cfg.rope_theta,
                                            like.device, like.dtype)
        return self._rope[key]

    def forward(self, ids):
        x = self.embed(ids)
        rope = self.rope(ids.shape[1], x)
        for b in self.blocks:
            x = b(x, rope)
        return self.lm_head(self.norm(x))


def build(cfg: LlamaConfig, device, seed: int = 0, dtype=torch.bfloat16) -> Llama:
    """Random-init weights ~ N(0, 0.02), made on the device (there is no checkpoint to load)."""
    with torch.device(device):
        model = Llama(cfg)
    g = torch.Generator(device=device).manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() >= 2:
                p.copy_(torch.randn(p.shape, generator=g, device=device) * 0.02)
    return model.to(dtype)


def quantize(model: Llama, weight_bitwidth: int = 4, block: int = 64, act_bitwidth: int = 16) -> int:
    """W<weight_bitwidth> blockwise (block along the input dimension) + A<act_bitwidth> per-tensor asymmetric at every
    Linear input and output.  Returns the number of wrapped layers."""
    dev = next(model.parameters()).device

    def make(_name, linear):
        out_f, in_f = linear.weight.shape
        wq = QuantizeDequantize((out_f, in_f // block), weight_bitwidth, symmetric=True, block_size=(1, block))
        iq = QuantizeDequantize((), act_bitwidth, symmetric=False)
        oq = QuantizeDequantize((), act_bitwidth, symmetric=False)
        return iq.to(dev), wq.to(dev), oq.to(dev)

    return qnn.wrap_linears(model, make)


def calibration_batches(cfg: LlamaConfig, device, batches: int = 8, seq: int = 2048, batch: int = 1, seed: int = 1):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, cfg.vocab, (batch, seq), generator=g).to(device) for _ in range(batches)]


def calibrate(model: nn.Module, batches):
    """compute_encodings over ``batches`` (the reference flow: aimet_torch.nn.compute_encodings around forward passes)."""
    from aimet_amd import nn as qnn

    with torch.no_grad(), qnn.compute_encodings(model):
        for b in batches:
            model(b)


def linear_flops(cfg: LlamaConfig, tokens: int) -> float:
    per_layer = 4 * cfg.hidden * cfg.hidden + 3 * cfg.hidden * cfg.ffn
    return 2.0 * tokens * (cfg.layers * per_layer + cfg.hidden * cfg.vocab)


def weight_elements(cfg: LlamaConfig) -> int:
    return cfg.layers * (4 * cfg.hidden * cfg.hidden + 3 * cfg.hidden * cfg.ffn) + cfg.hidden * cfg.vocab
