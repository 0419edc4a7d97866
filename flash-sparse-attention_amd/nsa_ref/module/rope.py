"""Rotary embedding for packed sequences under the reference's names (nsa_ref/module/rope.py:43-134).

The frequency table is computed here from the published "llama3" / default formulas (the
reference obtains it from `transformers`), the rotation itself runs in the gfx950 kernel."""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch
from torch import nn

from fsa_hip import ops as _ops


@dataclass
class RopeConfig:
    max_position_embeddings: int = 131072
    head_dim: int = 128
    rope_theta: float = 500000
    rope_scaling: dict = field(
        default_factory=lambda: {
            "factor": 8.0,
            "high_freq_factor": 4.0,
            "low_freq_factor": 1.0,
            "original_max_position_embeddings": 8192,
            "rope_type": "llama3",
        }
    )
    # unused, kept for compatibility with the reference's dataclass
    hidden_size: int = 4096
    num_attention_heads: int = 32


def _inv_freq(config: RopeConfig) -> torch.Tensor:
    d = config.head_dim
    inv = 1.0 / (config.rope_theta ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d))
    sc = config.rope_scaling
    rope_type = "default" if not sc else sc.get("rope_type", sc.get("type", "default"))
    if rope_type == "default":
        return inv
    if rope_type != "llama3":
        raise NotImplementedError(f"rope_type {rope_type!r}: only 'default' and 'llama3' are implemented")
    factor, lo, hi = sc["factor"], sc["low_freq_factor"], sc["high_freq_factor"]
    old = sc["original_max_position_embeddings"]
    wl = 2 * math.pi / inv
    out = torch.where(wl > old / lo, inv / factor, inv)
    smooth = (old / wl - lo) / (hi - lo)
    mid = (1 - smooth) * out / factor + smooth * out
    is_mid = ~(wl < old / hi) & ~(wl > old / lo)
    return torch.where(is_mid, mid, out)


class _Rotary(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cu_seqlens, inv_freq, scaling, start, stride):
        ctx.save_for_backward(cu_seqlens, inv_freq)
        ctx.args = (scaling, start, stride)
        return _ops.rope(x, cu_seqlens, inv_freq, scaling, start, stride)

    @staticmethod
    def backward(ctx, dy):
        cu_seqlens, inv_freq = ctx.saved_tensors
        scaling, start, stride = ctx.args
        if dy.stride(2) != 1:
            dy = dy.contiguous()
        return _ops.rope(dy, cu_seqlens, inv_freq, scaling, start, stride, inverse=True), None, None, None, None, None


class RotaryEmbedding(nn.Module):
    def __init__(self, config: RopeConfig, device=None):
        super().__init__()
        self.config = config
        self.attention_scaling = 1.0
        self.register_buffer("inv_freq", _inv_freq(config).to(device) if device else _inv_freq(config),
                             persistent=False)

    def forward(self, x: torch.Tensor, cu_seqlens: torch.Tensor, start: int = 0, stride: int = 1):
        """Token j of every sequence is rotated for position start + j * stride."""
        inv = self.inv_freq
        if inv.dtype != torch.float32:  # module.to(bf16) must not degrade the table
            inv = _inv_freq(self.config).to(x.device)
        return _Rotary.apply(x, cu_seqlens, inv.to(x.device), self.attention_scaling, start, stride)
