"""RMSNorm and fused residual-add + RMSNorm with the reference's rounding points
(lightvllm/layers/layernorm.py:28-80): fp32 math, one rounding to the activation dtype before the
weight multiply, the new residual rounded once from the fp32 sum. OffsetRMSNorm: the norm of models
that keep their residual in f32 and hold the norm weight as an offset from one. DynamicTanh: a norm without
statistics, tanh(alpha x) w + b, on the same kind of residual."""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops, ops
from .fused import use_fused


class RMSNorm(nn.Module):

    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))

    def rms_forward(self, x: torch.Tensor) -> torch.Tensor:
        dtype = x.dtype
        xf = x.to(torch.float32)
        var = xf.pow(2).mean(-1, True)
        xf = xf * torch.rsqrt(var + self.eps)
        return xf.to(dtype).mul_(self.weight)

    def add_rms_forward(self, x: torch.Tensor, residual: torch.Tensor):
        dtype = x.dtype
        xf = x.to(torch.float32) + residual.to(torch.float32)
        residual = xf.to(dtype)
        var = xf.pow(2).mean(-1, True)
        xf = xf * torch.rsqrt(var + self.eps)
        return xf.to(dtype).mul_(self.weight), residual

    def forward(self, x: torch.Tensor, residual: torch.Tensor | None = None):
        if use_fused(x):    # one HIP launch; the residual is updated in place
            out = ops.add_rms_norm(x, residual, self.weight, self.eps)
            return out if residual is None else (out, residual)
        if residual is None:
            return self.rms_forward(x)
        return self.add_rms_forward(x, residual)


class OffsetRMSNorm(nn.Module):
    """x / sqrt(mean(x^2) + eps) * (offset + w) on an f32 residual, fused with the residual update that
    precedes it: `forward(x, y1, y2)` adds up to two sublayer outputs to x in place and returns the normed
    row in the activation dtype (mix_ops.residual_add_norm, one launch). The weight is f32."""

    def __init__(self, hidden_size: int, eps: float = 1e-6, offset: float = 1.0):
        super().__init__()
        self.hidden_size, self.eps, self.offset = hidden_size, eps, float(offset)
        self.weight = nn.Parameter(torch.zeros(hidden_size, dtype=torch.float32))

    def forward(self, x: torch.Tensor, y1=None, y2=None, act_dtype=None) -> torch.Tensor:
        return mix_ops.residual_add_norm(x, y1, y2, self.weight, self.offset, self.eps, act_dtype)


class DynamicTanh(nn.Module):
    """tanh(alpha * x) * w + b, element by element, with a learned scalar alpha and vectors w, b (all f32): no mean and no
    variance are computed. Fused with the residual update that precedes it: `forward(x, y1, y2)` adds up to two sublayer
    outputs to the f32 residual x in place, or with post weights `pair_scale` times the sum of the two outputs each
    divided by its root mean square and weighted (two mixers side by side), and returns the normed row in the activation
    dtype (mix_ops.residual_dyt, one launch)."""

    def __init__(self, hidden_size: int):
        super().__init__()
        f32 = dict(dtype=torch.float32)
        self.weight = nn.Parameter(torch.ones(hidden_size, **f32))
        self.bias = nn.Parameter(torch.zeros(hidden_size, **f32))
        self.alpha = nn.Parameter(torch.ones(1, **f32))

    def forward(self, x: torch.Tensor, y1=None, y2=None, post_w1=None, post_w2=None, pair_scale: float = 1.0,
                pair_eps: float = 1e-6, act_dtype=None) -> torch.Tensor:
        return mix_ops.residual_dyt(x, y1, y2, post_w1, post_w2, pair_scale, pair_eps, self.alpha, self.weight, self.bias,
                                    act_dtype)
