"""SwiGLU: silu(gate) * up over the two halves of the last dim (reference "native" backend,
lightvllm/layers/activation.py:7-29), the clamped gated unit with a sigmoid of slope alpha, PolyNorm,
a learned cubic of the row-normalised powers of its input, and the gated unit with a choice of activation."""
import torch
import torch.nn.functional as F
from torch import nn

from .. import mix_ops, ops
from .fused import use_fused


class SiluAndMul(nn.Module):

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if use_fused(x):
            return ops.silu_and_mul(x)
        gate, up = torch.chunk(x, 2, dim=-1)
        return F.silu(gate) * up


class ClampedGLU(nn.Module):
    """min(g, L) * sigmoid(alpha * g) * (clamp(u, -L, L) + 1) over [gate | up] halves of the last dim."""

    def __init__(self, limit: float, alpha: float = 1.702):
        super().__init__()
        self.limit, self.alpha = float(limit), float(alpha)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return mix_ops.clamped_glu(x, self.limit, self.alpha)


class PolyNorm(nn.Module):
    """c1 R(z) + c2 R(z^2) + c3 R(z^3) + c0 over the last dim, powers element by element, R(u) = u / sqrt(mean(u^2) + eps)
    per token; coef = (c1, c2, c3, c0), f32."""

    def __init__(self, eps: float = 1e-6):
        super().__init__()
        self.eps = float(eps)
        self.coef = nn.Parameter(torch.tensor([1.0, 0.0, 0.0, 0.0], dtype=torch.float32))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return mix_ops.polynorm(x, self.coef, self.eps)


class GatedAct(nn.Module):
    """act(gate) * up over the [gate | up] halves of the last dim; act: "gelu_tanh" (0.5 z (1 + tanh(sqrt(2/pi) (z +
    0.044715 z^3)))), "gelu" (the exact form) or "relu2"."""

    def __init__(self, act: str = "gelu_tanh"):
        super().__init__()
        assert act in mix_ops.ACTS
        self.act = act

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return mix_ops.glu_act(x, self.act)
