"""Two sequence mixers side by side: both read the same normed layer input, each output is divided by its root mean
square over the model width and weighted, and the layer takes `scale` times their sum:

    y = scale * ( left(h) / rms(left(h)) * w_left + right(h) / rms(right(h)) * w_right )

The two mixers are built with `fused_input`: their input projections are ONE GEMM here (the left one's columns, then
the right one's; biases of a mixer that has none are zero). `forward` returns the two raw outputs; the norms, the
weights, the scale and the sum belong to the residual update that follows (mix_ops.residual_dyt), which reads
`left_out`, `right_out`, `scale` and `eps` from this module.
"""
from __future__ import annotations

import torch
from torch import nn

from .linear import MergedColumnParallelLinear


class ParallelMixers(nn.Module):

    def __init__(self, width: int, left: nn.Module, right: nn.Module, eps: float = 1e-6, scale: float = 0.5,
                 share: "ParallelMixers | None" = None):
        super().__init__()
        self.left, self.right, self.eps, self.scale = left, right, float(eps), float(scale)
        self.sizes = list(left.sizes) + list(right.sizes)
        self.split = sum(left.sizes)
        if share is None:
            bias = bool(getattr(left, "bias", False) or getattr(right, "bias", False))
            self.in_proj = MergedColumnParallelLinear(width, self.sizes, bias=bias)
            if bias:
                self.in_proj.bias.data.zero_()
            self.left_out = nn.Parameter(torch.ones(width, dtype=torch.float32))
            self.right_out = nn.Parameter(torch.ones(width, dtype=torch.float32))
        else:
            assert share.sizes == self.sizes
            self.in_proj, self.left_out, self.right_out = share.in_proj, share.left_out, share.right_out

    def forward(self, h: torch.Tensor):
        proj = self.in_proj(h)
        return self.left(h, proj, 0), self.right(h, proj, self.split)
