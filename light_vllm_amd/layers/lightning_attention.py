"""Lightning attention: linear attention whose state S [D, Dv] per head decays by a constant and takes the outer
product of every token's key and value:

    q = silu(W_q h), k = silu(W_k h)   (H heads of D),   v = silu(W_v h)   (H heads of Dv)
    S_t = decay_h * S_(t-1) + k_t v_t^T;   o_t = S_t^T q_t                (no other scale)
    y = W_o [ rms_norm(all heads of o together) * w * sigmoid(W_g h) ]

The decays are constants of the model (one per head), not parameters. Serving state per sequence (one slot of the
engine's state manager): S in f32. A ragged step carries any number of new tokens per sequence from that state; a
sequence without context starts from zeros without the slot being cleared. One GEMM for q | k | v | gate, the
recurrence with silu applied as it reads the projection (mix_ops.lightning_attention), the norm over the whole row
with the gate (mix_ops.head_norm_gate with the row as one head), and the output GEMM.

`share=`: the parameters of another module, a state of its own. `fused_input`: no input projection of its own; the
caller hands `forward` the columns of a wider projection.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops
from ..utils.context import get_context
from .linear import MergedColumnParallelLinear, RowParallelLinear
from .tp import tp_size


class LightningAttention(nn.Module):
    uses_state_slots = True

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, norm_eps: float = 1e-6,
                 share: "LightningAttention | None" = None, fused_input: bool = False):
        super().__init__()
        assert tp_size() == 1, "the lightning attention is not sharded: run it with tensor_parallel_size 1"
        decay = [float(d) for d in decay]
        assert len(decay) == heads and heads >= 1 and dim >= 1 and vdim >= 1
        self.H, self.D, self.Dv, self.decay_values, self.norm_eps = heads, dim, vdim, decay, float(norm_eps)
        self.sizes = [heads * dim, heads * dim, heads * vdim, heads * vdim]          # q | k | v | gate
        if share is None:
            self.in_proj = None if fused_input else MergedColumnParallelLinear(width, self.sizes, bias=False)
            self.o_proj = RowParallelLinear(heads * vdim, width, bias=False)
            self.out_norm_weight = nn.Parameter(torch.ones(heads * vdim, dtype=torch.float32))
        else:
            assert share.sizes == self.sizes and share.decay_values == decay
            self.in_proj, self.o_proj, self.out_norm_weight = share.in_proj, share.o_proj, share.out_norm_weight
        self.decay = torch.tensor([])           # f32 [H], made with the state
        self.state = torch.tensor([])           # [slots, H, D, Dv] f32

    # -- cache protocol of the model runner
    def cache_bytes(self, block_size: int, act_bytes: int) -> tuple[int, int]:
        """(bytes per cache page, bytes per state slot)."""
        return 0, self.H * self.D * self.Dv * 4

    def bind_cache(self, num_blocks: int, block_size: int, num_slots: int, device, dtype) -> None:
        self.state = torch.zeros(num_slots, self.H, self.D, self.Dv, dtype=torch.float32, device=device)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).float().to(device)

    def forward(self, h: torch.Tensor, proj: torch.Tensor | None = None, col0: int = 0) -> torch.Tensor:
        step = get_context().ragged
        if proj is None:
            proj, col0 = self.in_proj(h), 0
        hd, hv = self.H * self.D, self.H * self.Dv
        o = mix_ops.lightning_attention(proj, col0, col0 + hd, col0 + 2 * hd, self.decay, self.state, step, self.H, self.D,
                                        self.Dv)
        gate = proj[:, col0 + 2 * hd + hv:col0 + 2 * hd + 2 * hv]
        y = mix_ops.head_norm_gate(o.view(-1, 1, hv), gate, self.out_norm_weight, self.norm_eps, h.dtype, "sigmoid")
        return self.o_proj(y)
