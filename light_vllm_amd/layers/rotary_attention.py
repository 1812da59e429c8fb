"""Causal softmax attention with grouped key/value heads, rotated positions, a learned temperature per
query head and a sigmoid output gate, on the paged cache of ragged steps.

    q = W_q h + b_q, k = W_k h + b_k, v = W_v h + b_v            (biases optional)
    optionally every query and key head is divided by its root mean square, sqrt(mean(head^2) + unit_norm_eps)
    the first rot_dims entries of every query and key head are rotated: entry i pairs with i + rot_dims/2 (or, with
    `interleaved`, entry 2i with 2i + 1), angle = position * f_i, f_i = base^(-2i/rot_dims), optionally rescaled by
    wavelength (mix_ops.rotary_inv_freq)
    score_h(i, j) = q_h(i) . k_g(j) * scale * temp_h,  g = h / (H / G), over the positions j <= i that i sees:
        all of them; those with i - j < window; those of i's own chunk, floor(i / chunk) == floor(j / chunk);
        in each case also the first keep_first positions
    softmax over the visible keys, with `sink` the exponential of a learned number per head in the denominator as well
    o_h = sum_j p_h(i, j) v_g(j) * sigmoid(W_g h)_h              (gate: one number per head, per channel, or none)
    y = W_o [o_h]_h + b_o                                        (bias optional)

One GEMM for q | k | v | gate, one launch that rotates (f32 angles), folds the head temperature into the
queries and writes keys and values to the cache (mix_ops.rotary_store), the paged attention kernel with a
window no sequence reaches, no pooled blocks and no sink, which also applies the gate, and the output GEMM.
Prompts, portions of prompts and single decoded tokens are one code path.

A module built with `share=` runs with the parameters of another one and keeps a cache of its own: the same
layer applied again at another depth of the model. A module built with `fused_input` has no input projection: the
caller hands `forward` the columns of a wider projection that it computed for several mixers at once.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops
from ..utils.context import get_context
from .linear import MergedColumnParallelLinear, RowParallelLinear
from .tp import tp_size

NO_WINDOW = 1 << 30       # a window no sequence reaches: plain causal attention


class GatedRotaryAttention(nn.Module):
    uses_pages = True

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, rot_dims: int = 0,
                 rot_base: float = 10000.0, rot_scaling: dict | None = None, bias: bool = True, head_temp: bool = True,
                 gate: str | None = "head", share: "GatedRotaryAttention | None" = None, interleaved: bool = False,
                 window: int = NO_WINDOW, keep_first: int = 0, chunk: int = 0, sink: bool = False,
                 unit_norm_eps: float | None = None, out_bias: bool = False, fused_input: bool = False):
        super().__init__()
        assert tp_size() == 1, "the gated rotary attention is not sharded: run it with tensor_parallel_size 1"
        assert heads % kv_heads == 0 and gate in ("head", "channel", None)
        assert 0 <= rot_dims <= dim and rot_dims % 2 == 0 and window >= 1 and keep_first >= 0 and chunk >= 0
        self.H, self.G, self.D, self.Dv = heads, kv_heads, dim, vdim
        self.scale, self.rot_dims, self.rot_base, self.rot_scaling = float(scale), rot_dims, float(rot_base), rot_scaling
        self.gate, self.bias, self.interleaved = gate, bias, interleaved
        self.window, self.keep_first, self.chunk, self.unit_norm_eps = window, keep_first, chunk, unit_norm_eps
        gate_size = {"head": heads, "channel": heads * vdim, None: 0}[gate]
        self.sizes = [heads * dim, kv_heads * dim, kv_heads * vdim] + ([gate_size] if gate_size else [])
        if share is None:
            self.in_proj = None
            if not fused_input:
                self.in_proj = MergedColumnParallelLinear(width, self.sizes, bias=bias)       # q | k | v | gate
                if bias:
                    self.in_proj.bias.data.zero_()   # the gate's part has no bias in the checkpoint and stays 0
            self.o_proj = RowParallelLinear(heads * vdim, width, bias=out_bias)
            self.temp = nn.Parameter(torch.ones(heads, dtype=torch.float32)) if head_temp else None
            self.sink = nn.Parameter(torch.zeros(heads, dtype=torch.float32)) if sink else None
        else:
            assert (share.sizes, share.H, share.G, share.D, share.Dv) == (self.sizes, heads, kv_heads, dim, vdim)
            self.in_proj, self.o_proj, self.temp, self.sink = share.in_proj, share.o_proj, share.temp, share.sink
        self.inv_freq = None                         # f32 [rot_dims/2], made with the cache
        self.k_cache = self.v_cache = torch.tensor([])

    # -- cache protocol of the model runner
    def cache_bytes(self, block_size: int, act_bytes: int) -> tuple[int, int]:
        return block_size * self.G * (self.D + self.Dv) * act_bytes, 0

    def bind_cache(self, num_blocks: int, block_size: int, num_slots: int, device, dtype) -> None:
        kw = dict(dtype=dtype, device=device)
        self.k_cache = torch.zeros(num_blocks, block_size, self.G, self.D, **kw)
        self.v_cache = torch.zeros(num_blocks, block_size, self.G, self.Dv, **kw)
        self.inv_freq = mix_ops.rotary_inv_freq(max(self.rot_dims, 2), self.rot_base, device, self.rot_scaling)

    def forward(self, h: torch.Tensor, proj: torch.Tensor | None = None, col0: int = 0) -> torch.Tensor:
        """proj, col0: a projection of h computed by the caller whose columns from col0 on are this mixer's q | k | v | gate."""
        step = get_context().ragged
        if proj is None:
            proj, col0 = self.in_proj(h), 0
        a = col0 + self.sizes[0]
        b = a + self.sizes[1]
        c = b + self.sizes[2]
        q = mix_ops.rotary_store(proj, col0, a, b, self.inv_freq, self.temp, self.k_cache, self.v_cache, step,
                                 self.H, self.G, self.D, self.Dv, self.rot_dims, interleaved=self.interleaved,
                                 unit_eps=self.unit_norm_eps)
        gate = proj[:, c:c + self.sizes[3]] if self.gate is not None else None
        o = mix_ops.window_pool_attention(q, self.k_cache, self.v_cache, None, None, gate, step, self.H, self.G, self.D,
                                          self.Dv, self.window, 0, self.scale, has_sink=False,
                                          gate_per_head=self.gate == "head", keep_first=self.keep_first, chunk=self.chunk,
                                          sinks=self.sink)
        return self.o_proj(o)
