"""Mixture-of-experts feed-forward: `experts` small two-matrix feed-forward layers, of which each token
uses `top`, chosen by a sigmoid router.

    s = sigmoid(W_r h) (32-bit)          selection scores c = s + correction (the correction steers the
    selection only); the experts are split into `groups` consecutive blocks, a block is ranked by the sum of its two
    largest c, experts outside the `keep` highest-ranked blocks are excluded, and the `top` largest c that remain win.
    weights = s of the chosen / (their sum + 1e-20)      y = sum_chosen weight_e * W_down,e act(W_up,e h)

act is the squared relu (or, as a choice, a gelu). Other choices of the constructor: scores by softmax over all router
outputs instead of the sigmoid; a block ranked by its one largest c; `identity` more router outputs behind the experts'
that stand for experts without weights, whose output is their input (they take part in scores, blocks and choice like any
other; a token that chooses one gets weight * h from it). All experts' up matrices are one [experts * ff, width] weight and all down
matrices one [width, experts * ff] weight. Two forms compute the same sum:

  * gathered (bf16, width and ff in multiples of 32, at least GATHER_FROM experts per choice): the (token,
    choice) pairs are sorted by expert on the device and every expert multiplies only its own rows
    (mix_ops.moe_grouped_ff: sort, two grouped GEMMs on the matrix cores, weighted sum; four launches);
  * sorted (bf16, eager steps with at least SORTED_FROM rows per expert): the same device-side sort, then every
    expert's two products as vendor GEMMs on its slice of the sorted rows, after reading the experts' row counts
    back once (mix_ops.moe_sorted_ff); large prompt steps, where the vendor GEMM's rate outweighs the one host
    synchronisation. Steps captured into a hipGraph never take it;
  * masked (f32, other sizes, few experts per choice): the up projection of every expert in one vendor
    GEMM, one kernel applies the activation times the token's weight for the column's expert (zero for
    experts the token did not choose), and the down GEMM sums over experts by itself. It spends
    experts / top times the FLOPs of the gathered form.

The gathered and masked forms never synchronise with the host, so both can be captured into a hipGraph.

GLUSparseMoE is the same mixture with clamped gated experts (gate and up matrices), a router without correction
or groups whose weights are the chosen scores themselves, the weight applied to the expert's INPUT,
    y = sum_chosen expert_e(s_e * h),    expert(x) = W_down [min(W_gate x, L) * sigmoid(alpha min(W_gate x, L)) * (clamp(W_up x, -L, L) + 1)]
and an optional shared expert of the same form that every token uses, times sigmoid(w_sg . h). Because the
projections are linear, s * h enters as a factor on the pre-activations (mix_ops.expert_glu), and the shared
expert's token gate as a factor on its activations, so all of it is GEMMs on h plus one elementwise kernel.
Forms: masked (everything in one up GEMM and one down GEMM; any dtype and size), gathered (bf16: sort, two
grouped GEMMs on the matrix cores with the gated unit in the first one's epilogue, sum; the shared expert as
vendor GEMMs beside it) and sorted (bf16, eager steps with at least SORTED_FROM rows per expert: the same sort, then
every expert's products as vendor GEMMs on its slice of the sorted rows).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import mix_ops
from ..utils.context import get_context
from .tp import tp_size


GATHER_FROM = 2.0     # experts / top from which the gathered form is taken
SORTED_FROM = 256     # rows per expert from which an eager step runs the experts as vendor GEMMs on sorted rows
MOE_KERNEL = "auto"   # "auto" | "masked" | "gathered" | "sorted" (tests force one or the other)


class SparseMoE(nn.Module):

    def __init__(self, width: int, ff: int, experts: int, top: int, groups: int = 1, keep: int = 1,
                 share: "SparseMoE | None" = None, score: str = "sigmoid", group_rank: str = "top2", act: str = "relu2",
                 identity: int = 0, logits_kernel: bool = False):
        super().__init__()
        assert tp_size() == 1, "the mixture of experts is not sharded: run it with tensor_parallel_size 1"
        routed = experts + identity                  # outputs of the router
        assert 1 <= top <= routed and groups >= 1 and routed % groups == 0 and 1 <= keep <= groups and identity >= 0
        assert score in ("sigmoid", "softmax") and group_rank in ("top2", "max") and act in mix_ops.ACTS
        self.width, self.ff, self.E, self.top, self.groups, self.keep = width, ff, experts, top, groups, keep
        self.score, self.group_rank, self.act, self.identity, self.logits_kernel = score, group_rank, act, identity, logits_kernel
        if share is None:
            f32 = dict(dtype=torch.float32)
            self.router_weight = nn.Parameter(torch.empty(routed, width, **f32))
            self.correction = nn.Parameter(torch.zeros(routed, **f32))
            self.up_weight = nn.Parameter(torch.empty(experts * ff, width))
            self.down_weight = nn.Parameter(torch.empty(width, experts * ff))
        else:
            assert (share.width, share.ff, share.E, share.identity) == (width, ff, experts, identity)
            self.router_weight, self.correction = share.router_weight, share.correction
            self.up_weight, self.down_weight = share.up_weight, share.down_weight

    def route(self, h: torch.Tensor):
        # logits_kernel: small steps form their f32 logits straight from the activations (no widened copy)
        logits = mix_ops.router_logits(h, self.router_weight) if self.logits_kernel else F.linear(h.float(), self.router_weight)
        return mix_ops.moe_route(logits, self.correction, self.top, self.groups, self.keep, score=self.score,
                                 group_rank=self.group_rank)

    def form(self, h: torch.Tensor) -> str:
        if MOE_KERNEL != "auto":
            return MOE_KERNEL
        if not (mix_ops.moe_grouped_ok(h, self.ff) and self.E >= GATHER_FROM * self.top):
            return "masked"
        step = get_context().ragged
        captured = step is not None and step.static
        return "sorted" if not captured and h.size(0) * self.top >= SORTED_FROM * self.E else "gathered"

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ids, weights, dense = self.route(h)
        form = self.form(h)
        if form == "gathered":
            return mix_ops.moe_grouped_ff(h, ids, weights, self.up_weight, self.down_weight, self.E, self.ff, self.act,
                                          self.identity)
        if form == "sorted":
            return mix_ops.moe_sorted_ff(h, ids, weights, self.up_weight, self.down_weight, self.E, self.ff, self.act,
                                         self.identity)
        up = F.linear(h, self.up_weight)
        if self.act == "relu2" and not self.identity:
            return F.linear(mix_ops.relu2_scale(up, dense, self.E, self.ff), self.down_weight)
        y = F.linear(mix_ops.expert_act_scale(up, dense, self.E, self.ff, self.act), self.down_weight)
        return mix_ops.scaled_row_add(y, h, dense[:, self.E:])      # experts without weights hand h through


class GLUSparseMoE(nn.Module):
    """Weights: up_weight [E*2*ff + 2*shared_ff + 1, width] = per expert [gate | up] rows, then the shared
    expert's gate and up rows and the row of its token gate; down_weight [width, E*ff + shared_ff]."""

    def __init__(self, width: int, ff: int, experts: int, top: int, limit: float, alpha: float = 1.702,
                 shared_ff: int = 0, shared_limit: float = 0.0):
        super().__init__()
        assert tp_size() == 1, "the mixture of experts is not sharded: run it with tensor_parallel_size 1"
        assert 1 <= top <= experts and shared_ff >= 0
        self.width, self.ff, self.E, self.top = width, ff, experts, top
        self.limit, self.alpha, self.Fs, self.shared_limit = float(limit), float(alpha), shared_ff, float(shared_limit)
        self.router_weight = nn.Parameter(torch.empty(experts, width, dtype=torch.float32))
        self.up_weight = nn.Parameter(torch.empty(experts * 2 * ff + (2 * shared_ff + 1 if shared_ff else 0), width))
        self.down_weight = nn.Parameter(torch.empty(width, experts * ff + shared_ff))

    def route(self, h: torch.Tensor):
        return mix_ops.moe_route(mix_ops.router_logits(h, self.router_weight), None, self.top, 1, 1, normalize=False)

    def form(self, h: torch.Tensor) -> str:
        if MOE_KERNEL != "auto":
            return MOE_KERNEL
        ok = mix_ops.moe_grouped_ok(h, self.ff) and (self.E * self.ff + self.Fs) % 8 == 0
        if not (ok and self.E >= GATHER_FROM * self.top):
            return "masked"
        step = get_context().ragged
        captured = step is not None and step.static
        return "sorted" if not captured and h.size(0) * self.top >= SORTED_FROM * self.E else "gathered"

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ids, weights, dense = self.route(h)
        E, Fe, Fs, T = self.E, self.ff, self.Fs, h.size(0)
        form = self.form(h)
        if form in ("gathered", "sorted"):
            routed = mix_ops.moe_grouped_glu_ff if form == "gathered" else mix_ops.moe_sorted_glu_ff
            y = routed(h, ids, weights, self.up_weight[:E * 2 * Fe], self.down_weight[:, :E * Fe], E, Fe, self.limit, self.alpha)
            if Fs:
                up = F.linear(h, self.up_weight[E * 2 * Fe:])
                a = mix_ops.expert_glu(up[:, :2 * Fs], 1, Fs, self.shared_limit, self.alpha, out_gate=up[:, 2 * Fs])
                y = torch.addmm(y, a, self.down_weight[:, E * Fe:].t())
            return y
        up = F.linear(h, self.up_weight)
        act = torch.empty(T, E * Fe + Fs, dtype=h.dtype, device=h.device)
        mix_ops.expert_glu(up[:, :E * 2 * Fe], E, Fe, self.limit, self.alpha, in_scale=dense, out=act[:, :E * Fe])
        if Fs:
            mix_ops.expert_glu(up[:, E * 2 * Fe:E * 2 * Fe + 2 * Fs], 1, Fs, self.shared_limit, self.alpha,
                               out_gate=up[:, E * 2 * Fe + 2 * Fs], out=act[:, E * Fe:])
        return F.linear(act, self.down_weight)
