"""Givozen: a decoder-only model of gated rotary-attention layers with dense PolyNorm or mixture-of-experts
feed-forwards on one f32 residual, with a stretch of layers that is applied several times over.

config.json (`architecture: "Givozen"`) lists the layers. Each names its mixer type ("attention": causal
softmax attention with grouped key/value heads, biased q/k/v projections, rotation of part of every head with
wavelength-dependent frequency scaling, a temperature per query head and a sigmoid output gate per head), the
mixer's sizes, and its feed-forward: "dense" (up projection, PolyNorm, down projection), "moe" (clamped gated
experts behind a sigmoid router whose unnormalised scores scale the experts' inputs, plus an optional gated
shared expert), or none. Every sublayer is normed on both sides, x += norm_b(f(norm(x))), with norm weights
held as offsets from one. `loop` (start, stop, times) applies the stretch of layers start .. stop-1 `times` times back
to back with one set of weights, each pass on cache pages of its own; from the second pass on the token embeddings are
added to the residual once more, and ahead of every pass row t of `loop.step`. The output head is the embedding table.

Sizes, layer order and constants all come from the config; nothing here assumes a particular model.
The model runs ragged steps only (utils.context.RaggedStep). Checkpoint tensors: embed, loop.step, final.norm,
l<i>.norm1|norm1b|norm2|norm2b, l<i>.mix.q|k|v (+ .b) |temp|g|o, l<i>.mlp.up|down|act or
l<i>.mlp.router, l<i>.mlp.e<j>.gate|up|down, l<i>.mlp.shared.gate|up|down|sg; linear weights stored [out, in].
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Optional

import torch
from torch import nn

from .. import mix_ops
from ..layers.activation import PolyNorm
from ..layers.embed_head import ParallelLMHead, VocabParallelEmbedding
from ..layers.linear import ColumnParallelLinear, RowParallelLinear
from ..layers.moe import GLUSparseMoE
from ..layers.rotary_attention import GatedRotaryAttention

GLU_ALPHA = 1.702          # slope of the sigmoid in the experts' gate
NORM_WEIGHT_OFFSET = 1.0   # norm weights are offsets from one


@dataclass
class GivozenConfig:
    """config.json of a Givozen checkpoint. Attribute names the engine reads from any model config
    (vocab_size, hidden_size, max_position_embeddings, torch_dtype) are provided as well."""
    vocab: int
    width: int
    norm_eps: float
    layers: list = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    has_loop: bool = False                       # the config names a loop (its table of pass vectors exists even if the stretch is empty)
    torch_dtype: Any = torch.bfloat16
    max_position_embeddings: int = 1 << 30       # positions are rotated on the fly: any length the cache holds
    architectures: tuple = ("Givozen",)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def looped(self) -> bool:
        return self.loop_stop > self.loop_start

    def runs(self) -> list:
        """(layer index, pass number or None) in running order; a pass number marks the first layer of a pass."""
        n = len(self.layers)
        if not self.looped:
            return [(i, None) for i in range(n)]
        a, b = self.loop_start, self.loop_stop
        order = [(i, None) for i in range(a)]
        for t in range(self.loop_times):
            order += [(i, t if i == a else None) for i in range(a, b)]
        return order + [(i, None) for i in range(b, n)]

    @classmethod
    def from_dict(cls, d: dict) -> "GivozenConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise ValueError(f"Givozen config lacks '{key}'")
        layers = []
        for i, L in enumerate(d["layers"]):
            kind, m = L["type"], dict(L["mixer"])
            if kind != "attention":
                raise ValueError(f"layer {i}: unknown mixer type '{kind}'")
            missing = [k for k in ("heads", "kv_heads", "dim", "vdim", "scale") if k not in m]
            if missing:
                raise ValueError(f"layer {i} ({kind}): mixer lacks {missing}")
            mlp = L.get("mlp")
            if mlp is not None:
                mlp = dict(mlp)
                if mlp.get("kind") == "dense":
                    need = ("ff",)
                elif mlp.get("kind") == "moe":
                    need = ("expert", "router")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind '{mlp.get('kind')}'")
                missing = [k for k in need if k not in mlp]
                if missing:
                    raise ValueError(f"layer {i}: feed-forward lacks {missing}")
            layers.append({"type": kind, "mixer": m, "mlp": mlp})
        loop = d.get("loop") or {}
        start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
        if loop and not (0 <= start <= stop <= len(layers) and times >= 1):
            raise ValueError(f"loop {loop} does not fit {len(layers)} layers")
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=float(d["norm"]["eps"]), layers=layers,
                   loop_start=start, loop_stop=stop, loop_times=times, has_loop=bool(loop))

    @classmethod
    def from_pretrained(cls, path: str) -> "GivozenConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f))


class OffsetNormWeight(nn.Module):
    """Weight of an RMS norm applied as (1 + w); the norm itself runs fused with the residual update
    (mix_ops.sandwich_add_norm)."""

    def __init__(self, width: int):
        super().__init__()
        self.weight = nn.Parameter(torch.zeros(width, dtype=torch.float32))


class PolyNormMLP(nn.Module):

    def __init__(self, width: int, ff: int, eps: float):
        super().__init__()
        self.up_proj = ColumnParallelLinear(width, ff, bias=False)
        self.act_fn = PolyNorm(eps)
        self.down_proj = RowParallelLinear(ff, width, bias=False)

    def forward(self, x):
        return self.down_proj(self.act_fn(self.up_proj(x)))


def _make_mixer(config: GivozenConfig, spec: dict, share=None):
    m = spec["mixer"]
    rot = m.get("rot") or {}
    return GatedRotaryAttention(config.width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                float(m["scale"]), rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                                rot_scaling=rot.get("scaling") or None, bias=True, head_temp=True, gate="head", share=share)


class GivozenLayer(nn.Module):
    """One layer, or (with `source`) one more pass of a looped layer: the same parameters, cache pages of its own."""

    def __init__(self, config: GivozenConfig, spec: dict, source: "GivozenLayer | None" = None):
        super().__init__()
        W = config.width
        self.mix = _make_mixer(config, spec, source.mix if source is not None else None)
        if source is not None:
            self.norm1, self.norm1b, self.mlp = source.norm1, source.norm1b, source.mlp
            if self.mlp is not None:
                self.norm2, self.norm2b = source.norm2, source.norm2b
            return
        self.norm1, self.norm1b = OffsetNormWeight(W), OffsetNormWeight(W)
        mlp = spec["mlp"]
        self.mlp = None
        if mlp is not None:
            self.norm2, self.norm2b = OffsetNormWeight(W), OffsetNormWeight(W)
            if mlp["kind"] == "dense":
                self.mlp = PolyNormMLP(W, int(mlp["ff"]), config.norm_eps)
            else:
                shared = mlp.get("shared") or {}
                self.mlp = GLUSparseMoE(W, int(mlp["expert"]["ff"]), int(mlp["router"]["experts"]), int(mlp["router"]["top"]),
                                        float(mlp["expert"]["limit"]), GLU_ALPHA, int(shared.get("ff", 0)),
                                        float(shared.get("limit", 0.0)))


class GivozenForCausalLM(nn.Module):
    ragged_steps = True           # the runner feeds utils.context.RaggedStep batches
    config_class = GivozenConfig

    def __init__(self, config: GivozenConfig):
        super().__init__()
        self.config = config
        self.embed = VocabParallelEmbedding(config.vocab, config.width)
        self.layers = nn.ModuleList([GivozenLayer(config, spec) for spec in config.layers])
        # later passes of the looped layers: modules of their own (cache), parameters of the first pass
        self.repeats = nn.ModuleList()
        self.order: list = []                     # (layer module, pass number or None) in running order
        seen = set()
        for i, t in config.runs():
            layer = self.layers[i]
            if i in seen:
                layer = GivozenLayer(config, config.layers[i], layer)
                self.repeats.append(layer)
            seen.add(i)
            self.order.append((layer, t))
        self.loop_step = nn.Parameter(torch.zeros(config.loop_times, config.width, dtype=torch.float32)) if config.has_loop else None
        self.final_norm = OffsetNormWeight(config.width)
        self.lm_head = ParallelLMHead(config.vocab, config.width)
        self.lm_head.weight = self.embed.weight    # the output head is the embedding table
        self.layer_outputs: Optional[list] = None  # set to [] to record the residual after every layer run

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        emb = self.embed(input_ids)
        act, eps, off = emb.dtype, self.config.norm_eps, NORM_WEIGHT_OFFSET
        x = emb.float()                            # the residual, f32 throughout
        if x is emb:
            x = emb.clone()
        order = self.order

        def entry(r):
            """What is added to the residual ahead of run r, and the weight of the norm that reads it."""
            if r == len(order):
                return None, None, self.final_norm.weight
            layer, t = order[r]
            if t is None:
                return None, None, layer.norm1.weight
            return (emb if t > 0 else None), self.loop_step[t], layer.norm1.weight

        rows, vec, w = entry(0)
        h = mix_ops.sandwich_add_norm(x, None, None, rows, vec, w, off, eps, act)
        for r, (layer, _) in enumerate(order):
            y, post = layer.mix(h), layer.norm1b.weight
            if layer.mlp is not None:
                h = mix_ops.sandwich_add_norm(x, y, post, None, None, layer.norm2.weight, off, eps, act)
                y, post = layer.mlp(h), layer.norm2b.weight
            rows, vec, w = entry(r + 1)
            if self.layer_outputs is not None:     # the residual as the layer leaves it, before the next pass's additions
                mix_ops.sandwich_add_norm(x, y, post, None, None, None, off, eps, act)
                self.layer_outputs.append(x.clone())
                y = post = None
            h = mix_ops.sandwich_add_norm(x, y, post, rows, vec, w, off, eps, act)
        return h

    def compute_logits(self, hidden_states):
        return self.lm_head(hidden_states)

    def greedy_tokens(self, hidden_states):
        return self.lm_head.greedy_tokens(hidden_states)

    # ------------------------------------------------------------------ checkpoint
    def weight_targets(self) -> dict:
        """checkpoint tensor name -> (parameter, where, shape): where is None (the whole parameter), the
        index of a part of a merged projection, ("rows", offset, size) or ("cols", offset, size)."""
        t = {}
        W = self.config.width

        def whole(name, param, shape=None):
            t[name] = (param, None, tuple(shape or param.shape))

        whole("embed", self.embed.weight)
        whole("final.norm", self.final_norm.weight)
        if self.loop_step is not None:
            whole("loop.step", self.loop_step)
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            whole(p + "norm1", layer.norm1.weight)
            whole(p + "norm1b", layer.norm1b.weight)
            mix = layer.mix
            for j, nm in enumerate(("q", "k", "v")):
                t[p + "mix." + nm] = (mix.in_proj.weight, j, (mix.sizes[j], W))
                t[p + f"mix.{nm}.b"] = (mix.in_proj.bias, j, (mix.sizes[j],))
            t[p + "mix.g"] = (mix.in_proj.weight, 3, (mix.sizes[3], W))
            whole(p + "mix.temp", mix.temp)
            whole(p + "mix.o", mix.o_proj.weight)
            mlp = layer.mlp
            if mlp is None:
                continue
            whole(p + "norm2", layer.norm2.weight)
            whole(p + "norm2b", layer.norm2b.weight)
            if isinstance(mlp, PolyNormMLP):
                whole(p + "mlp.up", mlp.up_proj.weight)
                whole(p + "mlp.down", mlp.down_proj.weight)
                whole(p + "mlp.act", mlp.act_fn.coef)
                continue
            E, Fe, Fs = mlp.E, mlp.ff, mlp.Fs
            whole(p + "mlp.router", mlp.router_weight)
            for e in range(E):
                t[p + f"mlp.e{e}.gate"] = (mlp.up_weight, ("rows", e * 2 * Fe, Fe), (Fe, W))
                t[p + f"mlp.e{e}.up"] = (mlp.up_weight, ("rows", e * 2 * Fe + Fe, Fe), (Fe, W))
                t[p + f"mlp.e{e}.down"] = (mlp.down_weight, ("cols", e * Fe, Fe), (W, Fe))
            if Fs:
                base = E * 2 * Fe
                t[p + "mlp.shared.gate"] = (mlp.up_weight, ("rows", base, Fs), (Fs, W))
                t[p + "mlp.shared.up"] = (mlp.up_weight, ("rows", base + Fs, Fs), (Fs, W))
                t[p + "mlp.shared.sg"] = (mlp.up_weight, ("rows", base + 2 * Fs, 1), (1, W))
                t[p + "mlp.shared.down"] = (mlp.down_weight, ("cols", E * Fe, Fs), (W, Fs))
        return t

    def load_weights(self, tensors) -> None:
        """tensors: iterable of (checkpoint name, tensor). Every parameter must be covered."""
        targets = self.weight_targets()
        seen = set()
        for name, tensor in tensors:
            if name not in targets:
                raise KeyError(f"checkpoint tensor '{name}' has no place in this Givozen configuration")
            param, where, shape = targets[name]
            if tuple(tensor.shape) != shape:
                raise ValueError(f"'{name}': shape {tuple(tensor.shape)} does not fit {shape}")
            if where is None:
                loader = getattr(param, "weight_loader", None)
                if loader is not None:
                    loader(param, tensor)
                else:
                    param.data.copy_(tensor.reshape(param.shape))
            elif isinstance(where, tuple) and where[0] == "rows":
                param.data[where[1]:where[1] + where[2]].copy_(tensor)
            elif isinstance(where, tuple):
                param.data[:, where[1]:where[1] + where[2]].copy_(tensor)
            else:
                param.weight_loader(param, tensor, where)
            seen.add(name)
        missing = sorted(set(targets) - seen)
        if missing:
            raise KeyError(f"checkpoint lacks {missing[:8]}{' ...' if len(missing) > 8 else ''}")

    @staticmethod
    def _random_std(name: str, shape) -> Optional[float]:
        """Standard deviation of a random stand-in for checkpoint tensor `name` (None: drawn near 0, as the
        norm offsets are). Scales keep activations of order one through any depth."""
        leaf = name.rsplit(".", 1)[-1]
        if "norm" in leaf:
            return None
        if leaf in ("b", "act", "step"):
            return 0.5
        if leaf == "temp":
            return None
        return shape[-1] ** -0.5 if len(shape) == 2 else 0.5

    @torch.no_grad()
    def init_random_on_device(self, seed: int = 0) -> None:
        """Fast random fill on the parameters' own device (benchmarks: values differ between devices)."""
        gens, done = {}, set()
        for name, (param, _, shape) in self.weight_targets().items():
            if id(param) in done:
                continue                    # merged tensors are filled once
            done.add(id(param))
            g = gens.get(param.device)
            if g is None:
                g = gens[param.device] = torch.Generator(device=param.device).manual_seed(seed)
            std = self._random_std(name, shape)
            if name.endswith(".temp"):
                param.fill_(1.0)
            elif std is None:
                param.zero_()
            elif name.endswith(".act"):
                param.copy_(torch.tensor([0.6, 0.3, 0.1, 0.0]))
            else:
                param.normal_(0.0, std, generator=g)
        for layer in self.layers:           # the gate's part of the merged bias has no tensor: it is zero
            layer.mix.in_proj.bias[sum(layer.mix.sizes[:3]):].zero_()

    def random_weights(self, seed: int = 0):
        """(name, tensor) pairs of a seeded random checkpoint of this configuration, for runs without
        weights on disk."""
        from ..utils.loader import full_random_tensor
        for name, (_, _, shape) in self.weight_targets().items():
            std = self._random_std(name, shape)
            if name.endswith(".temp"):
                yield name, 1.0 + full_random_tensor(name, shape, seed, 0.2)
            else:
                yield name, full_random_tensor(name, shape, seed, 0.1 if std is None else std)
