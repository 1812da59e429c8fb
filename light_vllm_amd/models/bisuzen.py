"""Bisuzen: a decoder-only model on one f32 residual with dynamic-tanh norms, whose layers mix the sequence either with
two mixers side by side or with chunked attention, followed by a dense gated or a mixture-of-experts feed-forward; a
stretch of layers may be applied several times over.

config.json (`architecture: "Bisuzen"`) lists the layers. Each names its type:
  "parallel"   two mixers read the same normed input. Left: softmax attention with grouped key/value heads, biased
               q, k, v and output projections, pairwise rotation (entries 2i, 2i+1) of the first `rot.dims` entries of every
               head, a sliding window of `mask.size` positions that also keeps the first `mask.keep_first` ones, and a
               learned sink per head in the softmax denominator. Right: lightning attention (a state per head that decays
               by a constant of the config and takes k v^T of every token; q, k, v pass silu), its heads RMS-normed
               together, gated by a sigmoid of the input. The layer takes half the sum of the two outputs, each divided by
               its root mean square over the width and weighted.
  "attention"  softmax attention without biases or rotation, q and k divided by their root mean square per head, a query
               seeing the keys of its own chunk of `mask.size` positions (counted from position 0) up to itself.
and its feed-forward: "dense" (W_down (gelu_tanh(W_gate h) * W_up h)), "moe" (experts W_down gelu(W_up h) behind a softmax
router with a selection-only correction, groups ranked by their best expert, and identity experts that hand their
input through), or none. Norms are tanh(alpha x) w + b. `loop` (start, stop, times) applies the layers start .. stop-1
`times` times back to back with one set of weights, each pass on cache pages and state of its own. The logits are the
head's product times `logit_scale`.

Sizes, layer order and constants all come from the config; nothing here assumes a particular model. The model runs
ragged steps only (utils.context.RaggedStep). Checkpoint tensors: embed, head, final.norm (+ .b, .alpha),
l<i>.norm1|norm2 (+ .b, .alpha), parallel: l<i>.mix.left.q|k|v|o (+ .b) |sink|out, l<i>.mix.right.q|k|v|g|o|norm|out,
attention: l<i>.mix.q|k|v|o, dense: l<i>.mlp.gate|up|down, moe: l<i>.mlp.router|correction, l<i>.mlp.e<j>.up|down;
linear weights stored [out, in].
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Optional

import torch
from torch import nn

from ..layers.activation import GatedAct
from ..layers.embed_head import ParallelLMHead, VocabParallelEmbedding
from ..layers.layernorm import DynamicTanh
from ..layers.lightning_attention import LightningAttention
from ..layers.linear import MergedColumnParallelLinear, RowParallelLinear
from ..layers.moe import SparseMoE
from ..layers.parallel_mixer import ParallelMixers
from ..layers.rotary_attention import GatedRotaryAttention

PAIR_SCALE = 0.5           # the parallel mixer takes half the sum of its two normed outputs


@dataclass
class BisuzenConfig:
    """config.json of a Bisuzen checkpoint. Attribute names the engine reads from any model config
    (vocab_size, hidden_size, max_position_embeddings, torch_dtype) are provided as well."""
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float = 1.0
    layers: list = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    torch_dtype: Any = torch.bfloat16
    max_position_embeddings: int = 1 << 30       # positions are rotated on the fly: any length the cache holds
    architectures: tuple = ("Bisuzen",)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """Layer indices in running order."""
        n = len(self.layers)
        if self.loop_stop <= self.loop_start:
            return list(range(n))
        a, b = self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, n))

    @classmethod
    def from_dict(cls, d: dict) -> "BisuzenConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise ValueError(f"Bisuzen config lacks '{key}'")

        def need(i, what, m, keys):
            missing = [k for k in keys if k not in m]
            if missing:
                raise ValueError(f"layer {i} ({what}) lacks {missing}")

        layers = []
        for i, L in enumerate(d["layers"]):
            kind, m = L["type"], dict(L["mixer"])
            if kind == "parallel":
                need(i, kind, m, ("left", "right"))
                need(i, "left mixer", m["left"], ("heads", "kv_heads", "dim", "vdim", "scale", "mask"))
                need(i, "left mixer's mask", m["left"]["mask"], ("size",))
                need(i, "right mixer", m["right"], ("heads", "dim", "vdim", "decay"))
                if len(m["right"]["decay"]) != int(m["right"]["heads"]):
                    raise ValueError(f"layer {i}: {len(m['right']['decay'])} decays for {m['right']['heads']} heads")
            elif kind == "attention":
                need(i, kind, m, ("heads", "kv_heads", "dim", "vdim", "scale", "mask"))
                need(i, "mask", m["mask"], ("size",))
            else:
                raise ValueError(f"layer {i}: unknown mixer type '{kind}'")
            mlp = L.get("mlp")
            if mlp is not None:
                mlp = dict(mlp)
                if mlp.get("kind") == "dense":
                    need(i, "feed-forward", mlp, ("ff",))
                elif mlp.get("kind") == "moe":
                    need(i, "feed-forward", mlp, ("expert", "router"))
                    need(i, "router", mlp["router"], ("experts", "top"))
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind '{mlp.get('kind')}'")
            layers.append({"type": kind, "mixer": m, "mlp": mlp})
        loop = d.get("loop") or {}
        start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
        if loop and not (0 <= start <= stop <= len(layers) and times >= 1):
            raise ValueError(f"loop {loop} does not fit {len(layers)} layers")
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   logit_scale=float(d.get("logit_scale", 1.0)), layers=layers, loop_start=start, loop_stop=stop,
                   loop_times=times)

    @classmethod
    def from_pretrained(cls, path: str) -> "BisuzenConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f))


class GatedMLP(nn.Module):
    """W_down (act(W_gate h) * W_up h); the gate and up projections are one GEMM."""

    def __init__(self, width: int, ff: int, act: str = "gelu_tanh"):
        super().__init__()
        self.gate_up_proj = MergedColumnParallelLinear(width, [ff, ff], bias=False)
        self.act_fn = GatedAct(act)
        self.down_proj = RowParallelLinear(ff, width, bias=False)

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_up_proj(x)))


def _make_mixer(config: BisuzenConfig, spec: dict, share=None):
    W, m = config.width, spec["mixer"]
    if spec["type"] == "attention":
        return GatedRotaryAttention(W, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                                    rot_dims=0, bias=False, head_temp=False, gate=None, share=share,
                                    chunk=int(m["mask"]["size"]), unit_norm_eps=config.norm_eps)
    a, b = m["left"], m["right"]
    rot = a.get("rot") or {}
    left = GatedRotaryAttention(W, int(a["heads"]), int(a["kv_heads"]), int(a["dim"]), int(a["vdim"]), float(a["scale"]),
                                rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)), bias=True,
                                head_temp=False, gate=None, share=share.left if share is not None else None,
                                interleaved=True, window=int(a["mask"]["size"]), keep_first=int(a["mask"].get("keep_first", 0)),
                                sink=True, out_bias=True, fused_input=True)
    right = LightningAttention(W, int(b["heads"]), int(b["dim"]), int(b["vdim"]), b["decay"], norm_eps=config.norm_eps,
                               share=share.right if share is not None else None, fused_input=True)
    return ParallelMixers(W, left, right, eps=config.norm_eps, scale=PAIR_SCALE, share=share)


class BisuzenLayer(nn.Module):
    """One layer, or (with `source`) one more pass of a looped layer: the same parameters, cache pages and state of its own."""

    def __init__(self, config: BisuzenConfig, spec: dict, source: "BisuzenLayer | None" = None):
        super().__init__()
        W = config.width
        self.mix = _make_mixer(config, spec, source.mix if source is not None else None)
        if source is not None:
            self.norm1, self.mlp = source.norm1, source.mlp
            if self.mlp is not None:
                self.norm2 = source.norm2
            return
        self.norm1 = DynamicTanh(W)
        mlp = spec["mlp"]
        self.mlp = None
        if mlp is not None:
            self.norm2 = DynamicTanh(W)
            if mlp["kind"] == "dense":
                self.mlp = GatedMLP(W, int(mlp["ff"]), "gelu_tanh")
            else:
                r = mlp["router"]
                groups = r.get("groups") or {}
                count = int(groups.get("count", 1))
                self.mlp = SparseMoE(W, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), count,
                                     int(groups.get("keep", count)), score="softmax", group_rank="max", act="gelu",
                                     identity=int(r.get("identity", 0)), logits_kernel=True)


class BisuzenForCausalLM(nn.Module):
    ragged_steps = True           # the runner feeds utils.context.RaggedStep batches
    config_class = BisuzenConfig

    def __init__(self, config: BisuzenConfig):
        super().__init__()
        self.config = config
        self.embed = VocabParallelEmbedding(config.vocab, config.width)
        self.layers = nn.ModuleList([BisuzenLayer(config, spec) for spec in config.layers])
        # later passes of the looped layers: modules of their own (cache, state), parameters of the first pass
        self.repeats = nn.ModuleList()
        self.order: list = []                     # layer modules in running order
        seen = set()
        for i in config.runs():
            layer = self.layers[i]
            if i in seen:
                layer = BisuzenLayer(config, config.layers[i], layer)
                self.repeats.append(layer)
            seen.add(i)
            self.order.append(layer)
        self.final_norm = DynamicTanh(config.width)
        self.lm_head = ParallelLMHead(config.vocab, config.width)
        self.layer_outputs: Optional[list] = None  # set to [] to record the residual after every layer run

    @staticmethod
    def _sublayer(mix, out) -> dict:
        """Arguments of the residual update that takes a mixer's output."""
        if isinstance(mix, ParallelMixers):
            return dict(y1=out[0], y2=out[1], post_w1=mix.left_out, post_w2=mix.right_out, pair_scale=mix.scale, pair_eps=mix.eps)
        return dict(y1=out)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        emb = self.embed(input_ids)
        act = emb.dtype
        x = emb.float()                            # the residual, f32 throughout
        if x is emb:
            x = emb.clone()
        order = self.order
        norms = [layer.norm1 for layer in order] + [self.final_norm]
        h = norms[0](x, act_dtype=act)
        for r, layer in enumerate(order):
            update = self._sublayer(layer.mix, layer.mix(h))
            if layer.mlp is not None:
                h = layer.norm2(x, act_dtype=act, **update)
                update = dict(y1=layer.mlp(h))
            h = norms[r + 1](x, act_dtype=act, **update)     # x += this layer's last sublayer, then the next norm
            if self.layer_outputs is not None:
                self.layer_outputs.append(x.clone())
        return h

    def compute_logits(self, hidden_states):
        logits = self.lm_head(hidden_states)
        return logits.float() * self.config.logit_scale if logits is not None else None

    def greedy_tokens(self, hidden_states):
        if self.config.logit_scale > 0:           # a positive factor does not move the maximum
            return self.lm_head.greedy_tokens(hidden_states)
        return self.compute_logits(hidden_states).argmax(-1)

    # ------------------------------------------------------------------ checkpoint
    def weight_targets(self) -> dict:
        """checkpoint tensor name -> (parameter, where, shape): where is None (the whole parameter), the
        index of a part of a merged projection, ("rows", offset, size) or ("cols", offset, size)."""
        t = {}
        W = self.config.width

        def whole(name, param, shape=None):
            t[name] = (param, None, tuple(param.shape if shape is None else shape))

        def norm(name, mod):
            whole(name, mod.weight)
            whole(name + ".b", mod.bias)
            whole(name + ".alpha", mod.alpha, ())

        whole("embed", self.embed.weight)
        whole("head", self.lm_head.weight)
        norm("final.norm", self.final_norm)
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            norm(p + "norm1", layer.norm1)
            mix = layer.mix
            if isinstance(mix, ParallelMixers):
                left, right, proj = mix.left, mix.right, mix.in_proj
                for j, nm in enumerate(("q", "k", "v")):
                    t[p + f"mix.left.{nm}"] = (proj.weight, j, (left.sizes[j], W))
                    t[p + f"mix.left.{nm}.b"] = (proj.bias, j, (left.sizes[j],))
                whole(p + "mix.left.sink", left.sink)
                whole(p + "mix.left.o", left.o_proj.weight)
                whole(p + "mix.left.o.b", left.o_proj.bias)
                whole(p + "mix.left.out", mix.left_out)
                n = len(left.sizes)
                for j, nm in enumerate(("q", "k", "v", "g")):
                    t[p + f"mix.right.{nm}"] = (proj.weight, n + j, (right.sizes[j], W))
                whole(p + "mix.right.norm", right.out_norm_weight)
                whole(p + "mix.right.o", right.o_proj.weight)
                whole(p + "mix.right.out", mix.right_out)
            else:
                for j, nm in enumerate(("q", "k", "v")):
                    t[p + "mix." + nm] = (mix.in_proj.weight, j, (mix.sizes[j], W))
                whole(p + "mix.o", mix.o_proj.weight)
            mlp = layer.mlp
            if mlp is None:
                continue
            norm(p + "norm2", layer.norm2)
            if isinstance(mlp, GatedMLP):
                ff = mlp.gate_up_proj.output_sizes[0]
                t[p + "mlp.gate"] = (mlp.gate_up_proj.weight, 0, (ff, W))
                t[p + "mlp.up"] = (mlp.gate_up_proj.weight, 1, (ff, W))
                whole(p + "mlp.down", mlp.down_proj.weight)
                continue
            whole(p + "mlp.router", mlp.router_weight)
            whole(p + "mlp.correction", mlp.correction)
            for e in range(mlp.E):
                t[p + f"mlp.e{e}.up"] = (mlp.up_weight, ("rows", e * mlp.ff, mlp.ff), (mlp.ff, W))
                t[p + f"mlp.e{e}.down"] = (mlp.down_weight, ("cols", e * mlp.ff, mlp.ff), (W, mlp.ff))
        return t

    def load_weights(self, tensors) -> None:
        """tensors: iterable of (checkpoint name, tensor). Every parameter must be covered."""
        targets = self.weight_targets()
        seen = set()
        for name, tensor in tensors:
            if name not in targets:
                raise KeyError(f"checkpoint tensor '{name}' has no place in this Bisuzen configuration")
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
    def _random(name: str, shape):
        """(mean, standard deviation) of a random stand-in for checkpoint tensor `name`. Scales keep activations of
        order one through any depth."""
        leaf = name.rsplit(".", 1)[-1]
        if leaf == "alpha":
            return 0.7, 0.1
        if leaf in ("norm", "norm1", "norm2", "out"):
            return 1.0, 0.1
        if leaf == "b":
            return 0.0, 0.1
        if leaf == "sink":
            return 0.0, 1.0
        if leaf == "correction":
            return 0.0, 0.05
        return 0.0, (shape[-1] ** -0.5 if len(shape) == 2 else 0.5)

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
            mean, std = self._random(name, shape)
            param.normal_(mean, std, generator=g)
        for layer in self.layers:           # the right mixer's part of the merged bias has no tensor: it is zero
            if isinstance(layer.mix, ParallelMixers):
                layer.mix.in_proj.bias[sum(layer.mix.left.sizes[:3]):].zero_()

    def random_weights(self, seed: int = 0):
        """(name, tensor) pairs of a seeded random checkpoint of this configuration, for runs without
        weights on disk."""
        from ..utils.loader import full_random_tensor
        for name, (_, _, shape) in self.weight_targets().items():
            mean, std = self._random(name, shape)
            yield name, mean + full_random_tensor(name, shape, seed, std)
