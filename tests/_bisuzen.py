"""Shared pieces of the Bisuzen tests: small configurations made here (none of them a real model's sizes),
the engine or single kernels on one side, oracle/bisuzen_oracle.py on the other. Replay, step and comparison
helpers are the ones of tests/_kagalorn.py."""
from __future__ import annotations

import random

from tests._kagalorn import TOL, assert_close, make_step, rel_err, replay, tokens_for, write_model  # noqa: F401

LEFT_A = {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 10, "scale": 0.3, "mask": {"size": 9, "keep_first": 3},
          "rot": {"base": 5000.0, "dims": 8}}
RIGHT_A = {"heads": 3, "dim": 8, "vdim": 12, "decay": [0.5, 0.9, 0.995]}
LEFT_B = {"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 16, "scale": 0.35, "mask": {"size": 20, "keep_first": 1},
          "rot": {"base": 100.0, "dims": 8}}
RIGHT_B = {"heads": 2, "dim": 20, "vdim": 6, "decay": [0.97, 0.7]}
ATT_A = {"heads": 6, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.4, "mask": {"size": 7}}
ATT_B = {"heads": 2, "kv_heads": 1, "dim": 12, "vdim": 20, "scale": 0.3, "mask": {"size": 18}}
MOE_A = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 6, "identity": 2, "top": 2, "groups": {"count": 4, "keep": 2}}}
MOE_B = {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 4, "identity": 1, "top": 1}}
DENSE_A = {"kind": "dense", "ff": 40}

# the first two layers run three times; a dense and two expert feed-forwards, one layer without any
CFG_MAIN = {
    "architecture": "Bisuzen", "vocab": 67, "width": 48, "norm": {"eps": 1e-5}, "logit_scale": 1.5,
    "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [
        {"type": "parallel", "mixer": {"left": LEFT_A, "right": RIGHT_A}, "mlp": DENSE_A},
        {"type": "attention", "mixer": ATT_A, "mlp": MOE_A},
        {"type": "attention", "mixer": ATT_B, "mlp": None},
        {"type": "parallel", "mixer": {"left": LEFT_B, "right": RIGHT_B}, "mlp": MOE_B},
    ],
}
# values that a model may happen to make 1 or equal: one head, one kv head under five heads, every entry rotated, none
# rotated, no kept tokens, a window of one, a chunk of one, a chunk no prompt fills, a loop in the middle, every expert
# chosen, no identity expert, one group, every group kept, a value size above one wave, key size 40, a decay of 1 and of 0,
# no logit scale
CFG_ODD = {
    "architecture": "Bisuzen", "vocab": 37, "width": 40, "norm": {"eps": 1e-6},
    "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 1, "kv_heads": 1, "dim": 40, "vdim": 70, "scale": 0.15, "mask": {"size": 1, "keep_first": 0},
                            "rot": {"base": 300.0, "dims": 40}},
                   "right": {"heads": 1, "dim": 40, "vdim": 70, "decay": [1.0]}},
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "top": 3}}},
        {"type": "attention", "mixer": {"heads": 5, "kv_heads": 1, "dim": 6, "vdim": 4, "scale": 0.4, "mask": {"size": 1}}, "mlp": None},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.4, "mask": {"size": 1000, "keep_first": 5}},
                   "right": {"heads": 2, "dim": 6, "vdim": 5, "decay": [0.0, 0.8]}},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 2, "identity": 2, "top": 1, "groups": {"count": 2, "keep": 2}}}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.3, "mask": {"size": 1000}},
         "mlp": {"kind": "dense", "ff": 24}},
    ],
}
CFG_ONE_PASS = {
    "architecture": "Bisuzen", "vocab": 41, "width": 32, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
    "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [{"type": "attention", "mixer": ATT_B, "mlp": DENSE_A},
               {"type": "parallel", "mixer": {"left": LEFT_A, "right": RIGHT_B}, "mlp": MOE_B}],
}
CFG_NO_LOOP = {
    "architecture": "Bisuzen", "vocab": 41, "width": 32, "norm": {"eps": 1e-5},
    "layers": [{"type": "parallel", "mixer": {"left": LEFT_B, "right": RIGHT_A}, "mlp": MOE_A},
               {"type": "attention", "mixer": ATT_A, "mlp": None}],
}
# head and expert sizes in multiples of 16 / 32 (in bf16 the attention then runs on the matrix cores and the experts
# in the gathered form), five query heads a kv head, a looped last layer, windows and chunks beside the 16-token pages
CFG_WIDE = {
    "architecture": "Bisuzen", "vocab": 83, "width": 64, "norm": {"eps": 1e-6}, "logit_scale": 2.5,
    "loop": {"start": 2, "stop": 3, "times": 2},
    "layers": [
        {"type": "attention", "mixer": {"heads": 5, "kv_heads": 1, "dim": 32, "vdim": 16, "scale": 0.18, "mask": {"size": 17}},
         "mlp": {"kind": "moe", "expert": {"ff": 32}, "router": {"experts": 7, "identity": 1, "top": 3, "groups": {"count": 4, "keep": 3}}}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 48, "scale": 0.25, "mask": {"size": 15, "keep_first": 2},
                            "rot": {"base": 1000.0, "dims": 8}},
                   "right": {"heads": 2, "dim": 32, "vdim": 16, "decay": [0.9, 0.99]}},
         "mlp": {"kind": "dense", "ff": 96}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 48, "vdim": 32, "scale": 0.15, "mask": {"size": 33, "keep_first": 17},
                            "rot": {"base": 500.0, "dims": 48}},
                   "right": {"heads": 4, "dim": 16, "vdim": 16, "decay": [0.6, 0.8, 0.95, 0.999]}},
         "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 4, "top": 2}}},
    ],
}

# head sizes of a real model's order, windows, kept tokens and chunks longer than a 64-token page and a 64-key tile, prompts
# of a few hundred tokens (tests/_bisuzen_cases.py::case_engine_long_windows)
CFG_LONG = {
    "architecture": "Bisuzen", "vocab": 211, "width": 96, "norm": {"eps": 1e-6}, "logit_scale": 1.25,
    "loop": {"start": 0, "stop": 1, "times": 2},
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 6, "kv_heads": 3, "dim": 64, "vdim": 32, "scale": 0.125, "mask": {"size": 70, "keep_first": 3},
                            "rot": {"base": 20000.0, "dims": 32}},
                   "right": {"heads": 2, "dim": 32, "vdim": 96, "decay": [0.97, 0.999]}},
         "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 10, "identity": 2, "top": 3, "groups": {"count": 3, "keep": 2}}}},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 1, "dim": 32, "vdim": 64, "scale": 0.2, "mask": {"size": 90}},
         "mlp": {"kind": "dense", "ff": 160}},
    ],
}


def random_config(seed: int) -> dict:
    """A configuration drawn from lists of sizes: layer count and kinds, loop, head counts and sizes, rotated part,
    windows, kept tokens, chunks, decays, feed-forward kinds, expert, identity and group counts all vary."""
    r = random.Random(seed)
    width = r.choice([32, 48, 64])
    n = r.randint(2, 4)
    layers = []
    for _ in range(n):
        G = r.choice([1, 2])
        D = r.choice([8, 12, 16, 24])
        att = {"heads": G * r.choice([1, 2, 3]), "kv_heads": G, "dim": D, "vdim": r.choice([8, 16, 20]), "scale": r.choice([0.2, 0.3, 0.4])}
        if r.random() < 0.5:
            att["mask"] = {"size": r.choice([1, 5, 64, 70, 129])}
            layer = {"type": "attention", "mixer": att}
        else:
            att["mask"] = {"size": r.choice([1, 30, 64, 65, 100]), "keep_first": r.choice([0, 1, 4, 70])}
            dims = r.choice([0, 2, D // 2 // 2 * 2, D])
            if dims:
                att["rot"] = {"base": r.choice([50.0, 1000.0, 100000.0]), "dims": dims}
            H = r.choice([1, 2, 3])
            right = {"heads": H, "dim": r.choice([4, 8, 20]), "vdim": r.choice([6, 16]),
                     "decay": [r.choice([0.3, 0.8, 0.95, 0.999]) for _ in range(H)]}
            layer = {"type": "parallel", "mixer": {"left": att, "right": right}}
        kind = r.choice(["dense", "moe", "moe", None])
        if kind == "dense":
            layer["mlp"] = {"kind": "dense", "ff": r.choice([24, 40, 64])}
        elif kind == "moe":
            count = r.choice([1, 2, 3])
            per = r.choice([1, 2, 3])
            ident = r.randint(0, min(2, count * per - 1))
            E = count * per - ident
            router = {"experts": E, "identity": ident, "top": r.randint(1, min(per, 3))}
            if count > 1:
                router["groups"] = {"count": count, "keep": r.randint(1, count)}
            layer["mlp"] = {"kind": "moe", "expert": {"ff": r.choice([8, 16, 32])}, "router": router}
        else:
            layer["mlp"] = None
        layers.append(layer)
    cfg = {"architecture": "Bisuzen", "vocab": r.choice([53, 97]), "width": width, "norm": {"eps": r.choice([1e-6, 1e-5])},
           "logit_scale": r.choice([0.7, 1.0, 3.0]), "layers": layers}
    if r.random() < 0.8:
        a = r.randint(0, n - 1)
        cfg["loop"] = {"start": a, "stop": r.randint(a + 1, n), "times": r.randint(1, 3)}
    return cfg
