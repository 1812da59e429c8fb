"""Shared pieces of the Givozen tests: small configurations made here (none of them a real model's sizes),
the engine or single kernels on one side, oracle/givozen_oracle.py on the other. Replay, step and comparison
helpers are the ones of tests/_kagalorn.py."""
from __future__ import annotations

import random

from tests._kagalorn import TOL, assert_close, make_step, rel_err, replay, tokens_for, write_model  # noqa: F401

ROT_A = {"base": 5000.0, "dims": 8, "scaling": {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 40}}
ATT_A = {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 10, "scale": 0.3, "rot": ROT_A}
ATT_B = {"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 16, "scale": 0.35, "rot": {"base": 100.0, "dims": 8}}
MOE_A = {"kind": "moe", "expert": {"ff": 20, "limit": 0.8}, "router": {"experts": 6, "top": 2}, "shared": {"ff": 12, "limit": 1.2}}
MOE_B = {"kind": "moe", "expert": {"ff": 12, "limit": 2.0}, "router": {"experts": 4, "top": 1}}
DENSE_A = {"kind": "dense", "ff": 40}

# two layers of the middle run three times; a dense and two expert feed-forwards, one layer without any
CFG_MAIN = {
    "architecture": "Givozen", "vocab": 67, "width": 48, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "attention", "mixer": ATT_A, "mlp": DENSE_A},
        {"type": "attention", "mixer": ATT_B, "mlp": MOE_A},
        {"type": "attention", "mixer": ATT_A, "mlp": None},
        {"type": "attention", "mixer": ATT_B, "mlp": MOE_B},
    ],
}
# values that a model may happen to make 1 or equal: one head, one kv head under five heads, every entry rotated,
# none rotated, no frequency scaling, a loop from the first layer, a loop of one pass, every expert chosen, no shared
# expert, a value size above one wave, key size 40, two experts
CFG_ODD = {
    "architecture": "Givozen", "vocab": 37, "width": 40, "norm": {"eps": 1e-6},
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        {"type": "attention", "mixer": {"heads": 1, "kv_heads": 1, "dim": 40, "vdim": 70, "scale": 0.15,
                                        "rot": {"base": 300.0, "dims": 40}},
         "mlp": {"kind": "moe", "expert": {"ff": 8, "limit": 1.0}, "router": {"experts": 3, "top": 3}}},
        {"type": "attention", "mixer": {"heads": 5, "kv_heads": 1, "dim": 6, "vdim": 4, "scale": 0.4}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.4,
                                        "rot": {"base": 10.0, "dims": 2, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0,
                                                                                     "original": 16}}},
         "mlp": {"kind": "moe", "expert": {"ff": 16, "limit": 0.5}, "router": {"experts": 2, "top": 1},
                 "shared": {"ff": 4, "limit": 0.6}}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.3,
                                        "rot": {"base": 50.0, "dims": 4}}, "mlp": {"kind": "dense", "ff": 24}},
    ],
}
CFG_ONE_PASS = {
    "architecture": "Givozen", "vocab": 41, "width": 32, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [{"type": "attention", "mixer": ATT_B, "mlp": DENSE_A}, {"type": "attention", "mixer": ATT_A, "mlp": MOE_B}],
}
CFG_NO_LOOP = {
    "architecture": "Givozen", "vocab": 41, "width": 32, "norm": {"eps": 1e-5},
    "layers": [{"type": "attention", "mixer": ATT_A, "mlp": MOE_A}, {"type": "attention", "mixer": ATT_B, "mlp": None}],
}
# head and expert sizes in multiples of 16 / 32 (in bf16 the attention then runs on the matrix cores and the experts
# in the gathered form), five query heads a kv head, a looped last layer
CFG_WIDE = {
    "architecture": "Givozen", "vocab": 83, "width": 64, "norm": {"eps": 1e-6},
    "loop": {"start": 2, "stop": 3, "times": 2},
    "layers": [
        {"type": "attention", "mixer": {"heads": 5, "kv_heads": 1, "dim": 32, "vdim": 16, "scale": 0.18,
                                        "rot": {"base": 10000.0, "dims": 16}},
         "mlp": {"kind": "moe", "expert": {"ff": 32, "limit": 0.9}, "router": {"experts": 8, "top": 3},
                 "shared": {"ff": 48, "limit": 1.4}}},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 48, "scale": 0.25,
                                        "rot": {"base": 1000.0, "dims": 16, "scaling": {"factor": 6.0, "low": 0.5, "high": 3.0,
                                                                                        "original": 64}}},
         "mlp": {"kind": "dense", "ff": 96}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 48, "vdim": 32, "scale": 0.15,
                                        "rot": {"base": 500.0, "dims": 32}},
         "mlp": {"kind": "moe", "expert": {"ff": 64, "limit": 2.0}, "router": {"experts": 4, "top": 2}}},
    ],
}


def random_config(seed: int) -> dict:
    """A configuration drawn from lists of sizes: layer count, loop, head counts and sizes, rotated part, scaling,
    feed-forward kinds and expert counts all vary."""
    r = random.Random(seed)
    width = r.choice([32, 48, 64])
    n = r.randint(2, 4)
    layers = []
    for _ in range(n):
        G = r.choice([1, 2])
        D = r.choice([8, 12, 16, 24])
        m = {"heads": G * r.choice([1, 2, 3]), "kv_heads": G, "dim": D, "vdim": r.choice([8, 16, 20]),
             "scale": r.choice([0.2, 0.3, 0.4])}
        dims = r.choice([0, 2, D // 2 // 2 * 2, D])
        if dims:
            m["rot"] = {"base": r.choice([50.0, 1000.0, 100000.0]), "dims": dims}
            if r.random() < 0.5:
                m["rot"]["scaling"] = {"factor": r.choice([2.0, 5.0]), "low": r.choice([0.5, 1.0]), "high": r.choice([2.0, 3.0]),
                                       "original": r.choice([16, 64, 256])}
        kind = r.choice(["dense", "moe", "moe", None])
        if kind == "dense":
            mlp = {"kind": "dense", "ff": r.choice([24, 40, 64])}
        elif kind == "moe":
            E = r.choice([2, 4, 5, 8])
            mlp = {"kind": "moe", "expert": {"ff": r.choice([8, 16, 32]), "limit": r.choice([0.5, 1.0, 3.0])},
                   "router": {"experts": E, "top": r.randint(1, min(E, 3))}}
            if r.random() < 0.6:
                mlp["shared"] = {"ff": r.choice([8, 24]), "limit": r.choice([0.7, 1.5])}
        else:
            mlp = None
        layers.append({"type": "attention", "mixer": m, "mlp": mlp})
    cfg = {"architecture": "Givozen", "vocab": r.choice([53, 97]), "width": width, "norm": {"eps": r.choice([1e-6, 1e-5])},
           "layers": layers}
    if r.random() < 0.8:
        a = r.randint(0, n - 1)
        cfg["loop"] = {"start": a, "stop": r.randint(a + 1, n), "times": r.randint(1, 3)}
    return cfg
