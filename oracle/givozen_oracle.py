"""Plain, slow restatement of the Givozen layers in float64, one function per mechanism, whole
sequences at a time (no cache, no batching, no merged weights, no fused steps). Test infrastructure
only: it shares no code with the package and is what the engine's results are compared with.

W is a dict of float64 tensors under the checkpoint's names; cfg is the parsed config.json."""
from __future__ import annotations

import math

import torch

F64 = torch.float64
GLU_SLOPE = 1.702


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    """x / rms(x) * (1 + w)."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------------------------ rotation
def rotary_frequencies(rot: dict) -> list:
    """f_i = base^(-2i/dims), i < dims/2, rescaled by wavelength when `scaling` is given: short waves
    keep their frequency, long ones are slowed by `factor`, those between are blended."""
    dims, base = int(rot["dims"]), float(rot["base"])
    sc = rot.get("scaling")
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wave = 2.0 * math.pi / f
            if wave < orig / high:
                pass
            elif wave > orig / low:
                f = f / factor
            else:
                s = (orig / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x, positions, freqs):
    """x [T, d]: entries i and i + len(freqs) are a pair turned by position * freqs[i]; entries from
    2 len(freqs) on pass unchanged."""
    out = x.clone()
    half = len(freqs)
    for t in range(x.shape[0]):
        for i, f in enumerate(freqs):
            a = float(positions[t]) * f
            u, v = x[t, i], x[t, i + half]
            out[t, i] = u * math.cos(a) - v * math.sin(a)
            out[t, i + half] = v * math.cos(a) + u * math.sin(a)
    return out


# ----------------------------------------------------------------------------------- attention
def causal_softmax_head(q, k, v, factor):
    """One head: q [T, D], k [T, D], v [T, Dv]; query i sees keys 0..i; scores times `factor`."""
    out = []
    for i in range(q.shape[0]):
        s = (k[:i + 1] @ q[i]) * factor
        e = torch.exp(s - s.max())
        out.append((e / e.sum()) @ v[:i + 1])
    return torch.stack(out)


def attention_mixer(h, W, p, m, cache_round=None):
    """p: '<layer>.mix.'; m: the mixer's sizes. cache_round: optional function applied to what a cache holds."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, D)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, D)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, Dv)
    rot = m.get("rot")
    freqs = rotary_frequencies(rot) if rot and int(rot.get("dims", 0)) > 0 else []
    pos = list(range(T))
    gate = torch.sigmoid(h @ W[p + "g"].T)                      # [T, H]
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        qh, kh, vh = rotate(q[:, hh], pos, freqs), rotate(k[:, g], pos, freqs), v[:, g]
        if cache_round is not None:
            kh, vh = cache_round(kh), cache_round(vh)
        o = causal_softmax_head(qh, kh, vh, float(m["scale"]) * float(W[p + "temp"][hh]))
        heads.append(o * gate[:, hh:hh + 1])
    return torch.cat(heads, -1) @ W[p + "o"].T


# ------------------------------------------------------------------------------- feed-forwards
def polynorm(z, coef, eps):
    """c1 R(z) + c2 R(z^2) + c3 R(z^3) + c0, R = division of a token's row by its root mean square."""
    a, b, c, e = (float(x) for x in coef)
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def dense_ff(h, W, p, eps):
    return polynorm(h @ W[p + "up"].T, W[p + "act"], eps) @ W[p + "down"].T


def glu_expert(x, W, p, limit):
    g = (x @ W[p + "gate"].T).clamp(max=limit)
    u = (x @ W[p + "up"].T).clamp(-limit, limit)
    return (g * torch.sigmoid(GLU_SLOPE * g) * (u + 1.0)) @ W[p + "down"].T


def route(h, W, p, top):
    """-> (ids [T, top], weights [T, top], margin [T]): sigmoid scores, the `top` largest, their own
    scores as weights; margin = gap between the last chosen and the first left out."""
    s = torch.sigmoid(h @ W[p + "router"].T)
    srt = s.sort(-1, descending=True)
    margin = srt.values[:, top - 1] - srt.values[:, top] if s.shape[1] > top else torch.full((h.shape[0],), 1.0, dtype=F64)
    return srt.indices[:, :top], srt.values[:, :top], margin


def moe_ff(h, W, p, mlp, margins=None):
    """Each token: sum over its chosen experts of expert(weight * h), plus the shared expert on h times
    a sigmoid gate of its own. margins (a list per token) receives each token's routing margin."""
    top = int(mlp["router"]["top"])
    ids, ws, margin = route(h, W, p, top)
    if margins is not None:
        for t in range(h.shape[0]):
            margins[t].append(float(margin[t]))
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), ws[t]):
            out[t] += glu_expert((w * h[t])[None], W, p + f"e{e}.", float(mlp["expert"]["limit"]))[0]
    if mlp.get("shared"):
        sg = torch.sigmoid(h @ W[p + "shared.sg"].T)             # [T, 1]
        out = out + sg * glu_expert(h, W, p + "shared.", float(mlp["shared"]["limit"]))
    return out


def feed_forward(h, W, p, mlp, eps, margins=None):
    if mlp["kind"] == "dense":
        return dense_ff(h, W, p, eps)
    return moe_ff(h, W, p, mlp, margins)


# --------------------------------------------------------------------------------------- model
def layer_order(cfg) -> list:
    """(layer index, pass number or None) in running order; a pass number marks the first layer of a pass."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or int(loop["stop"]) <= int(loop["start"]):
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None) for i in range(a)]
    for t in range(times):
        order += [(i, t if i == a else None) for i in range(a, b)]
    return order + [(i, None) for i in range(b, n)]


def layer(x, W, i, spec, eps, cache_round=None, margins=None):
    p = f"l{i}."
    x = x + norm(attention_mixer(norm(x, W[p + "norm1"], eps), W, p + "mix.", spec["mixer"], cache_round), W[p + "norm1b"], eps)
    if spec.get("mlp") is not None:
        x = x + norm(feed_forward(norm(x, W[p + "norm2"], eps), W, p + "mlp.", spec["mlp"], eps, margins), W[p + "norm2b"], eps)
    return x


def forward(tokens, W, cfg, cache_round=None, margins=None):
    """-> (logits [T, vocab], [residual after every layer run]). margins: an empty list that receives, per token,
    the smallest routing margin over all expert layers it went through (1.0 without any)."""
    eps = float(cfg["norm"]["eps"])
    emb = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = emb.clone()
    trail = []
    per_token = [[1.0] for _ in tokens] if margins is not None else None
    for i, t in layer_order(cfg):
        if t is not None:
            if t > 0:
                x = x + emb
            x = x + W["loop.step"][t]
        x = layer(x, W, i, cfg["layers"][i], eps, cache_round, per_token)
        trail.append(x)
    if margins is not None:
        margins.extend(min(m) for m in per_token)
    return norm(x, W["final.norm"], eps) @ W["embed"].T, trail


# ------------------------------------------------------------------------------ random checkpoints
def tensor_shapes(cfg) -> dict:
    """name -> shape of every tensor a checkpoint of this configuration holds."""
    W = int(cfg["width"])
    t = {"embed": (int(cfg["vocab"]), W), "final.norm": (W,)}
    loop = cfg.get("loop")
    if loop and int(loop["stop"]) > int(loop["start"]):
        t["loop.step"] = (int(loop["times"]), W)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t.update({p + "norm1": (W,), p + "norm1b": (W,), p + "mix.q": (H * D, W), p + "mix.q.b": (H * D,),
                  p + "mix.k": (G * D, W), p + "mix.k.b": (G * D,), p + "mix.v": (G * Dv, W), p + "mix.v.b": (G * Dv,),
                  p + "mix.temp": (H,), p + "mix.g": (H, W), p + "mix.o": (W, H * Dv)})
        mlp = L.get("mlp")
        if mlp is None:
            continue
        t.update({p + "norm2": (W,), p + "norm2b": (W,)})
        if mlp["kind"] == "dense":
            t.update({p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"]), p + "mlp.act": (4,)})
            continue
        Fe = mlp["expert"]["ff"]
        t[p + "mlp.router"] = (mlp["router"]["experts"], W)
        for e in range(mlp["router"]["experts"]):
            t.update({p + f"mlp.e{e}.gate": (Fe, W), p + f"mlp.e{e}.up": (Fe, W), p + f"mlp.e{e}.down": (W, Fe)})
        if mlp.get("shared"):
            Fs = mlp["shared"]["ff"]
            t.update({p + "mlp.shared.gate": (Fs, W), p + "mlp.shared.up": (Fs, W), p + "mlp.shared.down": (W, Fs),
                      p + "mlp.shared.sg": (1, W)})
    return t


def random_weights(cfg, seed: int) -> dict:
    """A seeded checkpoint, float64 values that bfloat16 holds exactly. Scales keep activations of order one, make the
    rotation, the biases, the head temperatures, the gates and the clamps of the experts all matter."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        x = torch.randn(*shape, generator=g)
        if "norm" in leaf:
            x = 0.3 * x
        elif leaf == "temp":
            x = 1.0 + 0.4 * x
        elif leaf == "act":
            x = torch.tensor([0.7, 0.4, -0.2, 0.1]) + 0.1 * x
        elif leaf == "b" or leaf == "step":
            x = 0.5 * x
        elif leaf == "embed":
            x = x
        elif leaf == "router":
            x = 2.0 * x / shape[-1] ** 0.5
        elif ".mix.q" in name or ".mix.k" in name or ".mlp.e" in name or ".shared." in name:
            x = 1.5 * x / shape[-1] ** 0.5
        else:
            x = x / shape[-1] ** 0.5
        out[name] = x.to(torch.bfloat16).to(F64)
    return out
