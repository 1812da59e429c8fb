"""Plain, slow restatement of the Bisuzen layers in float64, one function per mechanism, whole
sequences at a time (no cache, no state slots, no batching, no merged weights, no fused steps). Test
infrastructure only: it shares no code with the package and is what the engine's results are compared with.

W is a dict of float64 tensors under the checkpoint's names; cfg is the parsed config.json."""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dyt(x, W, name):
    """Dynamic tanh: tanh(alpha x) w + b, element by element (no statistics of the row)."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


# ------------------------------------------------------------------------------------ rotation
def rotate_pairs(x, positions, dims, base):
    """x [T, d]: entries (2i, 2i+1), i < dims/2, are a pair turned by position * base^(-2i/dims); entries from
    `dims` on pass unchanged."""
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(dims // 2):
            a = float(positions[t]) * base ** (-2.0 * i / dims)
            u, v = x[t, 2 * i], x[t, 2 * i + 1]
            out[t, 2 * i] = u * math.cos(a) - v * math.sin(a)
            out[t, 2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


# ----------------------------------------------------------------------------------- attention
def masked_softmax_head(q, k, v, factor, visible, sink=None):
    """One head: q [T, D], k [T, D], v [T, Dv]. visible(i, j) says whether query i sees key j <= i.
    sink: a number whose exponential joins the denominator (no key, no value), or None."""
    out = []
    for i in range(q.shape[0]):
        js = [j for j in range(i + 1) if visible(i, j)]
        s = (k[js] @ q[i]) * factor
        m = s.max() if sink is None else torch.maximum(s.max(), sink)
        e = torch.exp(s - m)
        den = e.sum() if sink is None else e.sum() + torch.exp(sink - m)
        out.append((e / den) @ v[js])
    return torch.stack(out)


def window_visible(size, keep_first):
    return lambda i, j: (i - j < size) or (j < keep_first)


def chunk_visible(size):
    return lambda i, j: i // size == j // size


def sink_window_attention(h, W, p, m, cache_round=None):
    """The left half of the parallel mixer: biased projections, pairwise rotation of part of every head,
    a sliding window that also keeps the first tokens, a learned sink per head in the softmax."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, D)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, D)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, Dv)
    rot = m.get("rot")
    pos = list(range(T))
    heads = []
    vis = window_visible(int(m["mask"]["size"]), int(m["mask"].get("keep_first", 0)))
    for hq in range(H):
        g = hq // (H // G)
        qh, kh, vh = q[:, hq], k[:, g], v[:, g]
        if rot:
            qh = rotate_pairs(qh, pos, int(rot["dims"]), float(rot["base"]))
            kh = rotate_pairs(kh, pos, int(rot["dims"]), float(rot["base"]))
        if cache_round is not None:
            qh, kh, vh = cache_round(qh), cache_round(kh), cache_round(vh)
        heads.append(masked_softmax_head(qh, kh, vh, float(m["scale"]), vis, W[p + "sink"][hq]))
    return torch.cat(heads, -1) @ W[p + "o"].T + W[p + "o.b"]


def lightning_attention(h, W, p, m, eps):
    """The right half: a state per head that decays by a constant and takes k v^T of every token, read with q;
    heads normed together, gated by a sigmoid of the input, projected."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).view(T, H, D)
    k = silu(h @ W[p + "k"].T).view(T, H, D)
    v = silu(h @ W[p + "v"].T).view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        d = float(m["decay"][hd])
        for t in range(T):
            S = d * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = unit_rms(o.reshape(T, H * Dv), eps) * W[p + "norm"]
    return (y * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps, cache_round=None):
    left = sink_window_attention(h, W, p + "left.", m["left"], cache_round)
    right = lightning_attention(h, W, p + "right.", m["right"], eps)
    return 0.5 * (unit_rms(left, eps) * W[p + "left.out"] + unit_rms(right, eps) * W[p + "right.out"])


def chunked_attention(h, W, p, m, eps, cache_round=None):
    """No biases, no rotation; q and k divided by their root mean square per head; a query sees the keys of its own
    chunk of mask.size positions (counted from position 0) up to itself."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ W[p + "q"].T).view(T, H, D), eps)
    k = unit_rms((h @ W[p + "k"].T).view(T, G, D), eps)
    v = (h @ W[p + "v"].T).view(T, G, Dv)
    vis = chunk_visible(int(m["mask"]["size"]))
    heads = []
    for hq in range(H):
        g = hq // (H // G)
        qh, kh, vh = q[:, hq], k[:, g], v[:, g]
        if cache_round is not None:
            qh, kh, vh = cache_round(qh), cache_round(kh), cache_round(vh)
        heads.append(masked_softmax_head(qh, kh, vh, float(m["scale"]), vis))
    return torch.cat(heads, -1) @ W[p + "o"].T


# -------------------------------------------------------------------------------- feed-forwards
def dense_ff(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, r):
    """-> (ids [T, top], weights [T, top], margin [T]). Softmax scores over experts and identity experts; the choice
    goes by score + correction among the experts of the `keep` groups whose best such number is largest; weights are
    the chosen experts' scores over their sum. margin: the smallest gap that decided anything (between the last group
    kept and the first dropped, between the last expert chosen and the first left out)."""
    T = h.shape[0]
    top = int(r["top"])
    s = torch.softmax(h @ W[p + "router"].T, -1)
    c = s + W[p + "correction"]
    n = c.shape[1]
    margin = torch.full((T,), 1.0, dtype=F64)
    groups = r.get("groups") or {}
    count, keep = int(groups.get("count", 1)), int(groups.get("keep", 1))
    if count > 1 and keep < count:
        best = c.view(T, count, n // count).max(-1).values
        srt = best.sort(-1, descending=True)
        margin = torch.minimum(margin, srt.values[:, keep - 1] - srt.values[:, keep])
        allowed = torch.zeros(T, count, dtype=torch.bool).scatter_(1, srt.indices[:, :keep], True)
        c = c.view(T, count, n // count).masked_fill(~allowed[:, :, None], float("-inf")).reshape(T, n)
    srt = c.sort(-1, descending=True)
    if n > top:
        gap = srt.values[:, top - 1] - srt.values[:, top]
        margin = torch.minimum(margin, torch.where(torch.isfinite(gap), gap, torch.ones_like(gap)))
    ids = srt.indices[:, :top]
    ws = s.gather(1, ids)
    return ids, ws / (ws.sum(-1, keepdim=True) + 1e-20), margin


def moe_ff(h, W, p, mlp, margins=None):
    r = mlp["router"]
    E = int(r["experts"])
    ids, ws, margin = route(h, W, p, r)
    if margins is not None:
        for t in range(h.shape[0]):
            margins[t].append(float(margin[t]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), ws[t]):
            if e >= E:                       # an identity expert hands the token through
                out[t] += w * h[t]
            else:
                out[t] += w * (gelu_erf(h[t] @ W[p + f"e{e}.up"].T) @ W[p + f"e{e}.down"].T)
    return out


def feed_forward(h, W, p, mlp, margins=None):
    if mlp["kind"] == "dense":
        return dense_ff(h, W, p)
    return moe_ff(h, W, p, mlp, margins)


# --------------------------------------------------------------------------------------- model
def layer_order(cfg) -> list:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or int(loop["stop"]) <= int(loop["start"]):
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def mixer(h, W, p, spec, eps, cache_round=None):
    if spec["type"] == "parallel":
        return parallel_mixer(h, W, p, spec["mixer"], eps, cache_round)
    if spec["type"] == "attention":
        return chunked_attention(h, W, p, spec["mixer"], eps, cache_round)
    raise ValueError(spec["type"])


def layer(x, W, i, spec, eps, cache_round=None, margins=None):
    p = f"l{i}."
    x = x + mixer(dyt(x, W, p + "norm1"), W, p + "mix.", spec, eps, cache_round)
    if spec.get("mlp") is not None:
        x = x + feed_forward(dyt(x, W, p + "norm2"), W, p + "mlp.", spec["mlp"], margins)
    return x


def forward(tokens, W, cfg, cache_round=None, margins=None):
    """-> (logits [T, vocab], [residual after every layer run]). margins: an empty list that receives, per token,
    the smallest routing margin over all expert layers it went through (1.0 without any)."""
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)].clone()
    trail = []
    per_token = [[1.0] for _ in tokens] if margins is not None else None
    for i in layer_order(cfg):
        x = layer(x, W, i, cfg["layers"][i], eps, cache_round, per_token)
        trail.append(x)
    if margins is not None:
        margins.extend(min(m) for m in per_token)
    return (dyt(x, W, "final.norm") @ W["head"].T) * float(cfg.get("logit_scale", 1.0)), trail


# ------------------------------------------------------------------------------ random checkpoints
def tensor_shapes(cfg) -> dict:
    """name -> shape of every tensor a checkpoint of this configuration holds."""
    W = int(cfg["width"])
    t = {"embed": (int(cfg["vocab"]), W), "head": (int(cfg["vocab"]), W)}

    def norm(name):
        t.update({name: (W,), name + ".b": (W,), name + ".alpha": ()})

    norm("final.norm")
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        norm(p + "norm1")
        if L["type"] == "parallel":
            a, b = m["left"], m["right"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            t.update({q + "q": (H * D, W), q + "q.b": (H * D,), q + "k": (G * D, W), q + "k.b": (G * D,),
                      q + "v": (G * Dv, W), q + "v.b": (G * Dv,), q + "sink": (H,), q + "o": (W, H * Dv), q + "o.b": (W,),
                      q + "out": (W,)})
            H, D, Dv = b["heads"], b["dim"], b["vdim"]
            q = p + "mix.right."
            t.update({q + "q": (H * D, W), q + "k": (H * D, W), q + "v": (H * Dv, W), q + "g": (H * Dv, W),
                      q + "o": (W, H * Dv), q + "norm": (H * Dv,), q + "out": (W,)})
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            q = p + "mix."
            t.update({q + "q": (H * D, W), q + "k": (G * D, W), q + "v": (G * Dv, W), q + "o": (W, H * Dv)})
        mlp = L.get("mlp")
        if mlp is None:
            continue
        norm(p + "norm2")
        if mlp["kind"] == "dense":
            t.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
            continue
        Fe, r = mlp["expert"]["ff"], mlp["router"]
        n = int(r["experts"]) + int(r.get("identity", 0))
        t.update({p + "mlp.router": (n, W), p + "mlp.correction": (n,)})
        for e in range(int(r["experts"])):
            t.update({p + f"mlp.e{e}.up": (Fe, W), p + f"mlp.e{e}.down": (W, Fe)})
    return t


def random_weights(cfg, seed: int) -> dict:
    """A seeded checkpoint, float64 values that bfloat16 holds exactly. Scales keep activations of order one and make
    the biases, the sinks, the norms' slopes and offsets, the router's correction and the identity experts all matter."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        x = torch.randn(tuple(shape), generator=g)
        if leaf == "alpha":
            x = 0.8 + 0.2 * x
        elif leaf == "b":
            x = 0.3 * x
        elif leaf in ("norm", "norm1", "norm2", "out"):
            x = 1.0 + 0.3 * x
        elif leaf == "sink":
            x = 1.0 + x
        elif leaf == "correction":
            x = 0.05 * x
        elif leaf == "router":
            x = 3.0 * x / shape[-1] ** 0.5
        elif leaf == "embed":
            x = x
        elif ".mix." in name and leaf in ("q", "k"):
            x = 1.5 * x / shape[-1] ** 0.5
        else:
            x = x / shape[-1] ** 0.5
        out[name] = x.to(torch.bfloat16).to(F64)
    return out
