"""Cases of the Bisuzen tests, written once and run by the CPU test file (host logic with the package's torch
restatement of the kernels) and the GPU test file (the HIP kernels): every mechanism alone against
oracle/bisuzen_oracle.py, then the engine on whole prompts, token-by-token decoding, portions, mixed batches,
reused pages and slots, long decoding and greedy generation."""
from __future__ import annotations



import torch

from oracle import bisuzen_oracle as oracle
from tests import _bisuzen as K

F64 = torch.float64


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


# ------------------------------------------------------------------------------- single mechanisms
def case_residual_dyt(device, dtype):
    """The f32 residual receives one sublayer output, two, or half the sum of two normed and weighted ones; the tanh
    norm reads the sum. Every part alone and together, widths that are no multiple of the workgroup or of four."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(1)
    tol = 1e-5 if dtype == "float32" else 1e-2
    for T, W in ((7, 48), (3, 37), (5, 1000), (2, 256)):
        x = 2 * torch.randn(T, W, generator=g)
        y1, y2 = (3 * torch.randn(T, W, generator=g).to(_dt(dtype)) for _ in range(2))
        p1, p2, w, b = (1.0 + 0.4 * torch.randn(W, generator=g) for _ in range(4))
        alpha = torch.tensor([0.37])
        Wt = {"n": w.to(F64), "n.b": b.to(F64), "n.alpha": alpha[0].to(F64)}
        for use1, use2, normed, use_w in ((1, 1, 1, 1), (1, 0, 1, 1), (1, 1, 0, 1), (1, 0, 0, 1), (0, 0, 0, 1), (1, 1, 1, 0), (1, 0, 0, 0)):
            xd = x.clone().to(device)
            h = mix_ops.residual_dyt(xd, y1.to(device) if use1 else None, y2.to(device) if use2 else None,
                                     p1.to(device) if normed else None, p2.to(device) if normed and use2 else None, 0.5, 1e-5,
                                     alpha.to(device) if use_w else None, w.to(device) if use_w else None,
                                     b.to(device) if use_w else None, _dt(dtype))
            want = x.to(F64)
            if normed:
                add = oracle.unit_rms(y1.to(F64), 1e-5) * p1.to(F64)
                if use2:
                    add = add + oracle.unit_rms(y2.to(F64), 1e-5) * p2.to(F64)
                want = want + 0.5 * add
            else:
                want = want + (y1.to(F64) if use1 else 0) + (y2.to(F64) if use2 else 0)
            assert torch.allclose(xd.cpu().to(F64), want, rtol=2e-6, atol=2e-5), ("the residual is f32", T, W, use1, use2, normed)
            if use_w:
                assert torch.allclose(h.cpu().to(F64), oracle.dyt(want, Wt, "n"), rtol=tol, atol=tol)
            else:
                assert h is None


def case_qk_prep(device, dtype):
    """Division of every head by its root mean square and rotation of pairs of the first entries, (2i, 2i+1) or half the
    rotated part apart, written to pages in any order: whole prompts, portions, single tokens, a position far out; part
    of a head rotated, all of it, none; with and without the division; columns that start on a multiple of four (four
    entries per lane, several heads per wave) and columns that do not (one entry per lane)."""
    from light_vllm_amd import mix_ops
    from oracle import givozen_oracle
    g = torch.Generator().manual_seed(2)
    tol = 2e-5 if dtype == "float32" else 2e-2
    shapes = ((4, 2, 12, 10, 8, False, 16, True), (3, 1, 16, 8, 16, True, 16, True), (2, 2, 9, 5, 0, True, 8, True),
              (1, 1, 40, 70, 2, False, 16, True), (6, 2, 32, 32, 32, False, 64, True), (2, 1, 128, 64, 64, True, 16, True),
              (5, 5, 96, 32, 0, True, 16, True), (3, 1, 24, 8, 16, True, 16, False), (2, 2, 256, 16, 256, False, 16, True),
              (7, 1, 8, 4, 8, True, 16, False))
    for (H, G, D, Dv, dims, unit, page, inter) in shapes:
        for pad in (3, 4):
            base, eps = 700.0, 1e-5
            inv = mix_ops.rotary_inv_freq(max(dims, 2), base, device)
            ld = H * D + G * D + G * Dv + pad
            for lens, ctxs in (([21], [0]), ([2, 1, 5], [15, 70000, 3]), ([1], [16])):
                B, T = len(lens), sum(lens)
                proj = torch.randn(T, ld, generator=g).to(_dt(dtype))
                need = [-(-(c + n) // page) for n, c in zip(lens, ctxs)]
                perm = torch.randperm(sum(min(nb, 8) for nb in need) + 2, generator=g).tolist()
                tables, at = [], 0
                for nb in need:       # a far position: only its own page matters
                    tables.append([perm[at]] * (nb - min(nb, 8)) + perm[at:at + min(nb, 8)])
                    at += min(nb, 8)
                kc = torch.zeros(len(perm), page, G, D, dtype=_dt(dtype), device=device)
                vc = torch.zeros(len(perm), page, G, Dv, dtype=_dt(dtype), device=device)
                step = K.make_step(lens, ctxs, list(range(B)), tables, device)
                q = mix_ops.rotary_store(proj.to(device), pad, pad + H * D, pad + H * D + G * D, inv, None, kc, vc, step, H, G, D, Dv, dims,
                                         interleaved=inter, unit_eps=eps if unit else None).cpu().to(F64)
                pf = proj.to(F64)
                t0 = 0
                for b, (n, c) in enumerate(zip(lens, ctxs)):
                    pos = list(range(c, c + n))
                    for hd in range(H + G):
                        src = pf[t0:t0 + n, pad + hd * D:pad + (hd + 1) * D]
                        if unit:
                            src = oracle.unit_rms(src, eps)
                        if dims and inter:
                            want = oracle.rotate_pairs(src, pos, dims, base)
                        elif dims:
                            want = givozen_oracle.rotate(src, pos, [base ** (-2.0 * i / dims) for i in range(dims // 2)])
                        else:
                            want = src
                        if hd < H:
                            got = q[t0:t0 + n, hd * D:(hd + 1) * D]
                        else:
                            got = torch.stack([kc[tables[b][p // page], p % page, hd - H].cpu().to(F64) for p in pos])
                        # an f32 angle at position 70000 is itself only good to half a hundredth
                        lim = max(tol, 1e-2 if max(pos) > 60000 else 0.0) * max(1.0, want.abs().max().item())
                        assert (got - want).abs().max().item() <= lim, (H, G, D, dims, unit, inter, pad, lens, hd)
                    gotv = torch.stack([vc[tables[b][p // page], p % page].cpu().to(F64).reshape(-1) for p in pos])
                    assert torch.equal(gotv, pf[t0:t0 + n, pad + H * D + G * D:pad + H * D + G * D + G * Dv])
                    t0 += n


def _paged(k, v, page, dtype, device, g):
    L, G = k.shape[0], k.shape[1]
    num_pages = -(-L // page) + 3
    table = torch.randperm(num_pages, generator=g).tolist()[:-(-L // page)]
    kc = torch.zeros(num_pages, page, G, k.shape[2], dtype=_dt(dtype))
    vc = torch.zeros(num_pages, page, G, v.shape[2], dtype=_dt(dtype))
    for j in range(L):
        kc[table[j // page], j % page] = k[j].to(_dt(dtype))
        vc[table[j // page], j % page] = v[j].to(_dt(dtype))
    return kc.to(device), vc.to(device), table


def case_masked_attention(device, dtype):
    """Windows with kept first tokens and a learned sink, and chunks, over a paged cache. A few beacon keys score far
    above the hundreds of others: the last kept token and the first one not kept, rows either side of page borders and
    of chunk borders, one in the middle. A query that has a beacon just inside or just outside its window or chunk gives
    a result of another order when it sees one key too many or too few; one head's sink is large enough to take most of
    the weight where no beacon is seen, another's small enough to vanish. Prompt-shaped, decode-shaped and
    portion-shaped launches."""
    from light_vllm_amd import mix_ops
    shapes = ((4, 2, 12, 10, 16, 150, 9, 3, 0), (1, 1, 40, 70, 64, 200, 70, 0, 0), (10, 1, 6, 4, 16, 90, 1, 5, 0),
              (5, 1, 32, 16, 16, 170, 33, 17, 0), (4, 2, 16, 48, 32, 210, 64, 1, 0), (2, 2, 48, 32, 64, 200, 41, 6, 0),
              (6, 2, 8, 8, 16, 100, 1, 0, 7), (12, 4, 32, 64, 64, 260, 1, 0, 100), (2, 1, 16, 16, 16, 130, 1, 0, 16),
              (3, 3, 64, 64, 64, 300, 1, 0, 129), (2, 2, 16, 16, 16, 80, 1, 0, 1))
    for (H, G, D, Dv, page, L, window, keep, chunk) in shapes:
        g = torch.Generator().manual_seed(L + H)
        beacons = {keep - 1, keep, page - 1, page, 2 * page + 1, 50} | ({chunk - 1, chunk, 2 * chunk - 1, 2 * chunk} if chunk else set())
        beacons = sorted(j for j in beacons if 0 <= j < L)
        e = torch.zeros(D); e[D - 1] = 1.0
        k = 0.3 * torch.randn(L, G, D, generator=g)
        for j in beacons:
            k[j] += 6.0 * e
        v = torch.randn(L, G, Dv, generator=g)
        q = 0.3 * torch.randn(L, H, D, generator=g) + 3.0 * e
        sinks = torch.linspace(-6.0, 4.0, H) if H > 1 else torch.tensor([2.0])
        k, v, q = (t.to(_dt(dtype)).float() for t in (k, v, q))
        scale = 0.7
        vis = oracle.chunk_visible(chunk) if chunk else oracle.window_visible(window, keep)
        use_sink = chunk == 0
        want = torch.cat([oracle.masked_softmax_head(q[:, h].to(F64), k[:, h // (H // G)].to(F64), v[:, h // (H // G)].to(F64), scale,
                                                     vis, sinks[h].to(F64) if use_sink else None) for h in range(H)], -1)
        kc, vc, table = _paged(k, v, page, dtype, device, g)
        qd = q.reshape(L, H * D).to(_dt(dtype)).to(device)
        tol = 2e-4 if dtype == "float32" else 3e-2
        sd = sinks.to(device) if use_sink else None

        def run(step, rows):
            return mix_ops.window_pool_attention(qd[rows].contiguous(), kc, vc, None, None, None, step, H, G, D, Dv,
                                                 window if not chunk else 1 << 30, 0, scale, has_sink=False, keep_first=keep,
                                                 chunk=chunk, sinks=sd)

        def check(got, idx, what):
            err = (got.cpu().to(F64) - want[idx]).abs().max().item()
            assert err <= tol * want.abs().max().item(), (what, H, G, D, Dv, page, window, keep, chunk, err)

        every = list(range(L))
        check(run(K.make_step([L], [0], [0], [table], device), every), every, "prompt")
        # queries beside every beacon, queries that have one at the edge of their window, queries beside chunk borders
        near = {i for j in beacons for i in (j - 1, j, j + 1)}
        if chunk:
            near |= {c * chunk + d for c in range(1, 4) for d in (-2, -1, 0, 1)}
        else:
            near |= {j + window + d for j in beacons for d in (-2, -1, 0, 1)}
        idx = sorted({i for i in near if 0 <= i < L} | set(range(L - 12, L)))
        check(run(K.make_step([1] * len(idx), idx, [0] * len(idx), [table] * len(idx), device), idx), idx, "decode")
        few = idx[-3:]
        check(run(K.make_step([1] * 3, few, [0] * 3, [table] * 3, device), few), few, "decode, few sequences")
        check(run(K.make_step([2], [L - 2], [0], [table], device), [L - 2, L - 1]), [L - 2, L - 1], "two tokens behind a long context")
        # portions that straddle a page border and the edge at which the first beacons leave the window or chunk,
        # beside the start of a sequence and the end of another
        cut = (chunk or window) + keep
        a, b = max(page - 1, 1), min(max(page + 1, cut + 2), L)
        rows = list(range(a, b)) + list(range(5)) + list(range(L - 19, L))
        check(run(K.make_step([b - a, 5, 19], [a, 0, L - 19], [0, 1, 2], [table, table, table], device), rows), rows, "portions")


def case_lightning(device, dtype):
    """The decaying state against the token-by-token recurrence: whole prompts, the same prompts in portions and single
    tokens through state slots in any order, a slot that held another sequence before, decays of 0 and 1 and near 1,
    key sizes that are no multiple of four, value sizes above one wave, rows of heads short and long (the norm over all
    heads, with the gate behind it, has a form of its own for long rows), launches of few workgroups and of many (the state's
    rows are then split over eight waves or four)."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(3)
    tol = 2e-5 if dtype == "float32" else 2e-2
    for (H, D, Dv, decay) in ((3, 8, 12, [0.5, 0.9, 0.995]), (1, 40, 70, [1.0]), (2, 6, 5, [0.0, 0.8]), (4, 16, 16, [0.6, 0.8, 0.95, 0.999]),
                              (2, 128, 64, [0.99, 0.3]), (1, 130, 8, [0.9]), (4, 16, 160, [0.9, 0.5, 0.99, 0.7]), (1, 100, 128, [0.95]), (2, 24, 40, [0.9, 0.8]),
                              (128, 40, 512, [0.5 + 0.499 * i / 127 for i in range(128)]), (64, 100, 1024, [0.9] * 64)):
        Wd, eps = 24, 1e-5
        m = {"heads": H, "dim": D, "vdim": Dv, "decay": decay}
        shapes = {"q": (H * D, Wd), "k": (H * D, Wd), "v": (H * Dv, Wd), "g": (H * Dv, Wd), "o": (Wd, H * Dv), "norm": (H * Dv,)}
        Wt = {"r." + n: (torch.randn(*s, generator=g) / (1.0 if n == "norm" else s[-1] ** 0.5)).to(torch.bfloat16).to(F64) for n, s in shapes.items()}
        lens = {"a": 75, "b": 33}
        hs = {i: torch.randn(n, Wd, generator=g).to(_dt(dtype)) for i, n in lens.items()}
        want = {i: oracle.lightning_attention(h.to(F64), Wt, "r.", m, eps) for i, h in hs.items()}
        w_in = torch.cat([Wt["r.q"], Wt["r.k"], Wt["r.v"], Wt["r.g"]]).to(_dt(dtype)).to(device)
        state = torch.full((3, H, D, Dv), 7.0, device=device)            # what an earlier sequence left behind
        dec = torch.tensor(decay, dtype=torch.float32, device=device)
        nw = Wt["r.norm"].float().to(device)
        hd, hv = H * D, H * Dv

        def run(parts):
            """parts: [(id, lo, hi, slot)] of one step -> {id: rows}"""
            h = torch.cat([hs[i][lo:hi] for i, lo, hi, _ in parts]).to(device)
            proj = torch.nn.functional.linear(h, w_in)
            step = K.make_step([hi - lo for _, lo, hi, _ in parts], [lo for _, lo, _, _ in parts], [s for *_, s in parts],
                               [[0]] * len(parts), device)
            o = mix_ops.lightning_attention(proj, 0, hd, 2 * hd, dec, state, step, H, D, Dv)
            y = mix_ops.head_norm_gate(o.view(-1, 1, hv), proj[:, 2 * hd + hv:], nw, eps, _dt(dtype), "sigmoid")
            out = (y.to(F64).cpu() @ Wt["r.o"].T)
            res, at = {}, 0
            for i, lo, hi, _ in parts:
                res[i] = out[at:at + hi - lo]
                at += hi - lo
            return res

        def check(got, i, lo, what):
            ref = want[i][lo:lo + got.shape[0]]
            assert (got - ref).abs().max().item() <= tol * max(1.0, want[i].abs().max().item()), (what, H, D, Dv, i, lo)

        check(run([("a", 0, 75, 1)])["a"], "a", 0, "whole")
        r = run([("b", 0, 33, 1), ("a", 0, 40, 2)])                     # b starts on the slot a just used
        check(r["b"], "b", 0, "reused slot")
        check(r["a"], "a", 0, "first portion")
        check(run([("a", 40, 42, 2)])["a"], "a", 40, "two tokens")
        at = 42
        for n in (1, 1, 17, 1, 13):
            check(run([("a", at, at + n, 2)])["a"], "a", at, "portions and single tokens")
            at += n


def case_glu_act(device, dtype):
    """act(gate) * up with the tanh form of gelu, the exact one, and the squared relu; strided rows, odd sizes."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(4)
    tol = 1e-5 if dtype == "float32" else 1e-2
    for T, Fh, pad in ((5, 40, 0), (3, 37, 3), (2, 1024, 8)):
        x = (2.5 * torch.randn(T, 2 * Fh + pad, generator=g)).to(_dt(dtype))
        xs = x.to(device)[:, :2 * Fh]
        gate, up = x[:, :Fh].to(F64), x[:, Fh:2 * Fh].to(F64)
        for act, f in (("gelu_tanh", oracle.gelu_tanh), ("gelu", oracle.gelu_erf), ("relu2", lambda z: torch.relu(z) ** 2)):
            got = mix_ops.glu_act(xs, act).cpu().to(F64)
            want = f(gate) * up
            assert (got - want).abs().max().item() <= tol * max(1.0, want.abs().max().item()), (act, T, Fh)
    z = torch.tensor([0.3, -1.2, 2.0], dtype=F64)           # the two gelus differ: a test that mixes them up fails
    assert (oracle.gelu_tanh(z) - oracle.gelu_erf(z)).abs().max().item() > 1e-4


def _route_case(g, T, E, ident, top, count, keep, spread=3.0):
    n = E + ident
    r = {"experts": E, "identity": ident, "top": top}
    if count > 1:
        r["groups"] = {"count": count, "keep": keep}
    Wd = 16
    Wt = {"m.router": (spread * torch.randn(n, Wd, generator=g) / Wd ** 0.5).to(F64), "m.correction": (0.3 * torch.randn(n, generator=g) - 0.2).to(F64)}
    h = torch.randn(T, Wd, generator=g).to(F64)
    return r, Wt, h


def case_moe_route(device):
    """Softmax scores over experts and identity experts, the choice by score plus correction (negative numbers among
    them: a dropped group must count as minus infinity, not as zero), groups ranked by their best member, weights from
    the uncorrected scores of the chosen over their sum."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(5)
    for (E, ident, top, count, keep) in ((6, 2, 2, 4, 2), (4, 1, 1, 1, 1), (3, 0, 3, 1, 1), (2, 2, 1, 2, 2), (7, 1, 3, 4, 3), (14, 2, 2, 2, 1),
                                         (5, 3, 4, 4, 2), (60, 4, 6, 8, 3)):
        r, Wt, h = _route_case(g, 40, E, ident, top, count, keep)
        ids, ws, margin = oracle.route(h, Wt, "m.", r)
        logits = (h @ Wt["m.router"].T).float().to(device)
        gi, gw, dense = mix_ops.moe_route(logits, Wt["m.correction"].float().to(device), top, count, keep, score="softmax", group_rank="max")
        clear = (margin > 1e-4).nonzero().flatten().tolist()
        assert len(clear) >= 30
        for t in clear:
            a = dict(zip(ids[t].tolist(), ws[t].tolist()))
            b = dict(zip(gi[t].tolist(), gw[t].tolist()))
            assert set(a) == set(b), (E, ident, top, count, keep, t, a, b)
            for e in a:
                assert abs(a[e] - b[e]) <= 1e-5, (e, a, b)
                assert abs(dense[t, e].item() - a[e]) <= 1e-5
            assert abs(dense[t].sum().item() - 1.0) <= 1e-5 and (dense[t] != 0).sum().item() == top
    # choice scores below zero everywhere: the kept group's members must still beat the dropped ones
    logits = torch.tensor([[2.0, 1.0, 0.0, 0.5]], device=device)
    corr = torch.tensor([-5.0, -5.2, -0.9, -0.95], device=device)
    gi, gw, _ = mix_ops.moe_route(logits, corr, 2, 2, 1, score="softmax", group_rank="max")
    assert sorted(gi[0].tolist()) == [2, 3]
    s = torch.softmax(logits[0].double().cpu(), 0)
    assert abs(gw[0].sum().item() - 1.0) < 1e-6 and abs(gw[0, gi[0].tolist().index(2)].item() - (s[2] / (s[2] + s[3])).item()) < 1e-6
    # ranked by the best member, not by the best two: group 0 = (0.5, 0.1), group 1 = (0.39, 0.38) in choice scores
    logits = torch.log(torch.tensor([[0.5, 0.1, 0.39, 0.38]])).to(device)
    gi, _, _ = mix_ops.moe_route(logits, None, 1, 2, 1, score="softmax", group_rank="max")
    assert gi[0].tolist() == [0]
    gi, _, _ = mix_ops.moe_route(logits, None, 1, 2, 1, score="softmax", group_rank="top2")
    assert gi[0].tolist() == [2]


def case_moe_ff(device, dtype):
    """The experts' sum in every form the layer has (masked; gathered and sorted where they apply) with identity experts
    among the choices, against the oracle token by token; tokens whose routing is a close call are left out."""
    from light_vllm_amd.layers import moe as moe_mod
    from light_vllm_amd.utils.context import reset_context, set_context
    g = torch.Generator().manual_seed(6)
    forms = ["masked"] + (["gathered", "sorted"] if dtype == "bfloat16" and device != "cpu" else [])
    tol = 3e-5 if dtype == "float32" else 4e-2
    for (Wd, Fe, E, ident, top, count, keep, T) in ((32, 32, 6, 2, 2, 4, 2, 50), (64, 64, 3, 1, 4, 1, 1, 33), (32, 32, 4, 0, 1, 2, 1, 20),
                                                    (32, 32, 2, 2, 2, 2, 2, 300)):
        mlp = {"kind": "moe", "expert": {"ff": Fe}, "router": {"experts": E, "identity": ident, "top": top,
                                                               "groups": {"count": count, "keep": keep}}}
        n = E + ident
        Wt = {"m.router": (3.0 * torch.randn(n, Wd, generator=g) / Wd ** 0.5).to(torch.bfloat16).to(F64),
              "m.correction": (0.05 * torch.randn(n, generator=g)).to(torch.bfloat16).to(F64)}
        for e in range(E):
            Wt[f"m.e{e}.up"] = (1.5 * torch.randn(Fe, Wd, generator=g) / Wd ** 0.5).to(torch.bfloat16).to(F64)
            Wt[f"m.e{e}.down"] = (torch.randn(Wd, Fe, generator=g) / Fe ** 0.5).to(torch.bfloat16).to(F64)
        h = torch.randn(T, Wd, generator=g).to(_dt(dtype))
        margins = [[] for _ in range(T)]
        want = oracle.moe_ff(h.to(F64), Wt, "m.", mlp, margins)
        clear = [t for t in range(T) if margins[t][0] > (1e-5 if dtype == "float32" else 0.03)]
        assert len(clear) >= T // 3
        old = torch.get_default_dtype()
        torch.set_default_dtype(_dt(dtype))
        try:
            layer = moe_mod.SparseMoE(Wd, Fe, E, top, count, keep, score="softmax", group_rank="max", act="gelu", identity=ident,
                                      logits_kernel=True)
        finally:
            torch.set_default_dtype(old)
        with torch.no_grad():
            layer.router_weight.copy_(Wt["m.router"])
            layer.correction.copy_(Wt["m.correction"])
            for e in range(E):
                layer.up_weight[e * Fe:(e + 1) * Fe].copy_(Wt[f"m.e{e}.up"])
                layer.down_weight[:, e * Fe:(e + 1) * Fe].copy_(Wt[f"m.e{e}.down"])
        layer = layer.to(device)
        chosen_identity = 0
        for form in forms:
            moe_mod.MOE_KERNEL = form
            try:
                set_context(True)
                with torch.no_grad():
                    got = layer(h.to(device)).cpu().to(F64)
                    ids = layer.route(h.to(device))[0].cpu()
                chosen_identity += int((ids >= E).sum())
            finally:
                moe_mod.MOE_KERNEL = "auto"
                reset_context()
            err = (got[clear] - want[clear]).abs().max().item()
            assert err <= tol * max(1.0, want.abs().max().item()), (form, Wd, Fe, E, ident, top, err)
        assert ident == 0 or chosen_identity > 0, "no token chose an identity expert: pick another seed"


# ------------------------------------------------------------------------------------------- engine
def _model(tmp_path, cfg, seed):
    weights = oracle.random_weights(cfg, seed)
    return K.write_model(tmp_path / f"m{seed}", cfg, weights), weights


ROUTE_MARGIN = 0.03      # bf16 runs: a router decided by less than this (in score units) may choose otherwise after rounding


def _oracle_runs(cfg, weights, prompts, dtype):
    """id -> (logits [len, vocab], positions whose routing was no close call in the oracle; all but ties for f32 runs).
    A token whose experts differ is another computation, not a rounding of this one, so comparisons leave those out."""
    want, decided = {}, {}
    for i, t in prompts.items():
        margins = []
        want[i] = oracle.forward(t, weights, cfg, margins=margins)[0]
        decided[i] = [j for j, m in enumerate(margins) if m >= (1e-5 if dtype == "float32" else ROUTE_MARGIN)]
        assert len(decided[i]) >= max(2, len(t) // 10), "too many close calls: pick another seed"
    return want, decided


def case_checkpoint_placement(tmp_path):
    """Every tensor of a checkpoint lands where the oracle reads it: the two mixers' parts of one merged projection, its
    biases (zero where a mixer has none), the scalar of a norm, experts' row and column blocks, passes of a loop on the
    same parameters with caches and state of their own."""
    import json
    import os
    from light_vllm_amd.models.bisuzen import BisuzenConfig, BisuzenForCausalLM
    from light_vllm_amd.models.registry import load_config, model_class
    cfg = K.CFG_MAIN
    weights = oracle.random_weights(cfg, 3)
    assert sorted(weights) == sorted(oracle.tensor_shapes(cfg))
    model_dir = K.write_model(tmp_path / "m", cfg, weights)
    config = load_config(model_dir)
    assert isinstance(config, BisuzenConfig) and model_class(config) is BisuzenForCausalLM
    assert config.runs() == [0, 1, 0, 1, 0, 1, 2, 3] == oracle.layer_order(cfg) and config.logit_scale == 1.5
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float32)
    try:
        model = BisuzenForCausalLM(config)
    finally:
        torch.set_default_dtype(old)
    model.load_weights(weights.items())
    assert sorted(model.weight_targets()) == sorted(weights)
    assert len(model.order) == 8 and len(model.repeats) == 4
    first, again = model.order[0], model.order[2]
    assert again is not first and again.mix is not first.mix and again.mix.in_proj is first.mix.in_proj and again.mlp is first.mlp
    assert again.mix.left is not first.mix.left and again.mix.left.sink is first.mix.left.sink
    assert again.mix.right.o_proj is first.mix.right.o_proj and again.norm1 is first.norm1
    mix = model.layers[3].mix
    ls, rs = mix.left.sizes, mix.right.sizes
    a, b, c = ls[0], ls[0] + ls[1], sum(ls)
    assert torch.equal(mix.in_proj.weight[a:b].double(), weights["l3.mix.left.k"])
    assert torch.equal(mix.in_proj.bias[b:c].double(), weights["l3.mix.left.v.b"]) and mix.in_proj.bias[c:].abs().max().item() == 0
    assert torch.equal(mix.in_proj.weight[c + rs[0]:c + rs[0] + rs[1]].double(), weights["l3.mix.right.k"])
    assert torch.equal(mix.in_proj.weight[c + sum(rs[:3]):].double(), weights["l3.mix.right.g"])
    assert torch.equal(mix.left.o_proj.bias.double(), weights["l3.mix.left.o.b"])
    assert model.layers[1].norm2.alpha.shape == (1,) and model.layers[1].norm2.alpha.item() == weights["l1.norm2.alpha"].item()
    moe = model.layers[1].mlp
    assert moe.router_weight.shape[0] == 8 and moe.E == 6
    assert torch.equal(moe.up_weight[4 * moe.ff:5 * moe.ff].double(), weights["l1.mlp.e4.up"])
    assert torch.equal(moe.down_weight[:, 5 * moe.ff:].double(), weights["l1.mlp.e5.down"])
    short = dict(weights)
    del short["l0.mix.left.sink"]
    try:
        model.load_weights(short.items())
        raise AssertionError("a missing tensor went unnoticed")
    except KeyError:
        pass
    bad = json.load(open(os.path.join(model_dir, "config.json")))
    bad["layers"][0]["type"] = "recurrent"
    try:
        BisuzenConfig.from_dict(bad)
        raise AssertionError("an unknown mixer went unnoticed")
    except ValueError:
        pass


def case_layer_by_layer(device, tmp_path, cfg=None):
    """The f32 residual after every layer run of a whole prompt (a looped layer counts each time), against the oracle:
    names the first run that differs."""
    from light_vllm_amd.engine.trace_replay import TraceReplayer
    cfg = cfg or K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 4)
    tokens = K.tokens_for(cfg, 27, 5)
    margins = []
    want = oracle.forward(tokens, weights, cfg, margins=margins)[1]
    rows = [j for j, m in enumerate(margins) if m >= 1e-5]
    rp = TraceReplayer(model_dir, "float32", 64, device=device, slots=2, page=16)
    try:
        model = rp.engine.model_runner.model
        model.layer_outputs = []
        rp.step([{"id": "a", "tokens": tokens, "want": []}], ["a"])
        got = [x.cpu() for x in model.layer_outputs]
    finally:
        rp.close()
    assert len(got) == len(want) == len(oracle.layer_order(cfg))
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a.to(F64) - b)[rows].abs().max().item() <= 3e-4 * b.abs().max().item(), f"layer run {i}"


def case_engine_schedules(device, dtype, tmp_path, cfg=None, seed=5):
    """Whole prompts, token-by-token decoding, portions down to two tokens and mixed batches of unequal
    requests give the logits of the whole-sequence oracle at every position: the first tokens, every page border
    (pages of 16 tokens), and every edge of the small windows, kept tokens and chunks included."""
    cfg = cfg or K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, seed)
    prompts = {"a": K.tokens_for(cfg, 53, 1), "b": K.tokens_for(cfg, 21, 2), "c": K.tokens_for(cfg, 38, 3)}
    want, decided = _oracle_runs(cfg, weights, prompts, dtype)
    schedules = {
        "whole": [[("a", 53)], [("b", 21)], [("c", 38)]],
        "decode": [[("a", 9)]] + [[("a", 1)]] * 44 + [[("b", 1)]] * 21,
        "portions": [[("a", n)] for n in (2, 3, 11, 2, 16, 1, 17, 1)] + [[("c", n)] for n in (16, 16, 2, 2, 2)],
        "mixed": [[("a", 5), ("b", 2)], [("a", 1), ("b", 7), ("c", 30)], [("c", 1), ("a", 20)], [("b", 12), ("a", 1)],
                  [("a", 26), ("c", 2)], [("c", 5)]],
    }
    for name, schedule in schedules.items():
        got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=128, page=16, slots=3)
        for i, logits in got.items():
            rows = [j for j in decided[i] if j < len(logits)]
            if rows:
                err = K.rel_err(logits[rows], want[i][rows])
                assert err <= K.TOL[dtype], (name, i, err)


def case_engine_random_config(device, dtype, tmp_path, seed):
    """A drawn configuration, prompts of a few hundred tokens on pages of 64: whole, and cut into unequal portions beside
    single tokens of another request, against the oracle at every position."""
    cfg = K.random_config(seed)
    model_dir, weights = _model(tmp_path, cfg, seed)
    prompts = {"a": K.tokens_for(cfg, 210, seed), "b": K.tokens_for(cfg, 75, seed + 1)}
    want, decided = _oracle_runs(cfg, weights, prompts, dtype)
    schedules = {
        "whole": [[("a", 210)], [("b", 75)]],
        "mixed": [[("a", 63)], [("a", 2), ("b", 70)], [("a", 100), ("b", 1)], [("a", 1), ("b", 1)], [("a", 44), ("b", 1)], [("b", 2)]],
    }
    for name, schedule in schedules.items():
        got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=384, page=64, slots=2)
        for i, logits in got.items():
            rows = [j for j in decided[i] if j < len(logits)]
            err = K.rel_err(logits[rows], want[i][rows])
            assert err <= K.TOL[dtype], (seed, name, i, err, cfg)


def case_engine_long_windows(device, dtype, tmp_path):
    """Windows, kept tokens and chunks that span several pages and key tiles: a prompt of 330 tokens whole, cut into
    portions at odd places beside the single tokens of another request, and decoded token by token across the edges."""
    cfg = K.CFG_LONG
    model_dir, weights = _model(tmp_path, cfg, 11)
    prompts = {"a": K.tokens_for(cfg, 330, 41), "b": K.tokens_for(cfg, 100, 42)}
    want, decided = _oracle_runs(cfg, weights, prompts, dtype)
    schedules = {
        "whole": [[("a", 330)], [("b", 100)]],
        "mixed": [[("a", 67)], [("a", 2), ("b", 60)], [("a", 111), ("b", 1)], [("a", 1), ("b", 1)], [("a", 89), ("b", 1)]]
                 + [[("a", 1), ("b", 1)]] * 37 + [[("a", 23)]],
    }
    for name, schedule in schedules.items():
        got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=512, page=64, slots=2)
        for i, logits in got.items():
            rows = [j for j in decided[i] if j < len(logits)]
            err = K.rel_err(logits[rows], want[i][rows])
            assert err <= K.TOL[dtype], (name, i, err)


def case_engine_reuse(device, dtype, tmp_path):
    """More requests than state slots and more tokens than pages: both are given back and used again,
    in another order, and a sequence that starts on used pages and a used slot starts from nothing."""
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 6)
    prompts = {f"r{n}": K.tokens_for(cfg, length, 10 + n) for n, length in enumerate((30, 17, 33, 9, 26, 31))}
    want, decided = _oracle_runs(cfg, weights, prompts, dtype)
    schedule = [[("r0", 30), ("r1", 10)], [("r1", 7), ("r2", 20)], [("r3", 9), ("r2", 13)], [("r4", 13)],
                [("r5", 15), ("r4", 13)], [("r5", 16)]]
    got = K.replay(model_dir, dtype, device, prompts, schedule, max_tokens=64, page=16, slots=2)   # 4 pages, 2 slots
    for i, logits in got.items():
        K.assert_close(logits[decided[i]], want[i][decided[i]], dtype, i)


def case_engine_long_decode(device, dtype, tmp_path):
    """Hundreds of single-token steps through the caches and states of every pass: windows and chunks pass over decoded
    tokens many times."""
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 7)
    prompts = {"a": K.tokens_for(cfg, 140, 21)}
    want, decided = _oracle_runs(cfg, weights, prompts, dtype)
    got = K.replay(model_dir, dtype, device, prompts, [[("a", 3)]] + [[("a", 1)]] * 137, max_tokens=192, page=16, slots=1)
    K.assert_close(got["a"][decided["a"]], want["a"][decided["a"]], dtype, "long decode")


def case_generate(device, tmp_path, enforce_eager=True):
    """Greedy generation through LLM.generate: the scheduler admits, cuts prompts into portions under a small
    token budget, mixes them with decoding sequences, and every completion is the oracle's greedy continuation."""
    from light_vllm_amd.llm import LLM
    from light_vllm_amd.sampling_params import SamplingParams
    cfg = K.CFG_MAIN
    model_dir, weights = _model(tmp_path, cfg, 8)
    prompts = [K.tokens_for(cfg, n, 30 + n) for n in (19, 5, 33, 12, 8)]
    steps = 6
    llm = LLM(model_dir, dtype="float32", device=device, kvcache_block_size=16, max_num_seqs=3, max_cache_tokens=160,
              max_num_batched_tokens=24, long_prefill_token_threshold=10, max_model_len=64, enforce_eager=enforce_eager)
    assert llm.model_runner.enforce_eager == enforce_eager
    outs = llm.generate([list(p) for p in prompts], SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True))
    llm.exit()
    for p, out in zip(prompts, outs):
        seq = list(p)
        for _ in range(steps):
            logits = oracle.forward(seq, weights, cfg)[0][-1]
            top2 = logits.topk(2).values
            assert (top2[0] - top2[1]).item() > 2e-4 * logits.abs().max().item(), "oracle tie: pick another seed"
            seq.append(int(logits.argmax()))
        assert out["token_ids"] == seq[len(p):]


def case_generate_bf16_graphs_like_eager(device, tmp_path):
    """bf16, sizes that take the matrix-core attention and the gathered experts: single-token steps replayed from
    hipGraphs (launch geometry fixed at its bound, padded rows) continue every prompt like eager steps do, wherever
    the oracle's choice of the next token is no close call."""
    from light_vllm_amd.llm import LLM
    from light_vllm_amd.sampling_params import SamplingParams
    cfg = K.CFG_WIDE
    model_dir, weights = _model(tmp_path, cfg, 12)
    prompts = [K.tokens_for(cfg, n, 70 + n) for n in (40, 9, 23)]
    steps = 8
    outs = {}
    for eager in (True, False):
        llm = LLM(model_dir, dtype="bfloat16", device=device, kvcache_block_size=16, max_num_seqs=4, max_cache_tokens=256,
                  max_num_batched_tokens=64, max_model_len=64, enforce_eager=eager)
        outs[eager] = [o["token_ids"] for o in llm.generate([list(p) for p in prompts],
                                                           SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True))]
        llm.exit()
    compared = 0
    for p, a, b in zip(prompts, outs[True], outs[False]):
        seq = list(p)
        for x, y in zip(a, b):
            logits = oracle.forward(seq, weights, cfg)[0][-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() < 0.05 * logits.std().item() or x != int(logits.argmax()):
                break                       # a close call (or bf16 already chose otherwise): the continuations part ways
            assert x == y, (seq[len(p):], a, b)
            compared += 1
            seq.append(x)
    assert compared >= steps, "too few decided tokens: pick another seed"



