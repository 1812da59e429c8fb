"""Cases of the Givozen tests, written once and run by the CPU test file (host logic with the package's torch
restatement of the kernels) and the GPU test file (the HIP kernels): every mechanism alone against
oracle/givozen_oracle.py, then the engine on whole prompts, token-by-token decoding, portions, mixed batches,
reused pages and slots, long decoding and greedy generation."""
from __future__ import annotations

import torch

from oracle import givozen_oracle as oracle
from tests import _givozen as K

F64 = torch.float64


def _dt(name):
    return {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]


# ------------------------------------------------------------------------------- single mechanisms
def case_sandwich_norm(device, dtype):
    """The f32 residual receives the normed sublayer output, then a row of activations and a vector; the next
    norm reads the sum. Every part alone and all together, widths that are no multiple of the workgroup."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(1)
    tol = 1e-5 if dtype == "float32" else 1e-2
    for T, W in ((7, 48), (3, 37), (5, 1000), (2, 256)):
        x = 5 * torch.randn(T, W, generator=g)
        y, rows = (3 * torch.randn(T, W, generator=g).to(_dt(dtype)) for _ in range(2))
        post, w, vec = (0.4 * torch.randn(W, generator=g) for _ in range(3))
        for use_y, use_rows, use_vec, use_w in ((1, 1, 1, 1), (1, 0, 0, 1), (0, 1, 0, 1), (0, 0, 1, 1), (0, 0, 0, 1), (1, 0, 1, 0)):
            xd = x.clone().to(device)
            h = mix_ops.sandwich_add_norm(xd, y.to(device) if use_y else None, post.to(device) if use_y else None,
                                          rows.to(device) if use_rows else None, vec.to(device) if use_vec else None,
                                          w.to(device) if use_w else None, 1.0, 1e-5, _dt(dtype))
            want = x.to(F64)
            if use_y:
                want = want + oracle.norm(y.to(F64), post.to(F64), 1e-5)
            if use_rows:
                want = want + rows.to(F64)
            if use_vec:
                want = want + vec.to(F64)
            assert torch.allclose(xd.cpu().to(F64), want, rtol=2e-6, atol=2e-5), ("the residual is f32", T, W)
            if use_w:
                assert torch.allclose(h.cpu().to(F64), oracle.norm(want, w.to(F64), 1e-5), rtol=tol, atol=tol)
            else:
                assert h is None


def case_inv_freq(device):
    """The frequency table with and without wavelength-dependent scaling: short waves kept, long ones slowed, the band between blended."""
    from light_vllm_amd import mix_ops
    for rot in ({"base": 10000.0, "dims": 32}, {"base": 500.0, "dims": 16, "scaling": {"factor": 6.0, "low": 0.5, "high": 3.0, "original": 64}},
                {"base": 1e6, "dims": 64, "scaling": {"factor": 3.0, "low": 2.0, "high": 9.0, "original": 512}},
                {"base": 10.0, "dims": 2, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 16}}):
        got = mix_ops.rotary_inv_freq(rot["dims"], rot["base"], device, rot.get("scaling")).cpu().to(F64)
        want = torch.tensor(oracle.rotary_frequencies(rot), dtype=F64)
        assert torch.allclose(got, want, rtol=1e-6, atol=0), rot
        if "scaling" in rot and rot["dims"] >= 16:
            plain = torch.tensor(oracle.rotary_frequencies({"base": rot["base"], "dims": rot["dims"]}), dtype=F64)
            ratio = want / plain
            assert ratio.max() == 1.0 and abs(ratio.min().item() - 1.0 / rot["scaling"]["factor"]) < 1e-12
            assert ((ratio < 1.0) & (ratio > 1.0 / rot["scaling"]["factor"])).any(), "no frequency falls into the blended band"


def case_rotary_store(device, dtype):
    """Rotation of part of every query and key head at positions that continue a context across pages and far out,
    the head factor on queries only, keys and values in the cache rows the page table names."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(2)
    shapes = ((4, 2, 12, 10, K.ROT_A, 0), (1, 1, 40, 70, {"base": 300.0, "dims": 40}, 0), (5, 1, 6, 4, None, 0),
              (6, 3, 16, 32, {"base": 10.0, "dims": 2}, 0), (2, 2, 48, 16, {"base": 1e5, "dims": 32}, 0),
              # columns and sizes in multiples of four: the kernel's four-at-a-time form, part of a head rotated, all of it, none
              (2, 2, 48, 16, {"base": 1e5, "dims": 32}, 1), (3, 1, 8, 8, {"base": 40.0, "dims": 8}, 1), (2, 1, 16, 4, None, 1),
              (4, 2, 64, 32, {"base": 2000.0, "dims": 24, "scaling": {"factor": 5.0, "low": 1.0, "high": 3.0, "original": 128}}, 1))
    for (H, G, D, Dv, rot, lined_up) in shapes:
        for ctx in (29, 70000):
            page, T = 16, 21
            first = ctx // page
            table = {first + i: p for i, p in enumerate([2, 0, 3, 1])}
            row = [0] * (first + 4)
            for j, p in table.items():
                row[j] = p
            ld = 5 + H * D + G * D + G * Dv + 3
            off_q, off_k, off_v = 2, 2 + H * D + 1, 2 + H * D + 1 + G * D + 2
            if lined_up:
                ld, off_q, off_k, off_v = H * D + G * D + G * Dv + 4, 0, H * D, H * D + G * D
            proj = torch.randn(T, ld, generator=g).to(_dt(dtype))
            temp = 1 + 0.5 * torch.randn(H, generator=g)
            dims = int(rot["dims"]) if rot else 0
            inv_freq = mix_ops.rotary_inv_freq(max(dims, 2), rot["base"] if rot else 1.0, device, (rot or {}).get("scaling"))
            kc = torch.zeros(5, page, G, D, dtype=_dt(dtype), device=device)
            vc = torch.zeros(5, page, G, Dv, dtype=_dt(dtype), device=device)
            step = K.make_step([T - 2, 2], [ctx, ctx + T - 2], [0, 1], [row, row], device)      # two portions, one sequence's rows
            q = mix_ops.rotary_store(proj.to(device), off_q, off_k, off_v, inv_freq, temp.to(device), kc, vc, step, H, G, D, Dv, dims)
            q = q.cpu().to(F64).view(T, H, D)
            p64 = proj.to(F64)
            pos = list(range(ctx, ctx + T))
            freqs = oracle.rotary_frequencies(rot) if rot else []
            # f32 angles: position times a rounded frequency is good to 1e-7 of the angle
            tol = (2e-5 if ctx < 1000 else 2e-2) if dtype == "float32" else 2e-2
            for h in range(H):
                want = oracle.rotate(p64[:, off_q + h * D:off_q + (h + 1) * D], pos, freqs) * float(temp[h])
                assert torch.allclose(q[:, h], want, rtol=tol, atol=tol), ("q", H, D, ctx)
            for r in range(T):
                kr = kc.cpu()[table[pos[r] // page], pos[r] % page].to(F64)
                vr = vc.cpu()[table[pos[r] // page], pos[r] % page].to(F64)
                for gg in range(G):
                    want = oracle.rotate(p64[r:r + 1, off_k + gg * D:off_k + (gg + 1) * D], [pos[r]], freqs)[0]
                    assert torch.allclose(kr[gg], want, rtol=tol, atol=tol), ("k", r, gg, ctx)
                assert torch.equal(vr.reshape(-1), p64[r, off_v:off_v + G * Dv])


def case_attention_beacons(device, dtype):
    """Causal softmax over a paged cache with a temperature per head (folded into the queries) and a gate per head.
    A few beacon keys score far above the hundreds of others: the very first tokens, rows either side of page borders,
    one far back. Prompt-shaped, decode-shaped and portion-shaped launches; the head whose temperature is small
    barely sees the beacons, so a temperature applied to the wrong head shows."""
    from light_vllm_amd import mix_ops
    from light_vllm_amd.layers.rotary_attention import NO_WINDOW
    for (H, G, D, Dv, page, L) in ((4, 2, 12, 10, 16, 300), (1, 1, 40, 70, 64, 333), (10, 1, 6, 4, 16, 120),
                                   (5, 1, 32, 16, 16, 300), (4, 2, 16, 48, 32, 410), (2, 2, 48, 32, 64, 200),
                                   (12, 4, 32, 64, 64, 260)):
        g = torch.Generator().manual_seed(L + H)
        beacons = [0, 1, page - 1, page, 2 * page + 1, 50]
        e = torch.zeros(D); e[D - 1] = 1.0
        k = 0.3 * torch.randn(L, G, D, generator=g)
        for j in beacons:
            k[j] += 6.0 * e
        v = torch.randn(L, G, Dv, generator=g)
        q = 0.3 * torch.randn(L, H, D, generator=g) + 3.0 * e
        temp = torch.linspace(0.05, 1.6, H) if H > 1 else torch.tensor([1.3])
        gate = torch.randn(L, H, generator=g)
        k, v, q, gate = (t.to(_dt(dtype)).float() for t in (k, v, q, gate))
        scale = 0.7
        qs = (q * temp.view(1, H, 1)).to(_dt(dtype)).float()          # what the rotation kernel hands to the attention
        want = torch.cat([oracle.causal_softmax_head(qs[:, h].to(F64), k[:, h // (H // G)].to(F64), v[:, h // (H // G)].to(F64), scale)
                          * torch.sigmoid(gate[:, h:h + 1].to(F64)) for h in range(H)], -1)
        s = (k[:, G - 1].to(F64) @ qs[L - 1, H - 1].to(F64)) * scale
        p_last = torch.softmax(s, 0)                   # the beacons hold the weight of a late row, the far one a good part of it
        assert p_last[beacons].sum() > 0.9 and p_last[0] > 0.01, (p_last[beacons], H, L)
        num_pages = -(-L // page) + 3
        table = torch.randperm(num_pages, generator=g).tolist()[:-(-L // page)]
        kc = torch.zeros(num_pages, page, G, D, dtype=_dt(dtype))
        vc = torch.zeros(num_pages, page, G, Dv, dtype=_dt(dtype))
        for j in range(L):
            kc[table[j // page], j % page] = k[j].to(_dt(dtype))
            vc[table[j // page], j % page] = v[j].to(_dt(dtype))
        kc, vc = kc.to(device), vc.to(device)
        qd = qs.reshape(L, H * D).to(_dt(dtype)).to(device)
        gd = gate.to(_dt(dtype)).to(device)
        tol = 2e-4 if dtype == "float32" else 5e-2

        def run(step, rows):
            return mix_ops.window_pool_attention(qd[rows].contiguous(), kc, vc, None, None, gd[rows].contiguous(), step, H, G, D, Dv,
                                                 NO_WINDOW, 0, scale, has_sink=False, gate_per_head=True)

        def check(got, idx, what):
            err = (got.cpu().to(F64) - want[idx]).abs().max().item()
            assert err <= tol * want.abs().max().item(), (what, H, G, D, Dv, page, err)

        every = list(range(L))
        check(run(K.make_step([L], [0], [0], [table], device), every), every, "prompt")
        idx = sorted({i for j in beacons for i in (j - 1, j, j + 1) if 0 <= i < L} | set(range(L - 20, L)))
        check(run(K.make_step([1] * len(idx), idx, [0] * len(idx), [table] * len(idx), device), idx), idx, "decode")
        few = idx[-3:]
        check(run(K.make_step([1] * 3, few, [0] * 3, [table] * 3, device), few), few, "decode, few sequences")
        check(run(K.make_step([2], [L - 2], [0], [table], device), [L - 2, L - 1]), [L - 2, L - 1], "two tokens behind a long context")
        a, b = page - 1, page + 1           # a portion of two tokens across a page border beside the start of a sequence
        rows = list(range(a, b)) + list(range(5))
        check(run(K.make_step([b - a, 5], [a, 0], [0, 1], [table, table], device), rows), rows, "portions")


def case_polynorm(device, dtype):
    """The learned cubic of row-normalised powers: row lengths around and far above a workgroup, strided input, large values."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(3)
    tol = 2e-5 if dtype == "float32" else 2e-2
    for T, Fd, spread in ((5, 40, 1.0), (3, 257, 4.0), (2, 3000, 0.02), (4, 96, 30.0)):
        buf = (spread * torch.randn(T, Fd + 7, generator=g)).to(_dt(dtype))
        z = buf[:, 3:3 + Fd]
        coef = torch.tensor([0.7, 0.4, -0.2, 0.1]) + 0.1 * torch.randn(4, generator=g)
        want = oracle.polynorm(z.to(F64), coef.to(F64), 1e-5)
        for zd in (buf.to(device)[:, 3:3 + Fd], z.contiguous().to(device)):          # a view of wider rows, and rows of their own
            got = mix_ops.polynorm(zd, coef.to(device), 1e-5).cpu().to(F64)
            assert torch.allclose(got, want, rtol=tol, atol=tol * want.abs().max().item()), (T, Fd, spread)
    # the three norms are separate: a row with one large entry has R(z^3) close to a one-hot vector
    z = torch.full((1, 64), 0.1); z[0, 5] = 20.0
    got = mix_ops.polynorm(z.to(_dt(dtype)).to(device), torch.tensor([0.0, 0.0, 1.0, 0.0], device=device), 1e-6).cpu().float()
    assert abs(got[0, 5].item() - 8.0) < 0.05 and got[0, 0].abs().item() < 1e-4


def case_moe_route_raw(device):
    """Sigmoid scores, the largest win, weights are the winners' own scores (they do not sum to one); the kernel takes
    the lowest index first on ties."""
    from light_vllm_amd import mix_ops
    logits = torch.tensor([[2.0, -1.0, 0.5, 3.0, -4.0], [0.0, 0.0 if device != "cpu" else -0.01, -1.0, -2.0, -3.0],
                           [-9.0, -8.0, -7.0, -6.0, -5.0]])
    ids, w, dense = mix_ops.moe_route(logits.to(device), None, 2, 1, 1, normalize=False)
    assert ids.cpu().tolist() == [[3, 0], [0, 1], [4, 3]]
    s = torch.sigmoid(logits)
    assert torch.allclose(w.cpu(), torch.stack([s[0, [3, 0]], s[1, [0, 1]], s[2, [4, 3]]]), rtol=1e-6)
    assert torch.allclose(dense.cpu().sum(-1), w.cpu().sum(-1), rtol=1e-6) and (dense.cpu() > 0).sum().item() == 6
    _, wn, _ = mix_ops.moe_route(logits.to(device), None, 2, 1, 1)                      # the normalised form still sums to one
    assert torch.allclose(wn.cpu().sum(-1), torch.ones(3), rtol=1e-6)
    g = torch.Generator().manual_seed(4)
    for T, E, top in ((33, 6, 2), (9, 3, 3), (20, 70, 5), (5, 2, 1)):
        logits = 2 * torch.randn(T, E, generator=g)
        ids, w, _ = mix_ops.moe_route(logits.to(device), None, top, 1, 1, normalize=False)
        want = torch.sigmoid(logits).sort(dim=-1, descending=True, stable=True)
        assert torch.equal(ids.cpu().long(), want.indices[:, :top]) and torch.allclose(w.cpu(), want.values[:, :top], rtol=1e-6)


def case_router_logits(device):
    """The router's f32 logits from bf16 and f32 activations, in the kernel of small steps and through the GEMM of large
    ones, rows of a wider tensor, widths that are no multiple of four, expert counts that are no multiple of the group."""
    from light_vllm_amd import mix_ops
    g = torch.Generator().manual_seed(6)
    for T, W, E, dt in ((7, 48, 6, torch.float32), (40, 200, 33, torch.bfloat16), (300, 64, 8, torch.bfloat16),
                        (3, 1001, 5, torch.float32), (16, 2048, 32, torch.bfloat16), (5, 30, 1, torch.bfloat16)):
        buf = torch.randn(T, W + 8, generator=g).to(dt)
        rw = torch.randn(E, W, generator=g) / W ** 0.5
        want = buf[:, 8:].to(F64) @ rw.to(F64).T
        for hd in (buf.to(device)[:, 8:], buf[:, 8:].contiguous().to(device)):
            got = mix_ops.router_logits(hd, rw.to(device)).cpu().to(F64)
            assert got.shape == (T, E) and (got - want).abs().max().item() <= 2e-5 * max(1.0, want.abs().max().item()), (T, W, E, dt)


def case_moe_ff(device, dtype):
    """The mixture with gated experts in both forms against the oracle: the weight scales the expert's INPUT (with a small
    clamp the two readings differ by far), the shared expert and its token gate, every expert chosen, one expert."""
    from light_vllm_amd.layers import moe as moe_mod
    g = torch.Generator().manual_seed(5)
    cases = [(48, 20, 6, 2, 12, 37), (40, 8, 3, 3, 0, 9), (64, 32, 8, 3, 48, 50), (64, 64, 4, 1, 0, 300), (32, 32, 5, 2, 24, 1),
             (96, 32, 16, 4, 8, 700)]
    for (W, Fe, E, top, Fs, T) in cases:
        forms = ["masked"] + (["gathered", "sorted"] if device == "cpu" or (dtype == "bfloat16" and W % 32 == 0 and Fe % 32 == 0
                                                               and (E * Fe + Fs) % 8 == 0) else [])
        mlp = {"expert": {"ff": Fe, "limit": 0.6}, "router": {"experts": E, "top": top}}
        weights = {"router": 2 * torch.randn(E, W, generator=g) / W ** 0.5}
        for e in range(E):
            weights[f"e{e}.gate"] = 1.5 * torch.randn(Fe, W, generator=g) / W ** 0.5
            weights[f"e{e}.up"] = 1.5 * torch.randn(Fe, W, generator=g) / W ** 0.5
            weights[f"e{e}.down"] = torch.randn(W, Fe, generator=g) / Fe ** 0.5
        if Fs:
            mlp["shared"] = {"ff": Fs, "limit": 0.9}
            weights.update({"shared.gate": 1.5 * torch.randn(Fs, W, generator=g) / W ** 0.5, "shared.up": 1.5 * torch.randn(Fs, W, generator=g) / W ** 0.5,
                            "shared.down": torch.randn(W, Fs, generator=g) / Fs ** 0.5, "shared.sg": torch.randn(1, W, generator=g) / W ** 0.5})
        weights = {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
        h = torch.randn(T, W, generator=g).to(_dt(dtype))
        old = torch.get_default_dtype()
        torch.set_default_dtype(_dt(dtype))
        try:
            moe = moe_mod.GLUSparseMoE(W, Fe, E, top, 0.6, 1.702, Fs, 0.9)
        finally:
            torch.set_default_dtype(old)
        with torch.no_grad():
            moe.router_weight.copy_(weights["router"])
            for e in range(E):
                moe.up_weight[e * 2 * Fe:e * 2 * Fe + Fe].copy_(weights[f"e{e}.gate"])
                moe.up_weight[e * 2 * Fe + Fe:(e + 1) * 2 * Fe].copy_(weights[f"e{e}.up"])
                moe.down_weight[:, e * Fe:(e + 1) * Fe].copy_(weights[f"e{e}.down"])
            if Fs:
                b = E * 2 * Fe
                moe.up_weight[b:b + Fs].copy_(weights["shared.gate"])
                moe.up_weight[b + Fs:b + 2 * Fs].copy_(weights["shared.up"])
                moe.up_weight[b + 2 * Fs:].copy_(weights["shared.sg"])
                moe.down_weight[:, E * Fe:].copy_(weights["shared.down"])
        moe = moe.to(device)
        margins = [[] for _ in range(T)]
        w64 = {k: v.to(F64) for k, v in weights.items()}
        want = oracle.moe_ff(h.to(F64), w64, "", mlp, margins)
        rows = [t for t in range(T) if dtype == "float32" or min(margins[t]) >= 1e-2]
        for form in forms:
            old_kernel, moe_mod.MOE_KERNEL = moe_mod.MOE_KERNEL, form
            try:
                with torch.inference_mode():
                    got = moe(h.to(device)).cpu().to(F64)
            finally:
                moe_mod.MOE_KERNEL = old_kernel
            tol = 1e-4 if dtype == "float32" else 4e-2
            assert (got[rows] - want[rows]).abs().max().item() <= tol * want.abs().max().item(), (W, Fe, E, top, Fs, T, form)
        # the other reading (weight on the output) is far away: the test tells the two apart
        ids, ws, _ = oracle.route(h.to(F64), w64, "", top)
        other = torch.zeros_like(want)
        for t in range(T):
            for e, w in zip(ids[t].tolist(), ws[t]):
                other[t] += w * oracle.glu_expert(h[t].to(F64)[None], w64, f"e{e}.", 0.6)[0]
        if Fs:
            other = other + torch.sigmoid(h.to(F64) @ w64["shared.sg"].T) * oracle.glu_expert(h.to(F64), w64, "shared.", 0.9)
        assert (other - want).abs().max().item() > 0.05 * want.abs().max().item()


# ------------------------------------------------------------------------------------- the engine
def _model(tmp_path, cfg, seed):
    weights = oracle.random_weights(cfg, seed)
    return K.write_model(tmp_path / f"m{seed}", cfg, weights), weights


ROUTE_MARGIN = 0.03      # bf16 runs: a router decided by less than this (in score units) may choose otherwise after rounding


def _oracle_runs(cfg, weights, prompts, dtype):
    """id -> (logits [len, vocab], positions whose routing was no close call in the oracle; all of them for f32 runs).
    A token whose experts differ is another computation, not a rounding of this one, so bf16 comparisons leave those out."""
    want, decided = {}, {}
    for i, t in prompts.items():
        margins = []
        want[i] = oracle.forward(t, weights, cfg, margins=margins)[0]
        decided[i] = [j for j, m in enumerate(margins) if dtype == "float32" or m >= ROUTE_MARGIN]
        assert len(decided[i]) >= max(2, len(t) // 10), "too many close calls: pick another seed"
    return want, decided


def case_checkpoint_placement(tmp_path):
    """Every tensor of a checkpoint lands where the oracle reads it: merged projections, biases, experts' row and column
    blocks, the shared expert behind them, passes of a loop on the same parameters, the head on the embedding table."""
    import json
    import os
    from light_vllm_amd.models.givozen import GivozenConfig, GivozenForCausalLM
    cfg = K.CFG_MAIN
    weights = oracle.random_weights(cfg, 3)
    model_dir = K.write_model(tmp_path / "m", cfg, weights)
    config = GivozenConfig.from_pretrained(model_dir)
    assert [i for i, _ in config.runs()] == [0, 1, 2, 1, 2, 1, 2, 3] and [t for _, t in config.runs()] == [None, 0, None, 1, None, 2, None, None]
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float32)
    try:
        model = GivozenForCausalLM(config)
    finally:
        torch.set_default_dtype(old)
    model.load_weights(weights.items())
    assert model.lm_head.weight is model.embed.weight
    assert len(model.order) == 8 and len(model.repeats) == 4
    first, again = model.order[1][0], model.order[3][0]
    assert again is not first and again.mix is not first.mix and again.mix.in_proj is first.mix.in_proj and again.mlp is first.mlp
    mix = model.layers[1].mix
    a, b, c = mix.sizes[0], mix.sizes[0] + mix.sizes[1], mix.sizes[0] + mix.sizes[1] + mix.sizes[2]
    assert torch.equal(mix.in_proj.weight[a:b].double(), weights["l1.mix.k"]) and torch.equal(mix.in_proj.bias[b:c].double(), weights["l1.mix.v.b"])
    assert torch.equal(mix.in_proj.weight[c:].double(), weights["l1.mix.g"]) and mix.in_proj.bias[c:].abs().max().item() == 0
    moe = model.layers[1].mlp
    Fe, E, Fs = moe.ff, moe.E, moe.Fs
    assert torch.equal(moe.up_weight[4 * 2 * Fe + Fe:5 * 2 * Fe].double(), weights["l1.mlp.e4.up"])
    assert torch.equal(moe.down_weight[:, E * Fe:].double(), weights["l1.mlp.shared.down"])
    assert torch.equal(moe.up_weight[E * 2 * Fe + 2 * Fs:].double(), weights["l1.mlp.shared.sg"])
    short = dict(weights)
    del short["l2.mix.temp"]
    try:
        model.load_weights(short.items())
        raise AssertionError("a missing tensor went unnoticed")
    except KeyError:
        pass
    bad = json.load(open(os.path.join(model_dir, "config.json")))
    bad["layers"][0]["type"] = "recurrent"
    try:
        GivozenConfig.from_dict(bad)
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
    want = oracle.forward(tokens, weights, cfg)[1]
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
        assert (a.to(F64) - b).abs().max().item() <= 3e-4 * b.abs().max().item(), f"layer run {i}"


def case_engine_schedules(device, dtype, tmp_path, cfg=None, seed=5):
    """Whole prompts, token-by-token decoding, portions down to two tokens and mixed batches of unequal
    requests give the logits of the whole-sequence oracle at every position: the first tokens and every
    page border included (pages of 16 tokens)."""
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


def case_engine_reuse(device, dtype, tmp_path):
    """More requests than state slots and more tokens than pages: both are given back and used again,
    in another order, and a sequence that starts on used pages starts from nothing."""
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
    """Hundreds of single-token steps through the caches of every pass."""
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
