"""Tensor-level wrappers over liblvmix.so (include/lv_mixers.h), one function per kernel.

GPU tensors go to the HIP kernels (bf16 or f32 activations; streams, recurrent state and the small
parameter vectors always f32). CPU tensors, which only the plumbing tests of the engine produce,
take a restatement in torch ops ON THE SAME cache and state layouts, so that page tables, state
slots and ragged batching are exercised without a GPU. Nothing here synchronises.

`step` is the utils.context.RaggedStep of the running forward pass: device tensors cu_q [B+1],
ctx_lens [B], slots [B], tok_seq [T], block_tables [B, n] and the same lengths as python ints.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import _mixlib

_DT = {torch.bfloat16: 0, torch.float32: 1}
# windowed pooled attention: "auto" takes the matrix-core kernel where it applies (bf16, head sizes that
# are multiples of 16 up to 256) and the vector kernel elsewhere (f32, other head sizes); "valu" forces the latter
WINDOW_ATTN_KERNEL = "auto"


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


def _f32(*ts):
    for t in ts:
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous()), "expected a contiguous f32 tensor"


# ---------------------------------------------------------------------------------------- streams
def hc_update_norm(x, y=None, mix=None, out_w=None, in_w=None, norm_w=None, groups=1, eps=1e-6, act_dtype=None):
    """x [T, S, W] f32 is updated in place from the sublayer output y [T, W] (skipped when y is None);
    returns the grouped-RMS-normed read-out sum_s in_w[s] x[s] in act dtype (None when in_w is None)."""
    T, S, W = x.shape
    _f32(x, mix, out_w, in_w, norm_w)
    act_dtype = act_dtype or (y.dtype if y is not None else torch.bfloat16)
    out = torch.empty(T, W, dtype=act_dtype, device=x.device) if in_w is not None else None
    if x.is_cuda:
        if y is not None:
            assert y.is_contiguous() and y.dtype == act_dtype and y.shape == (T, W)
        lib = _mixlib.load()
        _mixlib.check(lib.lv_hc_update_norm(_p(x), _p(y), _p(mix), _p(out_w), _p(in_w), _p(norm_w), _p(out), T, S, W,
                                            groups, eps, _DT[act_dtype], _stream(x)), "lv_hc_update_norm")
        return out
    if y is not None:
        x.copy_(torch.einsum("sr,tsw->trw", mix, x) + out_w[None, :, None] * y.float()[:, None, :])
    if in_w is None:
        return None
    u = torch.einsum("s,tsw->tw", in_w, x)
    ug = u.view(T, groups, W // groups)
    ug = ug / torch.sqrt(ug.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_(ug.reshape(T, W) * norm_w)
    return out


def residual_add_norm(x, y1=None, y2=None, w=None, w_offset=0.0, eps=1e-6, act_dtype=None):
    """x [T, W] f32 (the one residual) += y1 + y2 in place (either may be None); returns
    x / sqrt(mean(x^2) + eps) * (w_offset + w) in act dtype, or None when w is None."""
    T, W = x.shape
    _f32(x, w)
    ys = [y for y in (y1, y2) if y is not None]
    act_dtype = act_dtype or (ys[0].dtype if ys else torch.bfloat16)
    out = torch.empty(T, W, dtype=act_dtype, device=x.device) if w is not None else None
    if x.is_cuda:
        for y in ys:
            assert y.is_contiguous() and y.dtype == act_dtype and y.shape == (T, W)
        lib = _mixlib.load()
        _mixlib.check(lib.lv_residual_add_norm(_p(x), _p(y1), _p(y2), _p(w), w_offset, _p(out), T, W, eps, _DT[act_dtype],
                                               _stream(x)), "lv_residual_add_norm")
        return out
    if ys:
        add = ys[0].float()
        if len(ys) > 1:
            add = add + ys[1].float()
        x.add_(add)
    if w is None:
        return None
    out.copy_(x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (w_offset + w))
    return out


def sandwich_add_norm(x, y=None, post_w=None, rows=None, vec=None, w=None, w_offset=1.0, eps=1e-6, act_dtype=None):
    """The residual update of a layer that norms each sublayer's output as well as its input, fused with
    what follows it. x [T, W] f32, in place:
        x += y / sqrt(mean(y^2) + eps) * (w_offset + post_w)      (y act [T, W]; skipped when y is None)
        x += rows + vec                                            (rows act [T, W], vec f32 [W]; either may be None)
    and returns x / sqrt(mean(x^2) + eps) * (w_offset + w) in act dtype (None when w is None). All sums and
    both norms are f32."""
    T, W = x.shape
    _f32(x, post_w, vec, w)
    assert (y is None) == (post_w is None)
    act_dtype = act_dtype or next((t.dtype for t in (y, rows) if t is not None), torch.bfloat16)
    out = torch.empty(T, W, dtype=act_dtype, device=x.device) if w is not None else None
    if x.is_cuda:
        for t in (y, rows):
            assert t is None or (t.is_contiguous() and t.dtype == act_dtype and t.shape == (T, W))
        lib = _mixlib.load()
        _mixlib.check(lib.lv_sandwich_add_norm(_p(x), _p(y), _p(post_w), _p(rows), _p(vec), _p(w), w_offset, _p(out), T, W,
                                               eps, _DT[act_dtype], _stream(x)), "lv_sandwich_add_norm")
        return out
    if y is not None:
        yf = y.float()
        x.add_(yf / torch.sqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * (w_offset + post_w))
    if rows is not None:
        x.add_(rows.float())
    if vec is not None:
        x.add_(vec)
    if w is None:
        return None
    out.copy_(x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (w_offset + w))
    return out


def polynorm(z, coef, eps):
    """z act [T, F] -> act [T, F] = c1 R(z) + c2 R(z^2) + c3 R(z^3) + c0 with coef = (c1, c2, c3, c0) f32 [4], powers
    element by element and R(u) = u / sqrt(mean_F(u^2) + eps) per token, in f32."""
    T, Fd = z.shape
    _f32(coef)
    out = torch.empty(T, Fd, dtype=z.dtype, device=z.device)
    if z.is_cuda:
        assert z.stride(1) == 1 and coef.numel() == 4
        lib = _mixlib.load()
        _mixlib.check(lib.lv_polynorm(_p(z), z.stride(0), _p(coef), _p(out), T, Fd, eps, _DT[z.dtype], _stream(z)), "lv_polynorm")
        return out
    zf = z.float()
    acc = coef[3].expand_as(zf).clone()
    for k in range(3):
        u = zf.pow(k + 1)
        acc = acc + coef[k] * u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_(acc)
    return out


def expert_glu(x, E, Fe, limit, alpha, in_scale=None, out_gate=None, out=None):
    """Clamped gated unit of E experts side by side. x act [T, E*2*Fe] (row stride free), expert e's columns
    [gate Fe | up Fe]. With in_scale f32 [T, E] the pre-activations are multiplied by in_scale[t, e] first (the
    expert ran on its input times that number; an expert whose number is 0 gives zeros). With out_gate (act [T],
    any stride) the result is multiplied by sigmoid(out_gate[t]).
        g = min(s * gate, L); u = clamp(s * up, -L, L); y = g * sigmoid(alpha * g) * (u + 1)
    Writes act [T, E*Fe] into `out` (a view with free row stride) or a new tensor; returns it."""
    T = x.size(0)
    assert x.size(1) == E * 2 * Fe and x.stride(1) == 1
    if out is None:
        out = torch.empty(T, E * Fe, dtype=x.dtype, device=x.device)
    assert out.shape == (T, E * Fe) and out.stride(1) == 1 and out.dtype == x.dtype
    if x.is_cuda:
        assert in_scale is None or (in_scale.dtype == torch.float32 and in_scale.is_contiguous() and in_scale.shape == (T, E))
        assert out_gate is None or (out_gate.dtype == x.dtype and out_gate.shape == (T,))
        lib = _mixlib.load()
        _mixlib.check(lib.lv_expert_glu(_p(x), x.stride(0), _p(in_scale), _p(out_gate), out_gate.stride(0) if out_gate is not None else 0,
                                        _p(out), out.stride(0), T, E, Fe, limit, alpha, _DT[x.dtype], _stream(x)), "lv_expert_glu")
        return out
    xe = x.float().view(T, E, 2, Fe)
    sc = in_scale.view(T, E, 1) if in_scale is not None else 1.0
    g = (xe[:, :, 0] * sc).clamp(max=limit)
    u = (xe[:, :, 1] * sc).clamp(-limit, limit)
    yv = g * torch.sigmoid(alpha * g) * (u + 1)
    if in_scale is not None:
        yv = torch.where(in_scale.view(T, E, 1) != 0, yv, torch.zeros_like(yv))
    if out_gate is not None:
        yv = yv * torch.sigmoid(out_gate.float()).view(T, 1, 1)
    out.copy_(yv.reshape(T, E * Fe))
    return out


def clamped_glu(x, limit: float, alpha: float):
    """x [T, 2F] = [gate | up] -> min(g, L) * sigmoid(alpha * g) * (clamp(u, -L, L) + 1), [T, F]."""
    T, F2 = x.shape
    Fh = F2 // 2
    out = torch.empty(T, Fh, dtype=x.dtype, device=x.device)
    if x.is_cuda:
        assert x.stride(1) == 1
        lib = _mixlib.load()
        _mixlib.check(lib.lv_clamped_glu(_p(x), x.stride(0), _p(out), T, Fh, limit, alpha, _DT[x.dtype], _stream(x)),
                      "lv_clamped_glu")
        return out
    g = x[:, :Fh].float().clamp(max=limit)
    u = x[:, Fh:].float().clamp(-limit, limit)
    out.copy_(g * torch.sigmoid(alpha * g) * (u + 1))
    return out


# ------------------------------------------------------------------------------------- delta rule
def delta_prep(proj, conv_w, conv_state, A_log, dt_bias, step, G, H, D, Dv, taps, off_b, a, unit_eps,
               decay_per_channel=False):
    """Short causal convolution + silu over the q | k | v channels of `proj` [T, ld] (taps from the
    portion's own rows, then from the carried state of the sequence's slot, zeros before position
    0), unit-norm q (times D^-1/2) and k per head, beta = sigmoid(b), decay = exp(-exp(A_log) *
    softplus(a + dt_bias)) with a [T, H] (a view of proj's columns or a tensor of its own), or
    [T, H*D] with decay_per_channel (dt_bias [H*D], A_log [H]).
    Returns f32 (qn [T,G,D], kn [T,G,D], v [T,H,Dv], beta [T,H], decay [T,H] or [T,H,D])."""
    T = proj.size(0)
    dev = proj.device
    _f32(conv_w, A_log, dt_bias)
    nd = D if decay_per_channel else 1
    assert a.shape == (T, H * nd) and a.dtype == proj.dtype and dt_bias.numel() == H * nd
    qn = torch.empty(T, G, D, dtype=torch.float32, device=dev)
    kn = torch.empty(T, G, D, dtype=torch.float32, device=dev)
    v = torch.empty(T, H, Dv, dtype=torch.float32, device=dev)
    beta = torch.empty(T, H, dtype=torch.float32, device=dev)
    decay = torch.empty((T, H, D) if decay_per_channel else (T, H), dtype=torch.float32, device=dev)
    C = 2 * G * D + H * Dv
    assert conv_state.is_contiguous() and conv_state.shape[1:] == (taps - 1, C) and conv_state.dtype == proj.dtype
    if proj.is_cuda:
        assert proj.stride(1) == 1 and a.stride(1) == 1
        lib = _mixlib.load()
        _mixlib.check(lib.lv_delta_prep(_p(proj), proj.stride(0), _p(conv_w), _p(conv_state), _p(A_log), _p(dt_bias),
                                        _p(step.cu_q), _p(step.ctx_lens), _p(step.slots), _p(step.tok_seq), _p(qn),
                                        _p(kn), _p(v), _p(beta), _p(decay), T, G, H, D, Dv, taps, off_b, _p(a),
                                        a.stride(0), int(decay_per_channel), unit_eps, _DT[proj.dtype], _stream(proj)),
                      "lv_delta_prep")
        return qn, kn, v, beta, decay
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        rows = proj[q0:q0 + n, :C].float()
        hist = conv_state[step.host_slots[b]].float() if ctx > 0 else torch.zeros(taps - 1, C)
        if 0 < ctx < taps - 1:
            hist = hist.clone()
            hist[:taps - 1 - ctx] = 0
        full = torch.cat([hist, rows])
        y = sum(full[i:i + n] * conv_w[:, i] for i in range(taps))
        y = F.silu(y)
        qq = y[:, :G * D].view(n, G, D)
        kk = y[:, G * D:2 * G * D].view(n, G, D)
        qn[q0:q0 + n] = qq / torch.sqrt(qq.pow(2).sum(-1, keepdim=True) + unit_eps) * D ** -0.5
        kn[q0:q0 + n] = kk / torch.sqrt(kk.pow(2).sum(-1, keepdim=True) + unit_eps)
        v[q0:q0 + n] = y[:, 2 * G * D:].view(n, H, Dv)
        beta[q0:q0 + n] = torch.sigmoid(proj[q0:q0 + n, off_b:off_b + H].float())
        sp = F.softplus(a[q0:q0 + n].float() + dt_bias.view(-1))
        rate = torch.exp(A_log)
        if decay_per_channel:
            decay[q0:q0 + n] = torch.exp(-rate[None, :, None] * sp.view(n, H, D))
        else:
            decay[q0:q0 + n] = torch.exp(-rate * sp)
        q0 += n
    return qn, kn, v, beta, decay


def conv_state_update(proj, conv_state, step, C, taps):
    """conv_state[slot] <- the last taps-1 convolution inputs of every sequence after this step."""
    if taps <= 1:
        return
    if proj.is_cuda:
        lib = _mixlib.load()
        _mixlib.check(lib.lv_conv_state_update(_p(proj), proj.stride(0), _p(conv_state), _p(step.cu_q),
                                               _p(step.ctx_lens), _p(step.slots), len(step.host_lens_q), C, taps,
                                               _DT[proj.dtype], _stream(proj)), "lv_conv_state_update")
        return
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        slot = step.host_slots[b]
        hist = conv_state[slot].clone() if ctx > 0 else torch.zeros_like(conv_state[slot])
        if 0 < ctx < taps - 1:
            hist[:taps - 1 - ctx] = 0
        full = torch.cat([hist, proj[q0:q0 + n, :C]])
        conv_state[slot] = full[-(taps - 1):]
        q0 += n


def gated_delta_rule(qn, kn, v, beta, decay, state, step):
    """Per head and token: S <- decay * S; u = beta * (v - S^T k); S <- S + k u^T; o = S^T q.
    decay [T, H] scales a head's whole state, decay [T, H, D] each of its rows (key channels) by its own number.
    state f32 [slots, H, D, Dv] (taken as zero for a sequence with no context), updated in place.
    Returns o f32 [T, H, Dv]."""
    T, G, D = qn.shape
    H, Dv = v.shape[1], v.shape[2]
    _f32(qn, kn, v, beta, decay, state)
    assert state.shape[1:] == (H, D, Dv)
    per_channel = decay.dim() == 3
    assert decay.shape == ((T, H, D) if per_channel else (T, H))
    o = torch.empty(T, H, Dv, dtype=torch.float32, device=qn.device)
    if qn.is_cuda:
        lib = _mixlib.load()
        _mixlib.check(lib.lv_gated_delta_rule(_p(qn), _p(kn), _p(v), _p(beta), _p(decay), _p(state), _p(step.cu_q),
                                              _p(step.ctx_lens), _p(step.slots), _p(o), len(step.host_lens_q), G, H, D,
                                              Dv, int(per_channel), _stream(qn)), "lv_gated_delta_rule")
        return o
    rep = H // G
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        slot = step.host_slots[b]
        S = state[slot].clone() if ctx > 0 else torch.zeros(H, D, Dv)
        for t in range(q0, q0 + n):
            k = kn[t].repeat_interleave(rep, 0)      # [H, D]
            q = qn[t].repeat_interleave(rep, 0)
            S = (decay[t][:, :, None] if per_channel else decay[t][:, None, None]) * S
            u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k))
            S = S + k[:, :, None] * u[:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q)
        state[slot] = S
        q0 += n
    return o


def head_norm_gate(o, gate, norm_w, eps, act_dtype, gate_act="silu"):
    """o f32 [T, H, Dv] -> act [T, H*Dv]: per-head RMS norm over Dv, times norm_w [Dv], times silu(gate)
    or sigmoid(gate)."""
    assert gate_act in ("silu", "sigmoid")
    T, H, Dv = o.shape
    _f32(o, norm_w)
    out = torch.empty(T, H * Dv, dtype=act_dtype, device=o.device)
    if o.is_cuda:
        assert gate.stride(1) == 1 and gate.dtype == act_dtype
        lib = _mixlib.load()
        _mixlib.check(lib.lv_head_norm_gate(_p(o), _p(gate), gate.stride(0), _p(norm_w), _p(out), T, H, Dv, eps,
                                            int(gate_act == "sigmoid"), _DT[act_dtype], _stream(o)), "lv_head_norm_gate")
        return out
    y = o / torch.sqrt(o.pow(2).mean(-1, keepdim=True) + eps) * norm_w
    g = F.silu(gate.float()) if gate_act == "silu" else torch.sigmoid(gate.float())
    out.copy_((y * g.view(T, H, Dv)).reshape(T, H * Dv))
    return out


# ------------------------------------------------------------------------- windowed pooled attention
def pooled_slots(page: int, P: int) -> int:
    """Pooled entries a page can own: blocks whose last token lies in it."""
    return -(-page // P) if P > 0 else 0


def _token_slot(bt_row, j, page):
    return bt_row[j // page] * page + j % page


def _pool_slot(bt_row, blk, page, P, PP):
    pj = (blk * P + P - 1) // page
    return bt_row[pj] * PP + blk - (page * pj) // P


def qk_fullnorm_store(q, k, v, q_w, k_w, k_cache, v_cache, step, H, G, D, Dv, eps):
    """RMS norm over the whole q row [H*D] and the whole k row [G*D] (weights q_w, k_w), normed K and
    V scattered into the paged caches [pages, page, G, D|Dv] at each token's position. Returns normed q."""
    T = q.size(0)
    page = k_cache.size(1)
    _f32(q_w, k_w)
    q_out = torch.empty(T, H * D, dtype=q.dtype, device=q.device)
    if q.is_cuda:
        ld = q.stride(0)
        assert k.stride(0) == ld and v.stride(0) == ld and q.stride(1) == 1 and k_cache.is_contiguous() and v_cache.is_contiguous()
        lib = _mixlib.load()
        _mixlib.check(lib.lv_qk_fullnorm_store(_p(q), _p(k), _p(v), ld, _p(q_w), _p(k_w), _p(q_out), _p(k_cache),
                                               _p(v_cache), _p(step.cu_q), _p(step.ctx_lens), _p(step.tok_seq),
                                               _p(step.block_tables), step.block_tables.stride(0), T, H, G, D, Dv, page,
                                               eps, _DT[q.dtype], _stream(q)), "lv_qk_fullnorm_store")
        return q_out
    qf, kf = q.float(), k.float()
    q_out.copy_(qf / torch.sqrt(qf.pow(2).mean(-1, keepdim=True) + eps) * q_w)
    kn = (kf / torch.sqrt(kf.pow(2).mean(-1, keepdim=True) + eps) * k_w).to(k_cache.dtype)
    kc, vc = k_cache.view(-1, G * D), v_cache.view(-1, G * Dv)
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        bt = step.host_block_tables[b]
        for r in range(n):
            s = _token_slot(bt, ctx + r, page)
            kc[s] = kn[q0 + r]
            vc[s] = v[q0 + r]
        q0 += n
    return q_out


def pool_update(k_cache, v_cache, kp, vp, step, G, D, Dv, P):
    """Means of the P cached keys / values of every block this step completed, stored with the page of
    the block's last token (kp, vp: [pages, pooled_slots(page, P), G, D|Dv])."""
    if P <= 0:
        return
    page = k_cache.size(1)
    new_blocks = [(c + n) // P - c // P for n, c in zip(step.host_lens_q, step.host_ctx_lens)]
    most = max(new_blocks, default=0)
    if step.static:        # a replayed graph cannot know: always launch, the kernel leaves when no block was completed
        most = max(-(-n // P) + 1 for n in step.host_lens_q)
    if most == 0:
        return
    if k_cache.is_cuda:
        lib = _mixlib.load()
        _mixlib.check(lib.lv_pool_update(_p(k_cache), _p(v_cache), _p(kp), _p(vp), _p(step.cu_q), _p(step.ctx_lens),
                                         _p(step.block_tables), step.block_tables.stride(0), len(new_blocks), most, G,
                                         D, Dv, page, P, _DT[k_cache.dtype], _stream(k_cache)), "lv_pool_update")
        return
    PP = pooled_slots(page, P)
    kc, vc = k_cache.view(-1, G * D), v_cache.view(-1, G * Dv)
    kpf, vpf = kp.view(-1, G * D), vp.view(-1, G * Dv)
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        bt = step.host_block_tables[b]
        for blk in range(ctx // P, (ctx + n) // P):
            rows = [_token_slot(bt, j, page) for j in range(blk * P, blk * P + P)]
            dst = _pool_slot(bt, blk, page, P, PP)
            kpf[dst] = kc[rows].float().mean(0)
            vpf[dst] = vc[rows].float().mean(0)


def window_pool_attention(q, k_cache, v_cache, kp, vp, gate, step, H, G, D, Dv, window, P, scale, has_sink=True,
                          gate_per_head=False, keep_first=0, chunk=0, sinks=None):
    """Query at position i attends to cached positions j with 0 <= i - j < window and to the pooled
    entry of every block b with b*P + P - 1 <= i - window, one softmax over both, `has_sink` adding 1
    to its denominator; the result is multiplied by sigmoid(gate) when a gate is given (gate rows hold
    H*Dv numbers, one per output channel, or H with `gate_per_head`).
    keep_first > 0: positions j < keep_first are seen from everywhere as well. chunk > 0: instead of a window, a
    query sees the positions of its own chunk, floor(i / chunk) == floor(j / chunk), j <= i (chunks count from
    position 0 of the sequence). sinks f32 [H]: the denominator of head h holds exp(sinks[h]) instead of 1.
    Neither combines with pooled blocks.
    q [T, H*D] contiguous act; returns act [T, H*Dv]. k_cache and v_cache [pages, page, G, D|Dv] may be
    views of wider token rows (one cache row serving as key and, in part, as value). A window that no
    sequence reaches, no pool and no sink give plain causal softmax attention."""
    T = q.size(0)
    page = k_cache.size(1)
    out = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
    k_ld, v_ld = k_cache.stride(1), v_cache.stride(1)
    assert P == 0 or (keep_first == 0 and chunk == 0)
    if sinks is not None:
        _f32(sinks)
        assert sinks.numel() == H
        has_sink = True
    if q.is_cuda:
        assert q.is_contiguous() and (gate is None or (gate.stride(1) == 1 and gate.size(1) == (H if gate_per_head else H * Dv)))
        for c, ld, d in ((k_cache, k_ld, D), (v_cache, v_ld, Dv)):
            assert c.stride(3) == 1 and (G == 1 or c.stride(2) == d) and c.stride(0) == page * ld and ld >= G * d
        lib = _mixlib.load()
        if (WINDOW_ATTN_KERNEL == "auto" and q.dtype == torch.bfloat16 and D % 16 == 0 and Dv % 16 == 0
                and D <= 256 and Dv <= 256 and k_ld % 8 == 0 and v_ld % 4 == 0 and k_cache.data_ptr() % 16 == 0
                and v_cache.data_ptr() % 8 == 0):
            # decode-shaped steps put one workgroup per (sequence, kv head) on the chip: cut each sequence's key
            # tiles over enough workgroups to fill it (partials merged by a second kernel)
            nsplit, ws = 1, None
            B = len(step.host_lens_q)
            if max(step.host_lens_q) <= 16:
                most = max(c + n for c, n in zip(step.host_ctx_lens, step.host_lens_q))
                span = min(most, chunk + 16) if chunk > 0 else min(most, window + 16 + keep_first)
                tiles = -(-span // 64) + (-(-(max(most - window, 0) // P) // 64) if P > 0 else 0)
                nsplit = max(1, min(tiles, 256 // max(B * G * -(-(H // G) // 4), 1), 32))      # one workgroup a CU: more splits cost more in the merge than they gain (measured)
                if nsplit > 1:
                    ws = torch.empty(T * H * nsplit * (Dv + 4), dtype=torch.float32, device=q.device)
            _mixlib.check(lib.lv_masked_attn_mfma(_p(q), _p(k_cache), _p(v_cache), _p(kp), _p(vp), _p(gate),
                                                  gate.stride(0) if gate is not None else 0, _p(out), _p(step.cu_q),
                                                  _p(step.ctx_lens), _p(step.block_tables),
                                                  step.block_tables.stride(0), len(step.host_lens_q),
                                                  max(step.host_lens_q), H, G, D, Dv, page, window, keep_first, chunk, P, scale,
                                                  int(has_sink), _p(sinks), nsplit, _p(ws), T, k_ld, v_ld,
                                                  0 if gate_per_head else 1, _stream(q)),
                          "lv_masked_attn_mfma")
            return out
        _mixlib.check(lib.lv_masked_attn(_p(q), _p(k_cache), _p(v_cache), _p(kp), _p(vp), _p(gate),
                                         gate.stride(0) if gate is not None else 0, _p(out), _p(step.cu_q),
                                         _p(step.ctx_lens), _p(step.tok_seq), _p(step.block_tables),
                                         step.block_tables.stride(0), T, H, G, D, Dv, page, window, keep_first, chunk, P, scale,
                                         int(has_sink), _p(sinks), k_ld, v_ld, 0 if gate_per_head else 1, _DT[q.dtype],
                                         _stream(q)),
                      "lv_masked_attn")
        return out
    PP = pooled_slots(page, P)
    rep = H // G
    kc, vc = k_cache.reshape(-1, G, D), v_cache.reshape(-1, G, Dv)
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        bt = step.host_block_tables[b]
        for r in range(n):
            i = ctx + r
            nb = max(0, (i - window + 1) // P) if P > 0 else 0
            j0 = (i // chunk) * chunk if chunk > 0 else max(0, i - window + 1)
            rows = [_token_slot(bt, j, page) for j in list(range(min(keep_first, j0))) + list(range(j0, i + 1))]
            K, V = kc[rows].float(), vc[rows].float()
            if nb:
                prow = [_pool_slot(bt, blk, page, P, PP) for blk in range(nb)]
                K = torch.cat([kp.view(-1, G, D)[prow].float(), K])
                V = torch.cat([vp.view(-1, G, Dv)[prow].float(), V])
            qi = q[q0 + r].float().view(G, rep, D)
            s = torch.einsum("grd,ngd->grn", qi, K) * scale
            m = s.max(-1, keepdim=True).values
            sk = sinks.view(G, rep, 1) if sinks is not None else torch.zeros(G, rep, 1)
            if has_sink:
                m = torch.maximum(m, sk)
            e = torch.exp(s - m)
            w = e / (e.sum(-1, keepdim=True) + (torch.exp(sk - m) if has_sink else 0))
            o = torch.einsum("grn,ngv->grv", w, V).reshape(H * Dv)
            if gate is not None:
                gr = torch.sigmoid(gate[q0 + r].float())
                o = o * (gr.repeat_interleave(Dv) if gate_per_head else gr)
            out[q0 + r] = o
        q0 += n
    return out


# ------------------------------------------------------------------------------- latent attention
def rotary_inv_freq(dims: int, base: float, device, scaling: dict | None = None) -> torch.Tensor:
    """f32 [dims/2]: base^(-2i/dims), computed in 64-bit and rounded once. `scaling` (factor, low, high,
    original) rescales by wavelength 2 pi / f: waves shorter than original / high keep their frequency,
    waves longer than original / low get f / factor, and those between are blended linearly in
    original / wavelength."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    if scaling:
        factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
        turns = float(scaling["original"]) * f / (2.0 * torch.pi)          # original / wavelength
        blend = ((turns - low) / (high - low)).clamp(0.0, 1.0) if high != low else (turns >= high).double()
        blend = torch.where(turns > high, torch.ones_like(blend), torch.where(turns < low, torch.zeros_like(blend), blend))
        f = (1.0 - blend) * f / factor + blend * f
    return f.float().to(device)


def _rotate(x, pos, inv_freq, dims, interleaved=False):
    """x f32 [n, ..., d]: the first `dims` entries rotated pairwise by pos * inv_freq[i]; pair i is (i, i + dims/2),
    or (2i, 2i + 1) with `interleaved`."""
    if dims == 0:
        return x
    half = dims // 2
    ang = pos.float().view(-1, *([1] * (x.dim() - 1))) * inv_freq.view(*([1] * (x.dim() - 1)), half)
    c, s = torch.cos(ang), torch.sin(ang)
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        turned = torch.stack([u * c - v * s, v * c + u * s], -1).flatten(-2)
        return torch.cat([turned, x[..., dims:]], -1)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def _positions(step, device):
    return torch.cat([torch.arange(c, c + n, device=device) for n, c in zip(step.host_lens_q, step.host_ctx_lens)])


def rotary_store(proj, off_q, off_k, off_v, inv_freq, head_scale, k_cache, v_cache, step, H, G, D, Dv, rot_dims,
                 interleaved=False, unit_eps=None):
    """proj act [T, ld]: queries at column off_q (H heads of D), keys at off_k (G heads of D), values at off_v
    (G heads of Dv). The first rot_dims entries of every query and key head are rotated (entry i pairs with
    i + rot_dims/2, or with `interleaved` entry 2i with 2i + 1; angle = position * inv_freq[i], f32); each query head is
    then multiplied by head_scale[h] (f32 [H], may be None). With unit_eps (a number) every query and key head is first
    divided by sqrt(mean(head^2) + unit_eps). Rotated keys and the values go to the token's row of the paged caches
    [pages, page, G, D|Dv]. Returns the queries, act [T, H*D]."""
    T = proj.size(0)
    page = k_cache.size(1)
    _f32(inv_freq, head_scale)
    q_out = torch.empty(T, H * D, dtype=proj.dtype, device=proj.device)
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == proj.dtype and v_cache.dtype == proj.dtype
    assert 0 <= rot_dims <= D and rot_dims % 2 == 0 and (rot_dims == 0 or inv_freq.numel() == rot_dims // 2)
    if proj.is_cuda:
        assert proj.stride(1) == 1
        lib = _mixlib.load()
        if interleaved or unit_eps is not None:
            _mixlib.check(lib.lv_qk_prep_store(_p(proj), proj.stride(0), off_q, off_k, off_v, _p(inv_freq), _p(head_scale),
                                               _p(q_out), _p(k_cache), _p(v_cache), _p(step.cu_q), _p(step.ctx_lens),
                                               _p(step.tok_seq), _p(step.block_tables), step.block_tables.stride(0), T, H, G, D,
                                               Dv, rot_dims, int(interleaved), int(unit_eps is not None),
                                               float(unit_eps or 0.0), page, _DT[proj.dtype], _stream(proj)), "lv_qk_prep_store")
            return q_out
        _mixlib.check(lib.lv_rotary_store(_p(proj), proj.stride(0), off_q, off_k, off_v, _p(inv_freq), _p(head_scale), _p(q_out),
                                          _p(k_cache), _p(v_cache), _p(step.cu_q), _p(step.ctx_lens), _p(step.tok_seq),
                                          _p(step.block_tables), step.block_tables.stride(0), T, H, G, D, Dv, rot_dims, page,
                                          _DT[proj.dtype], _stream(proj)), "lv_rotary_store")
        return q_out
    pos = _positions(step, proj.device)
    q, k = proj[:, off_q:off_q + H * D].float().view(T, H, D), proj[:, off_k:off_k + G * D].float().view(T, G, D)
    if unit_eps is not None:
        q = q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + unit_eps)
        k = k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + unit_eps)
    q = _rotate(q, pos, inv_freq, rot_dims, interleaved)
    if head_scale is not None:
        q = q * head_scale.view(1, H, 1)
    q_out.copy_(q.reshape(T, H * D))
    k = _rotate(k, pos, inv_freq, rot_dims, interleaved).reshape(T, G * D).to(k_cache.dtype)
    v = proj[:, off_v:off_v + G * Dv]
    kc, vc = k_cache.view(-1, G * D), v_cache.view(-1, G * Dv)
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        bt = step.host_block_tables[b]
        for r in range(n):
            sl = _token_slot(bt, ctx + r, page)
            kc[sl] = k[q0 + r]
            vc[sl] = v[q0 + r]
        q0 += n
    return q_out


def latent_prep(proj, off_q, off_kv, q_w, kv_w, inv_freq, cache, step, Rq, R, Dr, rot_dims, eps):
    """proj [T, ld]: query latent at column off_q (Rq wide), key/value latent at off_kv (R wide) followed
    by the positional key part (Dr wide). Returns the RMS-normed query latent [T, Rq]; writes
    [rms_norm(latent) * kv_w | rotated positional part] into each token's row of cache [pages, page, R + Dr]."""
    T = proj.size(0)
    page = cache.size(1)
    _f32(q_w, kv_w, inv_freq)
    cq = torch.empty(T, Rq, dtype=proj.dtype, device=proj.device)
    assert cache.is_contiguous() and cache.shape[2] == R + Dr and cache.dtype == proj.dtype
    if proj.is_cuda:
        assert proj.stride(1) == 1
        lib = _mixlib.load()
        _mixlib.check(lib.lv_latent_prep(_p(proj), proj.stride(0), off_q, off_kv, _p(q_w), _p(kv_w), _p(inv_freq), _p(cq),
                                         _p(cache), _p(step.cu_q), _p(step.ctx_lens), _p(step.tok_seq),
                                         _p(step.block_tables), step.block_tables.stride(0), T, Rq, R, Dr, rot_dims, page,
                                         eps, _DT[proj.dtype], _stream(proj)), "lv_latent_prep")
        return cq
    x = proj[:, off_q:off_q + Rq].float()
    cq.copy_(x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * q_w)
    c = proj[:, off_kv:off_kv + R].float()
    c = c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * kv_w
    pos = _positions(step, proj.device)
    kr = _rotate(proj[:, off_kv + R:off_kv + R + Dr].float(), pos, inv_freq, rot_dims)
    rows = torch.cat([c, kr], -1).to(cache.dtype)
    flat = cache.view(-1, R + Dr)
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        bt = step.host_block_tables[b]
        for r in range(n):
            flat[_token_slot(bt, ctx + r, page)] = rows[q0 + r]
        q0 += n
    return cq


def latent_q_finish(q, q_lat, inv_freq, step, H, Dn, Dr, R, rot_dims):
    """q [T, H*(Dn+Dr)] (per head: Dn unrotated entries, then Dr to rotate), q_lat [H, T, R] (the unrotated
    part multiplied into the latent space) -> [T, H*(R+Dr)] = per head [q_lat | rotated part]."""
    T = q.size(0)
    out = torch.empty(T, H * (R + Dr), dtype=q.dtype, device=q.device)
    assert q.is_contiguous() and q_lat.is_contiguous() and q_lat.shape == (H, T, R)
    if q.is_cuda:
        _f32(inv_freq)
        lib = _mixlib.load()
        _mixlib.check(lib.lv_latent_q_finish(_p(q), _p(q_lat), _p(inv_freq), _p(out), _p(step.cu_q), _p(step.ctx_lens),
                                             _p(step.tok_seq), T, H, Dn, Dr, R, rot_dims, _DT[q.dtype], _stream(q)),
                      "lv_latent_q_finish")
        return out
    o = out.view(T, H, R + Dr)
    o[:, :, :R] = q_lat.transpose(0, 1)
    if Dr:
        qr = q.view(T, H, Dn + Dr)[:, :, Dn:].float()
        o[:, :, R:] = _rotate(qr, _positions(step, q.device), inv_freq, rot_dims).to(q.dtype)
    return out


def latent_out_gate(o, gate, per_channel: bool):
    """o [H, T, Dv] -> [T, H*Dv] times sigmoid(gate); gate [T, H] (one per head) or [T, H*Dv]."""
    H, T, Dv = o.shape
    out = torch.empty(T, H * Dv, dtype=o.dtype, device=o.device)
    assert gate.shape == (T, H * Dv if per_channel else H) and gate.dtype == o.dtype
    if o.is_cuda:
        assert o.is_contiguous() and gate.stride(1) == 1
        lib = _mixlib.load()
        _mixlib.check(lib.lv_latent_out_gate(_p(o), _p(gate), gate.stride(0), int(per_channel), _p(out), T, H, Dv,
                                             _DT[o.dtype], _stream(o)), "lv_latent_out_gate")
        return out
    g = torch.sigmoid(gate.float())
    g = g.view(T, H, Dv) if per_channel else g.view(T, H, 1)
    out.copy_((o.float().transpose(0, 1) * g).reshape(T, H * Dv))
    return out


# ------------------------------------------------------------------------------ mixture of experts
def moe_route(logits, correction, top, groups=1, keep=1, normalize=True, score="sigmoid", group_rank="top2"):
    """logits f32 [T, E] -> (ids int32 [T, top], weights f32 [T, top], dense f32 [T, E]).
    Scores s = sigmoid(logits), or with score="softmax" the softmax over the row; the choice goes by s + correction; with
    `groups` > 1 only experts of the `keep` blocks of consecutive experts ranked highest by the sum of their two top selection
    scores (group_rank="max": by their top selection score) stay in the selection; weights are the
    chosen s over their sum (+ 1e-20), or the chosen s themselves without `normalize`; dense holds them at the
    chosen experts and 0 elsewhere. correction may be None."""
    T, E = logits.shape
    _f32(logits, correction)
    dev = logits.device
    ids = torch.empty(T, top, dtype=torch.int32, device=dev)
    w = torch.empty(T, top, dtype=torch.float32, device=dev)
    dense = torch.empty(T, E, dtype=torch.float32, device=dev)
    if logits.is_cuda:
        lib = _mixlib.load()
        _mixlib.check(lib.lv_moe_route_scored(_p(logits), _p(correction), _p(ids), _p(w), _p(dense), T, E, top, groups, keep,
                                              int(normalize), {"sigmoid": 0, "softmax": 1}[score],
                                              {"top2": 0, "max": 1}[group_rank], _stream(logits)), "lv_moe_route")
        return ids, w, dense
    s = torch.sigmoid(logits) if score == "sigmoid" else torch.softmax(logits, -1)
    c = s + correction if correction is not None else s.clone()
    if groups > 1 and keep < groups:
        cg = c.view(T, groups, E // groups)
        gs = cg.topk(min(2 if group_rank == "top2" else 1, E // groups), -1).values.sum(-1)
        best = gs.topk(keep, -1).indices
        kept = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
        c = cg.masked_fill(~kept[:, :, None], float("-inf")).reshape(T, E)
    idx = c.topk(top, -1).indices
    ws = s.gather(1, idx)
    if normalize:
        ws = ws / (ws.sum(-1, keepdim=True) + 1e-20)
    ids.copy_(idx)
    w.copy_(ws)
    dense.zero_().scatter_(1, idx, ws)
    return ids, w, dense


ROUTER_KERNEL_MAX_TOKENS = 256     # steps of at most this many tokens form their router logits in a kernel of their own


def router_logits(h, router_w):
    """f32 [T, E] = h router_w^T computed in f32 (h act [T, W], router_w f32 [E, W]). Steps of few tokens (decoded tokens,
    small portions, everything replayed from a graph) read the activations as they are, one workgroup per (token, four
    experts): one small launch instead of a widening copy and a GEMM. Larger steps take the f32 vendor GEMM."""
    T, W = h.shape
    E = router_w.size(0)
    _f32(router_w)
    if h.is_cuda and T <= ROUTER_KERNEL_MAX_TOKENS:
        assert h.stride(1) == 1
        logits = torch.empty(T, E, dtype=torch.float32, device=h.device)
        lib = _mixlib.load()
        _mixlib.check(lib.lv_router_logits(_p(h), h.stride(0), _p(router_w), _p(logits), T, W, E, _DT[h.dtype], _stream(h)),
                      "lv_router_logits")
        return logits
    return F.linear(h.float(), router_w)


def relu2_scale(up, dense, E, Fe):
    """up act [T, E*Fe] (all experts' up projections), dense f32 [T, E] -> relu(up)^2 * dense[t, e], act."""
    T = up.size(0)
    out = torch.empty_like(up)
    if up.is_cuda:
        assert up.is_contiguous() and dense.is_contiguous() and dense.dtype == torch.float32
        lib = _mixlib.load()
        _mixlib.check(lib.lv_relu2_scale(_p(up), _p(dense), _p(out), T, E, Fe, _DT[up.dtype], _stream(up)), "lv_relu2_scale")
        return out
    out.copy_((torch.relu(up.float()).pow(2).view(T, E, Fe) * dense[:, :, None]).reshape(T, E * Fe))
    return out


def moe_grouped_ok(h, Fe) -> bool:
    """Whether moe_grouped_ff serves these shapes (bf16, width and expert size in multiples of 32)."""
    return h.dtype == torch.bfloat16 and h.size(1) % 32 == 0 and Fe % 32 == 0


ACTS = {"relu2": 0, "gelu": 1, "gelu_tanh": 2}


def _act(x, act):
    """x f32 -> relu(x)^2, exact gelu, or the tanh form of gelu."""
    if act == "relu2":
        return torch.relu(x).pow(2)
    return F.gelu(x, approximate="tanh" if act == "gelu_tanh" else "none")


def glu_act(x, act="gelu_tanh"):
    """x act [T, 2F] = [gate | up] (row stride free) -> act [T, F] = act(gate) * up."""
    T, F2 = x.shape
    Fh = F2 // 2
    out = torch.empty(T, Fh, dtype=x.dtype, device=x.device)
    if x.is_cuda:
        assert x.stride(1) == 1
        lib = _mixlib.load()
        _mixlib.check(lib.lv_glu_act(_p(x), x.stride(0), _p(out), T, Fh, ACTS[act], _DT[x.dtype], _stream(x)), "lv_glu_act")
        return out
    out.copy_(_act(x[:, :Fh].float(), act) * x[:, Fh:].float())
    return out


def expert_act_scale(up, dense, E, Fe, act="relu2"):
    """up act [T, E*Fe] (all experts' up projections), dense f32 [T, >= E] (row stride free) -> act(up) * dense[t, e], act."""
    T = up.size(0)
    out = torch.empty_like(up)
    if up.is_cuda:
        assert up.is_contiguous() and dense.stride(1) == 1 and dense.dtype == torch.float32 and dense.size(1) >= E
        lib = _mixlib.load()
        _mixlib.check(lib.lv_expert_act_scale(_p(up), _p(dense), dense.stride(0), _p(out), T, E, Fe, ACTS[act], _DT[up.dtype],
                                              _stream(up)), "lv_expert_act_scale")
        return out
    out.copy_((_act(up.float(), act).view(T, E, Fe) * dense[:, :E, None]).reshape(T, E * Fe))
    return out


def scaled_row_add(y, h, factors):
    """y act [T, W] += (sum of factors[t, :]) * h[t], in place; factors f32 [T, n] (row stride free)."""
    T, W = y.shape
    if factors.size(1) == 0:
        return y
    if y.is_cuda:
        assert y.is_contiguous() and h.is_contiguous() and h.dtype == y.dtype and factors.stride(1) == 1
        lib = _mixlib.load()
        _mixlib.check(lib.lv_scaled_row_add(_p(y), _p(h), _p(factors), factors.stride(0), factors.size(1), T, W, _DT[y.dtype],
                                            _stream(y)), "lv_scaled_row_add")
        return y
    y.copy_(y.float() + factors.sum(-1, keepdim=True) * h.float())
    return y


def moe_grouped_ff(h, ids, weights, up_w, down_w, E, Fe, act="relu2", n_through=0):
    """y[t] = sum_k weights[t, k] * W_down,e act(W_up,e h[t]) with e = ids[t, k], computed expert by expert on rows
    sorted by expert: up_w [E*Fe, W], down_w [W, E*Fe]. The expert outputs are rounded to the activation dtype
    before the weighted sum, which is in f32. A choice e >= E (at most E + n_through - 1) stands for an expert without
    weights that hands h[t] through. Returns act [T, W]."""
    T, W = h.shape
    top = ids.size(1)
    out = torch.empty(T, W, dtype=h.dtype, device=h.device)
    if h.is_cuda:
        assert moe_grouped_ok(h, Fe) and h.is_contiguous() and up_w.is_contiguous() and down_w.is_contiguous()
        assert ids.dtype == torch.int32 and ids.is_contiguous() and weights.is_contiguous() and weights.dtype == torch.float32
        lib = _mixlib.load()
        ws = torch.empty(lib.lv_moe_grouped_workspace_bytes(T, W, Fe, E + n_through, top), dtype=torch.uint8, device=h.device)
        _mixlib.check(lib.lv_moe_grouped_act_ff(_p(h), _p(ids), _p(weights), _p(up_w), _p(down_w), _p(out), _p(ws), T, W, Fe, E,
                                                n_through, top, ACTS[act], _stream(h)), "lv_moe_grouped_act_ff")
        return out
    acc = torch.zeros(T, W)
    for e in range(E + n_through):
        t_idx, k_idx = (ids == e).nonzero(as_tuple=True)
        if t_idx.numel() == 0:
            continue
        if e >= E:
            y = h[t_idx].float()
        else:
            a = _act(F.linear(h[t_idx], up_w[e * Fe:(e + 1) * Fe]).float(), act).to(h.dtype)
            y = F.linear(a, down_w[:, e * Fe:(e + 1) * Fe]).float()
        acc.index_add_(0, t_idx, y * weights[t_idx, k_idx][:, None])
    out.copy_(acc)
    return out


def moe_grouped_glu_ff(h, ids, weights, up_w, down_w, E, Fe, limit, alpha):
    """y[t] = sum_k W_down,e glu(weights[t, k] * W_gu,e h[t]) with e = ids[t, k] and glu the clamped gated unit of
    expert_glu: the choice's weight scales what the expert reads, the outputs are summed as they are. Computed
    expert by expert on rows sorted by expert. up_w [E*2*Fe, W] (per expert gate rows, then up rows), down_w [W, E*Fe]
    (a column block of a wider weight is fine: its row stride is passed on). Returns act [T, W]."""
    T, W = h.shape
    top = ids.size(1)
    out = torch.empty(T, W, dtype=h.dtype, device=h.device)
    if h.is_cuda:
        assert moe_grouped_ok(h, Fe) and h.is_contiguous() and up_w.is_contiguous() and down_w.stride(1) == 1
        assert down_w.stride(0) % 8 == 0 and down_w.data_ptr() % 16 == 0 and up_w.data_ptr() % 16 == 0
        assert ids.dtype == torch.int32 and ids.is_contiguous() and weights.is_contiguous() and weights.dtype == torch.float32
        lib = _mixlib.load()
        ws = torch.empty(lib.lv_moe_grouped_workspace_bytes(T, W, Fe, E, top), dtype=torch.uint8, device=h.device)
        _mixlib.check(lib.lv_moe_grouped_glu_ff(_p(h), _p(ids), _p(weights), _p(up_w), _p(down_w), down_w.stride(0), _p(out),
                                                _p(ws), T, W, Fe, E, top, limit, alpha, _stream(h)), "lv_moe_grouped_glu_ff")
        return out
    acc = torch.zeros(T, W)
    for e in range(E):
        t_idx, k_idx = (ids == e).nonzero(as_tuple=True)
        if t_idx.numel() == 0:
            continue
        pre = F.linear(h[t_idx], up_w[e * 2 * Fe:(e + 1) * 2 * Fe])
        a = expert_glu(pre, 1, Fe, limit, alpha, in_scale=weights[t_idx, k_idx][:, None].contiguous())
        acc.index_add_(0, t_idx, F.linear(a, down_w[:, e * Fe:(e + 1) * Fe]).float())
    out.copy_(acc)
    return out


def moe_sort(ids, E, align=1):
    """ids int32 [T, top] -> (sorted_pair [M + E * align], inv [T, top], offsets [E + 1]), int32: the (token, choice)
    pairs in expert order, the row each pair got, and the first row of every expert. Every expert starts on a multiple
    of `align` rows: expert e owns rows offsets[e] .. offsets[e + 1], the last of which may be padding (pair 0)."""
    M = ids.numel()
    dev = ids.device
    if ids.is_cuda:
        sorted_pair = torch.zeros(M + E * align, dtype=torch.int32, device=dev)
        inv = torch.empty_like(ids)
        offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
        lib = _mixlib.load()
        _mixlib.check(lib.lv_moe_sort(_p(ids), M, E, align, _p(sorted_pair), _p(inv), _p(offsets), _stream(ids)), "lv_moe_sort")
        return sorted_pair, inv, offsets
    flat = ids.reshape(-1).long()
    order = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=E)
    padded = (counts + align - 1) // align * align
    offsets = torch.cat([torch.zeros(1, dtype=torch.long), padded.cumsum(0)])
    rank = torch.arange(M) - (counts.cumsum(0) - counts)[flat[order]]
    rows = offsets[flat[order]] + rank
    sorted_pair = torch.zeros(M + E * align, dtype=torch.int32)
    sorted_pair[rows] = order.to(torch.int32)
    inv = torch.empty(M, dtype=torch.int32)
    inv[order] = rows.to(torch.int32)
    return sorted_pair, inv.view_as(ids), offsets.to(torch.int32)


def moe_combine(rows, inv, weights=None, ids=None, n_real=0, h=None):
    """rows act [M, W] (expert outputs in sorted order) -> act [T, W] = sum_k weights[t, k] * rows[inv[t, k]], in f32
    (weights None: the plain sum). With ids [T, top], n_real and h [T, W]: a choice with ids[t, k] >= n_real takes h[t]
    in place of its row."""
    T, top = inv.shape
    W = rows.size(1)
    out = torch.empty(T, W, dtype=rows.dtype, device=rows.device)
    if rows.is_cuda:
        assert rows.dtype == torch.bfloat16 and rows.is_contiguous() and W % 4 == 0
        assert weights is None or (weights.dtype == torch.float32 and weights.is_contiguous())
        assert ids is None or (ids.dtype == torch.int32 and ids.is_contiguous() and h.is_contiguous() and h.dtype == rows.dtype)
        lib = _mixlib.load()
        _mixlib.check(lib.lv_moe_combine_through(_p(rows), _p(inv), _p(weights), _p(out), T, W, top, _p(ids), n_real, _p(h),
                                                 _stream(rows)), "lv_moe_combine")
        return out
    picked = rows[inv.long()].float()
    if ids is not None:
        picked = torch.where((ids >= n_real)[:, :, None], h.float()[:, None, :], picked)
    out.copy_((picked * weights[:, :, None] if weights is not None else picked).sum(1))
    return out


SORTED_ALIGN = 128


def moe_sorted_ff(h, ids, weights, up_w, down_w, E, Fe, act="relu2", n_through=0):
    """The same sum as moe_grouped_ff for large eager steps: rows sorted by expert on the device, the experts' row
    counts read back once, and each expert's two products run as vendor GEMMs on its slice of the sorted rows. One host
    synchronisation per call, so not for steps that are captured into a graph. Every expert's slice is padded to a
    multiple of SORTED_ALIGN rows (copies of token 0 that no one reads back): the GEMM library then sees a handful of
    shapes instead of a new one per expert and step, each of which would cost it a kernel selection on the host."""
    T, W = h.shape
    top = ids.size(1)
    sorted_pair, inv, offsets = moe_sort(ids, E + n_through, SORTED_ALIGN)
    off = offsets.tolist()
    xs = h.index_select(0, torch.div(sorted_pair[:off[E]], top, rounding_mode="floor"))
    mid = torch.empty(off[E], Fe, dtype=h.dtype, device=h.device)
    for e in range(E):
        if off[e + 1] > off[e]:
            torch.mm(xs[off[e]:off[e + 1]], up_w[e * Fe:(e + 1) * Fe].t(), out=mid[off[e]:off[e + 1]])
    if act == "relu2":
        mid.relu_().square_()
    else:
        mid = F.gelu(mid, approximate="tanh" if act == "gelu_tanh" else "none")
    rows = torch.empty(max(off[E], 1), W, dtype=h.dtype, device=h.device)    # rows of experts that hand through stay unread
    for e in range(E):
        if off[e + 1] > off[e]:
            torch.mm(mid[off[e]:off[e + 1]], down_w[:, e * Fe:(e + 1) * Fe].t(), out=rows[off[e]:off[e + 1]])
    if n_through:
        return moe_combine(rows, inv.clamp(max=rows.size(0) - 1), weights, ids, E, h)
    return moe_combine(rows, inv, weights)


def moe_sorted_glu_ff(h, ids, weights, up_w, down_w, E, Fe, limit, alpha):
    """The same sum as moe_grouped_glu_ff for large eager steps, the way moe_sorted_ff does it: rows sorted by expert on
    the device, the experts' row counts read back once, each expert's gate|up product and down product as vendor GEMMs on
    its slice of the sorted rows (slices padded to SORTED_ALIGN rows), the gated unit over all sorted rows in one launch
    with every row's routing weight as the factor on its pre-activations, and the plain sum of every token's rows."""
    T, W = h.shape
    top = ids.size(1)
    sorted_pair, inv, offsets = moe_sort(ids, E, SORTED_ALIGN)
    off = offsets.tolist()
    pairs = sorted_pair[:off[E]]
    xs = h.index_select(0, torch.div(pairs, top, rounding_mode="floor"))
    scale = weights.reshape(-1).index_select(0, pairs).unsqueeze(1).contiguous()
    pre = torch.empty(off[E], 2 * Fe, dtype=h.dtype, device=h.device)
    for e in range(E):
        if off[e + 1] > off[e]:
            torch.mm(xs[off[e]:off[e + 1]], up_w[e * 2 * Fe:(e + 1) * 2 * Fe].t(), out=pre[off[e]:off[e + 1]])
    act = expert_glu(pre, 1, Fe, limit, alpha, in_scale=scale)
    rows = torch.empty(off[E], W, dtype=h.dtype, device=h.device)
    for e in range(E):
        if off[e + 1] > off[e]:
            torch.mm(act[off[e]:off[e + 1]], down_w[:, e * Fe:(e + 1) * Fe].t(), out=rows[off[e]:off[e + 1]])
    return moe_combine(rows, inv, None)


# --------------------------------------------------------------------- tanh norm, two mixers side by side
def residual_dyt(x, y1=None, y2=None, post_w1=None, post_w2=None, pair_scale=1.0, eps=1e-6, alpha=None, w=None, b=None,
                 act_dtype=None):
    """x [T, W] f32 (the one residual), in place:
        post_w1 is None:  x += y1 + y2                                                   (either may be None)
        else:             x += pair_scale * (y1 / rms(y1) * post_w1 + y2 / rms(y2) * post_w2),  rms(y) = sqrt(mean(y^2) + eps)
    and returns the dynamic-tanh norm tanh(alpha * x) * w + b in act dtype (alpha f32 [1] or [], w and b f32 [W]), or None
    when w is None. All arithmetic f32."""
    T, W = x.shape
    _f32(x, post_w1, post_w2, alpha, w, b)
    ys = [y for y in (y1, y2) if y is not None]
    act_dtype = act_dtype or (ys[0].dtype if ys else torch.bfloat16)
    assert post_w1 is None or (y1 is not None and (post_w2 is not None) == (y2 is not None))
    assert post_w1 is not None or post_w2 is None
    out = torch.empty(T, W, dtype=act_dtype, device=x.device) if w is not None else None
    if x.is_cuda:
        for y in ys:
            assert y.is_contiguous() and y.dtype == act_dtype and y.shape == (T, W)
        lib = _mixlib.load()
        _mixlib.check(lib.lv_residual_dyt(_p(x), _p(y1), _p(post_w1), _p(y2), _p(post_w2), pair_scale, eps, _p(alpha), _p(w),
                                          _p(b), _p(out), T, W, _DT[act_dtype], _stream(x)), "lv_residual_dyt")
        return out
    if post_w1 is not None:
        def normed(y, pw):
            yf = y.float()
            return yf / torch.sqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * pw
        add = normed(y1, post_w1)
        if y2 is not None:
            add = add + normed(y2, post_w2)
        x.add_(pair_scale * add)
    else:
        for y in ys:
            x.add_(y.float())
    if w is None:
        return None
    out.copy_(torch.tanh(alpha * x) * w + b)
    return out


# ------------------------------------------------------------------------------- lightning attention
def lightning_attention(proj, off_q, off_k, off_v, decay, state, step, H, D, Dv):
    """Linear attention with a constant decay per head. proj act [T, ld]: H query heads of D at column off_q, H key heads of
    D at off_k, H value heads of Dv at off_v; q, k, v = silu of those columns. Per head and token
        S <- decay[h] * S + k v^T;   o = S^T q
    state f32 [slots, H, D, Dv] (taken as zero for a sequence with no context), updated in place; decay f32 [H].
    Returns o f32 [T, H, Dv]."""
    T = proj.size(0)
    _f32(decay, state)
    assert state.shape[1:] == (H, D, Dv) and decay.numel() == H
    o = torch.empty(T, H, Dv, dtype=torch.float32, device=proj.device)
    if proj.is_cuda:
        assert proj.stride(1) == 1
        lib = _mixlib.load()
        _mixlib.check(lib.lv_lightning_attn(_p(proj), proj.stride(0), off_q, off_k, off_v, _p(decay), _p(state), _p(step.cu_q),
                                            _p(step.ctx_lens), _p(step.slots), _p(o), len(step.host_lens_q), H, D, Dv,
                                            _DT[proj.dtype], _stream(proj)), "lv_lightning_attn")
        return o
    q = F.silu(proj[:, off_q:off_q + H * D].float()).view(T, H, D)
    k = F.silu(proj[:, off_k:off_k + H * D].float()).view(T, H, D)
    v = F.silu(proj[:, off_v:off_v + H * Dv].float()).view(T, H, Dv)
    q0 = 0
    for b, (n, ctx) in enumerate(zip(step.host_lens_q, step.host_ctx_lens)):
        slot = step.host_slots[b]
        S = state[slot].clone() if ctx > 0 else torch.zeros(H, D, Dv)
        for t in range(q0, q0 + n):
            S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S
        q0 += n
    return o
