"""Benchmark of the attention hot path on MI355X.

Metric (BASELINE.json): paged-decode attention HBM GB/s. One "step" is one decode pass of the hot
path over every layer of the model: per layer, lv_store_kvcache of the step's new token rows, then
lv_decode_attn over the paged cache (what Attention.forward does once per layer per decode step).

N = 1   BASELINE.json configs[1]: Qwen3-0.6B shapes (28 layers, 16 q / 8 kv heads, D=128), bf16,
        batch 256, every sequence at 1024 tokens of context, block size 256, a seeded random physical
        block permutation. `roofline` is its decode kernel (decode_attn_kernel<2,8>); `roofline_8b`
        is the same launch on Qwen3-8B TP=1 shapes (36 layers, 32 q / 8 kv heads: decode_mfma_kernel<4>),
        the configuration the 70 %-of-HBM-peak target is stated on.
N > 1   BASELINE.json configs[3]: Qwen3-8B under tensor parallelism TP = N. The path shards by KV
        head: rank r owns 8/N kv heads and 32/N q heads of every layer, a fixed GLOBAL batch of 32
        sequences at 32k tokens of context ([32, 128] block table), so the work per step is fixed
        and N divides it ("strong" scaling). What TP costs sits inside the timed step: per layer,
        after store + decode, one sum all-reduce of the [batch, 4096] bf16 activation (the o_proj
        all-reduce of RowParallelLinear, lightvllm/layers/linear.py:388-389) through the same
        layers.tp.all_reduce the model calls (direct IPC path when available, else RCCL). The 36
        layers of a step are captured in one hipGraph and the timed steps are replays.

`value` = algorithmic bytes of all attention launches of a step, summed over ranks, / max-over-ranks
step time. Inputs are resident in HBM before the timed region.

Auxiliary records on the same JSON line (never part of `value`): `cpu_baseline` (N=1: the CPU oracle
on the host cores), `prefill` (the prefill kernel on the 4 x 4096 configuration), `variants` (N=1: the
other launches the reference's call sites produce - ragged and outlier decode batches, a 32k-context
8q/1kv decode, varlen / prefix-cached / 8q/1kv prefill, the store at 16384 tokens), `config4_tp1`
(N=1: the N>1 step at TP=1, the base of the strong-scaling curve), `collectives` (N>1: all-reduce
latencies, direct path and RCCL) and `e2e` (the engine's tok/s at TP = N in child processes; a
failure there sets `e2e_failed`). `--no-aux` skips them, `--aux a,b` picks some.
At every N the line also carries `scale_value` / `scale_ms_per_step`: BASELINE config 4 at TP = N
(N = 1: the `config4_tp1` leg), one workload whose numbers are comparable across N, with
`scale_base_ms_per_step` (TP = 1, measured in the same run) and `scale_efficiency` against it.

    python bench.py [--gpus N] [--steps K] [--warmup W]
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import signal
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch  # noqa: E402

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E spec peak
MFMA_PEAK_TFLOPS = 2500.0   # dense bf16, MI355X
D, BLOCK = 128, 256
C2 = dict(name="Qwen3-0.6B", layers=28, hq=16, hkv=8, batch=256, ctx=1024)          # configs[1]
C2_8B = dict(name="Qwen3-8B", layers=36, hq=32, hkv=8, batch=256, ctx=1024)         # north-star shapes
C4 = dict(name="Qwen3-8B", layers=36, hq=32, hkv=8, batch=32, ctx=32768, hidden=4096)  # configs[3]
TUNED_GEMMS = os.path.join(ROOT, "tools", "tunable", "tunableop.csv")   # PyTorch appends the device ordinal


def decode_bytes(B, ctx, Hq, Hkv):
    """Algorithmic bytes of one decode launch: K and V rows of every context token once,
    q in + o out, context_lens, and the block-table entries touched."""
    nblk = (ctx + BLOCK - 1) // BLOCK
    return B * ctx * Hkv * D * 2 * 2 + 2 * B * Hq * D * 2 + 4 * B + 4 * B * nblk


def store_bytes(N, Hkv):
    return 2 * (N * Hkv * D * 2 * 2) + 4 * N


SETTLE_S = 1.0   # idle time between a leg's set-up and its first timed launch


class DecodeWorkload:
    """The per-layer tensors of one decode step on this rank: one KV tensor for all layers, as
    ModelRunner.allocate_kv_cache lays it out, so no layer's cache is served from the Infinity Cache
    of the layer before."""

    def __init__(self, ops, dev, layers, Hq, Hkv, B, ctx, seed):
        self.ops, self.dev, self.layers, self.Hq, self.Hkv, self.B, self.ctx = ops, dev, layers, Hq, Hkv, B, ctx
        bps = ctx // BLOCK
        nblk = B * bps
        gen = torch.Generator().manual_seed(seed)
        self.kv = torch.empty(2, layers, nblk, BLOCK, Hkv, D, dtype=torch.bfloat16, device=dev)
        for l in range(layers):
            self.kv[0, l].normal_()
            self.kv[1, l].normal_()
        self.q = torch.randn(B, Hq, D, device=dev).to(torch.bfloat16)
        self.k_new = torch.randn(B, Hkv, D, device=dev).to(torch.bfloat16)
        qkv = torch.randn(B, (Hq + 2 * Hkv) * D, device=dev).to(torch.bfloat16)
        self.v_new = qkv[:, (Hq + Hkv) * D:].view(B, Hkv, D)   # V is a view into the fused activation
        self.bt_cpu = torch.randperm(nblk, generator=gen).to(torch.int32).view(B, bps).contiguous()
        self.ctx_cpu = torch.full((B,), ctx, dtype=torch.int32)
        slots = (self.bt_cpu[:, -1].long() * BLOCK + (ctx - 1) % BLOCK).to(torch.int32)
        self.bt, self.ctx_t, self.slots = self.bt_cpu.to(dev), self.ctx_cpu.to(dev), slots.to(dev)
        self.scale = D ** -0.5
        self.out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=dev)
        self.nsplit = ops.decode_num_splits(B, Hkv, bps, BLOCK)
        ops.reserve_decode_workspace(dev, ops.decode_workspace_bytes(B, Hq, D, self.nsplit))
        self.decode_bytes = decode_bytes(B, ctx, Hq, Hkv)
        self.step_bytes = layers * (self.decode_bytes + store_bytes(B, Hkv))
        # For up to ~0.8 s after a large hipFree or fill (the previous leg's caches, this leg's random
        # numbers) the same launch on the same buffers runs 3-5 % slower, then returns to the time it
        # holds for thousands of back-to-back launches (tools/decode_state_probe.py). Every leg
        # starts from that settled state, not from the tail of its own set-up.
        torch.cuda.synchronize()
        time.sleep(SETTLE_S)

    def step(self, events=None, after_layer=None):
        ops, kv = self.ops, self.kv
        for l in range(self.layers):
            ops.store_kvcache(self.k_new, self.v_new, kv[0, l], kv[1, l], self.slots)
            if events is not None:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            ops.decode_attention(self.q, kv[0, l], kv[1, l], self.ctx_t, self.bt, self.scale, out=self.out)
            if events is not None:
                e1.record()
                events.append((e0, e1))
            if after_layer is not None:
                after_layer()

    def roofline(self, steps, kernel):
        """Events around every decode launch of `steps` eager passes, on the launch stream."""
        events = []
        self.step()
        torch.cuda.synchronize()
        for _ in range(steps):
            self.step(events)
        torch.cuda.synchronize()
        times = sorted(a.elapsed_time(b) for a, b in events)
        avg_s = sum(times) / len(times) / 1e3
        achieved = self.decode_bytes / avg_s / 1e9
        return {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "bytes_per_launch": self.decode_bytes, "avg_launch_us": round(avg_s * 1e6, 2),
                "median_launch_us": round(times[len(times) // 2] * 1e3, 2), "max_launch_us": round(times[-1] * 1e3, 2),
                "launches_timed": len(events),
                "shape": f"B={self.B} ctx={self.ctx} {self.Hq}q/{self.Hkv}kv x {self.layers} layers, splits {self.nsplit}"}

    def free(self):
        del self.kv, self.q, self.k_new, self.v_new, self.out
        torch.cuda.empty_cache()


def _sha16(path):
    return hashlib.sha256(open(path, "rb").read()).hexdigest()[:16]


def recorded_traffic(kernel="decode_attn_kernel<2", launch_bytes=None):
    """HBM bytes per launch of a decode kernel from the PMC passes of tools/pmc_decode.sh
    (profiles/decode_traffic.json). A recording, not a measurement of this run: returned only while
    the kernel source it was taken on is the one in the tree. launch_bytes: the algorithmic bytes of
    the launch in question; the recording of the same kernel whose algorithmic bytes match is used."""
    path = os.path.join(ROOT, "profiles", "decode_traffic.json")
    src = os.path.join(ROOT, "light_vllm_amd", "csrc", "decode_attn.hip")
    try:
        rec = json.load(open(path))
        sha = _sha16(src)
    except (OSError, ValueError):
        return None, {"kind": "none"}
    source = {"kind": "recorded PMC passes (FETCH_SIZE, WRITE_SIZE), not collected in this run",
              "file": "profiles/decode_traffic.json",
              "recorded_on_kernel_source": rec.get("kernel_source_sha16"), "current_kernel_source": sha}
    if rec.get("kernel_source_sha16") != sha:
        source["kind"] = "stale: recorded on another version of decode_attn.hip, dropped"
        return None, source
    for name, k in rec.get("kernels", {}).items():
        if kernel in name and (launch_bytes is None or k.get("algorithmic_bytes_per_launch") == launch_bytes):
            source["kernel"] = name
            return k.get("hbm_bytes_per_launch"), source
    source["kind"] = "no recording of this kernel on this launch"
    return None, source


def recorded_prefill_counters():
    """Matrix-pipe utilisation of the prefill kernel from rocprofv3 counters (tools/pmc_prefill.sh +
    tools/pmc_prefill_summary.py on the 4 x 4096, 32q/8kv launch): a recording, shown only while
    prefill_attn.hip is the source it was taken on."""
    path = os.path.join(ROOT, "profiles", "prefill_counters.json")
    src = os.path.join(ROOT, "light_vllm_amd", "csrc", "prefill_attn.hip")
    try:
        rec = json.load(open(path))
        sha = _sha16(src)
    except (OSError, ValueError):
        return None
    out = {"kind": "recorded rocprofv3 --pmc passes, not collected in this run", "file": "profiles/prefill_counters.json",
           "recorded_on_kernel_source": rec.get("kernel_source_sha16"), "current_kernel_source": sha}
    if rec.get("kernel_source_sha16") != sha:
        out["kind"] = "stale: recorded on another version of prefill_attn.hip, dropped"
        return out
    for key in ("kernel", "mfma_pipe_busy_fraction", "mfma_flops_over_algorithmic", "l2_hit_rate",
                "lds_instructions_per_wave_tile", "mfma_instructions_per_wave_tile", "kernel_shader_cycles"):
        if key in rec:
            out[key] = rec[key]
    return out


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(w, budget_s=10.0):
    """The CPU oracle (torch fp32 attention over block_table-gathered K/V, the reference's CPU
    plumbing path of BASELINE config 1) on one layer of the config-2 workload, on the threads this
    job owns; then a single-thread leg on 32 of the 256 sequences, and the config-3 prefill on
    1 x 4096 tokens (a quarter of its batch), each bounded in time."""
    from oracle.attention_oracle import decode_ref, prefill_ref
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    q, kc, vc = w.q.cpu(), w.kv[0, 0].cpu(), w.kv[1, 0].cpu()
    ctx, bt, scale = w.ctx_cpu, w.bt_cpu, w.scale

    def timed(fn, budget, max_reps):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            used = time.perf_counter() - t0
            if used >= budget or reps >= max_reps:
                return used / reps, reps

    per_call, reps = timed(lambda: decode_ref(q, kc, vc, ctx, bt, scale), budget_s, 50)
    rec = {"value": round(w.decode_bytes / per_call / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
           "sample": f"oracle decode_ref, 1 layer of the workload (B={w.B}, ctx={w.ctx}, Hq={w.Hq}, Hkv={w.Hkv}), "
                     f"{reps} calls, {per_call * 1e3:.1f} ms/call",
           "cpu_model": cpu_model(), "host_logical_cpus": os.cpu_count(),
           "threads_note": "threads = this job's CPU share (OMP_NUM_THREADS), not the host's core count"}
    torch.set_num_threads(1)
    nb = 32
    per1, reps1 = timed(lambda: decode_ref(q[:nb], kc, vc, ctx[:nb], bt[:nb], scale), 4.0, 10)
    rec["single_thread"] = {"value": round(decode_bytes(nb, w.ctx, w.Hq, w.Hkv) / per1 / 1e9, 3), "unit": "GB/s",
                            "cores": 1, "sample": f"first {nb} sequences of the same layer, {reps1} calls, {per1 * 1e3:.1f} ms/call"}
    torch.set_num_threads(threads)
    L, Hq, Hkv = 4096, 32, 8
    g = torch.Generator().manual_seed(3)
    pq = torch.randn(L, Hq, D, generator=g).to(torch.bfloat16)
    pk = torch.randn(L, Hkv, D, generator=g).to(torch.bfloat16)
    pv = torch.randn(L, Hkv, D, generator=g).to(torch.bfloat16)
    cu = torch.tensor([0, L], dtype=torch.int32)
    perp, repsp = timed(lambda: prefill_ref(pq, pk, pv, cu, cu, scale), 4.0, 10)
    flops = 4 * Hq * D * (L * L - L * (L - 1) // 2)
    rec["prefill"] = {"value": round(flops / perp / 1e12, 4), "unit": "TFLOP/s", "cores": threads,
                      "sample": f"oracle prefill_ref, 1 x {L} tokens of the 4 x 4096 configuration ({Hq}q/{Hkv}kv), "
                                f"{repsp} calls, {perp * 1e3:.0f} ms/call"}
    return rec


def prefill_leg(ops, dev, n, iters=50, warmup=20):
    """Varlen causal prefill attention of the Qwen3-8B prefill configuration (4 x 4096-token
    prompts, packed) on this rank's TP head share: TFLOP/s of the algorithmic causal FLOP count
    and the fraction of the dense bf16 matrix peak, timed with events on the launch stream.
    The untimed launches bring the clocks to what a busy engine sees: from an idle GPU the first
    ~10 ms of this matrix-bound kernel run ~19 % slower (measured: 10 launches 0.66 ms each, 100
    launches 0.555 ms each, same operands)."""
    Hq, Hkv, L, Bp = max(32 // n, 1), max(8 // n, 1), 4096, 4
    g = torch.Generator(device=dev).manual_seed(1)
    q = torch.randn(Bp * L, Hq, D, generator=g, device=dev).to(torch.bfloat16)
    k = torch.randn(Bp * L, Hkv, D, generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn(Bp * L, Hkv, D, generator=g, device=dev).to(torch.bfloat16)
    cu = torch.arange(0, (Bp + 1) * L, L, dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    for _ in range(warmup):
        ops.prefill_attention(q, k, v, cu, cu, L, L, D ** -0.5, out=out)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        ops.prefill_attention(q, k, v, cu, cu, L, L, D ** -0.5, out=out)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / iters
    flops = Bp * 4 * Hq * D * (L * L - L * (L - 1) // 2)
    tf = flops / (ms * 1e-3) / 1e12
    return {"workload": f"4 x 4096-token prompts, causal, packed, {Hq}q/{Hkv}kv heads, D=128",
            "launches": iters, "untimed_launches": warmup, "ms": round(ms, 4),
            "tflops": round(tf, 1), "peak": MFMA_PEAK_TFLOPS, "frac": round(tf / MFMA_PEAK_TFLOPS, 4),
            "bound": "mfma", "flops_per_launch": flops}


def _event_time(fn, iters, warmup=2):
    """Mean seconds per call of fn, events on the launch stream."""
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def ragged_decode_leg(ops, dev, Hq, Hkv, lens, how, layers=6, reps=3):
    """One paged-decode launch per layer cache on a batch of unequal lengths (python ints), blocks
    handed out as the block manager would (ceil(len / 256) per sequence, random physical order).
    how: "ordered" = lv_decode_attn with the longest-first launch order ModelRunner.prepare_decode
    passes, "planned" = lv_decode_attn_planned on the work list decode_plan.build_plan cuts."""
    from light_vllm_amd.decode_plan import build_plan
    B = len(lens)
    need = [-(-n // BLOCK) for n in lens]
    nblk, width = sum(need), max(need)
    perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(7)).to(torch.int32)
    bt = torch.zeros(B, width, dtype=torch.int32)
    pos = 0
    for i, n in enumerate(need):
        bt[i, :n] = perm[pos:pos + n]
        pos += n
    kv = torch.empty(layers, 2, nblk, BLOCK, Hkv, D, dtype=torch.bfloat16, device=dev).normal_()
    q = torch.randn(B, Hq, D, device=dev).to(torch.bfloat16)
    out = torch.empty_like(q)
    ctx_t, bt_d = torch.tensor(lens, dtype=torch.int32, device=dev), bt.to(dev)
    order = plan = None
    if how == "ordered":
        order = torch.tensor(sorted(range(B), key=lambda j: -lens[j]), dtype=torch.int32, device=dev)
    else:
        plan = build_plan(lens, Hkv, Hq // Hkv).to(dev)
    state = {"i": 0}

    def fn():
        l = state["i"] % layers
        state["i"] += 1
        ops.decode_attention(q, kv[l, 0], kv[l, 1], ctx_t, bt_d, D ** -0.5, num_splits=1 if how == "ordered" else 0,
                             out=out, seq_order=order, plan=plan)
    torch.cuda.synchronize()
    time.sleep(SETTLE_S)
    t = _event_time(fn, layers * reps, warmup=layers)
    nbytes = sum(lens) * Hkv * D * 4 + 2 * B * Hq * D * 2 + 4 * B + 4 * nblk
    rec = {"how": how, "heads": f"{Hq}q/{Hkv}kv", "batch": B, "tokens": sum(lens), "longest": max(lens),
           "bytes_per_launch": nbytes, "avg_launch_us": round(t * 1e6, 2), "achieved": round(nbytes / t / 1e9, 1),
           "unit": "GB/s", "peak": HBM_PEAK_GBS, "frac": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4), "bound": "hbm"}
    if plan is not None:
        rec["pieces"], rec["piece_tokens"], rec["most_pieces_per_sequence"] = plan.used, plan.piece_tokens, plan.max_splits
    del kv
    torch.cuda.empty_cache()
    return rec


def prefill_variant_leg(ops, dev, lens, Hq, Hkv, cached=0, iters=30, warmup=20):
    """Prefill attention on prompts of `lens` tokens whose first `cached` tokens each are already in
    the paged cache (0: packed K/V, no block table), with the query-tile launch order the runner
    builds from the lengths (ops.prefill_tile_order; None for 8 kv heads)."""
    lens_q = [n - cached for n in lens]
    tq = sum(lens_q)
    q = torch.randn(tq, Hq, D, device=dev).to(torch.bfloat16)
    out = torch.empty_like(q)
    cu_q = torch.tensor([0] + torch.tensor(lens_q).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    cu_k = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    order = ops.prefill_tile_order(lens_q, lens, Hq, Hkv, dev, paged=cached > 0)
    if cached:
        need = [-(-n // BLOCK) for n in lens]
        nblk = sum(need)
        kc = torch.randn(nblk, BLOCK, Hkv, D, device=dev).to(torch.bfloat16)
        vc = torch.randn(nblk, BLOCK, Hkv, D, device=dev).to(torch.bfloat16)
        perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(11)).to(torch.int32)
        bt = torch.full((len(lens), max(need)), -1, dtype=torch.int32)
        pos = 0
        for i, n in enumerate(need):
            bt[i, :n] = perm[pos:pos + n]
            pos += n
        bt = bt.to(dev)
        fn = lambda: ops.prefill_attention(q, kc, vc, cu_q, cu_k, max(lens_q), max(lens), D ** -0.5,   # noqa: E731
                                           block_table=bt, out=out, tile_order=order)
    else:
        k = torch.randn(tq, Hkv, D, device=dev).to(torch.bfloat16)
        v = torch.randn(tq, Hkv, D, device=dev).to(torch.bfloat16)
        fn = lambda: ops.prefill_attention(q, k, v, cu_q, cu_k, max(lens_q), max(lens), D ** -0.5,     # noqa: E731
                                           out=out, tile_order=order)
    t = _event_time(fn, iters, warmup)
    flops = sum(4 * Hq * D * (lq * lk - lq * (lq - 1) // 2) for lq, lk in zip(lens_q, lens))
    return {"prompts": lens, "cached_tokens_each": cached, "heads": f"{Hq}q/{Hkv}kv", "ms": round(t * 1e3, 4),
            "tflops": round(flops / t / 1e12, 1), "peak": MFMA_PEAK_TFLOPS, "frac": round(flops / t / 1e12 / MFMA_PEAK_TFLOPS, 4),
            "bound": "mfma", "flops_per_launch": flops, "tile_order": order is not None}


def store_leg(ops, dev, N=16384, Hq=32, Hkv=8, caches=4):
    """lv_store_kvcache at a prefill's size: N rows into random distinct slots, V a strided view into
    the fused qkv activation as the model hands it over."""
    qkv = torch.randn(N, (Hq + 2 * Hkv) * D, device=dev).to(torch.bfloat16)
    k = qkv[:, Hq * D:(Hq + Hkv) * D].contiguous().view(N, Hkv, D)
    v = qkv[:, (Hq + Hkv) * D:].view(N, Hkv, D)
    nblk = 2 * N // BLOCK
    kv = torch.zeros(caches, 2, nblk, BLOCK, Hkv, D, dtype=torch.bfloat16, device=dev)
    slots = torch.randperm(nblk * BLOCK, device=dev)[:N].to(torch.int32)
    state = {"i": 0}

    def fn():
        c = state["i"] % caches
        state["i"] += 1
        ops.store_kvcache(k, v, kv[c, 0], kv[c, 1], slots)
    t = _event_time(fn, 40, warmup=8)
    nbytes = store_bytes(N, Hkv)
    return {"tokens": N, "heads_kv": Hkv, "avg_launch_us": round(t * 1e6, 2), "bytes_per_launch": nbytes,
            "achieved": round(nbytes / t / 1e9, 1), "unit": "GB/s", "peak": HBM_PEAK_GBS,
            "frac": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4), "bound": "hbm"}


def variants_leg(ops, dev, sync_all):
    """The other launches the reference's two attention call sites and its store produce
    (lightvllm/layers/attention.py:104-108, 159-165, 172-175; engine/model_runner.py:369-370 for the
    prefix-cached mode), each with its own roofline fraction. Every entry stands alone: a failure
    is recorded in place."""
    out = {}

    def leg(name, fn):
        try:
            out[name] = fn()
        except Exception as exc:   # noqa: BLE001 - reported, never fatal for the headline number
            out[name] = {"error": repr(exc)[:300]}
        torch.cuda.empty_cache()

    ragged = torch.randint(1, 1025, (256,), generator=torch.Generator().manual_seed(0)).tolist()
    leg("decode_ragged_16q8kv", lambda: ragged_decode_leg(ops, dev, 16, 8, ragged, "ordered"))
    leg("decode_ragged_32q8kv", lambda: ragged_decode_leg(ops, dev, 32, 8, ragged, "ordered"))
    outl = [16384] * 4 + ragged[4:]
    leg("decode_outliers_32q8kv_one_split_count", lambda: ragged_decode_leg(ops, dev, 32, 8, outl, "ordered"))
    leg("decode_outliers_32q8kv_work_list", lambda: ragged_decode_leg(ops, dev, 32, 8, outl, "planned"))

    def c5_decode():
        w = DecodeWorkload(ops, dev, 4, 8, 1, 64, 32768, seed=77)
        w.step()
        r = w.roofline(5, "decode_mfma_kernel<8>")
        w.free()
        return r
    leg("decode_c5_8q1kv_b64_ctx32k", c5_decode)
    leg("prefill_varlen", lambda: prefill_variant_leg(ops, dev, [4096, 3000, 1024, 8264], 32, 8))
    leg("prefill_prefix_1024_cached", lambda: prefill_variant_leg(ops, dev, [4096] * 4, 32, 8, cached=1024))
    leg("prefill_c5_8q1kv", lambda: prefill_variant_leg(ops, dev, [4096] * 4, 8, 1))
    leg("prefill_c5_8q1kv_prefix_1024_cached", lambda: prefill_variant_leg(ops, dev, [4096] * 4, 8, 1, cached=1024))
    leg("store_16384_tokens", lambda: store_leg(ops, dev))
    return out


def sustained_mfma_peak():
    """tools/mfma_peak (built by __graft_entry__.build): every SIMD issues bf16 MFMAs back to back
    from registers for ~50 ms, operands random like attention's. What it reaches is the matrix rate
    the chip sustains at the clock its power management allows under that load, the practical
    ceiling under the 2.5 PFLOP/s the spec quotes at 2.4 GHz. None when the tool is not built."""
    exe = os.path.join(ROOT, "tools", "mfma_peak")
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe, "2", "1"], capture_output=True, text=True, timeout=60).stdout
        for line in out.splitlines():
            if line.startswith("RESULT "):
                return json.loads(line[len("RESULT "):])
    except (OSError, ValueError, subprocess.TimeoutExpired):
        pass
    return None


def time_all_reduce(fn, x, iters=50):
    for _ in range(5):
        fn(x)
        x.fill_(1.0)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn(x)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def collectives_leg(dist, dev, n, direct):
    """Average time of the in-place bf16 sum all-reduce of the TP model at its decode-sized
    messages ([32, 4096] and [256, 4096]) on the direct IPC path and on RCCL, and at the
    prefill-sized message ([16384, 4096], RCCL only); busbw = 2(n-1)/n * bytes / t. Then a sweep of
    the direct path from 64 KiB to 8 MiB under both of its algorithms, from which the one-shot /
    two-shot threshold (lv_comm_set_one_shot_inflow) is read off after a run across GPUs.
    A failure of the direct path on this rank is recorded per message and never skips a later
    RCCL call: every rank issues the same torch.distributed collectives in the same order."""
    out = {}

    def direct_time(x, algorithm):
        us = time_all_reduce(lambda t: direct.all_reduce(t, algorithm), x)
        if direct.failed():
            raise RuntimeError("a peer did not arrive within the communicator's timeout")
        return us

    for name, rows in (("decode_256KiB", 32), ("decode_2MiB", 256), ("prefill_128MiB", 16384)):
        x = torch.ones(rows, 4096, dtype=torch.bfloat16, device=dev)
        rec = {}
        if dist.get_backend() == "nccl":
            us = time_all_reduce(dist.all_reduce, x, iters=50 if rows <= 256 else 10)
            rec["rccl_us"] = round(us, 1)
            rec["rccl_busbw_GBs"] = round(2 * (n - 1) / n * x.numel() * 2 / (us * 1e-6) / 1e9, 1)
        if direct is not None and direct.usable(x):
            try:
                us = direct_time(x, "auto")
                rec["direct_us"] = round(us, 1)
                rec["direct_algorithm"] = direct.algorithm_for(x.numel() * 2)
                rec["direct_busbw_GBs"] = round(2 * (n - 1) / n * x.numel() * 2 / (us * 1e-6) / 1e9, 1)
            except Exception as exc:   # noqa: BLE001 - recorded; the RCCL sequence below stays in step
                rec["direct_error"] = repr(exc)[:200]
                torch.cuda.synchronize()
        out[name] = rec
        del x
    if direct is not None:
        sweep = {"one_shot_inflow_bytes": direct.one_shot_inflow, "sizes": {}}
        for kib in (64, 128, 256, 512, 1024, 2048, 4096, 8192):
            x = torch.ones(kib * 512, dtype=torch.bfloat16, device=dev)
            rec = {"auto": direct.algorithm_for(kib * 1024)}
            try:
                for algorithm in ("one_shot", "two_shot"):
                    rec[algorithm + "_us"] = round(direct_time(x, algorithm), 1)
            except Exception as exc:   # noqa: BLE001
                rec["error"] = repr(exc)[:200]
                torch.cuda.synchronize()
                sweep["sizes"][f"{kib}KiB"] = rec
                break
            sweep["sizes"][f"{kib}KiB"] = rec
            del x
        out["direct_sweep"] = sweep
    return out


def e2e_leg(n, port, mode, limit_s, tuned_gemms=False):
    """tools/e2e_bench.py in a child process group of its own (killed as a group at the limit).
    tuned_gemms: PyTorch's TunableOp picks the model's GEMM kernels from the committed selection
    file (read only, no tuning in the run; a file recorded for other library versions is ignored)."""
    cmd = [sys.executable, os.path.join(ROOT, "tools", "e2e_bench.py"), "--model", "8b", "--tp", str(n),
           "--batch", "256", "--prompt-len", "1024", "--new-tokens", "33", "--modes", mode,
           "--dist-port", str(port)]
    env = {k: v for k, v in os.environ.items()
           if k not in ("RANK", "LOCAL_RANK", "WORLD_SIZE", "LOCAL_WORLD_SIZE", "GROUP_RANK", "ROLE_RANK",
                        "MASTER_PORT", "TORCHELASTIC_RUN_ID")}
    if tuned_gemms:
        env.update(PYTORCH_TUNABLEOP_ENABLED="1", PYTORCH_TUNABLEOP_TUNING="0",
                   PYTORCH_TUNABLEOP_FILENAME=TUNED_GEMMS)
    t0 = time.perf_counter()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env,
                            start_new_session=True)
    try:
        out, err = proc.communicate(timeout=limit_s)
    except subprocess.TimeoutExpired:
        try:
            os.killpg(proc.pid, signal.SIGKILL)
        except ProcessLookupError:
            pass
        proc.communicate()
        return {"mode": mode, "error": f"no result within {limit_s} s"}
    for line in out.splitlines():
        if line.startswith("{"):
            try:
                rec = json.loads(line)
                rec["wall_s"] = round(time.perf_counter() - t0, 1)
                rec["gemm_selection"] = "tunableop file" if tuned_gemms else "library default"
                return rec
            except ValueError:
                pass
    return {"mode": mode, "error": f"exit code {proc.returncode}: {err.strip()[-300:]}"}


# ------------------------------------------------------------------------------------------------
# --mixers: the Kagalorn design (delta-rule and windowed pooled attention layers on hyper-connected
# streams) beside Qwen3 at equal width, depth and head counts, both with random weights, through the
# engine (LLM.generate: prefill and decode tok/s), and the design's kernels one by one at the same
# layer shapes beside the Qwen3 kernel that does the like job, each against its own roofline
# (HBM bytes at 8 TB/s for the memory-bound ones, dense bf16 MFMA rate for prompt attention).
MIXER_SIZES = {
    "2k": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, ff=6144, window=1024, pool=64, vocab=32000),
    "4k": dict(width=4096, layers=4, heads=32, kv_heads=8, dim=128, ff=12288, window=2048, pool=128, vocab=32000),
}
HBM_BPS, MFMA_FLOPS = 8.0e12, 2.5e15


def _kagalorn_config(z):
    from light_vllm_amd.models.kagalorn import KagalornConfig
    att = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"], "scale": z["dim"] ** -0.5,
           "mask": {"size": z["window"], "pool": z["pool"]}}
    dlt = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"], "conv": 4}
    mlp = {"kind": "dense", "ff": z["ff"], "limit": 7.0}
    layers = [{"type": "delta" if i % 2 == 0 else "attention", "mixer": dlt if i % 2 == 0 else att, "mlp": mlp}
              for i in range(z["layers"])]
    return KagalornConfig.from_dict({"vocab": z["vocab"], "width": z["width"], "streams": 4,
                                     "norm": {"eps": 1e-6, "groups": 4}, "layers": layers})


def _qwen3_config(z):
    from types import SimpleNamespace
    return SimpleNamespace(vocab_size=z["vocab"], head_dim=z["dim"], hidden_act="silu", max_position_embeddings=40960,
                           rms_norm_eps=1e-6, rope_theta=1000000, rope_scaling=None, attention_bias=False,
                           torch_dtype=torch.bfloat16, hidden_size=z["width"], intermediate_size=z["ff"],
                           num_hidden_layers=z["layers"], num_attention_heads=z["heads"],
                           num_key_value_heads=z["kv_heads"], tie_word_embeddings=False)


def _engine_rates(hf_config, batch, prompt_len, new_tokens, **kw):
    from light_vllm_amd.llm import LLM
    from light_vllm_amd.sampling_params import SamplingParams
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, hf_config.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    llm = LLM(None, hf_config=hf_config, max_num_seqs=batch, max_model_len=4096, max_num_batched_tokens=16384,
              random_seed=0, random_on_device=True, **kw)
    warm = [torch.randint(0, hf_config.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    llm.generate(warm, SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True))   # other prompts, the timed shapes
    llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=new_tokens, ignore_eos=True))
    st = dict(llm.last_stats)
    llm.exit()
    del llm
    torch.cuda.empty_cache()
    return {"prefill_tok_s": round(st["avg_prefill_tok_s"], 1), "decode_tok_s": round(st["avg_decode_tok_s"], 1)}


def _mixer_kernel_table(z, dev, batch, prompt_len):
    """Each kernel of the design alone, at one layer's shapes: a prompt step (batch x prompt_len new tokens)
    and a decode step (batch single tokens behind prompt_len tokens), with the Qwen3 kernel of the like job."""
    from light_vllm_amd import mix_ops, ops
    from light_vllm_amd.utils.context import RaggedStep
    bf = torch.bfloat16
    W, H, G, D, F_, S = z["width"], z["heads"], z["kv_heads"], z["dim"], z["ff"], 4
    window, P, page = z["window"], z["pool"], 256
    rows = []

    def step_of(lens_q, ctx):
        B = len(lens_q)
        cu = [0]
        tok = []
        for b, n_ in enumerate(lens_q):
            cu.append(cu[-1] + n_)
            tok += [b] * n_
        per = -(-(max(ctx) + max(lens_q)) // page)
        tables = [[b * per + j for j in range(per)] for b in range(B)]
        i32 = dict(dtype=torch.int32, device=dev)
        return RaggedStep(torch.tensor(cu, **i32), torch.tensor(ctx, **i32), torch.arange(B, **i32),
                          torch.tensor(tok, **i32), torch.tensor(tables, **i32), lens_q, ctx, list(range(B)), tables), B * per

    def add(name, phase, fn, nbytes=0, flops=0, like=None):
        us = _event_time(fn, 20, 3) * 1e6
        rec = {"kernel": name, "phase": phase, "us": round(us, 1)}
        if nbytes:
            rec["GBs"] = round(nbytes / us / 1e3, 1)
            rec["of_hbm_roofline"] = round(nbytes / us / 1e3 / (HBM_BPS / 1e9), 3)
        if flops:
            rec["TFLOPs"] = round(flops / us / 1e6, 2)
            rec["of_mfma_roofline"] = round(flops / us / 1e6 / (MFMA_FLOPS / 1e12), 4)
        if like:
            rec["like"] = like
        rows.append(rec)

    for phase, lens_q, ctx in (("prompt", [prompt_len] * batch, [0] * batch), ("decode", [1] * batch, [prompt_len] * batch)):
        step, pages = step_of(lens_q, ctx)
        T = sum(lens_q)
        x = torch.randn(T, S, W, device=dev)
        y = torch.randn(T, W, device=dev, dtype=bf)
        mixm, vec, nw = torch.eye(S, device=dev), torch.ones(S, device=dev), torch.ones(W, device=dev)
        add("hc_update_norm", phase, lambda: mix_ops.hc_update_norm(x, y, mixm, vec, vec, nw, 4, 1e-6, bf),
            nbytes=T * W * (8 * S + 4))
        res = torch.randn(T, W, device=dev, dtype=bf)
        nwb = torch.ones(W, device=dev, dtype=bf)
        add("qwen3 add_rms_norm", phase, lambda: ops.add_rms_norm(y, res, nwb, 1e-6), nbytes=T * W * 8, like="hc_update_norm")
        gu = torch.randn(T, 2 * F_, device=dev, dtype=bf)
        add("clamped_glu", phase, lambda: mix_ops.clamped_glu(gu, 7.0, 1.702), nbytes=T * F_ * 6)
        add("qwen3 silu_and_mul", phase, lambda: ops.silu_and_mul(gu), nbytes=T * F_ * 6, like="clamped_glu")
        # delta rule
        C = 2 * G * D + H * D
        ld = C + H * D + 2 * H
        proj = torch.randn(T, ld, device=dev, dtype=bf)
        conv_w = torch.randn(C, 4, device=dev) * 0.5
        conv_state = torch.zeros(batch, 3, C, device=dev, dtype=bf)
        A_log, dt_bias = torch.zeros(H, device=dev), torch.zeros(H, device=dev)
        state = torch.zeros(batch, H, D, D, device=dev)
        a_in = proj[:, C + H * D + H:C + H * D + 2 * H]
        add("delta_prep", phase, lambda: mix_ops.delta_prep(proj, conv_w, conv_state, A_log, dt_bias, step, G, H, D, D, 4,
                                                            C + H * D, a_in, 1e-6),
            nbytes=T * (C * 2 + C * 4 + 8 * H))
        qn, kn, v, beta, dec = mix_ops.delta_prep(proj, conv_w, conv_state, A_log, dt_bias, step, G, H, D, D, 4,
                                                  C + H * D, a_in, 1e-6)
        st_bytes = batch * H * D * D * 4 * 2
        add("gated_delta_rule", phase, lambda: mix_ops.gated_delta_rule(qn, kn, v, beta, dec, state, step),
            nbytes=st_bytes + T * (2 * G * D + 2 * H * D) * 4, flops=T * H * D * D * 2 * 3)
        o32 = torch.randn(T, H, D, device=dev)
        add("head_norm_gate", phase, lambda: mix_ops.head_norm_gate(o32, proj[:, C:C + H * D], nw[:D].contiguous(), 1e-6, bf),
            nbytes=T * H * D * 8)
        # windowed pooled attention
        qkv = torch.randn(T, (H + 2 * G) * D + H * D, device=dev, dtype=bf)
        kc = torch.zeros(pages, page, G, D, device=dev, dtype=bf)
        vc = torch.zeros(pages, page, G, D, device=dev, dtype=bf)
        pp = mix_ops.pooled_slots(page, P)
        kp, vp = torch.zeros(pages, pp, G, D, device=dev, dtype=bf), torch.zeros(pages, pp, G, D, device=dev, dtype=bf)
        qw, kw_ = torch.ones(H * D, device=dev), torch.ones(G * D, device=dev)
        a_, b_, c_ = H * D, (H + G) * D, (H + 2 * G) * D
        add("qk_fullnorm_store", phase, lambda: mix_ops.qk_fullnorm_store(qkv[:, :a_], qkv[:, a_:b_], qkv[:, b_:c_], qw, kw_, kc, vc,
                                                                         step, H, G, D, D, 1e-6),
            nbytes=T * (H + 2 * G) * D * 4)
        qn_ = mix_ops.qk_fullnorm_store(qkv[:, :a_], qkv[:, a_:b_], qkv[:, b_:c_], qw, kw_, kc, vc, step, H, G, D, D, 1e-6)
        add("pool_update", phase, lambda: mix_ops.pool_update(kc, vc, kp, vp, step, G, D, D, P))
        keys = sum(min(i + 1, window) + max(0, (i - window + 1) // P) for n_, c0 in zip(lens_q, ctx) for i in range(c0, c0 + n_))
        if phase == "prompt":
            add("window_pool_attn", phase, lambda: mix_ops.window_pool_attention(qn_, kc, vc, kp, vp, qkv[:, c_:], step, H, G, D, D,
                                                                               window, P, D ** -0.5, True),
                flops=keys * H * D * 4)
        else:
            add("window_pool_attn", phase, lambda: mix_ops.window_pool_attention(qn_, kc, vc, kp, vp, qkv[:, c_:], step, H, G, D, D,
                                                                               window, P, D ** -0.5, True),
                nbytes=keys * G * D * 4)
        # the Qwen3 attention at the same shapes: full causal prompt attention / full-context decode
        q3 = torch.randn(T, H, D, device=dev, dtype=bf)
        k3 = torch.randn(T, G, D, device=dev, dtype=bf)
        if phase == "prompt":
            cu3 = torch.tensor([i * prompt_len for i in range(batch + 1)], dtype=torch.int32, device=dev)
            add("qwen3 prefill_attn", phase, lambda: ops.prefill_attention(q3, k3, k3, cu3, cu3, prompt_len, prompt_len, D ** -0.5),
                flops=batch * prompt_len * (prompt_len + 1) // 2 * H * D * 4, like="window_pool_attn")
        else:
            cl = torch.full((batch,), prompt_len + 1, dtype=torch.int32, device=dev)
            bt3 = step.block_tables
            add("qwen3 decode_attn", phase, lambda: ops.decode_attention(q3, kc, vc, cl, bt3, D ** -0.5),
                nbytes=batch * (prompt_len + 1) * G * D * 4, like="window_pool_attn")
    return rows


# --mixers-design bokulorn: the Bokulorn design (latent attention, channel-wise delta rule, mixture-of-experts
# feed-forwards on one f32 residual) beside Kagalorn, the closest existing model (ragged steps, a delta rule and an
# attention over a paged cache), at equal width, depth, head counts and active feed-forward size.
BOKULORN_SIZES = {
    "2k": dict(q_rank=768, kv_rank=192, rot_dim=64, experts=32, top=4, groups=4, keep=2, thin=64),
    "4k": dict(q_rank=1536, kv_rank=192, rot_dim=64, experts=32, top=4, groups=4, keep=2, thin=128),
}


def _bokulorn_config(z, bz):
    from light_vllm_amd.models.bokulorn import BokulornConfig
    H, D = z["heads"], z["dim"]
    lat = {"heads": H, "dim": D, "vdim": D, "q_rank": bz["q_rank"], "kv_rank": bz["kv_rank"], "rot_dim": bz["rot_dim"],
           "rot": {"base": 10000.0, "dims": bz["rot_dim"]}, "scale": (D + bz["rot_dim"]) ** -0.5}
    lat2 = {"heads": H, "dim": D, "vdim": D, "q_rank": bz["q_rank"], "kv_rank": bz["kv_rank"] + bz["rot_dim"], "scale": D ** -0.5}
    dlt = {"heads": H, "kv_heads": z["kv_heads"], "dim": D, "vdim": D, "conv": 4, "decay_rank": bz["thin"], "gate_rank": bz["thin"]}
    mlp = {"kind": "moe", "expert": {"ff": z["ff"] // bz["top"]},
           "router": {"experts": bz["experts"], "top": bz["top"], "groups": {"count": bz["groups"], "keep": bz["keep"]}}}
    kinds = [("channel_delta", dlt), ("latent_attention", lat), ("channel_delta", dlt), ("latent_attention_2", lat2)]
    layers = [{"type": kinds[i % 4][0], "mixer": kinds[i % 4][1], "mlp": mlp} for i in range(z["layers"])]
    return BokulornConfig.from_dict({"vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6},
                                     "embedding": {"scale": z["width"] ** 0.5}, "layers": layers})


def _bokulorn_kernel_table(z, bz, dev, batch, prompt_len):
    """Each kernel of the design alone at one layer's shapes (prompt step and decode step), beside the Kagalorn
    kernel that does the like job."""
    from light_vllm_amd import mix_ops
    from light_vllm_amd.layers.latent_attention import NO_WINDOW
    from light_vllm_amd.layers.moe import SparseMoE
    from light_vllm_amd.utils.context import RaggedStep
    bf = torch.bfloat16
    W, H, G, D = z["width"], z["heads"], z["kv_heads"], z["dim"]
    R, Dr, Rq, E, top = bz["kv_rank"], bz["rot_dim"], bz["q_rank"], bz["experts"], bz["top"]
    Fe = z["ff"] // top
    page = 256
    rows = []

    def step_of(lens_q, ctx):
        B = len(lens_q)
        cu, tok = [0], []
        for b, n_ in enumerate(lens_q):
            cu.append(cu[-1] + n_)
            tok += [b] * n_
        per = -(-(max(ctx) + max(lens_q)) // page)
        tables = [[b * per + j for j in range(per)] for b in range(B)]
        i32 = dict(dtype=torch.int32, device=dev)
        return RaggedStep(torch.tensor(cu, **i32), torch.tensor(ctx, **i32), torch.arange(B, **i32),
                          torch.tensor(tok, **i32), torch.tensor(tables, **i32), lens_q, ctx, list(range(B)), tables), B * per

    def add(name, phase, fn, nbytes=0, flops=0, like=None):
        us = _event_time(fn, 20, 3) * 1e6
        rec = {"kernel": name, "phase": phase, "us": round(us, 1)}
        if nbytes:
            rec["of_hbm_roofline"] = round(nbytes / us / 1e3 / (HBM_BPS / 1e9), 3)
        if flops:
            rec["TFLOPs"] = round(flops / us / 1e6, 2)
            rec["of_mfma_roofline"] = round(flops / us / 1e6 / (MFMA_FLOPS / 1e12), 4)
        if like:
            rec["like"] = like
        rows.append(rec)

    old_default = torch.get_default_dtype()
    torch.set_default_dtype(bf)
    try:
        moe = SparseMoE(W, Fe, E, top, bz["groups"], bz["keep"]).to(dev)
    finally:
        torch.set_default_dtype(old_default)
    for prm in moe.parameters():
        prm.data.normal_(0.0, 0.02)
    for phase, lens_q, ctx in (("prompt", [prompt_len] * batch, [0] * batch), ("decode", [1] * batch, [prompt_len] * batch)):
        step, pages = step_of(lens_q, ctx)
        T = sum(lens_q)
        x = torch.randn(T, W, device=dev)
        y1, y2 = torch.randn(T, W, device=dev, dtype=bf), torch.randn(T, W, device=dev, dtype=bf)
        nw = torch.zeros(W, device=dev)
        add("residual_add_norm", phase, lambda: mix_ops.residual_add_norm(x, y1, y2, nw, 1.0, 1e-6, bf), nbytes=T * W * 14)
        xs = torch.randn(T, 4, W, device=dev)
        mixm, vec = torch.eye(4, device=dev), torch.ones(4, device=dev)
        add("kagalorn hc_update_norm", phase, lambda: mix_ops.hc_update_norm(xs, y1, mixm, vec, vec, nw, 4, 1e-6, bf),
            nbytes=T * W * 36, like="residual_add_norm")
        # latent attention
        proj = torch.randn(T, Rq + R + Dr + H, device=dev, dtype=bf)
        inv_freq = mix_ops.rotary_inv_freq(Dr, 10000.0, dev)
        cache = torch.zeros(pages, page, R + Dr, device=dev, dtype=bf)
        qw, kw_ = torch.ones(Rq, device=dev), torch.ones(R, device=dev)
        add("latent_prep", phase, lambda: mix_ops.latent_prep(proj, 0, Rq, qw, kw_, inv_freq, cache, step, Rq, R, Dr, Dr, 1e-6),
            nbytes=T * (Rq * 4 + (R + Dr) * 4))
        q = torch.randn(T, H * (D + Dr), device=dev, dtype=bf)
        q_lat = torch.randn(H, T, R, device=dev, dtype=bf)
        add("latent_q_finish", phase, lambda: mix_ops.latent_q_finish(q, q_lat, inv_freq, step, H, D, Dr, R, Dr),
            nbytes=T * H * ((R + Dr) * 4))
        q_abs = mix_ops.latent_q_finish(q, q_lat, inv_freq, step, H, D, Dr, R, Dr)
        kc = cache.unsqueeze(2)
        keys = sum(i + 1 for n_, c0 in zip(lens_q, ctx) for i in range(c0, c0 + n_))
        attn = lambda: mix_ops.window_pool_attention(q_abs, kc, kc[..., :R], None, None, None, step, H, 1, R + Dr, R,  # noqa: E731
                                                     NO_WINDOW, 0, 0.07, has_sink=False)
        if phase == "prompt":
            add("latent attention", phase, attn, flops=keys * H * (2 * R + Dr) * 2)
        else:
            add("latent attention", phase, attn, nbytes=keys * (R + Dr) * 2)
        o = torch.randn(H, T, D, device=dev, dtype=bf)
        add("latent_out_gate", phase, lambda: mix_ops.latent_out_gate(o, proj[:, Rq + R + Dr:], False), nbytes=T * H * D * 4)
        # the like kernel: windowed pooled attention of Kagalorn with the window open to the whole context
        kq = torch.randn(T, H * D, device=dev, dtype=bf)
        kk = torch.zeros(pages, page, G, D, device=dev, dtype=bf)
        kattn = lambda: mix_ops.window_pool_attention(kq, kk, kk, None, None, None, step, H, G, D, D, NO_WINDOW, 0,  # noqa: E731
                                                      D ** -0.5, True)
        if phase == "prompt":
            add("kagalorn window_pool_attn", phase, kattn, flops=keys * H * D * 4, like="latent attention")
        else:
            add("kagalorn window_pool_attn", phase, kattn, nbytes=keys * G * D * 4, like="latent attention")
        # channel-wise delta rule
        C = 2 * G * D + H * D
        dproj = torch.randn(T, C + H, device=dev, dtype=bf)
        a = torch.randn(T, H * D, device=dev, dtype=bf)
        conv_w = torch.randn(C, 4, device=dev) * 0.5
        conv_state = torch.zeros(batch, 3, C, device=dev, dtype=bf)
        A_log = torch.zeros(H, device=dev)
        state = torch.zeros(batch, H, D, D, device=dev)
        for ch in (True, False):
            dtb = torch.zeros(H * D if ch else H, device=dev)
            a_in = a if ch else a[:, :H]
            name = "channel" if ch else "kagalorn per-head"
            add(f"delta_prep ({name})", phase, lambda: mix_ops.delta_prep(dproj, conv_w, conv_state, A_log, dtb, step, G, H, D, D, 4, C,
                                                                         a_in, 1e-6, decay_per_channel=ch),
                nbytes=T * (C * 6 + (H * D * 6 if ch else 0)), like=None if ch else "delta_prep (channel)")
            qn, kn, v, beta, dec = mix_ops.delta_prep(dproj, conv_w, conv_state, A_log, dtb, step, G, H, D, D, 4, C, a_in, 1e-6,
                                                      decay_per_channel=ch)
            add(f"gated_delta_rule ({name})", phase, lambda: mix_ops.gated_delta_rule(qn, kn, v, beta, dec, state, step),
                nbytes=batch * H * D * D * 8 + T * (2 * G * D + 2 * H * D + (H * D if ch else 0)) * 4,
                like=None if ch else "gated_delta_rule (channel)")
        # mixture of experts
        h = torch.randn(T, W, device=dev, dtype=bf)
        logits = torch.randn(T, E, device=dev)
        add("moe_route", phase, lambda: mix_ops.moe_route(logits, moe.correction, top, bz["groups"], bz["keep"]))
        with torch.inference_mode():
            add("moe feed-forward (all of it)", phase, lambda: moe(h), flops=T * top * Fe * W * 4)
            wg = torch.randn(2 * z["ff"], W, device=dev, dtype=bf) * 0.02
            wd = torch.randn(W, z["ff"], device=dev, dtype=bf) * 0.02
            add("kagalorn dense feed-forward", phase,
                lambda: torch.nn.functional.linear(mix_ops.clamped_glu(torch.nn.functional.linear(h, wg), 7.0, 1.702), wd),
                flops=T * z["ff"] * W * 6, like="moe feed-forward (all of it)")
    return rows


def bokulorn_leg(sizes, batch, prompt_len, new_tokens):
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    out = {"metric": "mixers: Bokulorn beside Kagalorn at equal size", "dtype": "bf16", "data": "synthetic, random weights",
           "batch": batch, "prompt_len": prompt_len, "new_tokens": new_tokens, "sizes": []}
    for name in sizes:
        z, bz = MIXER_SIZES[name], BOKULORN_SIZES[name]
        rec = {"size": name, **z, **bz}
        cache_tokens = batch * 256 * (-(-(prompt_len + new_tokens) // 256))
        kw = dict(kvcache_block_size=256, max_cache_tokens=cache_tokens)
        rec["bokulorn"] = _engine_rates(_bokulorn_config(z, bz), batch, prompt_len, new_tokens, **kw)
        rec["bokulorn_graph"] = _engine_rates(_bokulorn_config(z, bz), batch, prompt_len, new_tokens, enforce_eager=False, **kw)
        rec["kagalorn"] = _engine_rates(_kagalorn_config(z), batch, prompt_len, new_tokens, **kw)
        rec["kagalorn_graph"] = _engine_rates(_kagalorn_config(z), batch, prompt_len, new_tokens, enforce_eager=False, **kw)
        rec["kernels"] = _bokulorn_kernel_table(z, bz, dev, batch, prompt_len)
        out["sizes"].append(rec)
    print(json.dumps(out), flush=True)


# --mixers-design givozen: the Givozen design (gated rotary attention with head temperatures, sublayers normed on
# both sides, PolyNorm and gated-expert feed-forwards, a looped stretch of layers) beside Bokulorn, the closest existing
# model (one f32 residual with offset norms, the same paged attention kernel without a window, a mixture of experts),
# at equal width, layer runs, head counts and active feed-forward parameters.
GIVOZEN_SIZES = {
    "2k": dict(experts=32, top=4, expert_ff=768, shared_ff=1024, rot_dims=64),
    "4k": dict(experts=32, top=4, expert_ff=1536, shared_ff=2048, rot_dims=64),
}


def _givozen_config(z, gz):
    from light_vllm_amd.models.givozen import GivozenConfig
    att = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"], "scale": z["dim"] ** -0.5,
           "rot": {"base": 500000.0, "dims": gz["rot_dims"], "scaling": {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 2048}}}
    moe = {"kind": "moe", "expert": {"ff": gz["expert_ff"], "limit": 7.0}, "router": {"experts": gz["experts"], "top": gz["top"]},
           "shared": {"ff": gz["shared_ff"], "limit": 7.0}}
    dense = {"kind": "dense", "ff": z["ff"]}
    looped = 2 if z["layers"] >= 6 else 1      # layers that run twice: as many layer runs as the other model has layers
    n = z["layers"] - looped
    layers = [{"type": "attention", "mixer": att, "mlp": dense if i == 0 else moe} for i in range(n)]
    return GivozenConfig.from_dict({"vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6}, "layers": layers,
                                    "loop": {"start": 1, "stop": 1 + looped, "times": 2}})


def _givozen_kernel_table(z, gz, bz, dev, batch, prompt_len):
    """Each kernel of the design alone at one layer's shapes (prompt step and decode step), beside the Bokulorn
    (or Kagalorn) kernel that does the like job."""
    from light_vllm_amd import mix_ops
    from light_vllm_amd.layers.moe import GLUSparseMoE, SparseMoE
    from light_vllm_amd.layers.rotary_attention import NO_WINDOW
    from light_vllm_amd.utils.context import RaggedStep
    bf = torch.bfloat16
    W, H, G, D = z["width"], z["heads"], z["kv_heads"], z["dim"]
    E, top, Fe, Fs, rd = gz["experts"], gz["top"], gz["expert_ff"], gz["shared_ff"], gz["rot_dims"]
    R, Dr, Rq = bz["kv_rank"], bz["rot_dim"], bz["q_rank"]
    page = 256
    rows = []

    def step_of(lens_q, ctx):
        B = len(lens_q)
        cu, tok = [0], []
        for b, n_ in enumerate(lens_q):
            cu.append(cu[-1] + n_)
            tok += [b] * n_
        per = -(-(max(ctx) + max(lens_q)) // page)
        tables = [[b * per + j for j in range(per)] for b in range(B)]
        i32 = dict(dtype=torch.int32, device=dev)
        return RaggedStep(torch.tensor(cu, **i32), torch.tensor(ctx, **i32), torch.arange(B, **i32),
                          torch.tensor(tok, **i32), torch.tensor(tables, **i32), lens_q, ctx, list(range(B)), tables), B * per

    def add(name, phase, fn, nbytes=0, flops=0, like=None):
        us = _event_time(fn, 20, 3) * 1e6
        rec = {"kernel": name, "phase": phase, "us": round(us, 1)}
        if nbytes:
            rec["of_hbm_roofline"] = round(nbytes / us / 1e3 / (HBM_BPS / 1e9), 3)
        if flops:
            rec["TFLOPs"] = round(flops / us / 1e6, 2)
            rec["of_mfma_roofline"] = round(flops / us / 1e6 / (MFMA_FLOPS / 1e12), 4)
        if like:
            rec["like"] = like
        rows.append(rec)

    old_default = torch.get_default_dtype()
    torch.set_default_dtype(bf)
    try:
        moe = GLUSparseMoE(W, Fe, E, top, 7.0, 1.702, Fs, 7.0).to(dev)
        bmoe = SparseMoE(W, z["ff"] // bz["top"], bz["experts"], bz["top"], bz["groups"], bz["keep"]).to(dev)
    finally:
        torch.set_default_dtype(old_default)
    for prm in list(moe.parameters()) + list(bmoe.parameters()):
        prm.data.normal_(0.0, 0.02)
    for phase, lens_q, ctx in (("prompt", [prompt_len] * batch, [0] * batch), ("decode", [1] * batch, [prompt_len] * batch)):
        step, pages = step_of(lens_q, ctx)
        T = sum(lens_q)
        x = torch.randn(T, W, device=dev)
        y1, y2 = torch.randn(T, W, device=dev, dtype=bf), torch.randn(T, W, device=dev, dtype=bf)
        nw = torch.zeros(W, device=dev)
        add("sandwich_add_norm", phase, lambda: mix_ops.sandwich_add_norm(x, y1, nw, None, None, nw, 1.0, 1e-6, bf), nbytes=T * W * 12)
        add("sandwich_add_norm (start of a pass)", phase, lambda: mix_ops.sandwich_add_norm(x, y1, nw, y2, nw, nw, 1.0, 1e-6, bf),
            nbytes=T * W * 14)
        add("bokulorn residual_add_norm", phase, lambda: mix_ops.residual_add_norm(x, y1, y2, nw, 1.0, 1e-6, bf), nbytes=T * W * 14,
            like="sandwich_add_norm")
        # attention: rotation + cache write, then the paged kernel
        cols = H * D + 2 * G * D + H
        proj = torch.randn(T, cols, device=dev, dtype=bf)
        inv_freq = mix_ops.rotary_inv_freq(rd, 500000.0, dev)
        temp = torch.ones(H, device=dev)
        kc = torch.zeros(pages, page, G, D, device=dev, dtype=bf)
        vc = torch.zeros(pages, page, G, D, device=dev, dtype=bf)
        add("rotary_store", phase, lambda: mix_ops.rotary_store(proj, 0, H * D, H * D + G * D, inv_freq, temp, kc, vc, step, H, G, D, D, rd),
            nbytes=T * (H * D + 2 * G * D) * 4)
        lproj = torch.randn(T, Rq + R + Dr + H, device=dev, dtype=bf)
        lcache = torch.zeros(pages, page, R + Dr, device=dev, dtype=bf)
        qw, kw_ = torch.ones(Rq, device=dev), torch.ones(R, device=dev)
        lfreq = mix_ops.rotary_inv_freq(Dr, 10000.0, dev)
        add("bokulorn latent_prep", phase, lambda: mix_ops.latent_prep(lproj, 0, Rq, qw, kw_, lfreq, lcache, step, Rq, R, Dr, Dr, 1e-6),
            nbytes=T * (Rq * 4 + (R + Dr) * 4), like="rotary_store")
        q = mix_ops.rotary_store(proj, 0, H * D, H * D + G * D, inv_freq, temp, kc, vc, step, H, G, D, D, rd)
        gate = proj[:, H * D + 2 * G * D:]
        keys = sum(i + 1 for n_, c0 in zip(lens_q, ctx) for i in range(c0, c0 + n_))
        attn = lambda: mix_ops.window_pool_attention(q, kc, vc, None, None, gate, step, H, G, D, D, NO_WINDOW, 0, D ** -0.5,  # noqa: E731
                                                     has_sink=False, gate_per_head=True)
        q_abs = torch.randn(T, H * (R + Dr), device=dev, dtype=bf)
        lc = lcache.unsqueeze(2)
        lattn = lambda: mix_ops.window_pool_attention(q_abs, lc, lc[..., :R], None, None, None, step, H, 1, R + Dr, R,  # noqa: E731
                                                      NO_WINDOW, 0, 0.07, has_sink=False)
        if phase == "prompt":
            add("gated rotary attention", phase, attn, flops=keys * H * D * 4)
            add("bokulorn latent attention", phase, lattn, flops=keys * H * (2 * R + Dr) * 2, like="gated rotary attention")
        else:
            add("gated rotary attention", phase, attn, nbytes=keys * G * D * 4)
            add("bokulorn latent attention", phase, lattn, nbytes=keys * (R + Dr) * 2, like="gated rotary attention")
        # feed-forwards
        h = torch.randn(T, W, device=dev, dtype=bf)
        zf = torch.randn(T, z["ff"], device=dev, dtype=bf)
        coef = torch.tensor([0.6, 0.3, 0.1, 0.0], device=dev)
        add("polynorm", phase, lambda: mix_ops.polynorm(zf, coef, 1e-6), nbytes=T * z["ff"] * 4)
        zg = torch.randn(T, 2 * z["ff"], device=dev, dtype=bf)
        add("kagalorn clamped_glu", phase, lambda: mix_ops.clamped_glu(zg, 7.0, 1.702), nbytes=T * z["ff"] * 6, like="polynorm")
        with torch.inference_mode():
            wu = torch.randn(z["ff"], W, device=dev, dtype=bf) * 0.02
            wd = torch.randn(W, z["ff"], device=dev, dtype=bf) * 0.02
            add("dense PolyNorm feed-forward", phase,
                lambda: torch.nn.functional.linear(mix_ops.polynorm(torch.nn.functional.linear(h, wu), coef, 1e-6), wd),
                flops=T * z["ff"] * W * 4)
            wg = torch.randn(2 * z["ff"], W, device=dev, dtype=bf) * 0.02
            add("kagalorn dense feed-forward", phase,
                lambda: torch.nn.functional.linear(mix_ops.clamped_glu(torch.nn.functional.linear(h, wg), 7.0, 1.702), wd),
                flops=T * z["ff"] * W * 6, like="dense PolyNorm feed-forward")
            weight_bytes = (min(T * top, E) * 3 * Fe + 3 * Fs) * W * 2
            bweight_bytes = min(T * bz["top"], bz["experts"]) * 2 * (z["ff"] // bz["top"]) * W * 2
            add("gated-expert feed-forward (router to sum, shared expert)", phase, lambda: moe(h),
                flops=T * (top * Fe + Fs) * W * 6, nbytes=weight_bytes if phase == "decode" else 0)
            add("bokulorn moe feed-forward", phase, lambda: bmoe(h), flops=T * bz["top"] * (z["ff"] // bz["top"]) * W * 4,
                nbytes=bweight_bytes if phase == "decode" else 0, like="gated-expert feed-forward (router to sum, shared expert)")
    return rows


def givozen_leg(sizes, batch, prompt_len, new_tokens):
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    out = {"metric": "mixers: Givozen beside Bokulorn at equal size", "dtype": "bf16", "data": "synthetic, random weights",
           "batch": batch, "prompt_len": prompt_len, "new_tokens": new_tokens, "sizes": []}
    for name in sizes:
        z, gz, bz = MIXER_SIZES[name], GIVOZEN_SIZES[name], BOKULORN_SIZES[name]
        rec = {"size": name, **z, **gz}
        cache_tokens = batch * 256 * (-(-(prompt_len + new_tokens) // 256))
        kw = dict(kvcache_block_size=256, max_cache_tokens=cache_tokens)
        rec["givozen"] = _engine_rates(_givozen_config(z, gz), batch, prompt_len, new_tokens, **kw)
        rec["givozen_graph"] = _engine_rates(_givozen_config(z, gz), batch, prompt_len, new_tokens, enforce_eager=False, **kw)
        rec["bokulorn"] = _engine_rates(_bokulorn_config(z, bz), batch, prompt_len, new_tokens, **kw)
        rec["bokulorn_graph"] = _engine_rates(_bokulorn_config(z, bz), batch, prompt_len, new_tokens, enforce_eager=False, **kw)
        rec["kernels"] = _givozen_kernel_table(z, gz, bz, dev, batch, prompt_len)
        out["sizes"].append(rec)
    print(json.dumps(out), flush=True)


# --mixers-design bisuzen: the Bisuzen design (layers whose mixer is a windowed attention with kept first tokens and learned
# sinks beside a lightning attention, layers of chunked attention with unit-normed heads, tanh norms, gated dense and
# softmax-routed expert feed-forwards with identity experts, a looped stretch of layers) beside Givozen, the closest existing
# model (one f32 residual, the same paged attention kernel, dense and expert feed-forwards, looped layers), at equal width,
# layer runs, head counts and active feed-forward parameters.
BISUZEN_SIZES = {
    "2k": dict(experts=30, identity=2, top=4, groups=4, keep=2, rot_dims=64, window=512, keep_first=4, chunk=512, state_heads=16),
    "4k": dict(experts=30, identity=2, top=4, groups=4, keep=2, rot_dims=64, window=512, keep_first=4, chunk=512, state_heads=32),
}


def _bisuzen_config(z, sz):
    from light_vllm_amd.models.bisuzen import BisuzenConfig
    H, G, D = z["heads"], z["kv_heads"], z["dim"]
    Hs = sz["state_heads"]
    left = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "rot": {"base": 500000.0, "dims": sz["rot_dims"]},
            "mask": {"size": sz["window"], "keep_first": sz["keep_first"]}}
    right = {"heads": Hs, "dim": D, "vdim": D, "decay": [1.0 - 2.0 ** (-5.0 - 5.0 * i / max(Hs - 1, 1)) for i in range(Hs)]}
    att = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "mask": {"size": sz["chunk"]}}
    moe = {"kind": "moe", "expert": {"ff": z["ff"] // sz["top"]},
           "router": {"experts": sz["experts"], "identity": sz["identity"], "top": sz["top"],
                      "groups": {"count": sz["groups"], "keep": sz["keep"]}}}
    dense = {"kind": "dense", "ff": z["ff"]}
    looped = 2 if z["layers"] >= 6 else 1      # layers that run twice: as many layer runs as the other model has
    n = z["layers"] - looped
    layers = [{"type": "parallel" if i % 2 == 0 else "attention", "mixer": {"left": left, "right": right} if i % 2 == 0 else att,
               "mlp": dense if i == 0 else moe} for i in range(n)]
    return BisuzenConfig.from_dict({"vocab": z["vocab"], "width": z["width"], "norm": {"eps": 1e-6}, "logit_scale": 1.0,
                                    "layers": layers, "loop": {"start": 1, "stop": 1 + looped, "times": 2}})


def _bisuzen_kernel_table(z, sz, gz, bz, dev, batch, prompt_len):
    """Each kernel of the design alone at one layer's shapes (prompt step and decode step), beside the kernel of Givozen
    (or, for the recurrence and the experts, of Kagalorn and Bokulorn) that does the like job."""
    from light_vllm_amd import mix_ops
    from light_vllm_amd.layers.moe import SparseMoE
    from light_vllm_amd.layers.rotary_attention import NO_WINDOW
    from light_vllm_amd.utils.context import RaggedStep
    bf = torch.bfloat16
    W, H, G, D, Hs = z["width"], z["heads"], z["kv_heads"], z["dim"], sz["state_heads"]
    E, ident, top, Fe, rd = sz["experts"], sz["identity"], sz["top"], z["ff"] // sz["top"], sz["rot_dims"]
    window, keep, chunk = sz["window"], sz["keep_first"], sz["chunk"]
    page = 256
    rows = []

    def step_of(lens_q, ctx):
        B = len(lens_q)
        cu, tok = [0], []
        for b, n_ in enumerate(lens_q):
            cu.append(cu[-1] + n_)
            tok += [b] * n_
        per = -(-(max(ctx) + max(lens_q)) // page)
        tables = [[b * per + j for j in range(per)] for b in range(B)]
        i32 = dict(dtype=torch.int32, device=dev)
        return RaggedStep(torch.tensor(cu, **i32), torch.tensor(ctx, **i32), torch.arange(B, **i32),
                          torch.tensor(tok, **i32), torch.tensor(tables, **i32), lens_q, ctx, list(range(B)), tables), B * per

    def add(name, phase, fn, nbytes=0, flops=0, like=None, matrix=True):
        us = _event_time(fn, 20, 3) * 1e6
        rec = {"kernel": name, "phase": phase, "us": round(us, 1)}
        if nbytes:
            rec["of_hbm_roofline"] = round(nbytes / us / 1e3 / (HBM_BPS / 1e9), 3)
        if flops:
            rec["TFLOPs"] = round(flops / us / 1e6, 2)
            if matrix:
                rec["of_mfma_roofline"] = round(flops / us / 1e6 / (MFMA_FLOPS / 1e12), 4)
        if like:
            rec["like"] = like
        rows.append(rec)

    old_default = torch.get_default_dtype()
    torch.set_default_dtype(bf)
    try:
        moe = SparseMoE(W, Fe, E, top, sz["groups"], sz["keep"], score="softmax", group_rank="max", act="gelu", identity=ident,
                        logits_kernel=True).to(dev)
        bmoe = SparseMoE(W, z["ff"] // bz["top"], bz["experts"], bz["top"], bz["groups"], bz["keep"]).to(dev)
    finally:
        torch.set_default_dtype(old_default)
    for prm in list(moe.parameters()) + list(bmoe.parameters()):
        prm.data.normal_(0.0, 0.02)
    for phase, lens_q, ctx in (("prompt", [prompt_len] * batch, [0] * batch), ("decode", [1] * batch, [prompt_len] * batch)):
        step, pages = step_of(lens_q, ctx)
        T = sum(lens_q)
        x = torch.randn(T, W, device=dev)
        y1, y2 = torch.randn(T, W, device=dev, dtype=bf), torch.randn(T, W, device=dev, dtype=bf)
        nw, alpha = torch.ones(W, device=dev), torch.full((1,), 0.5, device=dev)
        add("residual_dyt", phase, lambda: mix_ops.residual_dyt(x, y1, None, None, None, 1.0, 1e-6, alpha, nw, nw, bf), nbytes=T * W * 12)
        add("residual_dyt (two normed mixer outputs)", phase,
            lambda: mix_ops.residual_dyt(x, y1, y2, nw, nw, 0.5, 1e-6, alpha, nw, nw, bf), nbytes=T * W * 14)
        add("givozen sandwich_add_norm", phase, lambda: mix_ops.sandwich_add_norm(x, y1, nw, None, None, nw, 1.0, 1e-6, bf),
            nbytes=T * W * 12, like="residual_dyt")
        # attention inputs: unit norm or rotation, cache write
        cols = H * D + 2 * G * D
        proj = torch.randn(T, cols + H, device=dev, dtype=bf)
        inv_freq = mix_ops.rotary_inv_freq(rd, 500000.0, dev)
        temp = torch.ones(H, device=dev)
        kc = torch.zeros(pages, page, G, D, device=dev, dtype=bf)
        vc = torch.zeros(pages, page, G, D, device=dev, dtype=bf)
        prep_bytes = T * cols * 4
        add("qk_prep_store (pairs side by side rotated)", phase,
            lambda: mix_ops.rotary_store(proj, 0, H * D, H * D + G * D, inv_freq, None, kc, vc, step, H, G, D, D, rd, interleaved=True),
            nbytes=prep_bytes)
        add("qk_prep_store (heads divided by their rms)", phase,
            lambda: mix_ops.rotary_store(proj, 0, H * D, H * D + G * D, None, None, kc, vc, step, H, G, D, D, 0, unit_eps=1e-6),
            nbytes=prep_bytes)
        add("givozen rotary_store", phase,
            lambda: mix_ops.rotary_store(proj, 0, H * D, H * D + G * D, inv_freq, temp, kc, vc, step, H, G, D, D, rd),
            nbytes=prep_bytes, like="qk_prep_store")
        q = mix_ops.rotary_store(proj, 0, H * D, H * D + G * D, inv_freq, None, kc, vc, step, H, G, D, D, rd, interleaved=True)
        sinks = torch.zeros(H, device=dev)
        gate = proj[:, cols:]
        pos = [i for n_, c0 in zip(lens_q, ctx) for i in range(c0, c0 + n_)]
        keys_full = sum(i + 1 for i in pos)
        keys_win = sum(min(i + 1, window) + min(keep, max(i + 1 - window, 0)) for i in pos)
        keys_chunk = sum(i % chunk + 1 for i in pos)
        wattn = lambda: mix_ops.window_pool_attention(q, kc, vc, None, None, None, step, H, G, D, D, window, 0, D ** -0.5,  # noqa: E731
                                                      has_sink=False, keep_first=keep, sinks=sinks)
        cattn = lambda: mix_ops.window_pool_attention(q, kc, vc, None, None, None, step, H, G, D, D, NO_WINDOW, 0, D ** -0.5,  # noqa: E731
                                                      has_sink=False, chunk=chunk)
        gattn = lambda: mix_ops.window_pool_attention(q, kc, vc, None, None, gate, step, H, G, D, D, NO_WINDOW, 0, D ** -0.5,  # noqa: E731
                                                      has_sink=False, gate_per_head=True)
        if phase == "prompt":
            add("windowed attention with kept tokens and sinks", phase, wattn, flops=keys_win * H * D * 4)
            add("chunked attention", phase, cattn, flops=keys_chunk * H * D * 4)
            add("givozen gated rotary attention", phase, gattn, flops=keys_full * H * D * 4, like="windowed / chunked attention")
        else:
            add("windowed attention with kept tokens and sinks", phase, wattn, nbytes=keys_win * G * D * 4)
            add("chunked attention", phase, cattn, nbytes=keys_chunk * G * D * 4)
            add("givozen gated rotary attention", phase, gattn, nbytes=keys_full * G * D * 4, like="windowed / chunked attention")
        # the decaying state beside the delta rule
        B = len(lens_q)
        lproj = torch.randn(T, 4 * Hs * D, device=dev, dtype=bf)
        decay = torch.full((Hs,), 0.99, device=dev)
        state = torch.zeros(B, Hs, D, D, device=dev)
        state_bytes = B * Hs * D * D * 8 + T * Hs * D * (3 * 2 + 4)
        add("lightning_attention", phase, lambda: mix_ops.lightning_attention(lproj, 0, Hs * D, 2 * Hs * D, decay, state, step, Hs, D, D),
            flops=T * Hs * D * D * 4, nbytes=state_bytes if phase == "decode" else 0, matrix=False)
        qn, kn = torch.randn(T, G, D, device=dev) * D ** -0.5, torch.randn(T, G, D, device=dev) * D ** -0.5
        dv = torch.randn(T, Hs, D, device=dev)
        beta, dec = torch.rand(T, Hs, device=dev), torch.full((T, Hs), 0.99, device=dev)
        dstate = torch.zeros(B, Hs, D, D, device=dev)
        add("kagalorn gated_delta_rule", phase, lambda: mix_ops.gated_delta_rule(qn, kn, dv, beta, dec, dstate, step),
            flops=T * Hs * D * D * 6, nbytes=(B * Hs * D * D * 8 + T * (2 * G * D + 2 * Hs * D) * 4) if phase == "decode" else 0,
            like="lightning_attention", matrix=False)
        o = torch.randn(T, Hs, D, device=dev)
        gw = torch.ones(Hs * D, device=dev)
        lgate = lproj[:, 3 * Hs * D:]
        add("norm over all heads with gate", phase, lambda: mix_ops.head_norm_gate(o.view(T, 1, Hs * D), lgate, gw, 1e-6, bf, "sigmoid"),
            nbytes=T * Hs * D * 8)
        add("kagalorn norm per head with gate", phase, lambda: mix_ops.head_norm_gate(o, lgate, gw[:D], 1e-6, bf, "silu"),
            nbytes=T * Hs * D * 8, like="norm over all heads with gate")
        # feed-forwards
        h = torch.randn(T, W, device=dev, dtype=bf)
        zg = torch.randn(T, 2 * z["ff"], device=dev, dtype=bf)
        add("glu_act (tanh gelu)", phase, lambda: mix_ops.glu_act(zg, "gelu_tanh"), nbytes=T * z["ff"] * 6)
        add("kagalorn clamped_glu", phase, lambda: mix_ops.clamped_glu(zg, 7.0, 1.702), nbytes=T * z["ff"] * 6, like="glu_act")
        with torch.inference_mode():
            wg = torch.randn(2 * z["ff"], W, device=dev, dtype=bf) * 0.02
            wd = torch.randn(W, z["ff"], device=dev, dtype=bf) * 0.02
            add("dense gated feed-forward", phase,
                lambda: torch.nn.functional.linear(mix_ops.glu_act(torch.nn.functional.linear(h, wg), "gelu_tanh"), wd),
                flops=T * z["ff"] * W * 6)
            add("kagalorn dense feed-forward", phase,
                lambda: torch.nn.functional.linear(mix_ops.clamped_glu(torch.nn.functional.linear(h, wg), 7.0, 1.702), wd),
                flops=T * z["ff"] * W * 6, like="dense gated feed-forward")
            weight_bytes = min(T * top, E) * 2 * Fe * W * 2
            bweight_bytes = min(T * bz["top"], bz["experts"]) * 2 * (z["ff"] // bz["top"]) * W * 2
            add("expert feed-forward (softmax router to sum, identity experts)", phase, lambda: moe(h),
                flops=T * top * Fe * W * 4, nbytes=weight_bytes if phase == "decode" else 0)
            add("bokulorn moe feed-forward", phase, lambda: bmoe(h), flops=T * bz["top"] * (z["ff"] // bz["top"]) * W * 4,
                nbytes=bweight_bytes if phase == "decode" else 0, like="expert feed-forward (softmax router to sum, identity experts)")
    return rows


def bisuzen_leg(sizes, batch, prompt_len, new_tokens, engine_only=False):
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    out = {"metric": "mixers: Bisuzen beside Givozen at equal size", "dtype": "bf16", "data": "synthetic, random weights",
           "batch": batch, "prompt_len": prompt_len, "new_tokens": new_tokens, "sizes": []}
    for name in sizes:
        z, sz, gz, bz = MIXER_SIZES[name], BISUZEN_SIZES[name], GIVOZEN_SIZES[name], BOKULORN_SIZES[name]
        rec = {"size": name, **z, **sz}
        cache_tokens = batch * 256 * (-(-(prompt_len + new_tokens) // 256))
        kw = dict(kvcache_block_size=256, max_cache_tokens=cache_tokens)
        rec["bisuzen"] = _engine_rates(_bisuzen_config(z, sz), batch, prompt_len, new_tokens, **kw)
        rec["bisuzen_graph"] = _engine_rates(_bisuzen_config(z, sz), batch, prompt_len, new_tokens, enforce_eager=False, **kw)
        if engine_only:              # a run to be profiled: this design's kernels only
            out["sizes"].append(rec)
            continue
        rec["givozen"] = _engine_rates(_givozen_config(z, gz), batch, prompt_len, new_tokens, **kw)
        rec["givozen_graph"] = _engine_rates(_givozen_config(z, gz), batch, prompt_len, new_tokens, enforce_eager=False, **kw)
        rec["kernels"] = _bisuzen_kernel_table(z, sz, gz, bz, dev, batch, prompt_len)
        out["sizes"].append(rec)
    print(json.dumps(out), flush=True)


def mixers_leg(sizes, batch, prompt_len, new_tokens):
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    out = {"metric": "mixers: Kagalorn beside Qwen3 at equal size", "dtype": "bf16", "data": "synthetic, random weights",
           "batch": batch, "prompt_len": prompt_len, "new_tokens": new_tokens, "sizes": []}
    for name in sizes:
        z = MIXER_SIZES[name]
        rec = {"size": name, **z}
        cache_tokens = batch * 256 * (-(-(prompt_len + new_tokens) // 256))
        rec["kagalorn"] = _engine_rates(_kagalorn_config(z), batch, prompt_len, new_tokens, kvcache_block_size=256,
                                        max_cache_tokens=cache_tokens)
        rec["kagalorn_graph"] = _engine_rates(_kagalorn_config(z), batch, prompt_len, new_tokens, kvcache_block_size=256,
                                              max_cache_tokens=cache_tokens, enforce_eager=False)
        blocks = batch * (-(-(prompt_len + new_tokens) // 256)) + 8
        rec["qwen3_eager"] = _engine_rates(_qwen3_config(z), batch, prompt_len, new_tokens, num_kvcache_blocks=blocks,
                                           enforce_eager=True)
        rec["qwen3_graph"] = _engine_rates(_qwen3_config(z), batch, prompt_len, new_tokens, num_kvcache_blocks=blocks,
                                           enforce_eager=False)
        rec["kernels"] = _mixer_kernel_table(z, dev, batch, prompt_len)
        out["sizes"].append(rec)
    print(json.dumps(out), flush=True)


def tp_step_setup(ops, dev, n, rank, cfg, layers, batch):
    """The config-4 step on this rank: workload + the activation the per-layer all-reduce sums."""
    w = DecodeWorkload(ops, dev, layers, cfg["hq"] // n, cfg["hkv"] // n, batch, cfg["ctx"], seed=4321 + rank)
    hidden = torch.ones(batch, cfg["hidden"], dtype=torch.bfloat16, device=dev)
    return w, hidden


def run_steps(step, steps, warmup, sync_all, use_graph):
    """W untimed + exactly K timed steps, barrier + synchronize on both sides. With use_graph the
    step is captured once and the timed steps are replays. Returns (elapsed seconds, graph used, note)."""
    note = None
    graph = None
    if use_graph:
        try:
            step()                                   # warm run outside capture
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
        except Exception as exc:                      # reported on the line; the eager step still measures
            note = f"hipGraph capture failed, eager steps timed instead: {exc!r}"[:300]
            graph = None
            torch.cuda.synchronize()
    run = graph.replay if graph is not None else step
    for _ in range(warmup):
        run()
    sync_all()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    sync_all()
    return time.perf_counter() - t0, graph is not None, note


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-aux", action="store_true", help="skip the auxiliary legs")
    ap.add_argument("--aux", default="prefill,variants,config4,collectives,e2e",
                    help="comma list of auxiliary legs to run (prefill, variants, config4, collectives, e2e)")
    ap.add_argument("--rehearse", action="store_true",
                    help="N > 1 on ONE GPU: every rank on cuda:0, gloo group, 4 layers, batch 8 "
                         "(proves launcher, rendezvous, graph and JSON path; not a measurement)")
    ap.add_argument("--mixers", default="", help="comma list of sizes (2k, 4k): instead of the default workload, "
                    "run the Kagalorn design beside Qwen3 at equal size and time its kernels one by one")
    ap.add_argument("--mixers-design", default="kagalorn", choices=("kagalorn", "bokulorn", "givozen", "bisuzen"),
                    help="with --mixers: kagalorn (beside Qwen3), bokulorn (beside Kagalorn, its closest relative) or "
                         "givozen (beside Bokulorn, its closest relative) or bisuzen (beside Givozen, its closest relative)")
    ap.add_argument("--mixers-engine-only", action="store_true",
                    help="with --mixers-design bisuzen: only that design's engine runs (eager and from graphs), for a profiler")
    ap.add_argument("--mixers-batch", type=int, default=16)
    ap.add_argument("--mixers-prompt", type=int, default=1024)
    ap.add_argument("--mixers-new", type=int, default=17)
    args = ap.parse_args()
    if args.mixers and args.mixers_design == "bisuzen":
        return bisuzen_leg([x for x in args.mixers.split(",") if x], args.mixers_batch, args.mixers_prompt, args.mixers_new,
                           args.mixers_engine_only)
    if args.mixers and args.mixers_design == "givozen":
        return givozen_leg([x for x in args.mixers.split(",") if x], args.mixers_batch, args.mixers_prompt, args.mixers_new)
    if args.mixers and args.mixers_design == "bokulorn":
        return bokulorn_leg([x for x in args.mixers.split(",") if x], args.mixers_batch, args.mixers_prompt, args.mixers_new)
    if args.mixers:
        return mixers_leg([x for x in args.mixers.split(",") if x], args.mixers_batch, args.mixers_prompt, args.mixers_new)

    aux = set() if args.no_aux else {a for a in args.aux.split(",") if a}
    world = int(os.environ.get("WORLD_SIZE", "1"))
    rank = int(os.environ.get("RANK", "0"))
    local_rank = int(os.environ.get("LOCAL_RANK", "0"))
    n = args.gpus
    if world != n:
        if world == 1 and n > 1:
            raise SystemExit("launch with: python -m torch.distributed.run --nproc-per-node N bench.py --gpus N")
        raise SystemExit(f"--gpus {n} but WORLD_SIZE={world}")
    if C4["hkv"] % n != 0:
        raise SystemExit("--gpus must divide the 8 KV heads (1, 2, 4 or 8)")

    from light_vllm_amd import ops
    import torch.distributed as dist

    dev = torch.device("cuda:0" if args.rehearse else f"cuda:{local_rank}")
    torch.cuda.set_device(dev)
    direct = None
    backend = None
    if n > 1:
        from light_vllm_amd import comm as lvcomm
        os.environ.setdefault("MASTER_ADDR", "127.0.0.1")
        if args.rehearse:
            dist.init_process_group("gloo", world_size=world, rank=rank)
        else:
            dist.init_process_group("nccl", world_size=world, rank=rank, device_id=dev)
        backend = dist.get_backend()
        direct = lvcomm.create_for_group(dev)
        lvcomm.install(direct)

    def sync_all():
        torch.cuda.synchronize()
        if n > 1:
            dist.barrier()
            torch.cuda.synchronize()

    result = {"metric": "paged-decode attn HBM GB/s", "unit": "GB/s", "n_gpus": n, "steps": args.steps,
              "warmup": args.warmup, "higher_is_better": True, "vs_baseline": None, "dtype": "bf16",
              "data": "synthetic (seeded N(0,1) bf16 q/K/V, random physical block permutation)",
              "settle_s": SETTLE_S}

    if n == 1:
        c = C2
        w = DecodeWorkload(ops, dev, c["layers"], c["hq"], c["hkv"], c["batch"], c["ctx"], seed=1234)
        elapsed, _, _ = run_steps(w.step, args.steps, args.warmup, sync_all, use_graph=False)
        value = w.step_bytes * args.steps / elapsed / 1e9
        roof = w.roofline(args.steps, "decode_attn_kernel<2,8>")
        roof["traffic"], roof["traffic_source"] = recorded_traffic("decode_attn_kernel<2", w.decode_bytes)
        result.update({
            "value": round(value, 2), "ms_per_step": round(elapsed / args.steps * 1e3, 4), "scaling": "weak",
            "config": {"workload": f"BASELINE config 2: {c['name']} shapes TP=1: {c['layers']} layers x (store_kvcache + "
                                   f"paged decode), global batch {c['batch']}, ctx {c['ctx']}, block {BLOCK}, "
                                   f"heads {c['hq']}q/{c['hkv']}kv, D={D}, eager launches",
                       "global_batch": c["batch"], "context_len": c["ctx"], "parallelism": "tp1",
                       "decode_splits": w.nsplit},
            "pct_hbm_peak": round(100.0 * roof["frac"], 2), "roofline": roof})
        if not args.no_cpu_baseline:
            result["cpu_baseline"] = cpu_baseline(w)
        w.free()
        # the same launch on Qwen3-8B TP=1 shapes: the matrix-core decode kernel
        c8 = C2_8B
        w8 = DecodeWorkload(ops, dev, c8["layers"], c8["hq"], c8["hkv"], c8["batch"], c8["ctx"], seed=1235)
        el8, _, _ = run_steps(w8.step, max(args.steps // 2, 2), 2, sync_all, use_graph=False)
        r8 = w8.roofline(max(args.steps // 2, 2), "decode_mfma_kernel<4>")
        r8["step_GBs"] = round(w8.step_bytes * max(args.steps // 2, 2) / el8 / 1e9, 2)
        r8["workload"] = (f"{c8['name']} shapes TP=1: {c8['layers']} layers x (store_kvcache + paged decode), batch "
                          f"{c8['batch']}, ctx {c8['ctx']}, heads {c8['hq']}q/{c8['hkv']}kv")
        r8["traffic"], r8["traffic_source"] = recorded_traffic("decode_mfma_kernel<4", w8.decode_bytes)
        result["roofline_8b"] = r8
        w8.free()
    else:
        c = C4
        layers, batch = (4, 8) if args.rehearse else (c["layers"], c["batch"])
        from light_vllm_amd.layers import tp
        w, hidden = tp_step_setup(ops, dev, n, rank, c, layers, batch)
        use_graph = direct is not None or backend == "nccl"
        cpu_or_dev = dev if backend == "nccl" else "cpu"

        def timed_step():
            """(max elapsed over ranks, graph used, note, failed on any rank). A rank whose direct
            all-reduce gives up (bounded waits: every rank's kernels end) reports it instead of
            leaving; the ranks then agree through torch.distributed."""
            failed, el, graphed, note = 0.0, 0.0, False, None
            try:
                el, graphed, note = run_steps(lambda: w.step(after_layer=lambda: tp.all_reduce(hidden)),
                                              args.steps, args.warmup, sync_all, use_graph)
                if direct is not None and lvcomm.active() is not None and direct.failed():
                    raise RuntimeError("direct all-reduce: a peer did not arrive within the timeout")
            except Exception as exc:   # noqa: BLE001
                failed, note = 1.0, f"rank {rank}: {exc!r}"[:300]
                torch.cuda.synchronize()
            t = torch.tensor([el, failed], dtype=torch.float64, device=cpu_or_dev)
            dist.all_reduce(t, op=dist.ReduceOp.MAX)
            return float(t[0].item()), graphed, note, bool(t[1].item() > 0)

        elapsed, graphed, note, bad = timed_step()
        direct_fell_back = False
        if bad and direct is not None and backend == "nccl":
            # the direct transport failed on some rank: time the same step on RCCL instead
            lvcomm.install(None)
            direct_fell_back = True
            hidden.fill_(1.0)
            elapsed, graphed, note2, bad = timed_step()
            note = f"direct all-reduce failed ({note}); re-timed on RCCL" + (f"; {note2}" if note2 else "")
        if bad:
            raise SystemExit(f"bench: the timed step failed on some rank: {note}")
        value = n * w.step_bytes * args.steps / elapsed / 1e9
        kern = "decode_mfma_kernel<4>"
        roof = w.roofline(2, kern)
        msg = batch * c["hidden"] * 2
        result.update({
            "value": round(value, 2), "ms_per_step": round(elapsed / args.steps * 1e3, 4), "scaling": "strong",
            "config": {"workload": f"BASELINE config 4: {c['name']} shapes TP={n}: {layers} layers x (store_kvcache + "
                                   f"paged decode + all-reduce of [{batch}, {c['hidden']}] bf16), global batch {batch}, "
                                   f"ctx {c['ctx']}, block table [{batch}, {c['ctx'] // BLOCK}], per-rank heads "
                                   f"{w.Hq}q/{w.Hkv}kv, D={D}, " + ("hipGraph replay" if graphed else "eager launches"),
                       "global_batch": batch, "context_len": c["ctx"], "parallelism": f"tp{n}",
                       "decode_splits": w.nsplit, "hipgraph": graphed, "rehearsal": bool(args.rehearse),
                       "all_reduce": "direct (lv_comm over IPC-mapped peer buffers)"
                                     if direct is not None and not direct_fell_back else backend,
                       "all_reduce_bytes": msg,
                       "all_reduce_algorithm": direct.algorithm_for(msg)
                                               if direct is not None and not direct_fell_back else None,
                       "one_shot_inflow_bytes": direct.one_shot_inflow if direct is not None else None},
            "rccl_ranks": dist.get_world_size(), "dist_backend": backend,
            "pct_hbm_peak": round(100.0 * roof["frac"], 2), "roofline": roof})
        if note:
            result["config"]["graph_note"] = note
        if direct is not None and (direct_fell_back or direct.failed()):
            result["comm_failed"] = True
        del hidden
        w.free()

    t_aux = time.perf_counter()
    if rank == 0 and "prefill" in aux:
        try:
            result["prefill"] = prefill_leg(ops, dev, n)
            burn = sustained_mfma_peak()
            if burn:
                result["prefill"]["sustained_mfma"] = burn
                result["prefill"]["frac_of_sustained"] = round(result["prefill"]["tflops"] / burn["tflops"], 4)
            if n == 1:
                rp = recorded_prefill_counters()
                if rp:
                    result["prefill"]["rocprof"] = rp
        except Exception as exc:   # reported, never fatal for the headline number
            result["prefill"] = {"error": repr(exc)[:300]}
    if n == 1 and "variants" in aux:
        result["variants"] = variants_leg(ops, dev, sync_all)
    scale_base = None
    if "config4" in aux and (n == 1 or rank == 0):
        # the multi-GPU step at TP=1 (no all-reduce): the base of the strong-scaling curve
        # (a rehearsal keeps its reduced size: 4 layers, batch 8)
        try:
            l4, b4 = (4, 8) if args.rehearse else (C4["layers"], C4["batch"])
            w4, _ = tp_step_setup(ops, dev, 1, 0, C4, l4, b4)
            el4, graphed, note = run_steps(w4.step, 5, 2, lambda: torch.cuda.synchronize(), use_graph=True)
            r4 = w4.roofline(1, "decode_mfma_kernel<4>")
            r4["traffic"], r4["traffic_source"] = recorded_traffic("decode_mfma_kernel<4", w4.decode_bytes)
            result["config4_tp1"] = {"workload": f"BASELINE config 4 at TP=1: {l4} layers x (store_kvcache + paged "
                                                 f"decode), batch {b4}, ctx {C4['ctx']}, heads {C4['hq']}q/{C4['hkv']}kv",
                                     "value": round(w4.step_bytes * 5 / el4 / 1e9, 2), "unit": "GB/s",
                                     "ms_per_step": round(el4 / 5 * 1e3, 4), "hipgraph": graphed, "roofline": r4}
            scale_base = result["config4_tp1"]
            w4.free()
        except Exception as exc:
            result["config4_tp1"] = {"error": repr(exc)[:300]}
    if n > 1:
        sync_all()      # the other ranks wait here (process-group barrier) while rank 0 measures the TP = 1 base
    # One workload whose numbers are comparable at every N: BASELINE config 4 (global batch 32 at 32k
    # context) at TP = N. N = 1: the leg above; N > 1: the headline itself, beside the TP = 1 step
    # measured by rank 0 of this same run.
    if n == 1 and scale_base is not None:
        result.update(scale_value=scale_base["value"], scale_ms_per_step=scale_base["ms_per_step"])
    elif n > 1:
        result.update(scale_value=result["value"], scale_ms_per_step=result["ms_per_step"])
    if "scale_value" in result:
        result["scale_workload"] = (f"BASELINE config 4: Qwen3-8B shapes, global batch {8 if args.rehearse else C4['batch']}, "
                                    f"ctx {C4['ctx']}, TP={n}, hipGraph replay" + (" (rehearsal size)" if args.rehearse else ""))
        if scale_base is not None:
            result["scale_base_ms_per_step"] = scale_base["ms_per_step"]
            result["scale_efficiency"] = round(scale_base["ms_per_step"] / (n * result["scale_ms_per_step"]), 4)
    if n > 1 and "collectives" in aux:
        try:
            result["collectives"] = collectives_leg(dist, dev, n, None if direct_fell_back else direct)
        except Exception as exc:
            result["collectives"] = {"error": repr(exc)[:300]}
    torch.cuda.empty_cache()
    if n > 1:
        from light_vllm_amd import comm as lvcomm
        dist.barrier()
        lvcomm.install(None)
        if direct is not None:
            direct.close()
        dist.destroy_process_group()
    if rank == 0 and "e2e" in aux and not args.rehearse:
        # every bench rank has released its GPU memory; the engine starts its own one process per GPU
        port = int(os.environ.get("MASTER_PORT", "29500")) + 17
        legs = [e2e_leg(n, port, "eager", 150)]
        if "error" not in legs[0]:
            legs.append(e2e_leg(n, port + 1, "graph", 150))
            if n == 1 and "error" not in legs[-1] and os.path.exists(TUNED_GEMMS.replace(".csv", "0.csv")):
                legs.append(e2e_leg(n, port + 2, "graph", 120, tuned_gemms=True))
        result["e2e"] = {"what": "tools/e2e_bench.py: engine generate(), Qwen3-8B shapes, random weights, "
                                 f"TP={n}, batch 256 x 1024-token prompts, 33 new tokens, greedy",
                         "runs": legs}
        result["e2e_failed"] = any("error" in leg for leg in legs)
        result["aux_seconds"] = round(time.perf_counter() - t_aux, 1)
    if rank == 0:
        print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
