// Sliding-window attention with pooled blocks over a paged cache.
//
//   qk_fullnorm_store_kernel  one workgroup per token: RMS norm over the whole q projection and the whole k
//                             projection (before they are split into heads), K and V rows scattered into the cache.
//   pool_update_kernel        one workgroup per (sequence, block completed by this step): mean of its P cached
//                             keys and values, stored with the page of the block's last token.
//   window_pool_attn_kernel   one workgroup per (token, kv head, group of up to 8 query heads; 4 for value sizes above 256). The key list of a
//                             query is [pooled blocks wholly before the window | tokens of the window]; the four
//                             waves take 64-key chunks in turn (lane = key for the scores, lane = value column
//                             for the weighted sum), each with its own running maximum, and merge in LDS. The
//                             sink is one more term exp(0 - m) of the denominator, owned by wave 0.
#include "mix_common.h"

namespace lvmix {

template <typename T>
__global__ __launch_bounds__(256) void qk_fullnorm_store_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t ld,
    const float* __restrict__ q_w, const float* __restrict__ k_w, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int32_t* __restrict__ cu_q, const int32_t* __restrict__ ctx_lens,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ block_tables, int bt_stride, int HD, int GD,
    int GDv, int page, float eps) {
  __shared__ float red[2][4];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int b = tok_seq[t];
  const int pos = ctx_lens[b] + static_cast<int>(t) - cu_q[b];
  const int64_t slot = static_cast<int64_t>(block_tables[static_cast<int64_t>(b) * bt_stride + pos / page]) * page + pos % page;
  float sq = 0.0f, sk = 0.0f;
  for (int i = threadIdx.x; i < HD; i += blockDim.x) {
    const float x = ldf(q + t * ld + i);
    sq += x * x;
  }
  for (int i = threadIdx.x; i < GD; i += blockDim.x) {
    const float x = ldf(k + t * ld + i);
    sk += x * x;
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (lane == 0) {
    red[0][wave] = sq;
    red[1][wave] = sk;
  }
  __syncthreads();
  const float inv_q = 1.0f / sqrtf((red[0][0] + red[0][1] + red[0][2] + red[0][3]) / static_cast<float>(HD) + eps);
  const float inv_k = 1.0f / sqrtf((red[1][0] + red[1][1] + red[1][2] + red[1][3]) / static_cast<float>(GD) + eps);
  for (int i = threadIdx.x; i < HD; i += blockDim.x) stf(q_out + t * HD + i, ldf(q + t * ld + i) * inv_q * q_w[i]);
  for (int i = threadIdx.x; i < GD; i += blockDim.x) stf(k_cache + slot * GD + i, ldf(k + t * ld + i) * inv_k * k_w[i]);
  for (int i = threadIdx.x; i < GDv; i += blockDim.x) v_cache[slot * GDv + i] = v[t * ld + i];
}

template <typename T>
__global__ __launch_bounds__(256) void pool_update_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                          T* __restrict__ kp, T* __restrict__ vp,
                                                          const int32_t* __restrict__ cu_q,
                                                          const int32_t* __restrict__ ctx_lens,
                                                          const int32_t* __restrict__ block_tables, int bt_stride,
                                                          int GD, int GDv, int page, int P, int PP) {
  const int b = blockIdx.y;
  const int ctx = ctx_lens[b], n = cu_q[b + 1] - cu_q[b];
  const int blk = ctx / P + blockIdx.x;                 // blocks complete before the step: floor(ctx / P)
  if (blk >= (ctx + n) / P) return;
  const int32_t* bt = block_tables + static_cast<int64_t>(b) * bt_stride;
  const int last = blk * P + P - 1;
  const int pj = last / page;
  const int64_t dst = static_cast<int64_t>(bt[pj]) * PP + (blk - (page * pj) / P);
  const float invP = 1.0f / static_cast<float>(P);
  for (int i = threadIdx.x; i < GD + GDv; i += blockDim.x) {
    float acc = 0.0f;
    for (int j = blk * P; j <= last; ++j) {
      const int64_t slot = static_cast<int64_t>(bt[j / page]) * page + j % page;
      acc += i < GD ? ldf(k_cache + slot * GD + i) : ldf(v_cache + slot * GDv + (i - GD));
    }
    if (i < GD) stf(kp + dst * GD + i, acc * invP);
    else stf(vp + dst * GDv + (i - GD), acc * invP);
  }
}

struct WindowAttnParams {
  const void *q, *k_cache, *v_cache, *kp, *vp, *gate;
  int64_t ld_gate;
  int gate_dv;          // entries of a gate row per head: Dv (one per output channel) or 1 (one per head)
  void* out;
  const int32_t *cu_q, *ctx_lens, *tok_seq, *block_tables;
  int bt_stride, H, G, D, Dv, page, window, P, PP;
  float scale, sink;
  int64_t k_ld, v_ld;   // elements between the rows of two cached tokens (G*D and G*Dv unless the caches are views of wider rows)
  float m0;             // where the running maximum starts: the sink's score 0, or far below any score without a sink
  int keep_first;       // positions below this are seen from everywhere (with their own keys and values)
  int chunk;            // > 0: a query sees its own chunk of that many positions (counted from 0) up to itself; no window
  const float* sinks;   // [H] or NULL: a learned score per query head in place of the sink's 0
};

// kMaxRep: query heads of one kv head served by one workgroup; kMaxDvi: value columns per lane (Dv <= 64 * kMaxDvi).
// Instantiated for (8, 4): value sizes up to 256, and (4, 8): up to 512 with half the heads per workgroup.
template <typename T, int kMaxRep, int kMaxDvi>
__global__ __launch_bounds__(256) void window_pool_attn_kernel(WindowAttnParams p) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t t = blockIdx.x;
  const int g = blockIdx.y;
  const int rep_all = p.H / p.G;
  const int h0 = g * rep_all + blockIdx.z * kMaxRep;                 // first query head of this workgroup
  const int rep = min(kMaxRep, rep_all - static_cast<int>(blockIdx.z) * kMaxRep);
  const int D = p.D, Dv = p.Dv;
  float* q_lds = lds;                                   // [kMaxRep][D], scaled
  float* p_lds = q_lds + kMaxRep * D;                   // [4][kMaxRep][64]
  float* o_lds = p_lds + 4 * kMaxRep * kWave;           // [4][kMaxRep][Dv]
  float* ml_lds = o_lds + 4 * kMaxRep * Dv;             // [4][kMaxRep][2]

  const T* q = static_cast<const T*>(p.q) + t * p.H * D;
  for (int i = threadIdx.x; i < rep * D; i += blockDim.x) q_lds[i] = ldf(q + static_cast<int64_t>(h0) * D + i) * p.scale;
  __syncthreads();

  const int b = p.tok_seq[t];
  const int pos = p.ctx_lens[b] + static_cast<int>(t) - p.cu_q[b];
  const int32_t* bt = p.block_tables + static_cast<int64_t>(b) * p.bt_stride;
  const int j0 = p.chunk > 0 ? (pos / p.chunk) * p.chunk : max(0, pos - p.window + 1);
  const int nw = pos - j0 + 1;
  const int nb = (p.P > 0 && p.chunk == 0 && pos - p.window + 1 > 0) ? (pos - p.window + 1) / p.P : 0;
  const int nf = min(p.keep_first, j0);                 // kept first tokens that lie before the window
  const int nkeys = nb + nf + nw;                       // [pooled blocks | kept first tokens | window]
  const int GD = p.G * D, GDv = p.G * Dv;
  const T* kc = static_cast<const T*>(p.k_cache);
  const T* vc = static_cast<const T*>(p.v_cache);
  const T* kpool = static_cast<const T*>(p.kp);
  const T* vpool = static_cast<const T*>(p.vp);

  float m[kMaxRep], l[kMaxRep], o[kMaxRep][kMaxDvi];
#pragma unroll
  for (int h = 0; h < kMaxRep; ++h) {
    m[h] = (p.sinks != nullptr && h < rep) ? p.sinks[h0 + h] : p.m0;   // with a sink: never below its score
    l[h] = wave == 0 ? p.sink : 0.0f;
#pragma unroll
    for (int e = 0; e < kMaxDvi; ++e) o[h][e] = 0.0f;
  }
  float* pw = p_lds + wave * kMaxRep * kWave;

  for (int c0 = wave * kWave; c0 < nkeys; c0 += 4 * kWave) {
    const int idx = c0 + lane;
    const bool valid = idx < nkeys;
    // row of this lane's key in its cache
    const T* krow = kc;
    if (valid) {
      if (idx < nb) {
        const int pj = (idx * p.P + p.P - 1) / p.page;
        krow = kpool + (static_cast<int64_t>(bt[pj]) * p.PP + (idx - (p.page * pj) / p.P)) * GD + g * D;
      } else {
        const int j = idx < nb + nf ? idx - nb : j0 + idx - nb - nf;
        krow = kc + (static_cast<int64_t>(bt[j / p.page]) * p.page + j % p.page) * p.k_ld + g * D;
      }
    }
    float s[kMaxRep];
#pragma unroll
    for (int h = 0; h < kMaxRep; ++h) s[h] = 0.0f;
    if (valid) {
      for (int d = 0; d < D; ++d) {
        const float kd = ldf(krow + d);
#pragma unroll
        for (int h = 0; h < kMaxRep; ++h)
          if (h < rep) s[h] += kd * q_lds[h * D + d];
      }
    }
#pragma unroll
    for (int h = 0; h < kMaxRep; ++h) {
      if (h < rep) {
        const float cm = wave_max(valid ? s[h] : -INFINITY);
        const float nm = fmaxf(m[h], cm);
        const float corr = expf(m[h] - nm);
        const float e = valid ? expf(s[h] - nm) : 0.0f;
        l[h] = l[h] * corr + wave_sum(e);
        m[h] = nm;
#pragma unroll
        for (int x = 0; x < kMaxDvi; ++x) o[h][x] *= corr;
        pw[h * kWave + lane] = e;
      }
    }
    // lanes turn to value columns; the chunk's keys are walked by all of them together
    const int cn = min(kWave, nkeys - c0);
    for (int jj = 0; jj < cn; ++jj) {
      const int id2 = c0 + jj;
      const T* vrow;
      if (id2 < nb) {
        const int pj = (id2 * p.P + p.P - 1) / p.page;
        vrow = vpool + (static_cast<int64_t>(bt[pj]) * p.PP + (id2 - (p.page * pj) / p.P)) * GDv + g * Dv;
      } else {
        const int j = id2 < nb + nf ? id2 - nb : j0 + id2 - nb - nf;
        vrow = vc + (static_cast<int64_t>(bt[j / p.page]) * p.page + j % p.page) * p.v_ld + g * Dv;
      }
#pragma unroll
      for (int x = 0; x < kMaxDvi; ++x) {
        const int dv = x * kWave + lane;
        if (dv < Dv) {
          const float vv = ldf(vrow + dv);
#pragma unroll
          for (int h = 0; h < kMaxRep; ++h)
            if (h < rep) o[h][x] += pw[h * kWave + jj] * vv;
        }
      }
    }
  }
  // merge the four waves
#pragma unroll
  for (int h = 0; h < kMaxRep; ++h) {
    if (h < rep) {
      if (lane == 0) {
        ml_lds[(wave * kMaxRep + h) * 2] = m[h];
        ml_lds[(wave * kMaxRep + h) * 2 + 1] = l[h];
      }
#pragma unroll
      for (int x = 0; x < kMaxDvi; ++x) {
        const int dv = x * kWave + lane;
        if (dv < Dv) o_lds[(wave * kMaxRep + h) * Dv + dv] = o[h][x];
      }
    }
  }
  __syncthreads();
  T* out = static_cast<T*>(p.out) + t * p.H * Dv;
  const T* gate = p.gate != nullptr ? static_cast<const T*>(p.gate) + t * p.ld_gate : nullptr;
  for (int i = threadIdx.x; i < rep * Dv; i += blockDim.x) {
    const int h = i / Dv, dv = i - h * Dv;
    float mm = p.sinks != nullptr ? p.sinks[h0 + h] : p.m0;
    for (int w = 0; w < 4; ++w) mm = fmaxf(mm, ml_lds[(w * kMaxRep + h) * 2]);
    float ll = 0.0f, acc = 0.0f;
    for (int w = 0; w < 4; ++w) {
      const float c = expf(ml_lds[(w * kMaxRep + h) * 2] - mm);
      ll += ml_lds[(w * kMaxRep + h) * 2 + 1] * c;
      acc += o_lds[(w * kMaxRep + h) * Dv + dv] * c;
    }
    float r = ll > 0.0f ? acc / ll : 0.0f;
    if (gate != nullptr) r *= sigmoidf_(ldf(gate + static_cast<int64_t>(h0 + h) * p.gate_dv + (p.gate_dv > 1 ? dv : 0)));
    stf(out + static_cast<int64_t>(h0 + h) * Dv + dv, r);
  }
}

}  // namespace lvmix

using namespace lvmix;

extern "C" {

int lv_qk_fullnorm_store(const void* q, const void* k, const void* v, int64_t ld, const void* q_w, const void* k_w,
                         void* q_out, void* k_cache, void* v_cache, const int32_t* cu_q, const int32_t* ctx_lens,
                         const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int H, int G,
                         int D, int Dv, int page, float eps, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!q || !k || !v || !q_w || !k_w || !q_out || !k_cache || !v_cache || !cu_q || !ctx_lens || !tok_seq || !block_tables)
    return fail(-1, "lv_qk_fullnorm_store: null pointer");
  if (T < 0 || H <= 0 || G <= 0 || H % G != 0 || D <= 0 || Dv <= 0 || page <= 0 || bt_stride <= 0)
    return fail(-1, "lv_qk_fullnorm_store: bad sizes");
  dim3 grid(static_cast<unsigned>(T)), block(256);
  if (dtype == LV_MIX_BF16)
    qk_fullnorm_store_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k), static_cast<const bf16_t*>(v), ld,
        static_cast<const float*>(q_w), static_cast<const float*>(k_w), static_cast<bf16_t*>(q_out),
        static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), cu_q, ctx_lens, tok_seq, block_tables, bt_stride,
        H * D, G * D, G * Dv, page, eps);
  else if (dtype == LV_MIX_F32)
    qk_fullnorm_store_kernel<float><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(q), static_cast<const float*>(k), static_cast<const float*>(v), ld,
        static_cast<const float*>(q_w), static_cast<const float*>(k_w), static_cast<float*>(q_out),
        static_cast<float*>(k_cache), static_cast<float*>(v_cache), cu_q, ctx_lens, tok_seq, block_tables, bt_stride,
        H * D, G * D, G * Dv, page, eps);
  else
    return fail(-1, "lv_qk_fullnorm_store: dtype %d", dtype);
  return launched("lv_qk_fullnorm_store");
}

int lv_pool_update(const void* k_cache, const void* v_cache, void* kp, void* vp, const int32_t* cu_q,
                   const int32_t* ctx_lens, const int32_t* block_tables, int bt_stride, int B, int max_new_blocks, int G,
                   int D, int Dv, int page, int P, int dtype, void* stream) {
  if (B == 0 || max_new_blocks <= 0 || P <= 0) return 0;
  if (!k_cache || !v_cache || !kp || !vp || !cu_q || !ctx_lens || !block_tables)
    return fail(-1, "lv_pool_update: null pointer");
  if (B < 0 || G <= 0 || D <= 0 || Dv <= 0 || page <= 0 || bt_stride <= 0) return fail(-1, "lv_pool_update: bad sizes");
  const int PP = (page + P - 1) / P;
  dim3 grid(max_new_blocks, B), block(256);
  if (dtype == LV_MIX_BF16)
    pool_update_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const bf16_t*>(k_cache), static_cast<const bf16_t*>(v_cache), static_cast<bf16_t*>(kp),
        static_cast<bf16_t*>(vp), cu_q, ctx_lens, block_tables, bt_stride, G * D, G * Dv, page, P, PP);
  else if (dtype == LV_MIX_F32)
    pool_update_kernel<float><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(k_cache), static_cast<const float*>(v_cache), static_cast<float*>(kp),
        static_cast<float*>(vp), cu_q, ctx_lens, block_tables, bt_stride, G * D, G * Dv, page, P, PP);
  else
    return fail(-1, "lv_pool_update: dtype %d", dtype);
  return launched("lv_pool_update");
}

int lv_window_pool_attn(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                        const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                        const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int H, int G, int D,
                        int Dv, int page, int window, int P, float scale, int has_sink, int64_t k_ld, int64_t v_ld,
                        int gate_kind, int dtype, void* stream) {
  return lv_masked_attn(q, k_cache, v_cache, kp, vp, gate, ld_gate, out, cu_q, ctx_lens, tok_seq, block_tables, bt_stride, T, H,
                        G, D, Dv, page, window, 0, 0, P, scale, has_sink, nullptr, k_ld, v_ld, gate_kind, dtype, stream);
}

int lv_masked_attn(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                   const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                   const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int H, int G, int D,
                   int Dv, int page, int window, int keep_first, int chunk, int P, float scale, int has_sink,
                   const void* sinks, int64_t k_ld, int64_t v_ld, int gate_kind, int dtype, void* stream) {
  if (T == 0) return 0;
  if (keep_first < 0 || chunk < 0 || (P > 0 && (keep_first > 0 || chunk > 0)))
    return fail(-1, "lv_masked_attn: kept first tokens and chunks do not combine with pooled blocks");
  if (sinks != nullptr) has_sink = 1;
  if (!q || !k_cache || !v_cache || !out || !cu_q || !ctx_lens || !tok_seq || !block_tables)
    return fail(-1, "lv_window_pool_attn: null pointer");
  if (k_ld <= 0) k_ld = static_cast<int64_t>(G) * D;
  if (v_ld <= 0) v_ld = static_cast<int64_t>(G) * Dv;
  if (k_ld < static_cast<int64_t>(G) * D || v_ld < static_cast<int64_t>(G) * Dv) return fail(-1, "lv_window_pool_attn: row strides");
  if (P > 0 && (!kp || !vp)) return fail(-1, "lv_window_pool_attn: pooled blocks without their cache");
  if (T < 0 || H <= 0 || G <= 0 || H % G != 0 || D <= 0 || Dv <= 0 || page <= 0 || window <= 0 || bt_stride <= 0)
    return fail(-1, "lv_window_pool_attn: bad sizes");
  if (Dv > 8 * kWave) return fail(-2, "lv_window_pool_attn: value size %d above %d", Dv, 8 * kWave);
  if (gate_kind != LV_MIX_GATE_PER_HEAD && gate_kind != LV_MIX_GATE_PER_CHANNEL)
    return fail(-1, "lv_window_pool_attn: gate kind %d", gate_kind);
  const int gate_dv = gate_kind == LV_MIX_GATE_PER_HEAD ? 1 : Dv;
  if (gate != nullptr && ld_gate < static_cast<int64_t>(H) * gate_dv) return fail(-1, "lv_window_pool_attn: gate stride");
  const bool wide = Dv > 4 * kWave;
  const int kMaxRep = wide ? 4 : 8;
  const int rep = H / G;
  WindowAttnParams p{q, k_cache, v_cache, kp, vp, gate, ld_gate, gate_dv, out, cu_q, ctx_lens, tok_seq, block_tables,
                     bt_stride, H, G, D, Dv, page, window, P, P > 0 ? (page + P - 1) / P : 0, scale,
                     has_sink ? 1.0f : 0.0f, k_ld, v_ld, has_sink ? 0.0f : -1e30f, keep_first, chunk,
                     static_cast<const float*>(sinks)};
  const size_t shm = sizeof(float) * (static_cast<size_t>(kMaxRep) * D + 4 * kMaxRep * kWave +
                                      4 * static_cast<size_t>(kMaxRep) * Dv + 4 * kMaxRep * 2);
  if (shm > 64 * 1024) return fail(-2, "lv_window_pool_attn: head sizes %d / %d need %zu bytes of LDS", D, Dv, shm);
  dim3 grid(static_cast<unsigned>(T), G, (rep + kMaxRep - 1) / kMaxRep), block(256);
  if (dtype != LV_MIX_BF16 && dtype != LV_MIX_F32) return fail(-1, "lv_window_pool_attn: dtype %d", dtype);
  if (dtype == LV_MIX_BF16) {
    if (wide) window_pool_attn_kernel<bf16_t, 4, 8><<<grid, block, shm, as_stream(stream)>>>(p);
    else window_pool_attn_kernel<bf16_t, 8, 4><<<grid, block, shm, as_stream(stream)>>>(p);
  } else {
    if (wide) window_pool_attn_kernel<float, 4, 8><<<grid, block, shm, as_stream(stream)>>>(p);
    else window_pool_attn_kernel<float, 8, 4><<<grid, block, shm, as_stream(stream)>>>(p);
  }
  return launched("lv_window_pool_attn");
}

}  // extern "C"
