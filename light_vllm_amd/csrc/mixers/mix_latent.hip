// Latent attention around the paged attention kernel, and the mixture-of-experts router.
//
// Latent attention caches one row per token, [latent c (R) | rotated positional key part (Dr)], shared by all query
// heads. With the key up-projection multiplied into the query and the value up-projection applied after the weighted
// sum, every head attends to those rows directly: keys are the whole row, values its first R entries. The attention
// itself is the paged kernel of mix_window_attn.hip / mix_window_mfma.hip with one kv head and row strides; here are
// the steps either side of it.
//
//   latent_prep_kernel      one workgroup per token: RMS norm of the query latent; RMS norm of the key/value latent and
//                           rotation of the positional key part, both written into the token's cache row.
//   latent_q_finish_kernel  one workgroup per token: [absorbed query | rotated positional query part] per head.
//   latent_out_gate_kernel  elementwise: head-major outputs to token-major rows times sigmoid(gate).
//   moe_route_kernel        one wave per token: sigmoid scores, correction for the choice only, group limit, top-k,
//                           normalised (or raw) weights; the wave keeps its scores in LDS and picks maxima by shuffles.
//   router_logits_kernel    steps of few tokens: the f32 router logits straight from the activations, one workgroup per
//                           (token, four experts).
//   relu2_scale_kernel      elementwise: relu(x)^2 times the token's weight for the expert the column belongs to.
#include "mix_common.h"

namespace lvmix {

// Rotation of entry j (< rot_dims) of a vector x whose first rot_dims entries are paired (i, i + rot_dims/2).
// cs: [half] cosines then [half] sines of this token's angles.
template <typename T>
__device__ __forceinline__ float rotated(const T* x, int j, int half, const float* cs) {
  if (j >= 2 * half) return ldf(x + j);
  if (j < half) return ldf(x + j) * cs[j] - ldf(x + j + half) * cs[half + j];
  return ldf(x + j) * cs[j - half] + ldf(x + j - half) * cs[half + j - half];
}

__device__ __forceinline__ void fill_angles(float* cs, const float* inv_freq, int half, int pos) {
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float a = static_cast<float>(pos) * inv_freq[i];
    float s, c;
    sincosf(a, &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const T* __restrict__ proj, int64_t ld, int off_q, int off_kv,
                                                          const float* __restrict__ q_w, const float* __restrict__ kv_w,
                                                          const float* __restrict__ inv_freq, T* __restrict__ cq_out,
                                                          T* __restrict__ cache, const int32_t* __restrict__ cu_q,
                                                          const int32_t* __restrict__ ctx_lens,
                                                          const int32_t* __restrict__ tok_seq,
                                                          const int32_t* __restrict__ block_tables, int bt_stride, int Rq,
                                                          int R, int Dr, int rot_dims, int page, float eps) {
  extern __shared__ float cs[];                    // [rot_dims] cosines | sines
  __shared__ float red[2][4];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int b = tok_seq[t];
  const int pos = ctx_lens[b] + static_cast<int>(t) - cu_q[b];
  const int64_t slot = static_cast<int64_t>(block_tables[static_cast<int64_t>(b) * bt_stride + pos / page]) * page + pos % page;
  const T* row = proj + t * ld;
  const int half = rot_dims / 2;
  fill_angles(cs, inv_freq, half, pos);
  float sq = 0.0f, sk = 0.0f;
  for (int i = threadIdx.x; i < Rq; i += blockDim.x) {
    const float x = ldf(row + off_q + i);
    sq += x * x;
  }
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float x = ldf(row + off_kv + i);
    sk += x * x;
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (lane == 0) {
    red[0][wave] = sq;
    red[1][wave] = sk;
  }
  __syncthreads();
  const float inv_q = 1.0f / sqrtf((red[0][0] + red[0][1] + red[0][2] + red[0][3]) / static_cast<float>(Rq) + eps);
  const float inv_k = 1.0f / sqrtf((red[1][0] + red[1][1] + red[1][2] + red[1][3]) / static_cast<float>(R) + eps);
  for (int i = threadIdx.x; i < Rq; i += blockDim.x) stf(cq_out + t * Rq + i, ldf(row + off_q + i) * inv_q * q_w[i]);
  T* crow = cache + slot * (R + Dr);
  for (int i = threadIdx.x; i < R; i += blockDim.x) stf(crow + i, ldf(row + off_kv + i) * inv_k * kv_w[i]);
  for (int j = threadIdx.x; j < Dr; j += blockDim.x) stf(crow + R + j, rotated(row + off_kv + R, j, half, cs));
}

template <typename T>
__global__ __launch_bounds__(256) void latent_q_finish_kernel(const T* __restrict__ q, const T* __restrict__ q_lat,
                                                              const float* __restrict__ inv_freq, T* __restrict__ q_out,
                                                              const int32_t* __restrict__ cu_q,
                                                              const int32_t* __restrict__ ctx_lens,
                                                              const int32_t* __restrict__ tok_seq, int64_t Tn, int H, int Dn,
                                                              int Dr, int R, int rot_dims) {
  extern __shared__ float cs[];
  const int64_t t = blockIdx.x;
  const int half = rot_dims / 2;
  if (Dr > 0) {
    const int b = tok_seq[t];
    fill_angles(cs, inv_freq, half, ctx_lens[b] + static_cast<int>(t) - cu_q[b]);
    __syncthreads();
  }
  const int Dk = R + Dr;
  for (int i = threadIdx.x; i < H * Dk; i += blockDim.x) {
    const int h = i / Dk, c = i - h * Dk;
    T* dst = q_out + (t * H + h) * Dk + c;
    if (c < R) *dst = q_lat[(static_cast<int64_t>(h) * Tn + t) * R + c];
    else stf(dst, rotated(q + (t * H + h) * (Dn + Dr) + Dn, c - R, half, cs));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void latent_out_gate_kernel(const T* __restrict__ o, const T* __restrict__ gate,
                                                              int64_t ld_gate, int per_channel, T* __restrict__ out,
                                                              int64_t Tn, int H, int Dv) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t HD = static_cast<int64_t>(H) * Dv;
  if (idx >= Tn * HD) return;
  const int64_t t = idx / HD;
  const int c = static_cast<int>(idx - t * HD);
  const int h = c / Dv, d = c - h * Dv;
  const float g = ldf(gate + t * ld_gate + (per_channel ? c : h));
  stf(out + idx, ldf(o + (static_cast<int64_t>(h) * Tn + t) * Dv + d) * sigmoidf_(g));
}

// ------------------------------------------------------------------------------------------------
// (value, index) maximum over the wave: larger value wins, the lower index on equal values.
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, kWave);
    const int oi = __shfl_xor(i, o, kWave);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                                                        int32_t* __restrict__ ids, float* __restrict__ weights,
                                                        float* __restrict__ dense, int E, int top, int groups, int keep,
                                                        int normalize, int score_kind, int group_rank) {
  extern __shared__ float rl[];
  float* s_lds = rl;              // [E] scores
  float* c_lds = rl + E;          // [E] selection scores, -inf once out of the running
  float* g_lds = rl + 2 * E;      // [groups] group scores
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  float smax = -INFINITY, sden = 1.0f;
  if (score_kind == LV_MIX_SCORE_SOFTMAX) {            // over all experts of the row
    for (int e = lane; e < E; e += kWave) smax = fmaxf(smax, logits[t * E + e]);
    smax = wave_max(smax);
    float part = 0.0f;
    for (int e = lane; e < E; e += kWave) part += expf(logits[t * E + e] - smax);
    sden = wave_sum(part);
  }
  for (int e = lane; e < E; e += kWave) {
    const float s = score_kind == LV_MIX_SCORE_SOFTMAX ? expf(logits[t * E + e] - smax) / sden : sigmoidf_(logits[t * E + e]);
    s_lds[e] = s;
    c_lds[e] = s + (correction != nullptr ? correction[e] : 0.0f);
    if (dense != nullptr) dense[t * E + e] = 0.0f;
  }
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int gs = E / groups;
    for (int g = lane; g < groups; g += kWave) {
      float a = -INFINITY, b2 = -INFINITY;          // the two highest
      for (int e = g * gs; e < (g + 1) * gs; ++e) {
        const float c = c_lds[e];
        if (c > a) { b2 = a; a = c; }
        else if (c > b2) b2 = c;
      }
      g_lds[g] = (gs > 1 && group_rank == LV_MIX_GROUP_TOP2_SUM) ? a + b2 : a;
    }
    __syncthreads();
    // the `keep` best groups: their score is marked +inf, everything else leaves the choice
    for (int r = 0; r < keep; ++r) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < groups; g += kWave) {
        const float v = g_lds[g];
        if (v != INFINITY && (v > bv || bi == 0x7fffffff)) { bv = v; bi = g; }
      }
      wave_argmax(bv, bi);
      if (lane == 0 && bi != 0x7fffffff) g_lds[bi] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < E; e += kWave)
      if (g_lds[e / gs] != INFINITY) c_lds[e] = -INFINITY;
    __syncthreads();
  }
  float wsum = 0.0f;
  float mine = 0.0f;              // lane k keeps the score of the k-th choice (top <= 64)
  int mine_id = 0;
  for (int r = 0; r < top; ++r) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += kWave) {
      const float v = c_lds[e];
      if (v > bv) { bv = v; bi = e; }
    }
    wave_argmax(bv, bi);
    if (bi == 0x7fffffff) bi = 0;                  // fewer experts in the running than asked for
    const float s = s_lds[bi];
    wsum += s;
    if (lane == r) { mine = s; mine_id = bi; }
    __syncthreads();
    if (lane == 0) c_lds[bi] = -INFINITY;
    __syncthreads();
  }
  if (lane < top) {
    const float w = normalize ? mine / (wsum + 1e-20f) : mine;
    ids[t * top + lane] = mine_id;
    weights[t * top + lane] = w;
    if (dense != nullptr) dense[t * E + mine_id] = w;
  }
}

// Router logits of steps of few tokens: one workgroup per (token, group of kRouterGroup experts) forms the dot products of
// the token's row of activations with the experts' rows of the f32 router weight, in f32, without a widened copy of the
// activations; four elements per access when the rows allow it.
constexpr int kRouterGroup = 4;

template <typename T, bool VEC4>
__global__ __launch_bounds__(256) void router_logits_kernel(const T* __restrict__ h, int64_t ld_h, const float* __restrict__ router_w,
                                                            float* __restrict__ logits, int W, int E) {
  __shared__ float red[4][kRouterGroup];
  const int64_t t = blockIdx.x;
  const int e0 = blockIdx.y * kRouterGroup;
  const T* row = h + t * ld_h;
  float acc[kRouterGroup];
#pragma unroll
  for (int g = 0; g < kRouterGroup; ++g) acc[g] = 0.0f;
  if constexpr (VEC4) {
    for (int i = threadIdx.x * 4; i < W; i += blockDim.x * 4) {
      const float4 x = ld4(row + i);
#pragma unroll
      for (int g = 0; g < kRouterGroup; ++g) {
        if (e0 + g < E) {
          const float4 w = ld4(router_w + static_cast<int64_t>(e0 + g) * W + i);
          acc[g] += (x.x * w.x + x.y * w.y) + (x.z * w.z + x.w * w.w);
        }
      }
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      const float x = ldf(row + i);
#pragma unroll
      for (int g = 0; g < kRouterGroup; ++g)
        if (e0 + g < E) acc[g] += x * router_w[static_cast<int64_t>(e0 + g) * W + i];
    }
  }
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
  for (int g = 0; g < kRouterGroup; ++g) {
    const float v = wave_sum(acc[g]);
    if (lane == 0) red[wave][g] = v;
  }
  __syncthreads();
  if (threadIdx.x < kRouterGroup && e0 + threadIdx.x < E)
    logits[t * E + e0 + threadIdx.x] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

template <typename T>
__global__ __launch_bounds__(256) void relu2_scale_kernel(const T* __restrict__ up, const float* __restrict__ dense,
                                                          T* __restrict__ out, int64_t Tn, int E, int F) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t EF = static_cast<int64_t>(E) * F;
  if (idx >= Tn * EF) return;
  const int64_t t = idx / EF;
  const int e = static_cast<int>((idx - t * EF) / F);
  const float w = dense[t * E + e];
  const float x = fmaxf(ldf(up + idx), 0.0f);
  stf(out + idx, w != 0.0f ? x * x * w : 0.0f);
}

}  // namespace lvmix

using namespace lvmix;

extern "C" {

int lv_latent_prep(const void* proj, int64_t ld, int off_q, int off_kv, const void* q_w, const void* kv_w,
                   const void* inv_freq, void* cq_out, void* cache, const int32_t* cu_q, const int32_t* ctx_lens,
                   const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T, int Rq, int R, int Dr,
                   int rot_dims, int page, float eps, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!proj || !q_w || !kv_w || !cq_out || !cache || !cu_q || !ctx_lens || !tok_seq || !block_tables)
    return fail(-1, "lv_latent_prep: null pointer");
  if (T < 0 || Rq <= 0 || R <= 0 || Dr < 0 || rot_dims < 0 || rot_dims > Dr || rot_dims % 2 != 0 || page <= 0 ||
      bt_stride <= 0 || off_q < 0 || off_kv < 0 || off_q + Rq > ld || off_kv + R + Dr > ld || (rot_dims > 0 && !inv_freq))
    return fail(-1, "lv_latent_prep: bad sizes");
  const size_t shm = sizeof(float) * static_cast<size_t>(rot_dims > 0 ? rot_dims : 1);
  dim3 grid(static_cast<unsigned>(T)), block(256);
  if (dtype == LV_MIX_BF16)
    latent_prep_kernel<bf16_t><<<grid, block, shm, as_stream(stream)>>>(
        static_cast<const bf16_t*>(proj), ld, off_q, off_kv, static_cast<const float*>(q_w), static_cast<const float*>(kv_w),
        static_cast<const float*>(inv_freq), static_cast<bf16_t*>(cq_out), static_cast<bf16_t*>(cache), cu_q, ctx_lens,
        tok_seq, block_tables, bt_stride, Rq, R, Dr, rot_dims, page, eps);
  else if (dtype == LV_MIX_F32)
    latent_prep_kernel<float><<<grid, block, shm, as_stream(stream)>>>(
        static_cast<const float*>(proj), ld, off_q, off_kv, static_cast<const float*>(q_w), static_cast<const float*>(kv_w),
        static_cast<const float*>(inv_freq), static_cast<float*>(cq_out), static_cast<float*>(cache), cu_q, ctx_lens,
        tok_seq, block_tables, bt_stride, Rq, R, Dr, rot_dims, page, eps);
  else
    return fail(-1, "lv_latent_prep: dtype %d", dtype);
  return launched("lv_latent_prep");
}

int lv_latent_q_finish(const void* q, const void* q_lat, const void* inv_freq, void* q_out, const int32_t* cu_q,
                       const int32_t* ctx_lens, const int32_t* tok_seq, int64_t T, int H, int Dn, int Dr, int R,
                       int rot_dims, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!q || !q_lat || !q_out || !cu_q || !ctx_lens || !tok_seq) return fail(-1, "lv_latent_q_finish: null pointer");
  if (T < 0 || H <= 0 || Dn <= 0 || Dr < 0 || R <= 0 || rot_dims < 0 || rot_dims > Dr || rot_dims % 2 != 0 ||
      (rot_dims > 0 && !inv_freq))
    return fail(-1, "lv_latent_q_finish: bad sizes");
  const size_t shm = sizeof(float) * static_cast<size_t>(rot_dims > 0 ? rot_dims : 1);
  dim3 grid(static_cast<unsigned>(T)), block(256);
  if (dtype == LV_MIX_BF16)
    latent_q_finish_kernel<bf16_t><<<grid, block, shm, as_stream(stream)>>>(
        static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(q_lat), static_cast<const float*>(inv_freq),
        static_cast<bf16_t*>(q_out), cu_q, ctx_lens, tok_seq, T, H, Dn, Dr, R, rot_dims);
  else if (dtype == LV_MIX_F32)
    latent_q_finish_kernel<float><<<grid, block, shm, as_stream(stream)>>>(
        static_cast<const float*>(q), static_cast<const float*>(q_lat), static_cast<const float*>(inv_freq),
        static_cast<float*>(q_out), cu_q, ctx_lens, tok_seq, T, H, Dn, Dr, R, rot_dims);
  else
    return fail(-1, "lv_latent_q_finish: dtype %d", dtype);
  return launched("lv_latent_q_finish");
}

int lv_latent_out_gate(const void* o, const void* gate, int64_t ld_gate, int gate_kind, void* out, int64_t T, int H,
                       int Dv, int dtype, void* stream) {
  if (T == 0) return 0;
  const int per_channel = gate_kind == LV_MIX_GATE_PER_CHANNEL;
  if (!o || !gate || !out || T < 0 || H <= 0 || Dv <= 0 || (gate_kind != LV_MIX_GATE_PER_HEAD && !per_channel) ||
      ld_gate < (per_channel ? static_cast<int64_t>(H) * Dv : H))
    return fail(-1, "lv_latent_out_gate: bad arguments");
  const int64_t n = T * H * Dv;
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
  if (dtype == LV_MIX_BF16)
    latent_out_gate_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const bf16_t*>(o), static_cast<const bf16_t*>(gate), ld_gate, per_channel, static_cast<bf16_t*>(out), T, H, Dv);
  else if (dtype == LV_MIX_F32)
    latent_out_gate_kernel<float><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(o), static_cast<const float*>(gate), ld_gate, per_channel, static_cast<float*>(out), T, H, Dv);
  else
    return fail(-1, "lv_latent_out_gate: dtype %d", dtype);
  return launched("lv_latent_out_gate");
}

int lv_moe_route(const void* logits, const void* correction, void* ids, void* weights, void* dense, int64_t T, int E,
                 int top, int groups, int keep, int normalize, void* stream) {
  return lv_moe_route_scored(logits, correction, ids, weights, dense, T, E, top, groups, keep, normalize, LV_MIX_SCORE_SIGMOID,
                             LV_MIX_GROUP_TOP2_SUM, stream);
}

int lv_moe_route_scored(const void* logits, const void* correction, void* ids, void* weights, void* dense, int64_t T, int E,
                        int top, int groups, int keep, int normalize, int score_kind, int group_rank, void* stream) {
  if (T == 0) return 0;
  if ((score_kind != LV_MIX_SCORE_SIGMOID && score_kind != LV_MIX_SCORE_SOFTMAX) ||
      (group_rank != LV_MIX_GROUP_TOP2_SUM && group_rank != LV_MIX_GROUP_MAX))
    return fail(-1, "lv_moe_route: score kind %d, group rank %d", score_kind, group_rank);
  if (!logits || !ids || !weights || T < 0 || E <= 0 || top <= 0 || top > E || top > kWave)
    return fail(-1, "lv_moe_route: bad arguments (experts %d, top %d)", E, top);
  if (groups > 1 && (E % groups != 0 || keep <= 0 || keep > groups))
    return fail(-1, "lv_moe_route: %d groups (keep %d) of %d experts", groups, keep, E);
  const size_t shm = sizeof(float) * (2 * static_cast<size_t>(E) + static_cast<size_t>(groups > 1 ? groups : 1));
  if (shm > 64 * 1024) return fail(-2, "lv_moe_route: %d experts need %zu bytes of LDS", E, shm);
  moe_route_kernel<<<dim3(static_cast<unsigned>(T)), dim3(kWave), shm, as_stream(stream)>>>(
      static_cast<const float*>(logits), static_cast<const float*>(correction), static_cast<int32_t*>(ids),
      static_cast<float*>(weights), static_cast<float*>(dense), E, top, groups, keep, normalize, score_kind, group_rank);
  return launched("lv_moe_route");
}

int lv_router_logits(const void* h, int64_t ld_h, const void* router_w, void* logits, int64_t T, int W, int E, int dtype,
                     void* stream) {
  if (T == 0) return 0;
  if (!h || !router_w || !logits || T < 0 || W <= 0 || E <= 0 || ld_h < W) return fail(-1, "lv_router_logits: bad arguments");
  dim3 grid(static_cast<unsigned>(T), (E + kRouterGroup - 1) / kRouterGroup), block(256);
  const bool vec4 = W % 4 == 0 && ld_h % 4 == 0 && (reinterpret_cast<uintptr_t>(h) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(router_w) & 15) == 0;
#define LVMIX_ROUTER(TT, VV)                                                                                       \
  router_logits_kernel<TT, VV><<<grid, block, 0, as_stream(stream)>>>(static_cast<const TT*>(h), ld_h,             \
                                                                      static_cast<const float*>(router_w),         \
                                                                      static_cast<float*>(logits), W, E)
  if (dtype == LV_MIX_BF16) {
    if (vec4) LVMIX_ROUTER(bf16_t, true); else LVMIX_ROUTER(bf16_t, false);
  } else if (dtype == LV_MIX_F32) {
    if (vec4) LVMIX_ROUTER(float, true); else LVMIX_ROUTER(float, false);
  } else {
    return fail(-1, "lv_router_logits: dtype %d", dtype);
  }
#undef LVMIX_ROUTER
  return launched("lv_router_logits");
}

int lv_relu2_scale(const void* up, const void* dense, void* out, int64_t T, int E, int F, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!up || !dense || !out || T < 0 || E <= 0 || F <= 0) return fail(-1, "lv_relu2_scale: bad arguments");
  const int64_t n = T * E * F;
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
  if (dtype == LV_MIX_BF16)
    relu2_scale_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(static_cast<const bf16_t*>(up), static_cast<const float*>(dense),
                                                                    static_cast<bf16_t*>(out), T, E, F);
  else if (dtype == LV_MIX_F32)
    relu2_scale_kernel<float><<<grid, block, 0, as_stream(stream)>>>(static_cast<const float*>(up), static_cast<const float*>(dense),
                                                                   static_cast<float*>(out), T, E, F);
  else
    return fail(-1, "lv_relu2_scale: dtype %d", dtype);
  return launched("lv_relu2_scale");
}

}  // extern "C"
