// Layers whose mixer is two mixers side by side, tanh norms, a decaying linear-attention state, and the small steps
// around them.
//
//   residual_dyt_kernel      one workgroup per token: the f32 residual receives a sublayer output as it is, or the scaled
//                            sum of two sublayer outputs each divided by its root mean square and weighted; the
//                            dynamic-tanh norm tanh(alpha x) w + b of the updated row leaves in the activation dtype.
//   qk_prep_store_kernel     one wave per head of a token: optional division of a query or key head by its root mean
//                            square, optional rotation of the head's first entries (pairs side by side or half a
//                            rotated part apart), a factor per query head, keys and values written to the paged caches.
//                            A form with four entries per lane and several heads per wave serves aligned sizes.
//   lightning_attn_kernel    S <- decay_h S + k v^T, o = S^T q per head over the new tokens of every sequence, the state
//                            in f32 in the sequence's slot; q, k, v = silu of columns of the input projection. The four
//                            waves own a quarter of the state's rows each and never meet inside a chunk of tokens.
//   glu_act_kernel           act(gate) * up over [gate | up] rows.
//   expert_act_scale_kernel  act(up) * routing weight of the column's expert, zero for experts the token did not choose.
//   scaled_row_add_kernel    y[t] += (sum of a token's numbers) * h[t]: experts that hand their input through.
#include "mix_common.h"

namespace lvmix {

__device__ __forceinline__ float gelu_tanh_(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float gelu_erf_(float z) { return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f)); }

__device__ __forceinline__ float expert_act(float v, int act) {
  if (act == LV_MIX_ACT_GELU_ERF) return gelu_erf_(v);
  if (act == LV_MIX_ACT_GELU_TANH) return gelu_tanh_(v);
  v = fmaxf(v, 0.0f);
  return v * v;
}

// two sums over the workgroup's four waves at once
__device__ __forceinline__ void block_sum2(float& a, float& b, float (*red)[4]) {
  a = wave_sum(a);
  b = wave_sum(b);
  __syncthreads();
  if (threadIdx.x % kWave == 0) {
    red[0][threadIdx.x / kWave] = a;
    red[1][threadIdx.x / kWave] = b;
  }
  __syncthreads();
  a = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
  b = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void residual_dyt_kernel(float* __restrict__ x, const T* __restrict__ y1,
                                                            const float* __restrict__ pw1, const T* __restrict__ y2,
                                                            const float* __restrict__ pw2, float pair_scale, float eps,
                                                            const float* __restrict__ alpha, const float* __restrict__ w,
                                                            const float* __restrict__ bias, T* __restrict__ out, int W) {
  __shared__ float red[2][4];
  const int64_t t = blockIdx.x;
  float* xt = x + t * W;
  const T* a1 = y1 != nullptr ? y1 + t * W : nullptr;
  const T* a2 = y2 != nullptr ? y2 + t * W : nullptr;
  const int first = threadIdx.x * VEC, stride = blockDim.x * VEC;
  const bool normed = pw1 != nullptr;
  float f1 = 1.0f, f2 = 1.0f;
  if (normed) {
    float s1 = 0.0f, s2 = 0.0f;
    for (int i = first; i < W; i += stride) {
      if constexpr (VEC == 4) {
        const float4 u = ld4(a1 + i);
        s1 += (u.x * u.x + u.y * u.y) + (u.z * u.z + u.w * u.w);
        if (a2 != nullptr) {
          const float4 v = ld4(a2 + i);
          s2 += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
        }
      } else {
        const float u = ldf(a1 + i);
        s1 += u * u;
        if (a2 != nullptr) {
          const float v = ldf(a2 + i);
          s2 += v * v;
        }
      }
    }
    block_sum2(s1, s2, red);
    f1 = pair_scale / sqrtf(s1 / static_cast<float>(W) + eps);
    f2 = pair_scale / sqrtf(s2 / static_cast<float>(W) + eps);
  }
  const float al = alpha != nullptr ? alpha[0] : 1.0f;
  auto one = [&](float xv, float u, float v, float g1, float g2) {
    if (a1 != nullptr) xv += normed ? u * f1 * g1 : u;
    if (a2 != nullptr) xv += normed ? v * f2 * g2 : v;
    return xv;
  };
  for (int i = first; i < W; i += stride) {                    // the sublayer rows again: they are still in the cache
    if constexpr (VEC == 4) {
      float4 xv = ld4(xt + i);
      const float4 z = float4{0.0f, 0.0f, 0.0f, 0.0f};
      const float4 u = a1 != nullptr ? ld4(a1 + i) : z, v = a2 != nullptr ? ld4(a2 + i) : z;
      const float4 g1 = normed ? ld4(pw1 + i) : z, g2 = (normed && a2 != nullptr) ? ld4(pw2 + i) : z;
      xv = float4{one(xv.x, u.x, v.x, g1.x, g2.x), one(xv.y, u.y, v.y, g1.y, g2.y), one(xv.z, u.z, v.z, g1.z, g2.z),
                  one(xv.w, u.w, v.w, g1.w, g2.w)};
      if (a1 != nullptr || a2 != nullptr) st4(xt + i, xv);
      if (out != nullptr) {
        const float4 ww = ld4(w + i), bb = ld4(bias + i);
        st4(out + t * W + i, float4{tanhf(al * xv.x) * ww.x + bb.x, tanhf(al * xv.y) * ww.y + bb.y,
                                    tanhf(al * xv.z) * ww.z + bb.z, tanhf(al * xv.w) * ww.w + bb.w});
      }
    } else {
      const float xv = one(xt[i], a1 != nullptr ? ldf(a1 + i) : 0.0f, a2 != nullptr ? ldf(a2 + i) : 0.0f,
                           normed ? pw1[i] : 0.0f, (normed && a2 != nullptr) ? pw2[i] : 0.0f);
      if (a1 != nullptr || a2 != nullptr) xt[i] = xv;
      if (out != nullptr) stf(out + t * W + i, tanhf(al * xv) * w[i] + bias[i]);
    }
  }
}

// ------------------------------------------------------------------------------------------------
struct QkPrepParams {
  const void* proj;
  int64_t ld;
  int off_q, off_k, off_v;
  const float *inv_freq, *head_scale;
  void *q_out, *k_cache, *v_cache;
  const int32_t *cu_q, *ctx_lens, *tok_seq, *block_tables;
  int bt_stride, H, G, D, Dv, rot_dims, page, interleaved, unit_norm;
  float eps;
};

template <typename T>
__global__ __launch_bounds__(256) void qk_prep_store_kernel(QkPrepParams p) {
  extern __shared__ __attribute__((aligned(16))) float cs[];   // [rot_dims/2] cosines | [rot_dims/2] sines
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int b = p.tok_seq[t];
  const int pos = p.ctx_lens[b] + static_cast<int>(t) - p.cu_q[b];
  const int64_t slot = static_cast<int64_t>(p.block_tables[static_cast<int64_t>(b) * p.bt_stride + pos / p.page]) * p.page + pos % p.page;
  const int half = p.rot_dims / 2, D = p.D;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float s, c;
    sincosf(static_cast<float>(pos) * p.inv_freq[i], &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
  __syncthreads();
  const T* row = static_cast<const T*>(p.proj) + t * p.ld;
  T* q_out = static_cast<T*>(p.q_out) + t * p.H * D;
  T* k_out = static_cast<T*>(p.k_cache) + slot * p.G * D;
  for (int hd = wave; hd < p.H + p.G; hd += 4) {               // query heads, then key heads
    const bool is_q = hd < p.H;
    const T* head = row + (is_q ? p.off_q + hd * D : p.off_k + (hd - p.H) * D);
    T* dst = is_q ? q_out + hd * D : k_out + (hd - p.H) * D;
    float f = is_q && p.head_scale != nullptr ? p.head_scale[hd] : 1.0f;
    if (p.unit_norm) {
      float ss = 0.0f;
      for (int j = lane; j < D; j += kWave) {
        const float v = ldf(head + j);
        ss += v * v;
      }
      f /= sqrtf(wave_sum(ss) / static_cast<float>(D) + p.eps);
    }
    for (int j = lane; j < D; j += kWave) {
      float v = ldf(head + j);
      if (j < p.rot_dims) {
        // the entry's partner and place in the table of angles; the first of a pair gets u cos - v sin, the second v cos + u sin
        int i, other;
        bool lead;
        if (p.interleaved) { i = j >> 1; lead = (j & 1) == 0; other = j ^ 1; }
        else { lead = j < half; i = lead ? j : j - half; other = lead ? j + half : j - half; }
        const float u = ldf(head + other);
        v = lead ? v * cs[i] - u * cs[half + i] : v * cs[i] + u * cs[half + i];
      }
      stf(dst + j, v * f);
    }
  }
  const int GDv = p.G * p.Dv;
  T* v_out = static_cast<T*>(p.v_cache) + slot * GDv;
  for (int i = threadIdx.x; i < GDv; i += blockDim.x) v_out[i] = row[p.off_v + i];
}

// Four entries per lane: a head of D <= 256 entries sits in P lanes (the power of two at or above D / 4), so a wave holds
// 64 / P heads at once, each value is read once and stays in registers between the sum of squares and the rotation, and
// pairs that lie side by side need no second read at all. Taken when head sizes, the rotated part, column offsets and row
// strides are multiples of four (eight for the rotated part) and the rows are aligned.
template <typename T>
__global__ __launch_bounds__(256) void qk_prep_store_vec_kernel(QkPrepParams p, int P) {
  extern __shared__ __attribute__((aligned(16))) float cs[];   // [rot_dims/2] cosines | [rot_dims/2] sines
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int b = p.tok_seq[t];
  const int pos = p.ctx_lens[b] + static_cast<int>(t) - p.cu_q[b];
  const int64_t slot = static_cast<int64_t>(p.block_tables[static_cast<int64_t>(b) * p.bt_stride + pos / p.page]) * p.page + pos % p.page;
  const int half = p.rot_dims / 2, D = p.D;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float s, c;
    sincosf(static_cast<float>(pos) * p.inv_freq[i], &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
  __syncthreads();
  const T* row = static_cast<const T*>(p.proj) + t * p.ld;
  T* q_out = static_cast<T*>(p.q_out) + t * p.H * D;
  T* k_out = static_cast<T*>(p.k_cache) + slot * p.G * D;
  const int per_wave = kWave / P, sub = lane / P, j = 4 * (lane % P);
  const int heads = p.H + p.G;
  for (int hd0 = 0; hd0 < heads; hd0 += 4 * per_wave) {          // the same trip count for every lane: the sums below shuffle
    const int hd = hd0 + wave * per_wave + sub;
    const bool live = hd < heads && j < D;
    const bool is_q = hd < p.H;
    const T* head = row + (is_q ? p.off_q + hd * D : p.off_k + (hd - p.H) * D);
    float4 v = live ? ld4(head + j) : float4{0.0f, 0.0f, 0.0f, 0.0f};
    float f = (live && is_q && p.head_scale != nullptr) ? p.head_scale[hd] : 1.0f;
    if (p.unit_norm) {
      float ss = (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
      for (int o = P >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
      f /= sqrtf(ss / static_cast<float>(D) + p.eps);
    }
    if (!live) continue;
    if (j < p.rot_dims) {
      if (p.interleaved) {
        const int i = j >> 1;
        const float c0 = cs[i], s0 = cs[half + i], c1 = cs[i + 1], s1 = cs[half + i + 1];
        v = float4{v.x * c0 - v.y * s0, v.y * c0 + v.x * s0, v.z * c1 - v.w * s1, v.w * c1 + v.z * s1};
      } else if (j < half) {
        const float4 u = ld4(head + j + half), c = ld4(cs + j), sn = ld4(cs + half + j);
        v = float4{v.x * c.x - u.x * sn.x, v.y * c.y - u.y * sn.y, v.z * c.z - u.z * sn.z, v.w * c.w - u.w * sn.w};
      } else {
        const float4 u = ld4(head + j - half), c = ld4(cs + j - half), sn = ld4(cs + j);
        v = float4{v.x * c.x + u.x * sn.x, v.y * c.y + u.y * sn.y, v.z * c.z + u.z * sn.z, v.w * c.w + u.w * sn.w};
      }
    }
    st4((is_q ? q_out + hd * D : k_out + (hd - p.H) * D) + j, float4{v.x * f, v.y * f, v.z * f, v.w * f});
  }
  const int GDv = p.G * p.Dv;
  T* v_out = static_cast<T*>(p.v_cache) + slot * GDv;
  for (int i = threadIdx.x * 4; i < GDv; i += blockDim.x * 4) st4(v_out + i, ld4(row + p.off_v + i));
}

// ------------------------------------------------------------------------------------------------
struct LightningParams {
  const void* proj;        // act [T, ld]: q at off_q (H heads of D), k at off_k (H of D), v at off_v (H of Dv)
  int64_t ld;
  int off_q, off_k, off_v;
  const float* decay;      // [H]
  float* state;            // [slots, H, D, Dv]
  const int32_t *cu_q, *ctx_lens, *slots;
  float* o;                // [T, H, Dv]
  int H, D, Dv;
};


// NW waves a workgroup, DR = rows of the state each wave owns (NW * DR >= D; rows beyond D stay zero); lane = value column.
// Tokens come in chunks: the chunk's queries, keys and values are fetched into registers one chunk ahead and staged in LDS
// with silu applied; every wave then walks the chunk alone (its rows of S need nobody else's) and leaves its share of each
// read-out in LDS; the NW shares are added when the chunk is done. The token loop is a chain of LDS reads and multiply-adds
// that only other waves on the SIMD can overlap, so a launch with few workgroups (few sequences or heads) splits the rows
// over eight waves instead of four.
template <int DR, int NW>
struct LightningShape {
  static constexpr int kDP = NW * DR;
  static constexpr int kChunk = (kDP >= 128 || NW > 4) ? 16 : 32;     // what fits 64 KB of LDS with the shares of NW waves
  static constexpr size_t kLds = sizeof(float) * (2 * kChunk * kDP + kChunk * kWave + kChunk * NW * kWave);
};

template <typename T, int DR, int NW>
__global__ __launch_bounds__(NW * 64) void lightning_attn_kernel(LightningParams p) {
  extern __shared__ __attribute__((aligned(16))) float ll[];
  constexpr int DP = NW * DR, NT = NW * kWave;
  constexpr int kLightChunk = LightningShape<DR, NW>::kChunk;
  float* k_lds = ll;                               // [chunk][DP]
  float* q_lds = k_lds + kLightChunk * DP;         // [chunk][DP]
  float* v_lds = q_lds + kLightChunk * DP;         // [chunk][64]
  float* part_o = v_lds + kLightChunk * kWave;     // [chunk][NW][64]
  const int lane = threadIdx.x % kWave, rp = threadIdx.x / kWave;
  const int col = blockIdx.x * kWave + lane;
  const int h = blockIdx.y, b = blockIdx.z;
  const int q0 = p.cu_q[b], n = p.cu_q[b + 1] - q0;
  if (n <= 0) return;
  const bool live = col < p.Dv;
  const int row0 = rp * DR;
  const float dec = p.decay[h];
  float* sbase = p.state + (static_cast<int64_t>(p.slots[b]) * p.H + h) * p.D * p.Dv;
  const bool carry = p.ctx_lens[b] > 0;
  float s[DR];
#pragma unroll
  for (int r = 0; r < DR; ++r)
    s[r] = (carry && live && row0 + r < p.D) ? sbase[static_cast<int64_t>(row0 + r) * p.Dv + col] : 0.0f;
  const T* proj = static_cast<const T*>(p.proj);
  constexpr int NKQ = kLightChunk * DP / NT, NV = (kLightChunk * kWave + NT - 1) / NT;
  float kreg[NKQ], qreg[NKQ], vreg[NV];
  auto fetch = [&](int c0) {
    const int cn = min(kLightChunk, n - c0);
#pragma unroll
    for (int it = 0; it < NKQ; ++it) {
      const int x = threadIdx.x + it * NT;
      const int tok = x / DP, d = x - tok * DP;
      const T* row = proj + (static_cast<int64_t>(q0) + c0 + tok) * p.ld + h * p.D + d;
      const bool in = tok < cn && d < p.D;
      kreg[it] = in ? ldf(row + p.off_k) : 0.0f;
      qreg[it] = in ? ldf(row + p.off_q) : 0.0f;
    }
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int x = threadIdx.x + it * NT;
      const int tok = x / kWave, cc = blockIdx.x * kWave + (x % kWave);
      vreg[it] = (tok < cn && cc < p.Dv) ? ldf(proj + (static_cast<int64_t>(q0) + c0 + tok) * p.ld + p.off_v + h * p.Dv + cc) : 0.0f;
    }
  };
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += kLightChunk) {
    const int cn = min(kLightChunk, n - c0);
    // every wave is past the previous chunk's token loop: behind the barrier that followed it
#pragma unroll
    for (int it = 0; it < NKQ; ++it) {
      k_lds[threadIdx.x + it * NT] = siluf_(kreg[it]);
      q_lds[threadIdx.x + it * NT] = siluf_(qreg[it]);
    }
#pragma unroll
    for (int it = 0; it < NV; ++it)
      if (threadIdx.x + it * NT < kLightChunk * kWave) v_lds[threadIdx.x + it * NT] = siluf_(vreg[it]);
    __syncthreads();
    if (c0 + kLightChunk < n) fetch(c0 + kLightChunk);
    for (int i = 0; i < cn; ++i) {
      const float vv = v_lds[i * kWave + lane];
      float po4[4] = {0.0f, 0.0f, 0.0f, 0.0f};     // four chains: one sum would be bound by its own latency
#pragma unroll
      for (int r = 0; r < DR; r += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(k_lds + i * DP + row0 + r);
        const float4 q4 = *reinterpret_cast<const float4*>(q_lds + i * DP + row0 + r);
        s[r] = dec * s[r] + k4.x * vv;
        s[r + 1] = dec * s[r + 1] + k4.y * vv;
        s[r + 2] = dec * s[r + 2] + k4.z * vv;
        s[r + 3] = dec * s[r + 3] + k4.w * vv;
        po4[0] += s[r] * q4.x;
        po4[1] += s[r + 1] * q4.y;
        po4[2] += s[r + 2] * q4.z;
        po4[3] += s[r + 3] * q4.w;
      }
      part_o[(i * NW + rp) * kWave + lane] = (po4[0] + po4[1]) + (po4[2] + po4[3]);
    }
    __syncthreads();
    for (int x = threadIdx.x; x < cn * kWave; x += NT) {
      const int tok = x / kWave, ln = x % kWave, cc = blockIdx.x * kWave + ln;
      const float* po = part_o + tok * NW * kWave + ln;
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; w += 2) sum += po[w * kWave] + po[(w + 1) * kWave];
      if (cc < p.Dv) p.o[((static_cast<int64_t>(q0) + c0 + tok) * p.H + h) * p.Dv + cc] = sum;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < DR; ++r)
      if (row0 + r < p.D) sbase[static_cast<int64_t>(row0 + r) * p.Dv + col] = s[r];
  }
}

template <typename T, int DR, int NW>
static void lightning_launch(const LightningParams& p, dim3 grid, hipStream_t s) {
  lightning_attn_kernel<T, DR, NW><<<grid, dim3(NW * kWave), LightningShape<DR, NW>::kLds, s>>>(p);
}

template <typename T>
static int lightning_dispatch(const LightningParams& p, int B, hipStream_t s) {
  dim3 grid((p.Dv + kWave - 1) / kWave, p.H, B);
  // fewer than four workgroups a compute unit: eight waves each, so that a SIMD still holds four
  const bool eight = static_cast<int64_t>(grid.x) * grid.y * grid.z < 4 * 256 && p.D > 16 && p.D <= 128;
  if (eight) {
    if (p.D <= 32) lightning_launch<T, 4, 8>(p, grid, s);
    else if (p.D <= 64) lightning_launch<T, 8, 8>(p, grid, s);
    else lightning_launch<T, 16, 8>(p, grid, s);
  } else {
    if (p.D <= 32) lightning_launch<T, 8, 4>(p, grid, s);
    else if (p.D <= 64) lightning_launch<T, 16, 4>(p, grid, s);
    else if (p.D <= 128) lightning_launch<T, 32, 4>(p, grid, s);
    else lightning_launch<T, 64, 4>(p, grid, s);
  }
  return 0;
}

// ------------------------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void glu_act_kernel(const T* __restrict__ in, int64_t ld_in, T* __restrict__ out, int64_t Tn,
                                                      int F, int act) {
  const int64_t idx = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
  if (idx >= Tn * F) return;
  const int64_t t = idx / F;
  const int f = static_cast<int>(idx - t * F);
  const T* row = in + t * ld_in;
  if constexpr (VEC == 4) {
    const float4 g = ld4(row + f), u = ld4(row + F + f);
    st4(out + idx, float4{expert_act(g.x, act) * u.x, expert_act(g.y, act) * u.y, expert_act(g.z, act) * u.z,
                          expert_act(g.w, act) * u.w});
  } else {
    stf(out + idx, expert_act(ldf(row + f), act) * ldf(row + F + f));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void expert_act_scale_kernel(const T* __restrict__ up, const float* __restrict__ dense,
                                                               int64_t ld_dense, T* __restrict__ out, int64_t Tn, int E, int F,
                                                               int act) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t EF = static_cast<int64_t>(E) * F;
  if (idx >= Tn * EF) return;
  const int64_t t = idx / EF;
  const int e = static_cast<int>((idx - t * EF) / F);
  const float w = dense[t * ld_dense + e];
  stf(out + idx, w != 0.0f ? expert_act(ldf(up + idx), act) * w : 0.0f);
}

template <typename T>
__global__ __launch_bounds__(256) void scaled_row_add_kernel(T* __restrict__ y, const T* __restrict__ h,
                                                             const float* __restrict__ f, int64_t ld_f, int nf, int64_t Tn,
                                                             int W) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= Tn * W) return;
  const int64_t t = idx / W;
  float s = 0.0f;
  for (int i = 0; i < nf; ++i) s += f[t * ld_f + i];
  if (s != 0.0f) stf(y + idx, ldf(y + idx) + s * ldf(h + idx));
}

}  // namespace lvmix

using namespace lvmix;

extern "C" {

int lv_residual_dyt(void* x, const void* y1, const void* post_w1, const void* y2, const void* post_w2, float pair_scale,
                    float eps, const void* alpha, const void* w, const void* b, void* out, int64_t T, int W, int dtype,
                    void* stream) {
  if (T == 0) return 0;
  if (x == nullptr || T < 0 || W <= 0 || (out != nullptr && (w == nullptr || b == nullptr || alpha == nullptr)) ||
      (post_w1 != nullptr && y1 == nullptr) || ((post_w2 != nullptr) != (post_w1 != nullptr && y2 != nullptr)))
    return fail(-1, "lv_residual_dyt: bad arguments");
  if (out == nullptr && y1 == nullptr && y2 == nullptr) return 0;
  dim3 grid(static_cast<unsigned>(T)), block(256);
  auto aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec4 = W % 4 == 0 && aligned(x) && aligned(y1) && aligned(y2) && aligned(post_w1) && aligned(post_w2) && aligned(w) &&
                    aligned(b) && aligned(out);
#define LVMIX_DYT(TT, VV)                                                                                                   \
  residual_dyt_kernel<TT, VV><<<grid, block, 0, as_stream(stream)>>>(                                                      \
      static_cast<float*>(x), static_cast<const TT*>(y1), static_cast<const float*>(post_w1), static_cast<const TT*>(y2),   \
      static_cast<const float*>(post_w2), pair_scale, eps, static_cast<const float*>(alpha), static_cast<const float*>(w),  \
      static_cast<const float*>(b), static_cast<TT*>(out), W)
  if (dtype == LV_MIX_BF16) {
    if (vec4) LVMIX_DYT(bf16_t, 4); else LVMIX_DYT(bf16_t, 1);
  } else if (dtype == LV_MIX_F32) {
    if (vec4) LVMIX_DYT(float, 4); else LVMIX_DYT(float, 1);
  } else {
    return fail(-1, "lv_residual_dyt: dtype %d", dtype);
  }
#undef LVMIX_DYT
  return launched("lv_residual_dyt");
}

int lv_qk_prep_store(const void* proj, int64_t ld, int off_q, int off_k, int off_v, const void* inv_freq,
                     const void* head_scale, void* q_out, void* k_cache, void* v_cache, const int32_t* cu_q,
                     const int32_t* ctx_lens, const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T,
                     int H, int G, int D, int Dv, int rot_dims, int interleaved, int unit_norm, float eps, int page, int dtype,
                     void* stream) {
  if (T == 0) return 0;
  if (!proj || !q_out || !k_cache || !v_cache || !cu_q || !ctx_lens || !tok_seq || !block_tables)
    return fail(-1, "lv_qk_prep_store: null pointer");
  if (T < 0 || H <= 0 || G <= 0 || H % G != 0 || D <= 0 || Dv <= 0 || page <= 0 || bt_stride <= 0 || rot_dims < 0 ||
      rot_dims > D || rot_dims % 2 != 0 || (rot_dims > 0 && !inv_freq) || off_q < 0 || off_k < 0 || off_v < 0 ||
      off_q + static_cast<int64_t>(H) * D > ld || off_k + static_cast<int64_t>(G) * D > ld ||
      off_v + static_cast<int64_t>(G) * Dv > ld)
    return fail(-1, "lv_qk_prep_store: bad sizes");
  const size_t shm = sizeof(float) * static_cast<size_t>(rot_dims > 0 ? rot_dims : 4);
  if (shm > 64 * 1024) return fail(-2, "lv_qk_prep_store: %d rotated entries", rot_dims);
  QkPrepParams p{proj, ld, off_q, off_k, off_v, static_cast<const float*>(inv_freq), static_cast<const float*>(head_scale),
                 q_out, k_cache, v_cache, cu_q, ctx_lens, tok_seq, block_tables, bt_stride, H, G, D, Dv, rot_dims, page,
                 interleaved != 0, unit_norm != 0, eps};
  dim3 grid(static_cast<unsigned>(T)), block(256);
  if (dtype != LV_MIX_BF16 && dtype != LV_MIX_F32) return fail(-1, "lv_qk_prep_store: dtype %d", dtype);
  auto aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec4 = D % 4 == 0 && D <= 4 * kWave && Dv % 4 == 0 && rot_dims % 8 == 0 && ld % 4 == 0 && off_q % 4 == 0 &&
                    off_k % 4 == 0 && off_v % 4 == 0 && aligned(proj) && aligned(q_out) && aligned(k_cache) && aligned(v_cache);
  if (vec4) {
    int P = 1;
    while (4 * P < D) P <<= 1;                       // lanes that hold one head
    if (dtype == LV_MIX_BF16) qk_prep_store_vec_kernel<bf16_t><<<grid, block, shm, as_stream(stream)>>>(p, P);
    else qk_prep_store_vec_kernel<float><<<grid, block, shm, as_stream(stream)>>>(p, P);
  } else if (dtype == LV_MIX_BF16) {
    qk_prep_store_kernel<bf16_t><<<grid, block, shm, as_stream(stream)>>>(p);
  } else {
    qk_prep_store_kernel<float><<<grid, block, shm, as_stream(stream)>>>(p);
  }
  return launched("lv_qk_prep_store");
}

int lv_lightning_attn(const void* proj, int64_t ld, int off_q, int off_k, int off_v, const void* decay, void* state,
                      const int32_t* cu_q, const int32_t* ctx_lens, const int32_t* slots, void* o, int B, int H, int D, int Dv,
                      int dtype, void* stream) {
  if (B == 0) return 0;
  if (!proj || !decay || !state || !cu_q || !ctx_lens || !slots || !o) return fail(-1, "lv_lightning_attn: null pointer");
  if (B < 0 || H <= 0 || D <= 0 || Dv <= 0 || off_q < 0 || off_k < 0 || off_v < 0 || off_q + static_cast<int64_t>(H) * D > ld ||
      off_k + static_cast<int64_t>(H) * D > ld || off_v + static_cast<int64_t>(H) * Dv > ld)
    return fail(-1, "lv_lightning_attn: bad sizes");
  if (D > 256) return fail(-2, "lv_lightning_attn: key size %d above 256", D);
  LightningParams p{proj, ld, off_q, off_k, off_v, static_cast<const float*>(decay), static_cast<float*>(state), cu_q, ctx_lens,
                    slots, static_cast<float*>(o), H, D, Dv};
  if (dtype == LV_MIX_BF16) lightning_dispatch<bf16_t>(p, B, as_stream(stream));
  else if (dtype == LV_MIX_F32) lightning_dispatch<float>(p, B, as_stream(stream));
  else return fail(-1, "lv_lightning_attn: dtype %d", dtype);
  return launched("lv_lightning_attn");
}

int lv_glu_act(const void* in, int64_t ld_in, void* out, int64_t T, int F, int act, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!in || !out || T < 0 || F <= 0 || ld_in < 2 * static_cast<int64_t>(F) || act < 0 || act > LV_MIX_ACT_GELU_TANH)
    return fail(-1, "lv_glu_act: bad arguments");
  const bool vec4 = F % 4 == 0 && ld_in % 4 == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  const int64_t n = T * F / (vec4 ? 4 : 1);
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
#define LVMIX_GLU(TT, VV)                                                                                                  \
  glu_act_kernel<TT, VV><<<grid, block, 0, as_stream(stream)>>>(static_cast<const TT*>(in), ld_in, static_cast<TT*>(out), T, F, act)
  if (dtype == LV_MIX_BF16) {
    if (vec4) LVMIX_GLU(bf16_t, 4); else LVMIX_GLU(bf16_t, 1);
  } else if (dtype == LV_MIX_F32) {
    if (vec4) LVMIX_GLU(float, 4); else LVMIX_GLU(float, 1);
  } else {
    return fail(-1, "lv_glu_act: dtype %d", dtype);
  }
#undef LVMIX_GLU
  return launched("lv_glu_act");
}

int lv_expert_act_scale(const void* up, const void* dense, int64_t ld_dense, void* out, int64_t T, int E, int F, int act,
                        int dtype, void* stream) {
  if (T == 0) return 0;
  if (!up || !dense || !out || T < 0 || E <= 0 || F <= 0 || ld_dense < E || act < 0 || act > LV_MIX_ACT_GELU_TANH)
    return fail(-1, "lv_expert_act_scale: bad arguments");
  const int64_t n = T * E * F;
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
  if (dtype == LV_MIX_BF16)
    expert_act_scale_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const bf16_t*>(up), static_cast<const float*>(dense), ld_dense, static_cast<bf16_t*>(out), T, E, F, act);
  else if (dtype == LV_MIX_F32)
    expert_act_scale_kernel<float><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(up), static_cast<const float*>(dense), ld_dense, static_cast<float*>(out), T, E, F, act);
  else
    return fail(-1, "lv_expert_act_scale: dtype %d", dtype);
  return launched("lv_expert_act_scale");
}

int lv_scaled_row_add(void* y, const void* h, const void* factors, int64_t ld_f, int nf, int64_t T, int W, int dtype,
                      void* stream) {
  if (T == 0 || nf == 0) return 0;
  if (!y || !h || !factors || T < 0 || W <= 0 || nf < 0 || ld_f < nf) return fail(-1, "lv_scaled_row_add: bad arguments");
  const int64_t n = T * W;
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
  if (dtype == LV_MIX_BF16)
    scaled_row_add_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(static_cast<bf16_t*>(y), static_cast<const bf16_t*>(h),
                                                                       static_cast<const float*>(factors), ld_f, nf, T, W);
  else if (dtype == LV_MIX_F32)
    scaled_row_add_kernel<float><<<grid, block, 0, as_stream(stream)>>>(static_cast<float*>(y), static_cast<const float*>(h),
                                                                      static_cast<const float*>(factors), ld_f, nf, T, W);
  else
    return fail(-1, "lv_scaled_row_add: dtype %d", dtype);
  return launched("lv_scaled_row_add");
}

}  // extern "C"
