// Layers that norm both sides of every sublayer, rotated attention inputs, and gated experts.
//
//   sandwich_add_norm_kernel  one workgroup per token: the f32 residual receives the RMS-normed sublayer output
//                             (times offset + post weight), optionally a row of activations and a vector, and the
//                             RMS norm of the updated row (times offset + weight) leaves in the activation dtype.
//                             The sublayer output and the updated residual are staged in LDS between the passes.
//   rotary_store_kernel       one workgroup per token: rotation of the first rot_dims entries of every query and key
//                             head (angles in f32 from the token's position), a factor per query head, keys and
//                             values written to the token's row of the paged caches.
//   polynorm_kernel           one workgroup per token: c1 R(z) + c2 R(z^2) + c3 R(z^3) + c0, R = division by the root
//                             mean square of the row; the three sums of squares in one pass, f32.
//   expert_glu_kernel         elementwise: clamped gated unit of E experts side by side, the pre-activations times
//                             a number per (token, expert), the result times a sigmoid per token.
#include "mix_common.h"

namespace lvmix {

__device__ __forceinline__ float block_sum4(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();                                   // red may still be read from an earlier reduction
  if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void sandwich_add_norm_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                 const float* __restrict__ post_w, const T* __restrict__ rows,
                                                                 const float* __restrict__ vec, const float* __restrict__ w,
                                                                 float w_offset, T* __restrict__ out, int W, float eps) {
  extern __shared__ __attribute__((aligned(16))) float lds[];          // [W] row being worked on, then [4] partial sums
  float* red = lds + W;
  const int64_t t = blockIdx.x;
  float* xt = x + t * W;
  const int first = threadIdx.x * VEC, stride = blockDim.x * VEC;      // VEC = 4 when W % 4 == 0 and all rows are aligned
  float inv_y = 0.0f;
  if (y != nullptr) {
    float ss = 0.0f;
    for (int i = first; i < W; i += stride) {
      if constexpr (VEC == 4) {
        const float4 v = ld4(y + t * W + i);
        st4(lds + i, v);
        ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
      } else {
        const float v = ldf(y + t * W + i);
        lds[i] = v;
        ss += v * v;
      }
    }
    inv_y = 1.0f / sqrtf(block_sum4(ss, red) / static_cast<float>(W) + eps);
  }
  float ss = 0.0f;
  const bool changes = y != nullptr || rows != nullptr || vec != nullptr;
  for (int i = first; i < W; i += stride) {                            // every thread reads back its own entries of lds
    if constexpr (VEC == 4) {
      float4 v = ld4(xt + i);
      if (y != nullptr) {
        const float4 a = ld4(lds + i), g = ld4(post_w + i);
        v.x += a.x * inv_y * (w_offset + g.x); v.y += a.y * inv_y * (w_offset + g.y);
        v.z += a.z * inv_y * (w_offset + g.z); v.w += a.w * inv_y * (w_offset + g.w);
      }
      if (rows != nullptr) {
        const float4 a = ld4(rows + t * W + i);
        v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
      }
      if (vec != nullptr) {
        const float4 a = ld4(vec + i);
        v.x += a.x; v.y += a.y; v.z += a.z; v.w += a.w;
      }
      if (changes) st4(xt + i, v);
      st4(lds + i, v);
      ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    } else {
      float v = xt[i];
      if (y != nullptr) v += lds[i] * inv_y * (w_offset + post_w[i]);
      if (rows != nullptr) v += ldf(rows + t * W + i);
      if (vec != nullptr) v += vec[i];
      if (changes) xt[i] = v;
      lds[i] = v;
      ss += v * v;
    }
  }
  if (out == nullptr) return;
  const float inv = 1.0f / sqrtf(block_sum4(ss, red) / static_cast<float>(W) + eps);
  for (int i = first; i < W; i += stride) {
    if constexpr (VEC == 4) {
      const float4 v = ld4(lds + i), g = ld4(w + i);
      st4(out + t * W + i, float4{v.x * inv * (w_offset + g.x), v.y * inv * (w_offset + g.y), v.z * inv * (w_offset + g.z),
                                  v.w * inv * (w_offset + g.w)});
    } else {
      stf(out + t * W + i, lds[i] * inv * (w_offset + w[i]));
    }
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void rotary_store_kernel(const T* __restrict__ proj, int64_t ld, int off_q, int off_k,
                                                           int off_v, const float* __restrict__ inv_freq,
                                                           const float* __restrict__ head_scale, T* __restrict__ q_out,
                                                           T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                           const int32_t* __restrict__ cu_q,
                                                           const int32_t* __restrict__ ctx_lens,
                                                           const int32_t* __restrict__ tok_seq,
                                                           const int32_t* __restrict__ block_tables, int bt_stride, int H,
                                                           int G, int D, int Dv, int rot_dims, int page) {
  extern __shared__ __attribute__((aligned(16))) float cs[];   // [rot_dims/2] cosines | [rot_dims/2] sines
  const int64_t t = blockIdx.x;
  const int b = tok_seq[t];
  const int pos = ctx_lens[b] + static_cast<int>(t) - cu_q[b];
  const int64_t slot = static_cast<int64_t>(block_tables[static_cast<int64_t>(b) * bt_stride + pos / page]) * page + pos % page;
  const int half = rot_dims / 2;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float a = static_cast<float>(pos) * inv_freq[i];
    float s, c;
    sincosf(a, &s, &c);
    cs[i] = c;
    cs[half + i] = s;
  }
  __syncthreads();
  const T* row = proj + t * ld;
  const int HD = H * D, GD = G * D, GDv = G * Dv;
  if constexpr (VEC == 4) {
    // four consecutive entries of a head lie wholly in its first rotated half, its second, or its unrotated rest
    auto turned4 = [&](const T* head, int j) -> float4 {
      const float4 v = ld4(head + j);
      if (j >= rot_dims) return v;
      if (j < half) {
        const float4 u = ld4(head + j + half), c = ld4(cs + j), sn = ld4(cs + half + j);
        return float4{v.x * c.x - u.x * sn.x, v.y * c.y - u.y * sn.y, v.z * c.z - u.z * sn.z, v.w * c.w - u.w * sn.w};
      }
      const float4 u = ld4(head + j - half), c = ld4(cs + j - half), sn = ld4(cs + j);
      return float4{v.x * c.x + u.x * sn.x, v.y * c.y + u.y * sn.y, v.z * c.z + u.z * sn.z, v.w * c.w + u.w * sn.w};
    };
    for (int i = threadIdx.x * 4; i < HD; i += blockDim.x * 4) {
      const int h = i / D, j = i - h * D;
      float4 v = turned4(row + off_q + h * D, j);
      if (head_scale != nullptr) {
        const float f = head_scale[h];
        v.x *= f; v.y *= f; v.z *= f; v.w *= f;
      }
      st4(q_out + t * HD + i, v);
    }
    for (int i = threadIdx.x * 4; i < GD; i += blockDim.x * 4) {
      const int g = i / D, j = i - g * D;
      st4(k_cache + slot * GD + i, turned4(row + off_k + g * D, j));
    }
    for (int i = threadIdx.x * 4; i < GDv; i += blockDim.x * 4) st4(v_cache + slot * GDv + i, ld4(row + off_v + i));
    return;
  }
  auto turned = [&](const T* head, int j) -> float {
    if (j >= rot_dims) return ldf(head + j);
    if (j < half) return ldf(head + j) * cs[j] - ldf(head + j + half) * cs[half + j];
    return ldf(head + j) * cs[j - half] + ldf(head + j - half) * cs[j];     // cs[half + (j - half)]
  };
  for (int i = threadIdx.x; i < HD; i += blockDim.x) {
    const int h = i / D, j = i - h * D;
    const float v = turned(row + off_q + h * D, j);
    stf(q_out + t * HD + i, head_scale != nullptr ? v * head_scale[h] : v);
  }
  for (int i = threadIdx.x; i < GD; i += blockDim.x) {
    const int g = i / D, j = i - g * D;
    stf(k_cache + slot * GD + i, turned(row + off_k + g * D, j));
  }
  for (int i = threadIdx.x; i < GDv; i += blockDim.x) v_cache[slot * GDv + i] = row[off_v + i];
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void polynorm_kernel(const T* __restrict__ in, int64_t ld_in, const float* __restrict__ coef,
                                                       T* __restrict__ out, int F, float eps) {
  __shared__ float red[3][4];
  const int64_t t = blockIdx.x;
  const T* z = in + t * ld_in;
  const int first = threadIdx.x * VEC, stride = blockDim.x * VEC;      // VEC = 4 when F and ld_in are multiples of 4 and the rows aligned
  float s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  auto take = [&](float v) {
    const float v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  };
  for (int i = first; i < F; i += stride) {
    if constexpr (VEC == 4) {
      const float4 v = ld4(z + i);
      take(v.x); take(v.y); take(v.z); take(v.w);
    } else {
      take(ldf(z + i));
    }
  }
  s1 = wave_sum(s1);
  s2 = wave_sum(s2);
  s3 = wave_sum(s3);
  if (threadIdx.x % kWave == 0) {
    const int wv = threadIdx.x / kWave;
    red[0][wv] = s1;
    red[1][wv] = s2;
    red[2][wv] = s3;
  }
  __syncthreads();
  const float n = static_cast<float>(F);
  const float a = coef[0] / sqrtf(((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) / n + eps);
  const float b = coef[1] / sqrtf(((red[1][0] + red[1][1]) + (red[1][2] + red[1][3])) / n + eps);
  const float c = coef[2] / sqrtf(((red[2][0] + red[2][1]) + (red[2][2] + red[2][3])) / n + eps);
  const float e = coef[3];
  auto poly = [&](float v) { return ((c * v + b) * v + a) * v + e; };
  for (int i = first; i < F; i += stride) {                            // the row again: it is still in the cache
    if constexpr (VEC == 4) {
      const float4 v = ld4(z + i);
      st4(out + t * F + i, float4{poly(v.x), poly(v.y), poly(v.z), poly(v.w)});
    } else {
      stf(out + t * F + i, poly(ldf(z + i)));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void expert_glu_kernel(const T* __restrict__ in, int64_t ld_in, const float* __restrict__ in_scale,
                                                         const T* __restrict__ out_gate, int64_t ld_gate, T* __restrict__ out,
                                                         int64_t ld_out, int64_t Tn, int E, int F, float limit, float alpha) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t EF = static_cast<int64_t>(E) * F;
  if (idx >= Tn * EF) return;
  const int64_t t = idx / EF;
  const int c = static_cast<int>(idx - t * EF);
  const int e = c / F, f = c - e * F;
  const float s = in_scale != nullptr ? in_scale[t * E + e] : 1.0f;
  float r = 0.0f;
  if (s != 0.0f) {
    const T* x = in + t * ld_in + static_cast<int64_t>(e) * 2 * F;
    const float g = fminf(ldf(x + f) * s, limit);
    const float u = fminf(fmaxf(ldf(x + F + f) * s, -limit), limit);
    r = g * sigmoidf_(alpha * g) * (u + 1.0f);
    if (out_gate != nullptr) r *= sigmoidf_(ldf(out_gate + t * ld_gate));
  }
  stf(out + t * ld_out + c, r);
}

}  // namespace lvmix

using namespace lvmix;

extern "C" {

int lv_sandwich_add_norm(void* x, const void* y, const void* post_w, const void* rows, const void* vec, const void* w,
                         float w_offset, void* out, int64_t T, int W, float eps, int dtype, void* stream) {
  if (T == 0) return 0;
  if (x == nullptr || T < 0 || W <= 0 || (out != nullptr && w == nullptr) || (y != nullptr && post_w == nullptr))
    return fail(-1, "lv_sandwich_add_norm: bad arguments");
  if (out == nullptr && y == nullptr && rows == nullptr && vec == nullptr) return 0;
  const size_t shm = static_cast<size_t>(W + 4) * sizeof(float);
  if (shm > 64 * 1024) return fail(-2, "lv_sandwich_add_norm: width %d too large", W);
  dim3 grid(static_cast<unsigned>(T)), block(256);
  auto aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec4 = W % 4 == 0 && aligned(x) && aligned(y) && aligned(post_w) && aligned(rows) && aligned(vec) && aligned(w) &&
                    aligned(out);
#define LVMIX_SANDWICH(TT, VV)                                                                                  \
  sandwich_add_norm_kernel<TT, VV><<<grid, block, shm, as_stream(stream)>>>(                                   \
      static_cast<float*>(x), static_cast<const TT*>(y), static_cast<const float*>(post_w), static_cast<const TT*>(rows), \
      static_cast<const float*>(vec), static_cast<const float*>(w), w_offset, static_cast<TT*>(out), W, eps)
  if (dtype == LV_MIX_BF16) {
    if (vec4) LVMIX_SANDWICH(bf16_t, 4); else LVMIX_SANDWICH(bf16_t, 1);
  } else if (dtype == LV_MIX_F32) {
    if (vec4) LVMIX_SANDWICH(float, 4); else LVMIX_SANDWICH(float, 1);
  } else {
    return fail(-1, "lv_sandwich_add_norm: dtype %d", dtype);
  }
#undef LVMIX_SANDWICH
  return launched("lv_sandwich_add_norm");
}

int lv_rotary_store(const void* proj, int64_t ld, int off_q, int off_k, int off_v, const void* inv_freq,
                    const void* head_scale, void* q_out, void* k_cache, void* v_cache, const int32_t* cu_q,
                    const int32_t* ctx_lens, const int32_t* tok_seq, const int32_t* block_tables, int bt_stride, int64_t T,
                    int H, int G, int D, int Dv, int rot_dims, int page, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!proj || !q_out || !k_cache || !v_cache || !cu_q || !ctx_lens || !tok_seq || !block_tables)
    return fail(-1, "lv_rotary_store: null pointer");
  if (T < 0 || H <= 0 || G <= 0 || H % G != 0 || D <= 0 || Dv <= 0 || page <= 0 || bt_stride <= 0 || rot_dims < 0 ||
      rot_dims > D || rot_dims % 2 != 0 || (rot_dims > 0 && !inv_freq) || off_q < 0 || off_k < 0 || off_v < 0 ||
      off_q + static_cast<int64_t>(H) * D > ld || off_k + static_cast<int64_t>(G) * D > ld ||
      off_v + static_cast<int64_t>(G) * Dv > ld)
    return fail(-1, "lv_rotary_store: bad sizes");
  const size_t shm = sizeof(float) * static_cast<size_t>(rot_dims > 0 ? rot_dims : 4);
  dim3 grid(static_cast<unsigned>(T)), block(256);
  auto aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  // groups of four: head sizes, both halves of the rotated part and every column offset in multiples of 4
  const bool vec4 = D % 4 == 0 && Dv % 4 == 0 && rot_dims % 8 == 0 && ld % 4 == 0 && off_q % 4 == 0 && off_k % 4 == 0 &&
                    off_v % 4 == 0 && aligned(proj) && aligned(q_out) && aligned(k_cache) && aligned(v_cache);
#define LVMIX_ROTARY(TT, VV)                                                                                          \
  rotary_store_kernel<TT, VV><<<grid, block, shm, as_stream(stream)>>>(                                               \
      static_cast<const TT*>(proj), ld, off_q, off_k, off_v, static_cast<const float*>(inv_freq),                     \
      static_cast<const float*>(head_scale), static_cast<TT*>(q_out), static_cast<TT*>(k_cache), static_cast<TT*>(v_cache), \
      cu_q, ctx_lens, tok_seq, block_tables, bt_stride, H, G, D, Dv, rot_dims, page)
  if (dtype == LV_MIX_BF16) {
    if (vec4) LVMIX_ROTARY(bf16_t, 4); else LVMIX_ROTARY(bf16_t, 1);
  } else if (dtype == LV_MIX_F32) {
    if (vec4) LVMIX_ROTARY(float, 4); else LVMIX_ROTARY(float, 1);
  } else {
    return fail(-1, "lv_rotary_store: dtype %d", dtype);
  }
#undef LVMIX_ROTARY
  return launched("lv_rotary_store");
}

int lv_polynorm(const void* in, int64_t ld_in, const void* coef, void* out, int64_t T, int F, float eps, int dtype,
                void* stream) {
  if (T == 0) return 0;
  if (!in || !coef || !out || T < 0 || F <= 0 || ld_in < F) return fail(-1, "lv_polynorm: bad arguments");
  dim3 grid(static_cast<unsigned>(T)), block(256);
  const bool vec4 = F % 4 == 0 && ld_in % 4 == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0 &&
                    (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#define LVMIX_POLY(TT, VV)                                                                                   \
  polynorm_kernel<TT, VV><<<grid, block, 0, as_stream(stream)>>>(static_cast<const TT*>(in), ld_in,          \
                                                                 static_cast<const float*>(coef), static_cast<TT*>(out), F, eps)
  if (dtype == LV_MIX_BF16) {
    if (vec4) LVMIX_POLY(bf16_t, 4); else LVMIX_POLY(bf16_t, 1);
  } else if (dtype == LV_MIX_F32) {
    if (vec4) LVMIX_POLY(float, 4); else LVMIX_POLY(float, 1);
  } else {
    return fail(-1, "lv_polynorm: dtype %d", dtype);
  }
#undef LVMIX_POLY
  return launched("lv_polynorm");
}

int lv_expert_glu(const void* in, int64_t ld_in, const void* in_scale, const void* out_gate, int64_t ld_gate, void* out,
                  int64_t ld_out, int64_t T, int E, int F, float limit, float alpha, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!in || !out || T < 0 || E <= 0 || F <= 0 || ld_in < static_cast<int64_t>(E) * 2 * F || ld_out < static_cast<int64_t>(E) * F)
    return fail(-1, "lv_expert_glu: bad arguments");
  const int64_t n = T * E * F;
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
  if (dtype == LV_MIX_BF16)
    expert_glu_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const bf16_t*>(in), ld_in, static_cast<const float*>(in_scale), static_cast<const bf16_t*>(out_gate),
        ld_gate, static_cast<bf16_t*>(out), ld_out, T, E, F, limit, alpha);
  else if (dtype == LV_MIX_F32)
    expert_glu_kernel<float><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(in), ld_in, static_cast<const float*>(in_scale), static_cast<const float*>(out_gate),
        ld_gate, static_cast<float*>(out), ld_out, T, E, F, limit, alpha);
  else
    return fail(-1, "lv_expert_glu: dtype %d", dtype);
  return launched("lv_expert_glu");
}

}  // extern "C"
