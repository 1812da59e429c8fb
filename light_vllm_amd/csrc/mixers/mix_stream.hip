// Residual-stream kernels and the gated delta rule.
//
//   hc_update_norm_kernel     one workgroup per token: the S residual streams are remixed and receive the
//                             sublayer output, and in the same pass the next sublayer's input is read out
//                             of them and normalised in groups. Streams and all arithmetic are f32.
//   residual_add_norm_kernel  one workgroup per token: the single f32 residual receives the sum of up to two
//                             sublayer outputs and is normalised for the next layer, weight (offset + w).
//   clamped_glu_kernel        elementwise gate of the feed-forward.
//   delta_prep_kernel         one wave per (token, head slot): convolution taps from the step's own rows
//                             or the carried state, silu, unit norm; one more wave per token for the
//                             write strength and the decay (one per head, or one wave per head when every
//                             key channel has a decay of its own).
//   conv_state_update_kernel  one thread per (sequence, channel) shifts the carried inputs.
//   gated_delta_rule_kernel   one workgroup per (64 value columns, head, sequence) walks the step's tokens;
//                             each lane owns one column of the state, the four waves own a quarter of the
//                             rows each, partial dot products meet in LDS once per token. The decay is one
//                             number per head, or one for each key channel of it (a row of the state).
//   head_norm_gate_kernel     one wave per (token, head).
#include "mix_common.h"

namespace lvmix {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int launched(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(-3, "%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

// ------------------------------------------------------------------------------------------------
template <typename T, int S>
__global__ __launch_bounds__(256) void hc_update_norm_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                              const float* __restrict__ mix,
                                                              const float* __restrict__ out_w,
                                                              const float* __restrict__ in_w,
                                                              const float* __restrict__ norm_w, T* __restrict__ out,
                                                              int W, int groups, float eps) {
  extern __shared__ float lds[];          // [W] read-out, then [groups] inverse rms
  float* u_lds = lds;
  float* inv_lds = lds + W;
  const int64_t t = blockIdx.x;
  float* xt = x + t * S * W;
  float m[S][S], ow[S], iw[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    ow[s] = y != nullptr ? out_w[s] : 0.0f;
    iw[s] = out != nullptr ? in_w[s] : 0.0f;
#pragma unroll
    for (int r = 0; r < S; ++r) m[s][r] = y != nullptr ? mix[s * S + r] : 0.0f;
  }
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float xs[S];
#pragma unroll
    for (int s = 0; s < S; ++s) xs[s] = xt[s * W + i];
    if (y != nullptr) {
      const float yv = ldf(y + t * W + i);
      float nx[S];
#pragma unroll
      for (int r = 0; r < S; ++r) {
        float acc = ow[r] * yv;
#pragma unroll
        for (int s = 0; s < S; ++s) acc += m[s][r] * xs[s];
        nx[r] = acc;
      }
#pragma unroll
      for (int s = 0; s < S; ++s) {
        xs[s] = nx[s];
        xt[s * W + i] = nx[s];
      }
    }
    if (out != nullptr) {
      float u = 0.0f;
#pragma unroll
      for (int s = 0; s < S; ++s) u += iw[s] * xs[s];
      u_lds[i] = u;
    }
  }
  if (out == nullptr) return;
  __syncthreads();
  const int gs = W / groups;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, nwaves = blockDim.x / kWave;
  for (int g = wave; g < groups; g += nwaves) {
    float ss = 0.0f;
    for (int i = lane; i < gs; i += kWave) {
      const float v = u_lds[g * gs + i];
      ss += v * v;
    }
    ss = wave_sum(ss);
    if (lane == 0) inv_lds[g] = 1.0f / sqrtf(ss / static_cast<float>(gs) + eps);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    stf(out + t * W + i, u_lds[i] * inv_lds[i / gs] * norm_w[i]);
}

template <typename T>
static int hc_launch(void* x, const void* y, const void* mix, const void* out_w, const void* in_w,
                     const void* norm_w, void* out, int64_t Tn, int S, int W, int groups, float eps,
                     hipStream_t stream) {
  const size_t shm = static_cast<size_t>(W + groups) * sizeof(float);
  dim3 grid(static_cast<unsigned>(Tn)), block(256);
#define LVMIX_HC(SS)                                                                                            \
  case SS:                                                                                                      \
    hc_update_norm_kernel<T, SS><<<grid, block, shm, stream>>>(                                                 \
        static_cast<float*>(x), static_cast<const T*>(y), static_cast<const float*>(mix),                       \
        static_cast<const float*>(out_w), static_cast<const float*>(in_w), static_cast<const float*>(norm_w),   \
        static_cast<T*>(out), W, groups, eps);                                                                  \
    break;
  switch (S) {
    LVMIX_HC(1) LVMIX_HC(2) LVMIX_HC(3) LVMIX_HC(4) LVMIX_HC(5) LVMIX_HC(6) LVMIX_HC(7) LVMIX_HC(8)
    default: return fail(-2, "lv_hc_update_norm: %d streams (1..%d supported)", S, LV_MIX_MAX_STREAMS);
  }
#undef LVMIX_HC
  return launched("lv_hc_update_norm");
}

// ------------------------------------------------------------------------------------------------
// x f32 [T, W] += y1 + y2 (either may be absent); out = x / sqrt(mean(x^2) + eps) * (w_offset + w).
// Four elements per thread and access (16-byte loads of the residual, 8-byte loads of bf16 rows) when W is a multiple of 4.

template <typename T, int VEC>
__global__ __launch_bounds__(256) void residual_add_norm_kernel(float* __restrict__ x, const T* __restrict__ y1,
                                                                 const T* __restrict__ y2, const float* __restrict__ w,
                                                                 float w_offset, T* __restrict__ out, int W, float eps) {
  extern __shared__ __attribute__((aligned(16))) float lds[];          // [W] the updated row, then [4] partial sums
  float* red = lds + W;
  const int64_t t = blockIdx.x;
  float* xt = x + t * W;
  float ss = 0.0f;
  if (VEC == 4) {
    for (int i = threadIdx.x * 4; i < W; i += blockDim.x * 4) {
      float4 v = ld4(xt + i);
      if (y1 != nullptr || y2 != nullptr) {
        float4 add = y1 != nullptr ? ld4(y1 + t * W + i) : float4{0.0f, 0.0f, 0.0f, 0.0f};
        if (y2 != nullptr) {
          const float4 b = ld4(y2 + t * W + i);
          add.x += b.x; add.y += b.y; add.z += b.z; add.w += b.w;
        }
        v.x += add.x; v.y += add.y; v.z += add.z; v.w += add.w;
        st4(xt + i, v);
      }
      st4(lds + i, v);
      ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float v = xt[i];
      if (y1 != nullptr || y2 != nullptr) {
        float add = y1 != nullptr ? ldf(y1 + t * W + i) : 0.0f;
        if (y2 != nullptr) add += ldf(y2 + t * W + i);
        v += add;
        xt[i] = v;
      }
      lds[i] = v;
      ss += v * v;
    }
  }
  if (out == nullptr) return;
  ss = wave_sum(ss);
  if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = ss;
  __syncthreads();
  const float inv = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / static_cast<float>(W) + eps);
  if (VEC == 4) {
    for (int i = threadIdx.x * 4; i < W; i += blockDim.x * 4) {       // each thread reads back what it wrote itself
      const float4 v = ld4(lds + i), g = ld4(w + i);
      st4(out + t * W + i, float4{v.x * inv * (w_offset + g.x), v.y * inv * (w_offset + g.y), v.z * inv * (w_offset + g.z),
                                  v.w * inv * (w_offset + g.w)});
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + t * W + i, lds[i] * inv * (w_offset + w[i]));
  }
}

// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const T* __restrict__ in, int64_t ld_in, T* __restrict__ out,
                                                          int64_t Tn, int F, float limit, float alpha) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= Tn * F) return;
  const int64_t t = idx / F;
  const int f = static_cast<int>(idx - t * F);
  const float g = fminf(ldf(in + t * ld_in + f), limit);
  const float u = fminf(fmaxf(ldf(in + t * ld_in + F + f), -limit), limit);
  stf(out + idx, g * sigmoidf_(alpha * g) * (u + 1.0f));
}

// bf16 rows whose halves start on 16-byte boundaries: eight elements per thread, 16-byte loads and stores.
__global__ __launch_bounds__(256) void clamped_glu_bf16x8_kernel(const uint16_t* __restrict__ in, int64_t ld_in,
                                                                 uint16_t* __restrict__ out, int64_t Tn, int F8,
                                                                 float limit, float alpha) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= Tn * F8) return;
  const int64_t t = idx / F8;
  const int f = static_cast<int>(idx - t * F8) * 8;
  const uint4 gv = *reinterpret_cast<const uint4*>(in + t * ld_in + f);
  const uint4 uv = *reinterpret_cast<const uint4*>(in + t * ld_in + static_cast<int64_t>(F8) * 8 + f);
  const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
  uint32_t ow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float r[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const float gx = __builtin_bit_cast(float, half ? (gw[i] & 0xffff0000u) : (gw[i] << 16));
      const float ux = __builtin_bit_cast(float, half ? (uw[i] & 0xffff0000u) : (uw[i] << 16));
      const float g = fminf(gx, limit);
      const float u = fminf(fmaxf(ux, -limit), limit);
      r[half] = g * sigmoidf_(alpha * g) * (u + 1.0f);
    }
    bf16_t lo, hi;
    stf(&lo, r[0]);
    stf(&hi, r[1]);
    ow[i] = static_cast<uint32_t>(lo.bits) | (static_cast<uint32_t>(hi.bits) << 16);
  }
  *reinterpret_cast<uint4*>(out + idx * 8) = uint4{ow[0], ow[1], ow[2], ow[3]};
}

// ------------------------------------------------------------------------------------------------
struct DeltaPrepParams {
  const void* proj;
  int64_t ld;
  const float* conv_w;
  const void* conv_state;
  const float* A_log;
  const float* dt_bias;
  const int32_t *cu_q, *ctx_lens, *slots, *tok_seq;
  float *qn, *kn, *v, *beta, *decay;
  int64_t T;
  int G, H, D, Dv, taps, off_b;
  float unit_eps;
  const void* a;      // decay inputs, rows of stride ld_a: H numbers, or H * D when dec_dim == D
  int64_t ld_a;
  int dec_dim;        // 1: one decay per head; D: one for each of its key channels (dt_bias is as wide as a row of a)
};

template <typename T>
__global__ __launch_bounds__(256) void delta_prep_kernel(DeltaPrepParams p) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t t = blockIdx.x;
  const int unit = blockIdx.y * (blockDim.x / kWave) + wave;
  const int base_units = 2 * p.G + p.H + 1;
  const int units = base_units + (p.dec_dim > 1 ? p.H : 0);
  if (unit >= units) return;
  const T* proj = static_cast<const T*>(p.proj);
  const T* arow = static_cast<const T*>(p.a) + blockIdx.x * p.ld_a;
  if (unit >= base_units) {                       // decays of one head, one per key channel
    const int h = unit - base_units;
    const float rate = expf(p.A_log[h]);
    for (int d = lane; d < p.dec_dim; d += kWave) {
      const int i = h * p.dec_dim + d;
      p.decay[blockIdx.x * static_cast<int64_t>(p.H) * p.dec_dim + i] = expf(-rate * softplusf_(ldf(arow + i) + p.dt_bias[i]));
    }
    return;
  }
  const int b = p.tok_seq[t];
  const int q0 = p.cu_q[b];
  const int r = static_cast<int>(t) - q0;         // index of the token inside its sequence's portion
  const int ctx = p.ctx_lens[b];
  if (unit == base_units - 1) {                   // write strength and (per-head) decay, one lane per head
    for (int h = lane; h < p.H; h += kWave) {
      const float bv = ldf(proj + t * p.ld + p.off_b + h);
      p.beta[t * p.H + h] = sigmoidf_(bv);
      if (p.dec_dim == 1) p.decay[t * p.H + h] = expf(-expf(p.A_log[h]) * softplusf_(ldf(arow + h) + p.dt_bias[h]));
    }
    return;
  }
  const int C = 2 * p.G * p.D + p.H * p.Dv;
  const int taps = p.taps;
  const T* state = static_cast<const T*>(p.conv_state) + static_cast<int64_t>(p.slots[b]) * (taps - 1) * C;
  int c0, n;
  float* dst;
  bool unit_norm = true;
  float post = 1.0f;
  if (unit < p.G) {
    c0 = unit * p.D; n = p.D; dst = p.qn + (t * p.G + unit) * p.D; post = 1.0f / sqrtf(static_cast<float>(p.D));
  } else if (unit < 2 * p.G) {
    c0 = p.G * p.D + (unit - p.G) * p.D; n = p.D; dst = p.kn + (t * p.G + (unit - p.G)) * p.D;
  } else {
    const int h = unit - 2 * p.G;
    c0 = 2 * p.G * p.D + h * p.Dv; n = p.Dv; dst = p.v + (t * p.H + h) * p.Dv; unit_norm = false;
  }
  float ss = 0.0f;
  for (int e = lane; e < n; e += kWave) {
    const int c = c0 + e;
    float acc = 0.0f;
    for (int i = 0; i < taps; ++i) {
      const int rr = r - (taps - 1 - i);          // row of the portion this tap reads
      float xin = 0.0f;
      if (rr >= 0) xin = ldf(proj + static_cast<int64_t>(q0 + rr) * p.ld + c);
      else if (ctx + rr >= 0) xin = ldf(state + static_cast<int64_t>(taps - 1 + rr) * C + c);
      acc += p.conv_w[c * taps + i] * xin;
    }
    const float a = siluf_(acc);
    dst[e] = a;
    ss += a * a;
  }
  if (!unit_norm) return;
  ss = wave_sum(ss);
  const float inv = post / sqrtf(ss + p.unit_eps);
  for (int e = lane; e < n; e += kWave) dst[e] *= inv;    // each lane rescales what it wrote itself
}

template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(const T* __restrict__ proj, int64_t ld,
                                                                T* __restrict__ conv_state,
                                                                const int32_t* __restrict__ cu_q,
                                                                const int32_t* __restrict__ ctx_lens,
                                                                const int32_t* __restrict__ slots, int C, int taps) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int q0 = cu_q[b], n = cu_q[b + 1] - q0, ctx = ctx_lens[b];
  if (n <= 0) return;
  T* state = conv_state + static_cast<int64_t>(slots[b]) * (taps - 1) * C;
  // new row s holds the input of position ctx + n - (taps-1) + s; ascending s reads old rows above s only
  for (int s = 0; s < taps - 1; ++s) {
    const int rr = n - (taps - 1) + s;
    float v = 0.0f;
    if (rr >= 0) v = ldf(proj + static_cast<int64_t>(q0 + rr) * ld + c);
    else if (ctx + rr >= 0) v = ldf(state + static_cast<int64_t>(taps - 1 + rr) * C + c);
    stf(state + static_cast<int64_t>(s) * C + c, v);
  }
}

// ------------------------------------------------------------------------------------------------
struct DeltaRuleParams {
  const float *qn, *kn, *v, *beta, *decay;
  float* state;
  const int32_t *cu_q, *ctx_lens, *slots;
  float* o;
  int G, H, D, Dv;
};
// decay: [T, H] (one number per head) or, in the kernel's CH form, [T, H, D] (one per row of the state).

// DR = rows of the state each of the four waves owns (4 * DR >= D; rows beyond D stay zero).
// Tokens are taken in chunks of kDeltaChunk: the chunk's unit keys and queries, values, write strengths and
// decays are staged in LDS by all threads at once (one round of global latency per chunk instead of one
// per token), then each token costs LDS reads, 2 * DR multiply-adds per lane and one barrier.
constexpr int kDeltaChunk = 16;

template <int DR, bool CH>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(DeltaRuleParams p) {
  extern __shared__ __attribute__((aligned(16))) float dl[];
  constexpr int DP = 4 * DR;                       // padded key size
  float* k_lds = dl;                               // [chunk][DP]
  float* q_lds = k_lds + kDeltaChunk * DP;         // [chunk][DP]
  float* v_lds = q_lds + kDeltaChunk * DP;         // [chunk][64]
  float* bd_lds = v_lds + kDeltaChunk * kWave;     // [chunk][2]: beta, decay
  float* part_k = bd_lds + kDeltaChunk * 2;        // [2][4][64]
  float* part_o = part_k + 2 * 4 * kWave;          // [2][4][64]
  float* o_lds = part_o + 2 * 4 * kWave;           // [chunk][64]: read-outs leave for memory once per chunk
  float* g_lds = o_lds + kDeltaChunk * kWave;      // CH: [chunk][DP] decays per row
  const int lane = threadIdx.x % kWave, rp = threadIdx.x / kWave;
  const int col = blockIdx.x * kWave + lane;
  const int h = blockIdx.y, b = blockIdx.z;
  const int g = h / (p.H / p.G);
  const int q0 = p.cu_q[b], n = p.cu_q[b + 1] - q0;
  if (n <= 0) return;
  const bool live = col < p.Dv;
  const int row0 = rp * DR;
  float* sbase = p.state + (static_cast<int64_t>(p.slots[b]) * p.H + h) * p.D * p.Dv;
  float s[DR];
  const bool carry = p.ctx_lens[b] > 0;
#pragma unroll
  for (int r = 0; r < DR; ++r)
    s[r] = (carry && live && row0 + r < p.D) ? sbase[static_cast<int64_t>(row0 + r) * p.Dv + col] : 0.0f;

  for (int c0 = 0; c0 < n; c0 += kDeltaChunk) {
    const int cn = min(kDeltaChunk, n - c0);
    __syncthreads();                               // the previous chunk is consumed (its last read-out included)
    for (int x = threadIdx.x; x < cn * DP; x += blockDim.x) {
      const int tok = x / DP, d = x - tok * DP;
      const int64_t t = q0 + c0 + tok;
      const bool in = d < p.D;
      k_lds[x] = in ? p.kn[(t * p.G + g) * p.D + d] : 0.0f;
      q_lds[x] = in ? p.qn[(t * p.G + g) * p.D + d] : 0.0f;
      if (CH) g_lds[x] = in ? p.decay[(t * p.H + h) * p.D + d] : 1.0f;
    }
    for (int x = threadIdx.x; x < cn * kWave; x += blockDim.x) {
      const int tok = x / kWave, cc = blockIdx.x * kWave + (x % kWave);
      const int64_t t = q0 + c0 + tok;
      v_lds[x] = cc < p.Dv ? p.v[(t * p.H + h) * p.Dv + cc] : 0.0f;
    }
    if (threadIdx.x < cn) {
      const int64_t t = q0 + c0 + threadIdx.x;
      bd_lds[threadIdx.x * 2] = p.beta[t * p.H + h];
      bd_lds[threadIdx.x * 2 + 1] = CH ? 1.0f : p.decay[t * p.H + h];
    }
    __syncthreads();
    for (int i = 0; i < cn; ++i) {
      const int buf = i & 1;
      float kr[DR], qr[DR];
#pragma unroll
      for (int r = 0; r < DR; r += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(k_lds + i * DP + row0 + r);
        const float4 q4 = *reinterpret_cast<const float4*>(q_lds + i * DP + row0 + r);
        kr[r] = k4.x; kr[r + 1] = k4.y; kr[r + 2] = k4.z; kr[r + 3] = k4.w;
        qr[r] = q4.x; qr[r + 1] = q4.y; qr[r + 2] = q4.z; qr[r + 3] = q4.w;
      }
      if (CH) {                                     // rows decay one by one, before anything reads them
#pragma unroll
        for (int r = 0; r < DR; r += 4) {
          const float4 g4 = *reinterpret_cast<const float4*>(g_lds + i * DP + row0 + r);
          s[r] *= g4.x; s[r + 1] *= g4.y; s[r + 2] *= g4.z; s[r + 3] *= g4.w;
        }
      }
      const float beta = bd_lds[i * 2], dec = bd_lds[i * 2 + 1];
      const float vv = v_lds[i * kWave + lane];
      float pk4[4] = {0.0f, 0.0f, 0.0f, 0.0f};     // four chains: the sums are latency-bound otherwise
#pragma unroll
      for (int r = 0; r < DR; ++r) pk4[r & 3] += s[r] * kr[r];
      part_k[(buf * 4 + rp) * kWave + lane] = (pk4[0] + pk4[1]) + (pk4[2] + pk4[3]);
      __syncthreads();
      // the previous token's read-out partials are complete behind this barrier as well
      if (i > 0 && rp == ((i - 1) & 3)) {
        const float* po_ = part_o + (buf ^ 1) * 4 * kWave + lane;
        o_lds[(i - 1) * kWave + lane] = po_[0] + po_[kWave] + po_[2 * kWave] + po_[3 * kWave];
      }
      const float* pk_ = part_k + buf * 4 * kWave + lane;
      const float ks = pk_[0] + pk_[kWave] + pk_[2 * kWave] + pk_[3 * kWave];
      const float u = beta * (vv - dec * ks);       // the state is decayed before it is read
      float po4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int r = 0; r < DR; ++r) {
        s[r] = dec * s[r] + kr[r] * u;
        po4[r & 3] += s[r] * qr[r];
      }
      part_o[(buf * 4 + rp) * kWave + lane] = (po4[0] + po4[1]) + (po4[2] + po4[3]);
    }
    __syncthreads();
    if (rp == 0) {                                  // the chunk's last token
      const float* po_ = part_o + ((cn - 1) & 1) * 4 * kWave + lane;
      o_lds[(cn - 1) * kWave + lane] = po_[0] + po_[kWave] + po_[2 * kWave] + po_[3 * kWave];
    }
    __syncthreads();
    for (int x = threadIdx.x; x < cn * kWave; x += blockDim.x) {
      const int tok = x / kWave, cc = blockIdx.x * kWave + (x % kWave);
      if (cc < p.Dv) p.o[((static_cast<int64_t>(q0) + c0 + tok) * p.H + h) * p.Dv + cc] = o_lds[x];
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < DR; ++r)
      if (row0 + r < p.D) sbase[static_cast<int64_t>(row0 + r) * p.Dv + col] = s[r];
  }
}

template <int DR>
static void delta_rule_launch(const DeltaRuleParams& p, dim3 grid, hipStream_t s, bool per_channel) {
  const size_t shm = sizeof(float) * ((per_channel ? 3 : 2) * kDeltaChunk * 4 * DR + 2 * kDeltaChunk * kWave +
                                      kDeltaChunk * 2 + 4 * 4 * kWave);
  if (per_channel) gated_delta_rule_kernel<DR, true><<<grid, dim3(256), shm, s>>>(p);
  else gated_delta_rule_kernel<DR, false><<<grid, dim3(256), shm, s>>>(p);
}

// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                             int64_t ld_gate, const float* __restrict__ norm_w,
                                                             T* __restrict__ out, int64_t items, int H, int Dv,
                                                             float eps, int gate_act) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + wave;   // (token, head)
  if (item >= items) return;
  const int64_t t = item / H;
  const int h = static_cast<int>(item - t * H);
  const float* row = o + item * Dv;
  float ss = 0.0f;
  for (int e = lane; e < Dv; e += kWave) ss += row[e] * row[e];
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(Dv) + eps);
  for (int e = lane; e < Dv; e += kWave) {
    const float gv = ldf(gate + t * ld_gate + h * Dv + e);
    stf(out + item * Dv + e, row[e] * inv * norm_w[e] * (gate_act == LV_MIX_GATE_SILU ? siluf_(gv) : sigmoidf_(gv)));
  }
}

// The same for heads of many entries (a norm over a whole row of heads is one such head): one workgroup per (token, head),
// four entries per thread and access.
template <typename T>
__global__ __launch_bounds__(256) void wide_head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                                  int64_t ld_gate, const float* __restrict__ norm_w,
                                                                  T* __restrict__ out, int H, int Dv, float eps, int gate_act) {
  __shared__ float red[4];
  const int64_t item = blockIdx.x;
  const int64_t t = item / H;
  const int h = static_cast<int>(item - t * H);
  const float* row = o + item * Dv;
  float ss = 0.0f;
  for (int e = threadIdx.x * 4; e < Dv; e += blockDim.x * 4) {
    const float4 v = ld4(row + e);
    ss += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
  }
  ss = wave_sum(ss);
  if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = ss;
  __syncthreads();
  const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / static_cast<float>(Dv) + eps);
  const T* grow = gate + t * ld_gate + static_cast<int64_t>(h) * Dv;
  auto act = [&](float g) { return gate_act == LV_MIX_GATE_SILU ? siluf_(g) : sigmoidf_(g); };
  for (int e = threadIdx.x * 4; e < Dv; e += blockDim.x * 4) {
    const float4 v = ld4(row + e), w = ld4(norm_w + e), g = ld4(grow + e);
    st4(out + item * Dv + e, float4{v.x * inv * w.x * act(g.x), v.y * inv * w.y * act(g.y), v.z * inv * w.z * act(g.z),
                                    v.w * inv * w.w * act(g.w)});
  }
}

}  // namespace lvmix

using namespace lvmix;

extern "C" {

int lv_mix_abi_version(void) { return LV_MIX_ABI_VERSION; }
const char* lv_mix_last_error(void) { return lvmix::g_err; }

int lv_hc_update_norm(void* x, const void* y, const void* mix, const void* out_w, const void* in_w,
                      const void* norm_w, void* out, int64_t T, int S, int W, int groups, float eps, int dtype,
                      void* stream) {
  if (T == 0) return 0;
  if (x == nullptr || T < 0 || W <= 0) return fail(-1, "lv_hc_update_norm: bad arguments");
  if (y != nullptr && (mix == nullptr || out_w == nullptr)) return fail(-1, "lv_hc_update_norm: y without mix/out_w");
  if (out != nullptr && (in_w == nullptr || norm_w == nullptr || groups <= 0 || W % groups != 0))
    return fail(-1, "lv_hc_update_norm: read-out needs in_w, norm_w and groups dividing W (%d, %d)", W, groups);
  if (static_cast<size_t>(W + groups) * 4 > 160 * 1024) return fail(-2, "lv_hc_update_norm: width %d too large", W);
  if (dtype == LV_MIX_BF16)
    return hc_launch<bf16_t>(x, y, mix, out_w, in_w, norm_w, out, T, S, W, groups > 0 ? groups : 1, eps, as_stream(stream));
  if (dtype == LV_MIX_F32)
    return hc_launch<float>(x, y, mix, out_w, in_w, norm_w, out, T, S, W, groups > 0 ? groups : 1, eps, as_stream(stream));
  return fail(-1, "lv_hc_update_norm: dtype %d", dtype);
}

int lv_residual_add_norm(void* x, const void* y1, const void* y2, const void* w, float w_offset, void* out, int64_t T,
                         int W, float eps, int dtype, void* stream) {
  if (T == 0) return 0;
  if (x == nullptr || T < 0 || W <= 0 || (out != nullptr && w == nullptr)) return fail(-1, "lv_residual_add_norm: bad arguments");
  if (out == nullptr && y1 == nullptr && y2 == nullptr) return 0;
  const size_t shm = static_cast<size_t>(W + 4) * sizeof(float);
  if (shm > 64 * 1024) return fail(-2, "lv_residual_add_norm: width %d too large", W);
  dim3 grid(static_cast<unsigned>(T)), block(256);
  auto aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec = W % 4 == 0 && aligned(x) && aligned(y1) && aligned(y2) && aligned(w) && aligned(out);
#define LVMIX_RES(TT, VV)                                                                                       \
  residual_add_norm_kernel<TT, VV><<<grid, block, shm, as_stream(stream)>>>(                                   \
      static_cast<float*>(x), static_cast<const TT*>(y1), static_cast<const TT*>(y2), static_cast<const float*>(w), \
      w_offset, static_cast<TT*>(out), W, eps)
  if (dtype == LV_MIX_BF16) {
    if (vec) LVMIX_RES(bf16_t, 4); else LVMIX_RES(bf16_t, 1);
  } else if (dtype == LV_MIX_F32) {
    if (vec) LVMIX_RES(float, 4); else LVMIX_RES(float, 1);
  } else {
    return fail(-1, "lv_residual_add_norm: dtype %d", dtype);
  }
#undef LVMIX_RES
  return launched("lv_residual_add_norm");
}

int lv_clamped_glu(const void* in, int64_t ld_in, void* out, int64_t T, int F, float limit, float alpha, int dtype,
                   void* stream) {
  if (T == 0) return 0;
  if (in == nullptr || out == nullptr || T < 0 || F <= 0 || ld_in < 2 * F) return fail(-1, "lv_clamped_glu: bad arguments");
  const int64_t n = T * F;
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), block(256);
  if (dtype == LV_MIX_BF16 && F % 8 == 0 && ld_in % 8 == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    dim3 grid8(static_cast<unsigned>((n / 8 + 255) / 256));
    clamped_glu_bf16x8_kernel<<<grid8, block, 0, as_stream(stream)>>>(static_cast<const uint16_t*>(in), ld_in,
                                                                     static_cast<uint16_t*>(out), T, F / 8, limit, alpha);
  } else if (dtype == LV_MIX_BF16)
    clamped_glu_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(static_cast<const bf16_t*>(in), ld_in,
                                                                    static_cast<bf16_t*>(out), T, F, limit, alpha);
  else if (dtype == LV_MIX_F32)
    clamped_glu_kernel<float><<<grid, block, 0, as_stream(stream)>>>(static_cast<const float*>(in), ld_in,
                                                                   static_cast<float*>(out), T, F, limit, alpha);
  else
    return fail(-1, "lv_clamped_glu: dtype %d", dtype);
  return launched("lv_clamped_glu");
}

int lv_delta_prep(const void* proj, int64_t ld, const void* conv_w, const void* conv_state, const void* A_log,
                  const void* dt_bias, const int32_t* cu_q, const int32_t* ctx_lens, const int32_t* slots,
                  const int32_t* tok_seq, void* qn, void* kn, void* v, void* beta, void* decay, int64_t T, int G,
                  int H, int D, int Dv, int taps, int off_b, const void* a, int64_t ld_a, int decay_per_channel,
                  float unit_eps, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!proj || !conv_w || (!conv_state && taps > 1) || !A_log || !dt_bias || !cu_q || !ctx_lens || !slots || !tok_seq || !qn ||
      !kn || !v || !beta || !decay || !a)
    return fail(-1, "lv_delta_prep: null pointer");
  if (G <= 0 || H <= 0 || H % G != 0 || D <= 0 || Dv <= 0 || taps < 1) return fail(-1, "lv_delta_prep: bad sizes");
  const int C = 2 * G * D + H * Dv;
  const int dec_dim = decay_per_channel ? D : 1;
  if (ld < C || off_b + H > ld || ld_a < static_cast<int64_t>(H) * dec_dim)
    return fail(-1, "lv_delta_prep: row stride %lld / %lld too small", (long long)ld, (long long)ld_a);
  DeltaPrepParams p{proj, ld, static_cast<const float*>(conv_w), conv_state, static_cast<const float*>(A_log),
                    static_cast<const float*>(dt_bias), cu_q, ctx_lens, slots, tok_seq, static_cast<float*>(qn),
                    static_cast<float*>(kn), static_cast<float*>(v), static_cast<float*>(beta),
                    static_cast<float*>(decay), T, G, H, D, Dv, taps, off_b, unit_eps, a, ld_a, dec_dim};
  const int units = 2 * G + H + 1 + (dec_dim > 1 ? H : 0);
  dim3 grid(static_cast<unsigned>(T), (units + 3) / 4), block(256);
  if (dtype == LV_MIX_BF16) delta_prep_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(p);
  else if (dtype == LV_MIX_F32) delta_prep_kernel<float><<<grid, block, 0, as_stream(stream)>>>(p);
  else return fail(-1, "lv_delta_prep: dtype %d", dtype);
  return launched("lv_delta_prep");
}

int lv_conv_state_update(const void* proj, int64_t ld, void* conv_state, const int32_t* cu_q, const int32_t* ctx_lens,
                         const int32_t* slots, int B, int C, int taps, int dtype, void* stream) {
  if (B == 0 || taps <= 1) return 0;
  if (!proj || !conv_state || !cu_q || !ctx_lens || !slots || B < 0 || C <= 0 || ld < C)
    return fail(-1, "lv_conv_state_update: bad arguments");
  dim3 grid((C + 255) / 256, B), block(256);
  if (dtype == LV_MIX_BF16)
    conv_state_update_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const bf16_t*>(proj), ld, static_cast<bf16_t*>(conv_state), cu_q, ctx_lens, slots, C, taps);
  else if (dtype == LV_MIX_F32)
    conv_state_update_kernel<float><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(proj), ld, static_cast<float*>(conv_state), cu_q, ctx_lens, slots, C, taps);
  else
    return fail(-1, "lv_conv_state_update: dtype %d", dtype);
  return launched("lv_conv_state_update");
}

int lv_gated_delta_rule(const void* qn, const void* kn, const void* v, const void* beta, const void* decay, void* state,
                        const int32_t* cu_q, const int32_t* ctx_lens, const int32_t* slots, void* o, int B, int G,
                        int H, int D, int Dv, int decay_per_channel, void* stream) {
  if (B == 0) return 0;
  if (!qn || !kn || !v || !beta || !decay || !state || !cu_q || !ctx_lens || !slots || !o)
    return fail(-1, "lv_gated_delta_rule: null pointer");
  if (B < 0 || G <= 0 || H <= 0 || H % G != 0 || D <= 0 || Dv <= 0) return fail(-1, "lv_gated_delta_rule: bad sizes");
  if (D > 256) return fail(-2, "lv_gated_delta_rule: key size %d above 256", D);
  DeltaRuleParams p{static_cast<const float*>(qn), static_cast<const float*>(kn), static_cast<const float*>(v),
                    static_cast<const float*>(beta), static_cast<const float*>(decay), static_cast<float*>(state),
                    cu_q, ctx_lens, slots, static_cast<float*>(o), G, H, D, Dv};
  dim3 grid((Dv + kWave - 1) / kWave, H, B);
  hipStream_t s = as_stream(stream);
  const bool ch = decay_per_channel != 0;
  if (D <= 32) delta_rule_launch<8>(p, grid, s, ch);
  else if (D <= 64) delta_rule_launch<16>(p, grid, s, ch);
  else if (D <= 128) delta_rule_launch<32>(p, grid, s, ch);
  else delta_rule_launch<64>(p, grid, s, ch);
  return launched("lv_gated_delta_rule");
}

int lv_head_norm_gate(const void* o, const void* gate, int64_t ld_gate, const void* norm_w, void* out, int64_t T,
                      int H, int Dv, float eps, int gate_act, int dtype, void* stream) {
  if (T == 0) return 0;
  if (!o || !gate || !norm_w || !out || T < 0 || H <= 0 || Dv <= 0 || ld_gate < static_cast<int64_t>(H) * Dv ||
      (gate_act != LV_MIX_GATE_SILU && gate_act != LV_MIX_GATE_SIGMOID))
    return fail(-1, "lv_head_norm_gate: bad arguments");
  const int64_t items = T * H;
  auto aligned = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  if (Dv >= 512 && Dv % 4 == 0 && ld_gate % 4 == 0 && aligned(o) && aligned(gate) && aligned(norm_w) && aligned(out) &&
      (dtype == LV_MIX_BF16 || dtype == LV_MIX_F32)) {
    dim3 wgrid(static_cast<unsigned>(items)), wblock(256);
    if (dtype == LV_MIX_BF16)
      wide_head_norm_gate_kernel<bf16_t><<<wgrid, wblock, 0, as_stream(stream)>>>(
          static_cast<const float*>(o), static_cast<const bf16_t*>(gate), ld_gate, static_cast<const float*>(norm_w),
          static_cast<bf16_t*>(out), H, Dv, eps, gate_act);
    else
      wide_head_norm_gate_kernel<float><<<wgrid, wblock, 0, as_stream(stream)>>>(
          static_cast<const float*>(o), static_cast<const float*>(gate), ld_gate, static_cast<const float*>(norm_w),
          static_cast<float*>(out), H, Dv, eps, gate_act);
    return launched("lv_head_norm_gate");
  }
  dim3 grid(static_cast<unsigned>((items + 3) / 4)), block(256);
  if (dtype == LV_MIX_BF16)
    head_norm_gate_kernel<bf16_t><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(o), static_cast<const bf16_t*>(gate), ld_gate, static_cast<const float*>(norm_w),
        static_cast<bf16_t*>(out), items, H, Dv, eps, gate_act);
  else if (dtype == LV_MIX_F32)
    head_norm_gate_kernel<float><<<grid, block, 0, as_stream(stream)>>>(
        static_cast<const float*>(o), static_cast<const float*>(gate), ld_gate, static_cast<const float*>(norm_w),
        static_cast<float*>(out), items, H, Dv, eps, gate_act);
  else
    return fail(-1, "lv_head_norm_gate: dtype %d", dtype);
  return launched("lv_head_norm_gate");
}

}  // extern "C"
