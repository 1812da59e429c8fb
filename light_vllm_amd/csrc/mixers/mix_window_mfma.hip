// Matrix-core form of the windowed pooled attention for bf16 activations and caches.
//
// One workgroup = one tile of 16 consecutive new tokens of one sequence, one kv head, up to four of its
// query heads (one per wave). Keys are walked in tiles of 64 entries, first the pooled blocks that any
// query of the tile may see, then the tokens from the first window start to the last query; what a
// query does not see (outside its window, a block not yet wholly before it, the future) is masked.
//
// Everything is computed transposed so that no operand changes layout between the two products:
//   S^T = K Q^T   v_mfma_f32_16x16x32_bf16 (one 16x16x16 step more when D is an odd multiple of 16), A = 16 keys x 32
//                 of D read straight from the cache rows with 16-byte loads, B = the wave's Q fragments (registers,
//                 loaded once); a lane ends up with 4 keys of ONE query, so the softmax statistics of a query live
//                 in 4 lanes (two shuffles) and
//   O^T += V^T P^T  takes the probabilities of two 16-key blocks as its B operand exactly as they lie (keys x
//                 queries), with A = V^T read as two 8-byte runs of keys from the 64-entry V tile that the four
//                 waves stage TRANSPOSED in LDS together.
// The sink is the initial state of the running softmax: maximum 0, sum 1.
#include "mix_common.h"

namespace lvmix {

typedef __attribute__((ext_vector_type(4))) short bf16x4_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

struct WindowMfmaParams {
  const uint16_t *q, *k_cache, *v_cache, *kp, *vp, *gate;
  int64_t ld_gate;
  int gate_dv;         // entries of a gate row per head: Dv (one per output channel) or 1 (one per head)
  uint16_t* out;
  const int32_t *cu_q, *ctx_lens, *block_tables;
  int bt_stride, H, G, D, Dv, page, window, P, PP, ngroups;
  float scale, sink;
  uint32_t m_page, m_P, m_nseg;   // floor(2^32 / d) of the three divisors the tile loop divides by (see fdiv)
  int nsplit;          // > 1 (launches of at most one query tile per sequence): grid.x = split of the key tiles
  float* ws;           // [T, H, nsplit, Dv + 4] partial read-outs, running maximum and sum
  int64_t k_ld, v_ld;  // elements between the rows of two cached tokens (G*D, G*Dv unless the caches are views of wider rows)
  float m0;            // start of the running maximum: the sink's score 0, or far below any score without a sink
  int keep_first;      // positions below this are seen from everywhere; they take the place of the pooled tiles (P == 0)
  int chunk;           // > 0: a query sees its own chunk of that many positions (counted from 0) up to itself; no window
  const float* sinks;  // [H] or NULL: a learned score per query head in place of the sink's 0
};

constexpr int kTileQ = 16;
constexpr int kTileK = 64;
constexpr int kMaxK32 = 8;     // D <= 256: 32-wide steps over D (template K32: 4 up to D = 128), plus one 16-wide when D % 32 == 16
constexpr int kLdk = kTileK + 4; // row stride (in keys) of the transposed V tile: rows stay 8-byte aligned
constexpr int kMaxDvb = 16;    // Dv <= 256
constexpr int kBtCache = 2048; // page ids of a sequence kept in LDS (longer sequences look them up in memory)

// n / d for 0 <= n < 2^31 with magic = floor(2^32 / d) (0xffffffff for d = 1): the estimate is the quotient or one
// less. The tile loop divides by the page size, the pool size and the row's segment count for every row address;
// the compiler's general 32-bit division is some forty instructions each and dominated the kernel.
__device__ __forceinline__ int fdiv(int n, int d, uint32_t magic) {
  const uint32_t q = __umulhi(static_cast<uint32_t>(n), magic);
  const uint32_t r = static_cast<uint32_t>(n) - q * static_cast<uint32_t>(d);
  return static_cast<int>(r >= static_cast<uint32_t>(d) ? q + 1 : q);
}

__device__ __forceinline__ short bf16_bits(float x) {
  __bf16 b = static_cast<__bf16>(x);
  return __builtin_bit_cast(short, b);
}

// AHEAD: the next tile's V rows, key-row addresses and (once the current scores are done) K fragments are fetched while
// the current tile is computed. That pays when a launch has few workgroups per compute unit (decoded tokens). A prompt's
// many tiles hide latency by occupancy instead, and every register counts there: with the 32 registers of a V tile held
// ahead the kernel fell from two waves a SIMD to one and ran 1.7x slower; K32 and DVB size the fragment arrays for the
// head sizes at hand for the same reason.
template <bool AHEAD, int K32, int DVB>
__global__ __launch_bounds__(256, (AHEAD || DVB > 8) ? 1 : 4) void window_pool_mfma_kernel(WindowMfmaParams p) {
  extern __shared__ uint16_t vs[];                      // V^T tile [Dv][kLdk]
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int ln = lane & 15, lg = lane >> 4;
  const int b = blockIdx.z;
  const int g = blockIdx.y / p.ngroups, hg = blockIdx.y % p.ngroups;
  const int q0 = p.cu_q[b], n = p.cu_q[b + 1] - q0;
  const int split = p.nsplit > 1 ? blockIdx.x : 0;
  const int r0 = p.nsplit > 1 ? 0 : blockIdx.x * kTileQ;
  if (r0 >= n) return;
  const int ctx = p.ctx_lens[b];
  const int nvalid = min(kTileQ, n - r0);
  const int i0 = ctx + r0, i1 = i0 + nvalid - 1;
  const bool qvalid = ln < nvalid;
  const int r = r0 + min(ln, nvalid - 1);
  const int pos = ctx + r;
  const int64_t t = q0 + r;
  const int rep = p.H / p.G;
  const int hloc = hg * 4 + wave;
  const bool active = hloc < rep;
  const int h = g * rep + min(hloc, rep - 1);
  const int D = p.D, Dv = p.Dv, page = p.page, P = p.P, W = p.window;
  const int nk32 = D / 32, ndvb = Dv / 16;
  const bool tail16 = (D & 16) != 0;
  const int64_t GD = static_cast<int64_t>(p.G) * D, GDv = static_cast<int64_t>(p.G) * Dv;
  const int32_t* bt_global = p.block_tables + static_cast<int64_t>(b) * p.bt_stride;
  // the sequence's page ids up to the last query's page, once, so that no row address waits for a second trip to memory
  __shared__ int32_t bt_lds[kBtCache];
  const int nbt = (ctx + r0 + nvalid - 1) / page + 1;
  const bool bt_cached = nbt <= kBtCache;
  if (bt_cached) {
    for (int x = threadIdx.x; x < nbt; x += blockDim.x) bt_lds[x] = bt_global[x];
    __syncthreads();
  }
  auto bt = [&](int idx) { return bt_cached ? bt_lds[idx] : bt_global[idx]; };

  bf16x8_t qf[K32];
  bf16x4_t qtail = bf16x4_t{0, 0, 0, 0};
  {
    const uint16_t* qrow = p.q + (t * p.H + h) * D;
#pragma unroll
    for (int kk = 0; kk < K32; ++kk)
      if (kk < nk32) qf[kk] = *reinterpret_cast<const bf16x8_t*>(qrow + 32 * kk + 8 * lg);
    if (tail16) qtail = *reinterpret_cast<const bf16x4_t*>(qrow + 32 * nk32 + 4 * lg);
  }
  f32x4_t acc_o[DVB];
#pragma unroll
  for (int d = 0; d < DVB; ++d) acc_o[d] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m = p.sinks != nullptr ? p.sinks[h] : p.m0, l = split == 0 ? p.sink : 0.0f;

  const int chunk = p.chunk, keep = p.keep_first;
  const int jlo = chunk > 0 ? (i0 / chunk) * chunk : max(0, i0 - W + 1);
  const int cstart = chunk > 0 ? (pos / chunk) * chunk : 0;                // first position of this lane's query's chunk
  // entries of the first phase: pooled blocks the last query sees, or (without a pool) kept first tokens before the token tiles
  const int nbmax = P > 0 ? ((chunk == 0 && i1 - W + 1 > 0) ? (i1 - W + 1) / P : 0) : min(keep, jlo);

  // The tiles of both phases as one list: [pooled tiles | token tiles]. The V rows of the next tile and the
  // addresses of its key rows are fetched while the current tile is computed; they meet LDS behind a barrier.
  const int npt = (nbmax + kTileK - 1) / kTileK;
  const int ntt = (i1 + 1 - jlo + kTileK - 1) / kTileK;
  const int ntiles = npt + ntt;
  const int nseg = Dv / 4;                                                // 8-byte segments of a row

  auto entry_rows = [&](int tile, int e, const uint16_t*& kr_, const uint16_t*& vr_) {
    if (tile < npt && P == 0) {
      const int ec = min(e, nbmax - 1);
      const int pj = fdiv(ec, page, p.m_page);
      const int64_t slot = static_cast<int64_t>(bt(pj)) * page + (ec - pj * page);
      kr_ = p.k_cache + slot * p.k_ld + g * D;
      vr_ = p.v_cache + slot * p.v_ld + g * Dv;
    } else if (tile < npt) {
      const int ec = min(e, nbmax - 1);
      const int pj = fdiv(ec * P + P - 1, page, p.m_page);
      const int64_t slot = static_cast<int64_t>(bt(pj)) * p.PP + (ec - fdiv(page * pj, P, p.m_P));
      kr_ = p.kp + slot * GD + g * D;
      vr_ = p.vp + slot * GDv + g * Dv;
    } else {
      const int ec = min(e, i1);
      const int pj = fdiv(ec, page, p.m_page);
      const int64_t slot = static_cast<int64_t>(bt(pj)) * page + (ec - pj * page);
      kr_ = p.k_cache + slot * p.k_ld + g * D;
      vr_ = p.v_cache + slot * p.v_ld + g * Dv;
    }
  };
  auto tile_start = [&](int tile) { return tile < npt ? tile * kTileK : jlo + (tile - npt) * kTileK; };

  // V rows of a tile: consecutive threads take consecutive 8-byte segments of a row (whole cache lines per load
  // instruction). AHEAD: all of a thread's loads are issued together, one tile ahead of their use, and wait in registers.
  uint2 vreg[AHEAD ? DVB : 1];
  const uint16_t* knext[4];
  auto prefetch = [&](int tile) {
    const int e0 = tile_start(tile);
#pragma unroll
    for (int x = 0; x < (AHEAD ? DVB : 0); ++x) {
      const int c = threadIdx.x + 256 * x;
      if (c < kTileK * nseg) {
        const int row = fdiv(c, nseg, p.m_nseg), seg = c - row * nseg;
        const uint16_t *kr_, *vr_;
        entry_rows(tile, e0 + row, kr_, vr_);
        vreg[x] = *reinterpret_cast<const uint2*>(vr_ + seg * 4);
      }
    }
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const uint16_t* unused;
      entry_rows(tile, e0 + kb * 16 + ln, knext[kb], unused);
    }
  };
  auto store_v = [&](uint16_t* dst, uint2 v4) {
    dst[0] = static_cast<uint16_t>(v4.x & 0xffffu);
    dst[kLdk] = static_cast<uint16_t>(v4.x >> 16);
    dst[2 * kLdk] = static_cast<uint16_t>(v4.y & 0xffffu);
    dst[3 * kLdk] = static_cast<uint16_t>(v4.y >> 16);
  };
  // Only LDS traffic meets at the barriers of the tile loop. The fetch-ahead variant waits for that alone, so that the
  // vector loads of the next tile stay in flight across them (a full __syncthreads would drain them every tile).
  auto tile_barrier = [&]() {
    if (AHEAD) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else __syncthreads();
  };
  bf16x8_t kdata[AHEAD ? 4 : 1][K32];
  bf16x4_t ktail[4];
  auto fetch_k = [&]() {                                                    // the K fragments of the tile knext points to
#pragma unroll
    for (int kb = 0; kb < (AHEAD ? 4 : 0); ++kb) {
#pragma unroll
      for (int kk = 0; kk < K32; ++kk)
        if (kk < nk32) kdata[kb][kk] = *reinterpret_cast<const bf16x8_t*>(knext[kb] + 32 * kk + 8 * lg);
      if (tail16) ktail[kb] = *reinterpret_cast<const bf16x4_t*>(knext[kb] + 32 * nk32 + 4 * lg);
    }
  };
  // a split takes a contiguous share of the tiles
  const int per_split = p.nsplit > 1 ? (ntiles + p.nsplit - 1) / p.nsplit : ntiles;
  const int t_begin = split * per_split, t_end = min(ntiles, t_begin + per_split);
  if (AHEAD && t_begin < t_end) {
    prefetch(t_begin);
    if (active) fetch_k();
  }
  for (int tile = t_begin; tile < t_end; ++tile) {
    const int phase = tile < npt ? 0 : 1;
    const int e0 = tile_start(tile);
    const int e_end = phase == 0 ? nbmax : i1 + 1;
    const uint16_t* kcur[4];
    tile_barrier();                                                         // the previous tile's V reads are done
    if constexpr (AHEAD) {
#pragma unroll
      for (int x = 0; x < DVB; ++x) {
        const int c = threadIdx.x + 256 * x;
        if (c < kTileK * nseg) {
          const int row = fdiv(c, nseg, p.m_nseg), seg = c - row * nseg;
          store_v(vs + (seg * 4) * kLdk + row, vreg[x]);
        }
      }
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) kcur[kb] = knext[kb];
    } else {
      for (int c = threadIdx.x; c < kTileK * nseg; c += blockDim.x) {
        const int row = fdiv(c, nseg, p.m_nseg), seg = c - row * nseg;
        const uint16_t *kr_, *vr_;
        entry_rows(tile, e0 + row, kr_, vr_);
        store_v(vs + (seg * 4) * kLdk + row, *reinterpret_cast<const uint2*>(vr_ + seg * 4));
      }
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const uint16_t* unused;
        entry_rows(tile, e0 + kb * 16 + ln, kcur[kb], unused);
      }
    }
    tile_barrier();
    if (AHEAD && tile + 1 < t_end) prefetch(tile + 1);
    if (!active) continue;
    {
      float s[4][4];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const uint16_t* krow = kcur[kb];
        f32x4_t acc = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int kk = 0; kk < K32; ++kk)
          if (kk < nk32)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                AHEAD ? kdata[AHEAD ? kb : 0][kk] : *reinterpret_cast<const bf16x8_t*>(krow + 32 * kk + 8 * lg), qf[kk], acc, 0, 0, 0);
        if (tail16)
          acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
              AHEAD ? ktail[kb] : *reinterpret_cast<const bf16x4_t*>(krow + 32 * nk32 + 4 * lg), qtail, acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int ke = e0 + kb * 16 + 4 * lg + i;                         // the key of result row 4*lg + i
          bool vis = ke < e_end;
          if (phase == 0) vis = vis && (P == 0 || ke * P + P - 1 <= pos - W);
          else vis = vis && ke <= pos && ((chunk > 0 ? ke >= cstart : pos - ke < W) || ke < keep);
          s[kb][i] = vis ? acc[i] * p.scale : -INFINITY;
        }
      }
      if (AHEAD && tile + 1 < t_end) fetch_k();                            // in flight across the softmax, PV and the barriers
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[kb][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
      const float nm = fmaxf(m, mx);
      const float corr = expf(m - nm);
      float rs = 0.0f;
      bf16x8_t pb[2];                                                       // key blocks (0, 1) and (2, 3) side by side
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = expf(s[kb][i] - nm);                              // exp(-inf) = 0 for what is not seen
          rs += e;
          pb[kb >> 1][(kb & 1) * 4 + i] = static_cast<__bf16>(e);
        }
      }
      rs += __shfl_xor(rs, 16, kWave);
      rs += __shfl_xor(rs, 32, kWave);
      l = l * corr + rs;
      m = nm;
#pragma unroll
      for (int d = 0; d < DVB; ++d)
        if (d < ndvb) acc_o[d] *= corr;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const uint16_t* vt = vs + ln * kLdk + c * 32 + 4 * lg;              // value column ln: keys 4lg.. of blocks 2c, 2c+1
#pragma unroll
        for (int d = 0; d < DVB; ++d) {
          if (d < ndvb) {
            const uint2 lo = *reinterpret_cast<const uint2*>(vt + 16 * d * kLdk);
            const uint2 hi = *reinterpret_cast<const uint2*>(vt + 16 * d * kLdk + 16);
            const uint4 both = uint4{lo.x, lo.y, hi.x, hi.y};
            acc_o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, both), pb[c], acc_o[d], 0, 0, 0);
          }
        }
      }
    }
  }
  if (!active || !qvalid) return;
  if (p.nsplit > 1) {                                                       // unnormalised partials; window_pool_merge_kernel ends the job
    float* w = p.ws + ((t * p.H + h) * p.nsplit + split) * (Dv + 4);
#pragma unroll
    for (int d = 0; d < DVB; ++d)
      if (d < ndvb)
        *reinterpret_cast<f32x4_t*>(w + 16 * d + 4 * lg) = acc_o[d];
    if (lg == 0) {
      w[Dv] = m;
      w[Dv + 1] = l;
    }
    return;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  uint16_t* orow = p.out + (t * p.H + h) * Dv;
  const uint16_t* grow = p.gate != nullptr ? p.gate + t * p.ld_gate + static_cast<int64_t>(h) * p.gate_dv : nullptr;
  const int gstep = p.gate_dv > 1 ? 1 : 0;
#pragma unroll
  for (int d = 0; d < DVB; ++d) {
    if (d < ndvb) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int dv = 16 * d + 4 * lg + i;
        float val = acc_o[d][i] * inv;
        if (grow != nullptr) val *= sigmoidf_(__builtin_bit_cast(float, static_cast<uint32_t>(grow[dv * gstep]) << 16));
        orow[dv] = static_cast<uint16_t>(bf16_bits(val));
      }
    }
  }
}

// One wave per (token, query head): combines the splits' partials (each with its own running maximum), applies the gate.
__global__ __launch_bounds__(256) void window_pool_merge_kernel(const float* __restrict__ ws, const uint16_t* __restrict__ gate,
                                                                int64_t ld_gate, int gate_dv, uint16_t* __restrict__ out,
                                                                int64_t items, int H, int Dv, int nsplit, float m0,
                                                                const float* __restrict__ sinks) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + wave;
  if (item >= items) return;
  const int64_t t = item / H;
  const int h = static_cast<int>(item - t * H);
  const float* w = ws + item * nsplit * (Dv + 4);
  float mm = sinks != nullptr ? sinks[h] : m0;
  for (int s = 0; s < nsplit; ++s) mm = fmaxf(mm, w[s * (Dv + 4) + Dv]);
  float ll = 0.0f;
  for (int s = 0; s < nsplit; ++s) ll += w[s * (Dv + 4) + Dv + 1] * expf(w[s * (Dv + 4) + Dv] - mm);
  const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;
  for (int dv = lane; dv < Dv; dv += kWave) {
    float acc = 0.0f;
    for (int s = 0; s < nsplit; ++s) acc += w[s * (Dv + 4) + dv] * expf(w[s * (Dv + 4) + Dv] - mm);
    float val = acc * inv;
    if (gate != nullptr)
      val *= sigmoidf_(__builtin_bit_cast(float, static_cast<uint32_t>(gate[t * ld_gate + static_cast<int64_t>(h) * gate_dv +
                                                                            (gate_dv > 1 ? dv : 0)]) << 16));
    out[item * Dv + dv] = static_cast<uint16_t>(bf16_bits(val));
  }
}

}  // namespace lvmix

using namespace lvmix;

static uint32_t magic(int d) { return d <= 1 ? 0xffffffffu : static_cast<uint32_t>((1ull << 32) / static_cast<uint64_t>(d)); }

extern "C" int lv_window_pool_attn_mfma(const void* q, const void* k_cache, const void* v_cache, const void* kp,
                                        const void* vp, const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q,
                                        const int32_t* ctx_lens, const int32_t* block_tables, int bt_stride, int B,
                                        int max_new_tokens, int H, int G, int D, int Dv, int page, int window, int P,
                                        float scale, int has_sink, int nsplit, void* workspace, int64_t T, int64_t k_ld,
                                        int64_t v_ld, int gate_kind, void* stream) {
  return lv_masked_attn_mfma(q, k_cache, v_cache, kp, vp, gate, ld_gate, out, cu_q, ctx_lens, block_tables, bt_stride, B,
                             max_new_tokens, H, G, D, Dv, page, window, 0, 0, P, scale, has_sink, nullptr, nsplit, workspace, T,
                             k_ld, v_ld, gate_kind, stream);
}

extern "C" int lv_masked_attn_mfma(const void* q, const void* k_cache, const void* v_cache, const void* kp, const void* vp,
                                   const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q, const int32_t* ctx_lens,
                                   const int32_t* block_tables, int bt_stride, int B, int max_new_tokens, int H, int G, int D,
                                   int Dv, int page, int window, int keep_first, int chunk, int P, float scale, int has_sink,
                                   const void* sinks, int nsplit, void* workspace, int64_t T, int64_t k_ld, int64_t v_ld,
                                   int gate_kind, void* stream) {
  if (B == 0 || max_new_tokens <= 0) return 0;
  if (keep_first < 0 || chunk < 0 || (P > 0 && (keep_first > 0 || chunk > 0)))
    return fail(-1, "lv_masked_attn_mfma: kept first tokens and chunks do not combine with pooled blocks");
  if (sinks != nullptr) has_sink = 1;
  if (!q || !k_cache || !v_cache || !out || !cu_q || !ctx_lens || !block_tables)
    return fail(-1, "lv_window_pool_attn_mfma: null pointer");
  if (P > 0 && (!kp || !vp)) return fail(-1, "lv_window_pool_attn_mfma: pooled blocks without their cache");
  if (B < 0 || H <= 0 || G <= 0 || H % G != 0 || page <= 0 || window <= 0 || bt_stride <= 0)
    return fail(-1, "lv_window_pool_attn_mfma: bad sizes");
  if (D % 16 != 0 || Dv % 16 != 0 || D <= 0 || Dv <= 0 || D > 32 * kMaxK32 || Dv > 16 * kMaxDvb)
    return fail(-2, "lv_window_pool_attn_mfma: head sizes %d / %d (multiples of 16 up to 256)", D, Dv);
  if (gate_kind != LV_MIX_GATE_PER_HEAD && gate_kind != LV_MIX_GATE_PER_CHANNEL)
    return fail(-1, "lv_window_pool_attn_mfma: gate kind %d", gate_kind);
  const int gate_dv = gate_kind == LV_MIX_GATE_PER_HEAD ? 1 : Dv;
  if (gate != nullptr && ld_gate < static_cast<int64_t>(H) * gate_dv) return fail(-1, "lv_window_pool_attn_mfma: gate stride");
  if (k_ld <= 0) k_ld = static_cast<int64_t>(G) * D;
  if (v_ld <= 0) v_ld = static_cast<int64_t>(G) * Dv;
  if (k_ld < static_cast<int64_t>(G) * D || v_ld < static_cast<int64_t>(G) * Dv || k_ld % 8 != 0 || v_ld % 4 != 0 ||
      (reinterpret_cast<uintptr_t>(k_cache) & 15) != 0 || (reinterpret_cast<uintptr_t>(v_cache) & 7) != 0)
    return fail(-1, "lv_window_pool_attn_mfma: row strides or alignment of the caches");
  const float m0 = has_sink ? 0.0f : -1e30f;
  const int rep = H / G;
  const int ngroups = (rep + 3) / 4;
  WindowMfmaParams p{static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k_cache),
                     static_cast<const uint16_t*>(v_cache), static_cast<const uint16_t*>(kp),
                     static_cast<const uint16_t*>(vp), static_cast<const uint16_t*>(gate), ld_gate, gate_dv,
                     static_cast<uint16_t*>(out), cu_q, ctx_lens, block_tables, bt_stride, H, G, D, Dv, page, window, P,
                     P > 0 ? (page + P - 1) / P : 0, ngroups, scale, has_sink ? 1.0f : 0.0f,
                     magic(page), magic(P > 0 ? P : 1), magic(Dv / 4), nsplit > 1 ? nsplit : 1, static_cast<float*>(workspace),
                     k_ld, v_ld, m0, keep_first, chunk, static_cast<const float*>(sinks)};
  if (nsplit > 1 && (max_new_tokens > kTileQ || workspace == nullptr || T <= 0))
    return fail(-1, "lv_window_pool_attn_mfma: key splits need one query tile per sequence and a workspace");
  const size_t shm = static_cast<size_t>(Dv) * kLdk * sizeof(uint16_t);
  dim3 grid(nsplit > 1 ? nsplit : (max_new_tokens + kTileQ - 1) / kTileQ, G * ngroups, B), block(256);
  hipStream_t st = as_stream(stream);
  const bool small = D <= 128 && Dv <= 128;
  if (max_new_tokens <= kTileQ) {
    if (small) window_pool_mfma_kernel<true, 4, 8><<<grid, block, shm, st>>>(p);
    else window_pool_mfma_kernel<true, kMaxK32, kMaxDvb><<<grid, block, shm, st>>>(p);
  } else {
    if (small) window_pool_mfma_kernel<false, 4, 8><<<grid, block, shm, st>>>(p);
    else window_pool_mfma_kernel<false, kMaxK32, kMaxDvb><<<grid, block, shm, st>>>(p);
  }
  if (nsplit > 1) {
    const int64_t items = T * H;
    window_pool_merge_kernel<<<dim3(static_cast<unsigned>((items + 3) / 4)), block, 0, st>>>(
        static_cast<const float*>(workspace), static_cast<const uint16_t*>(gate), ld_gate, gate_dv,
        static_cast<uint16_t*>(out), items, H, Dv, nsplit, m0, static_cast<const float*>(sinks));
  }
  return launched("lv_window_pool_attn_mfma");
}
