// Mixture of experts, gathered form, for bf16: tokens are sorted by expert on the device and every expert multiplies
// only its own rows.
//
//   moe_sort_kernel      one workgroup: counts the (token, choice) pairs of every expert, gives each pair a row in
//                        expert order, and lists the row tiles (expert, first row, rows) that the GEMM launches walk.
//                        No host round trip: the GEMM grids are sized for the most tiles a step can have and
//                        workgroups beyond the list leave at once.
//   moe_gemm_kernel      grouped GEMM on the matrix cores, one workgroup per (row tile of one expert, column tile):
//                        C[row, n] = sum_k A[row, k] * B_e[n, k], both operands with k contiguous, so MFMA fragments
//                        (v_mfma_f32_16x16x32_bf16) are 16-byte loads straight from memory; the four waves share the
//                        tile's rows and split its columns. The weights are the MFMA's first operand: a lane then holds
//                        four consecutive columns of one row and stores them as 8 bytes.
//                        UP: rows are gathered from the tokens' activations, epilogue relu(x)^2, or (GLU) the clamped
//                        gated unit of a gate and an up block of the same columns.
//                        DOWN: rows are the sorted activations, B_e is a column block of the one [width, experts*ff] weight.
//   moe_combine_kernel   one workgroup per token: sum over its choices of weight * expert output row, in f32.
// A row's result does not depend on where the sort put it or on what else is in the tile: every output element is
// its own chain of MFMA accumulations over k.
// lv_moe_sort and lv_moe_combine are also exported alone: large eager steps run the experts' products as vendor GEMMs
// on the sorted rows in between (mix_ops.moe_sorted_ff).
#include "mix_common.h"

namespace lvmix {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int kSortThreads = 1024;

// ids [M] (expert of pair p = token * top + choice).  Outputs: sorted_pair [M] (pair of each row in expert order),
// inv [M] (row of each pair), tiles [max_tiles][3] (expert, first row, rows), num_tiles [1].
__global__ __launch_bounds__(kSortThreads) void moe_sort_kernel(const int32_t* __restrict__ ids, int M, int E, int BM,
                                                                 int32_t* __restrict__ sorted_pair, int32_t* __restrict__ inv,
                                                                 int32_t* __restrict__ tiles, int32_t* __restrict__ num_tiles,
                                                                 int max_tiles, int32_t* __restrict__ offsets, int align) {
  extern __shared__ int32_t sl[];
  int32_t* cnt = sl;              // [E] pairs per expert
  int32_t* off = sl + E;          // [E + 1] first row per expert
  int32_t* toff = sl + 2 * E + 1; // [E + 1] first tile per expert
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < M; p += blockDim.x) inv[p] = atomicAdd(&cnt[ids[p]], 1);     // rank inside the expert
  __syncthreads();
  if (threadIdx.x == 0) {
    int r = 0, t = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = r;
      toff[e] = t;
      r = (r + cnt[e] + align - 1) / align * align;           // every expert starts on a multiple of `align` rows
      t += (cnt[e] + BM - 1) / BM;
    }
    off[E] = r;
    toff[E] = t;
    if (num_tiles != nullptr) num_tiles[0] = t < max_tiles ? t : max_tiles;
  }
  __syncthreads();
  if (offsets != nullptr)
    for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = off[e];
  for (int p = threadIdx.x; p < M; p += blockDim.x) {
    const int row = off[ids[p]] + inv[p];
    sorted_pair[row] = p;
    inv[p] = row;
  }
  if (tiles == nullptr) return;
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    const int n = cnt[e];
    for (int j = 0, t = toff[e]; j * BM < n && t < max_tiles; ++j, ++t) {
      tiles[3 * t] = e;
      tiles[3 * t + 1] = off[e] + j * BM;
      tiles[3 * t + 2] = min(BM, n - j * BM);
    }
  }
}

struct MoeGemmParams {
  const uint16_t* A;       // UP: activations [T, K]; DOWN: sorted expert activations [M, K]
  const uint16_t* B;       // UP: [E * N, K]; DOWN: [N, E * K]
  uint16_t* C;             // [M, N] in sorted row order
  const int32_t *sorted_pair, *tiles, *num_tiles;
  int N, K, top;
  int64_t lda, ldb, ldc;
  int64_t b_expert;        // elements from one expert's B to the next
  const float* row_scale;  // GLU: [pairs] factor on the pre-activations of a (token, choice) pair
  float limit, alpha;      // GLU: clamp and sigmoid slope of the gated unit
  int act;                 // UP without GLU: LV_MIX_ACT_* applied to the product
  int n_real;              // tiles of buckets from this number on have no weights (experts that hand their input through) and are skipped
};

// MB x NB blocks of 16 x 16 per wave; WM waves along the rows (1 or 2), the others along the columns: the workgroup's
// tile is (16 MB WM) rows x (16 NB 4 / WM) columns. The fragments of the next 32-wide step over k are loaded before the
// matrix instructions of the current one are issued, so that memory latency is covered by them. KU > 0 (tiles of a few
// rows, where the weights are read once and the launch is bound by memory): the fragments of KU steps are requested
// together instead, and many small workgroups keep the memory system full.
// GLU (with UP; NB even): an expert's B holds N gate rows followed by N up rows; blocks 2c and 2c + 1 of a wave are the
// gate and the up pre-activations of the SAME 16 columns, so the gated unit
//   g = min(s * gate, L); u = clamp(s * up, -L, L); y = g * sigmoid(alpha * g) * (u + 1),  s = row_scale[pair of the row]
// is formed in registers and one N-wide row is stored.
template <int MB, int NB, int WM, bool UP, int KU = 0, bool GLU = false>
__global__ __launch_bounds__(256) void moe_gemm_kernel(MoeGemmParams p) {
  static_assert(!GLU || (UP && NB % 2 == 0), "the gated unit pairs column blocks of the up projection");
  constexpr int CB = GLU ? NB / 2 : NB;             // distinct 16-column blocks of a wave
  const int tile = blockIdx.y, bx = blockIdx.x;
  if (tile >= p.num_tiles[0]) return;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int ln = lane & 15, lg = lane >> 4;
  const int wm = wave % WM, wn = wave / WM;
  const int e = p.tiles[3 * tile], row0 = p.tiles[3 * tile + 1], nrows = p.tiles[3 * tile + 2];
  if (e >= p.n_real) return;
  const int m0 = wm * 16 * MB;
  const int n0 = (bx * (4 / WM) + wn) * 16 * CB;
  if (n0 >= p.N || m0 >= nrows) return;
  const uint16_t* arow[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int r = row0 + min(m0 + mb * 16 + ln, nrows - 1);     // rows past the tile's end repeat its last row; never stored
    const int64_t src = UP ? p.sorted_pair[r] / p.top : r;
    arow[mb] = p.A + src * p.lda + 8 * lg;
  }
  const uint16_t* brow[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int n = min(n0 + (GLU ? nb / 2 : nb) * 16 + ln, p.N - 1) + (GLU && (nb & 1) ? p.N : 0);
    brow[nb] = p.B + static_cast<int64_t>(e) * p.b_expert + static_cast<int64_t>(n) * p.ldb + 8 * lg;
  }
  f32x4_t acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  bf16x8_t a0[MB], b0[NB], a1[MB], b1[NB];
  auto load = [&](bf16x8_t* a, bf16x8_t* b, int k) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) a[mb] = *reinterpret_cast<const bf16x8_t*>(arow[mb] + k);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) b[nb] = *reinterpret_cast<const bf16x8_t*>(brow[nb] + k);
  };
  auto multiply = [&](const bf16x8_t* a, const bf16x8_t* b) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[nb], a[mb], acc[mb][nb], 0, 0, 0);
  };
  if constexpr (KU > 0) {
    bf16x8_t au[KU][MB], bu[KU][NB];
    for (int k = 0; k < p.K; k += 32 * KU) {
#pragma unroll
      for (int u = 0; u < KU; ++u)
        if (k + 32 * u < p.K) load(au[u], bu[u], k + 32 * u);
#pragma unroll
      for (int u = 0; u < KU; ++u)
        if (k + 32 * u < p.K) multiply(au[u], bu[u]);
    }
  } else {
    load(a0, b0, 0);
    for (int k = 0; k < p.K; k += 64) {
      if (k + 32 < p.K) load(a1, b1, k + 32);
      multiply(a0, b0);
      if (k + 32 >= p.K) break;
      if (k + 64 < p.K) load(a0, b0, k + 64);
      multiply(a1, b1);
    }
  }
  // acc[mb][nb][i] = C[row = m0 + 16 mb + ln][n = n0 + 16 nb + 4 lg + i]
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int r = m0 + mb * 16 + ln;
    if (r >= nrows) continue;
    uint16_t* crow = p.C + static_cast<int64_t>(row0 + r) * p.ldc;
    float rs = 1.0f;
    if constexpr (GLU) rs = p.row_scale[p.sorted_pair[row0 + r]];
#pragma unroll
    for (int nb = 0; nb < CB; ++nb) {
      const int n = n0 + nb * 16 + 4 * lg;
      if (n >= p.N) continue;                                   // N is a multiple of 4: a lane's four columns are in or out together
      uint16_t o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v;
        if constexpr (GLU) {
          const float g = fminf(acc[mb][2 * nb][i] * rs, p.limit);
          const float u = fminf(fmaxf(acc[mb][2 * nb + 1][i] * rs, -p.limit), p.limit);
          v = g * sigmoidf_(p.alpha * g) * (u + 1.0f);
        } else {
          v = acc[mb][nb][i];
          if (UP) {
            if (p.act == LV_MIX_ACT_GELU_ERF) {
              v = 0.5f * v * (1.0f + erff(v * 0.7071067811865476f));
            } else if (p.act == LV_MIX_ACT_GELU_TANH) {
              v = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
            } else {
              v = fmaxf(v, 0.0f);
              v = v * v;
            }
          }
        }
        bf16_t t;
        stf(&t, v);
        o[i] = t.bits;
      }
      *reinterpret_cast<uint2*>(crow + n) = uint2{static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16),
                                                  static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16)};
    }
  }
}

// ids, n_real, h (all or none): a choice whose expert number is n_real or above hands the token's own row h[t] through
// instead of a row of `rows`.
__global__ __launch_bounds__(256) void moe_combine_kernel(const uint16_t* __restrict__ rows, const int32_t* __restrict__ inv,
                                                          const float* __restrict__ weights, uint16_t* __restrict__ out,
                                                          int W, int top, const int32_t* __restrict__ ids, int n_real,
                                                          const uint16_t* __restrict__ h) {
  const int64_t t = blockIdx.x;
  for (int c = threadIdx.x * 4; c < W; c += blockDim.x * 4) {
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int k = 0; k < top; ++k) {
      const float w = weights != nullptr ? weights[t * top + k] : 1.0f;
      const bool through = ids != nullptr && ids[t * top + k] >= n_real;
      const uint2 v = *reinterpret_cast<const uint2*>(through ? h + t * W + c : rows + static_cast<int64_t>(inv[t * top + k]) * W + c);
      acc[0] += w * __builtin_bit_cast(float, v.x << 16);
      acc[1] += w * __builtin_bit_cast(float, v.x & 0xffff0000u);
      acc[2] += w * __builtin_bit_cast(float, v.y << 16);
      acc[3] += w * __builtin_bit_cast(float, v.y & 0xffff0000u);
    }
    bf16_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) stf(&o[i], acc[i]);
    *reinterpret_cast<uint2*>(out + t * W + c) = uint2{static_cast<uint32_t>(o[0].bits) | (static_cast<uint32_t>(o[1].bits) << 16),
                                                        static_cast<uint32_t>(o[2].bits) | (static_cast<uint32_t>(o[3].bits) << 16)};
  }
}

template <bool UP, bool GLU = false>
static void gemm_launch(const MoeGemmParams& p, int max_tiles, int BM, hipStream_t s) {
  if (BM == 128) {                 // 128 rows x 128 columns (gated: 64, each from a gate and an up block)
    const int cols = GLU ? 64 : 128;
    dim3 grid((p.N + cols - 1) / cols, max_tiles);
    moe_gemm_kernel<4, 4, 2, UP, 0, GLU><<<grid, dim3(256), 0, s>>>(p);
  } else if (BM == 64) {           // 64 rows x 256 columns (gated: 128)
    const int cols = GLU ? 128 : 256;
    dim3 grid((p.N + cols - 1) / cols, max_tiles);
    moe_gemm_kernel<4, 4, 1, UP, 0, GLU><<<grid, dim3(256), 0, s>>>(p);
  } else {                         // 16 rows x 64 columns, four steps over k requested at once
    dim3 grid((p.N + 63) / 64, max_tiles);
    moe_gemm_kernel<1, GLU ? 2 : 1, 1, UP, 4, GLU><<<grid, dim3(256), 0, s>>>(p);
  }
}

}  // namespace lvmix

using namespace lvmix;

extern "C" {

int lv_moe_tile_rows(int64_t pairs, int E) {
  // few rows per expert (decoded tokens): tiles of 16 rows read each weight once and waste little of the matrix cores;
  // prompts: 64 or 128 rows share every weight fragment
  if (pairs >= static_cast<int64_t>(E) * 256) return 128;
  return pairs >= static_cast<int64_t>(E) * 48 ? 64 : 16;
}

int lv_moe_max_tiles(int64_t pairs, int E, int BM) {
  const int64_t full = pairs / BM + E;            // every expert can end on a partial tile
  const int64_t hit = pairs < E ? pairs : E;
  const int64_t most = pairs / BM + hit;
  return static_cast<int>(most < full ? most : full);
}

int lv_moe_grouped_ff(const void* h, const void* ids, const void* weights, const void* up_w, const void* down_w, void* out,
                      void* workspace, int64_t T, int W, int F, int E, int top, void* stream) {
  return lv_moe_grouped_act_ff(h, ids, weights, up_w, down_w, out, workspace, T, W, F, E, 0, top, LV_MIX_ACT_RELU2, stream);
}

int lv_moe_grouped_act_ff(const void* h, const void* ids, const void* weights, const void* up_w, const void* down_w, void* out,
                          void* workspace, int64_t T, int W, int F, int E_real, int n_through, int top, int act, void* stream) {
  if (T == 0) return 0;
  if (!h || !ids || !weights || !up_w || !down_w || !out || !workspace) return fail(-1, "lv_moe_grouped_ff: null pointer");
  const int E = E_real + n_through;                 // buckets of the sort; the last n_through have no weights
  if (T < 0 || W <= 0 || F <= 0 || E_real <= 0 || n_through < 0 || top <= 0 || W % 32 != 0 || F % 32 != 0 || E > 4096 ||
      act < 0 || act > LV_MIX_ACT_GELU_TANH)
    return fail(-1, "lv_moe_grouped_ff: width %d and expert size %d must be multiples of 32 (experts %d)", W, F, E);
  const int64_t M = T * top;
  if (M > (1 << 30)) return fail(-2, "lv_moe_grouped_ff: %lld rows", (long long)M);
  const int BM = lv_moe_tile_rows(M, E);
  const int max_tiles = lv_moe_max_tiles(M, E, BM);
  // workspace: sorted_pair [M] | inv [M] | tiles [3 max_tiles] | num_tiles [1] (int32, padded to 16 bytes) | act [M, F] | rows [M, W]
  int32_t* sorted_pair = static_cast<int32_t*>(workspace);
  int32_t* inv = sorted_pair + M;
  int32_t* tiles = inv + M;
  int32_t* num_tiles = tiles + 3 * static_cast<int64_t>(max_tiles);
  const int64_t ints = (2 * M + 3 * static_cast<int64_t>(max_tiles) + 1 + 3) / 4 * 4;
  uint16_t* act_rows = reinterpret_cast<uint16_t*>(sorted_pair + ints);
  uint16_t* rows = act_rows + M * F;
  hipStream_t s = as_stream(stream);
  const size_t shm = sizeof(int32_t) * (3 * static_cast<size_t>(E) + 2);
  moe_sort_kernel<<<dim3(1), dim3(kSortThreads), shm, s>>>(static_cast<const int32_t*>(ids), static_cast<int>(M), E, BM,
                                                          sorted_pair, inv, tiles, num_tiles, max_tiles, nullptr, 1);
  MoeGemmParams up{static_cast<const uint16_t*>(h), static_cast<const uint16_t*>(up_w), act_rows, sorted_pair, tiles, num_tiles,
                   F, W, top, W, W, F, static_cast<int64_t>(F) * W, nullptr, 0.0f, 0.0f, act, E_real};
  gemm_launch<true>(up, max_tiles, BM, s);
  MoeGemmParams down{act_rows, static_cast<const uint16_t*>(down_w), rows, sorted_pair, tiles, num_tiles,
                     W, F, top, F, static_cast<int64_t>(E_real) * F, W, F, nullptr, 0.0f, 0.0f, 0, E_real};
  gemm_launch<false>(down, max_tiles, BM, s);
  moe_combine_kernel<<<dim3(static_cast<unsigned>(T)), dim3(256), 0, s>>>(
      rows, inv, static_cast<const float*>(weights), static_cast<uint16_t*>(out), W, top,
      n_through > 0 ? static_cast<const int32_t*>(ids) : nullptr, E_real, static_cast<const uint16_t*>(h));
  return launched("lv_moe_grouped_ff");
}

int lv_moe_grouped_glu_ff(const void* h, const void* ids, const void* weights, const void* up_w, const void* down_w,
                          int64_t down_ld, void* out, void* workspace, int64_t T, int W, int F, int E, int top, float limit,
                          float alpha, void* stream) {
  if (T == 0) return 0;
  if (!h || !ids || !weights || !up_w || !down_w || !out || !workspace) return fail(-1, "lv_moe_grouped_glu_ff: null pointer");
  if (T < 0 || W <= 0 || F <= 0 || E <= 0 || top <= 0 || W % 32 != 0 || F % 32 != 0 || E > 4096)
    return fail(-1, "lv_moe_grouped_glu_ff: width %d and expert size %d must be multiples of 32 (experts %d)", W, F, E);
  if (down_ld <= 0) down_ld = static_cast<int64_t>(E) * F;
  if (down_ld < static_cast<int64_t>(E) * F || down_ld % 8 != 0 || (reinterpret_cast<uintptr_t>(down_w) & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(up_w) & 15) != 0 || (reinterpret_cast<uintptr_t>(h) & 15) != 0)
    return fail(-1, "lv_moe_grouped_glu_ff: row stride or alignment of the weights");
  const int64_t M = T * top;
  if (M > (1 << 30)) return fail(-2, "lv_moe_grouped_glu_ff: %lld rows", (long long)M);
  const int BM = lv_moe_tile_rows(M, E);
  const int max_tiles = lv_moe_max_tiles(M, E, BM);
  // workspace as in lv_moe_grouped_ff
  int32_t* sorted_pair = static_cast<int32_t*>(workspace);
  int32_t* inv = sorted_pair + M;
  int32_t* tiles = inv + M;
  int32_t* num_tiles = tiles + 3 * static_cast<int64_t>(max_tiles);
  const int64_t ints = (2 * M + 3 * static_cast<int64_t>(max_tiles) + 1 + 3) / 4 * 4;
  uint16_t* act = reinterpret_cast<uint16_t*>(sorted_pair + ints);
  uint16_t* rows = act + M * F;
  hipStream_t s = as_stream(stream);
  const size_t shm = sizeof(int32_t) * (3 * static_cast<size_t>(E) + 2);
  moe_sort_kernel<<<dim3(1), dim3(kSortThreads), shm, s>>>(static_cast<const int32_t*>(ids), static_cast<int>(M), E, BM,
                                                          sorted_pair, inv, tiles, num_tiles, max_tiles, nullptr, 1);
  MoeGemmParams up{static_cast<const uint16_t*>(h), static_cast<const uint16_t*>(up_w), act, sorted_pair, tiles, num_tiles,
                   F, W, top, W, W, F, 2 * static_cast<int64_t>(F) * W, static_cast<const float*>(weights), limit, alpha, 0, E};
  gemm_launch<true, true>(up, max_tiles, BM, s);
  MoeGemmParams down{act, static_cast<const uint16_t*>(down_w), rows, sorted_pair, tiles, num_tiles,
                     W, F, top, F, down_ld, W, F, nullptr, 0.0f, 0.0f, 0, E};
  gemm_launch<false>(down, max_tiles, BM, s);
  moe_combine_kernel<<<dim3(static_cast<unsigned>(T)), dim3(256), 0, s>>>(rows, inv, nullptr, static_cast<uint16_t*>(out), W, top, nullptr, 0, nullptr);
  return launched("lv_moe_grouped_glu_ff");
}

int lv_moe_sort(const void* ids, int64_t M, int E, int align, void* sorted_pair, void* inv, void* offsets, void* stream) {
  if (M == 0) return 0;
  if (!ids || !sorted_pair || !inv || !offsets || M < 0 || M > (1 << 29) || E <= 0 || E > 4096 || align <= 0 || align > 4096)
    return fail(-1, "lv_moe_sort: bad arguments");
  const size_t shm = sizeof(int32_t) * (3 * static_cast<size_t>(E) + 2);
  moe_sort_kernel<<<dim3(1), dim3(kSortThreads), shm, as_stream(stream)>>>(
      static_cast<const int32_t*>(ids), static_cast<int>(M), E, 1 << 30, static_cast<int32_t*>(sorted_pair),
      static_cast<int32_t*>(inv), nullptr, nullptr, 0, static_cast<int32_t*>(offsets), align);
  return launched("lv_moe_sort");
}

int lv_moe_combine(const void* rows, const void* inv, const void* weights, void* out, int64_t T, int W, int top, void* stream) {
  return lv_moe_combine_through(rows, inv, weights, out, T, W, top, nullptr, 0, nullptr, stream);
}

int lv_moe_combine_through(const void* rows, const void* inv, const void* weights, void* out, int64_t T, int W, int top,
                           const void* ids, int n_real, const void* h, void* stream) {
  if (T == 0) return 0;
  if (!rows || !inv || !out || T < 0 || W <= 0 || W % 4 != 0 || top <= 0 || ((ids != nullptr) != (h != nullptr)))
    return fail(-1, "lv_moe_combine: bad arguments");
  moe_combine_kernel<<<dim3(static_cast<unsigned>(T)), dim3(256), 0, as_stream(stream)>>>(
      static_cast<const uint16_t*>(rows), static_cast<const int32_t*>(inv), static_cast<const float*>(weights),
      static_cast<uint16_t*>(out), W, top, static_cast<const int32_t*>(ids), n_real, static_cast<const uint16_t*>(h));
  return launched("lv_moe_combine");
}

int64_t lv_moe_grouped_workspace_bytes(int64_t T, int W, int F, int E, int top) {
  const int64_t M = T * top;
  const int BM = lv_moe_tile_rows(M, E);
  const int64_t ints = (2 * M + 3 * static_cast<int64_t>(lv_moe_max_tiles(M, E, BM)) + 1 + 3) / 4 * 4;
  return ints * 4 + M * (static_cast<int64_t>(F) + W) * 2;
}

}  // extern "C"
