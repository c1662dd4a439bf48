// Fused per-module gradient collection for gfx950 (MI355X).
//
// For a tile of tokens of one sequence of one module the kernels
//   1. project the activations  a'[t, j] = sum_k a[t, k] * (R_in[j, k] * col_scale[k])
//   2. project the output grads g'[t, i] = sum_k g[t, k] * (R_out[i, k] * row_scale[k])
//      both with MFMA tiles whose A operand is loaded straight from global memory (a and g are
//      read exactly once),
//   3. per-sequence: reduce P[i, j] = sum_t g'[t, i] * a'[t, j] over the tile's tokens and write one
//      fp32 partial; a second tiny kernel adds the partials of a sequence in a fixed order, clamps,
//      casts and writes the store row.
//      per-token: write flatten(g'[t] (x) a'[t]) for every valid token.
//
// Reference op sequence: bergson/collector/collector.py:518-543 (forward
// hook), :646-742 (backward hook), bergson/builder.py:17-32 (concatenation).
//
// Two kernels share that arithmetic:
//   collect_persist_kernel  p <= 16, aligned operands, no bias, projection matrices small enough for
//                           LDS: one workgroup per CU walks an equal share of all (module, tile) items.
//   collect_kernel          everything else: one workgroup per (module, tile); its 4 waves split K
//                           and combine their partial projections through LDS in the fixed order
//                           (w0+w2)+(w1+w3); the projection matrices come from L2.

#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <type_traits>
#include <queue>
#include <vector>

#include "common.hpp"
#include "mma16.hpp"
#include "stream.hpp"

namespace bgx {


// 16-byte fragment of row `row` starting at element k0 (zero beyond K).
template <typename T, bool ALIGNED>
__device__ inline uint4 load_frag(const T* __restrict__ row, int k0, int K) {
  using M = Mma<T>;
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (ALIGNED) {
    if (k0 < K) v = *reinterpret_cast<const uint4*>(row + k0);
  } else {
#pragma unroll
    for (int e = 0; e < M::EPL; ++e)
      if (k0 + e < K) M::set(v, e, Elem<T>::load(row + k0 + e));
  }
  return v;
}

// x' = x @ (R * scale)^T for the 16*MT tokens of the tile, this wave's share of K (k-steps wave, wave+4, ...).
//   xrow0: pointer to the tile's first token.
//   acc[mt][pb][i] belongs to token mt*16 + (lane/16)*4 + i, column pb*16 + lane%16.
// ALIGNED (the fast path; K is a multiple of the k-step and everything is 16-byte aligned): every load is
// unconditional.  Token rows past rows_valid and projection rows past p re-read a valid row instead of
// being masked -- a select on loaded data would make the wave wait for each load before issuing the
// next -- so those accumulator entries hold garbage; the caller zeroes the token rows, and columns >= p
// are never read.  !ALIGNED: element-wise guarded loads, rows and columns out of range read as zero.
template <typename T, int PB, bool ALIGNED, int MT, int U>
__device__ inline void project_tile(const T* __restrict__ xrow0, int64_t tok_stride, int rows_valid,
                                    int K, const T* __restrict__ R, int p,
                                    const float* __restrict__ scale, int wave, int lane,
                                    f32x4 (&acc)[MT][PB]) {
  using M = Mma<T>;  // U = k-steps kept in flight per wave
  const int r = lane & 15;
  const int q = lane >> 4;

  const T* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int t = mt * 16 + r;
    xok[mt] = t < rows_valid;
    xrow[mt] = xrow0 + (int64_t)(ALIGNED ? min(t, rows_valid - 1) : t) * tok_stride;
  }
  const T* rrow[PB];
  bool rok[PB];
#pragma unroll
  for (int pb = 0; pb < PB; ++pb) {
    const int j = pb * 16 + r;
    rok[pb] = j < p;
    rrow[pb] = R + (int64_t)(ALIGNED ? min(j, p - 1) : j) * K;
  }

  const int nsteps = (K + M::KS - 1) / M::KS;

  // UU consecutive k-steps of this wave starting at step ks0: all loads first, then the MFMAs
  auto run = [&](int ks0, auto uu_tag) {
    constexpr int UU = decltype(uu_tag)::value;
    uint4 xf[UU][MT];
    uint4 rf[UU][PB];
    float sc[UU][M::EPL];
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      const int k0 = (ks0 + 4 * u) * M::KS + q * M::EPL;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (ALIGNED) {
          xf[u][mt] = *reinterpret_cast<const uint4*>(xrow[mt] + k0);
        } else {
          xf[u][mt] = make_uint4(0u, 0u, 0u, 0u);
          if (xok[mt]) xf[u][mt] = load_frag<T, false>(xrow[mt], k0, K);
        }
      }
#pragma unroll
      for (int pb = 0; pb < PB; ++pb) {
        if (ALIGNED) {
          rf[u][pb] = *reinterpret_cast<const uint4*>(rrow[pb] + k0);
        } else {
          rf[u][pb] = make_uint4(0u, 0u, 0u, 0u);
          if (rok[pb]) rf[u][pb] = load_frag<T, false>(rrow[pb], k0, K);
        }
      }
      if (scale != nullptr) {
        if (ALIGNED) {
#pragma unroll
          for (int e = 0; e < M::EPL; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(scale + k0 + e);
            sc[u][e] = v.x;
            sc[u][e + 1] = v.y;
            sc[u][e + 2] = v.z;
            sc[u][e + 3] = v.w;
          }
        } else {
#pragma unroll
          for (int e = 0; e < M::EPL; ++e) sc[u][e] = (k0 + e < K) ? scale[k0 + e] : 0.f;
        }
      }
    }
    if (scale != nullptr) {
#pragma unroll
      for (int u = 0; u < UU; ++u)
#pragma unroll
        for (int e = 0; e < M::EPL; ++e)
#pragma unroll
          for (int pb = 0; pb < PB; ++pb) M::set(rf[u][pb], e, M::get(rf[u][pb], e) * sc[u][e]);
    }
#pragma unroll
    for (int u = 0; u < UU; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) M::mma(xf[u][mt], rf[u][pb], acc[mt][pb]);
  };

  int ks0 = wave;
  for (; ks0 + 4 * (U - 1) < nsteps; ks0 += 4 * U) run(ks0, std::integral_constant<int, U>{});
  for (; ks0 < nsteps; ks0 += 4) run(ks0, std::integral_constant<int, 1>{});
}

struct CollectArgs {
  const bgx_module_desc* mods;  // device copy
  const int32_t* lengths;
  int N, S, p, tiles_per_seq;  // tiles_per_seq = ceil(S / tokens per workgroup)
  // per-sequence
  float* partials;  // [n_modules][N][tiles_per_seq][p*p]
  // per-token
  const int64_t* row_offsets;
  void* out;
  int64_t out_row_stride;
  int out_dtype;
  float lo, hi;
};

__device__ inline int seq_token_limit(const int32_t* lengths, int n, int S) {
  if (lengths == nullptr) return S;
  const int l = lengths[n] - 1;
  return l < S ? (l < 0 ? 0 : l) : S;
}

// BIAS: the launch contains modules whose bias gradient is collected (bias_col != NULL).  The bias adds
// (sum_t gb'_t) (x) bias_col to P, where gb' = g' when the module has no bias_scale and otherwise a second
// projection of g scaled by bias_scale (the Adafactor bias factor applies to the unscaled g).
template <typename T, int PB, bool ALIGNED, bool PER_TOKEN, int MT, int U, bool BIAS = false>
__global__ __launch_bounds__(COLLECT_THREADS) void collect_kernel(CollectArgs args) {
  constexpr int TILE_T = 16 * MT;  // tokens per workgroup
  constexpr int PP = PB * 16;      // padded projection dim
  constexpr int LDP = PP + 1;      // LDS row stride (floats)
  __shared__ float sm[BIAS ? 3 : 2][2][TILE_T][LDP];  // [a/g/gb][slot][token][col]

  const int tile = blockIdx.x;
  const int m = blockIdx.y;
  const int n = tile / args.tiles_per_seq;
  const int ts = tile - n * args.tiles_per_seq;
  const int s0 = ts * TILE_T;
  const int s_limit = seq_token_limit(args.lengths, n, args.S);
  if (s0 >= s_limit) return;  // whole tile is padding: g is exactly zero there
  const int rows_valid = min(TILE_T, s_limit - s0);

  const bgx_module_desc d = args.mods[m];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int p = args.p;

  f32x4 accA[MT][PB];
  f32x4 accG[MT][PB];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int pb = 0; pb < PB; ++pb) {
      accA[mt][pb] = f32x4{0.f, 0.f, 0.f, 0.f};
      accG[mt][pb] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  const T* a0 = (const T*)d.a + (int64_t)n * d.a_seq_stride + (int64_t)s0 * d.a_tok_stride;
  const T* g0 = (const T*)d.g + (int64_t)n * d.g_seq_stride + (int64_t)s0 * d.g_tok_stride;
  project_tile<T, PB, ALIGNED, MT, U>(a0, d.a_tok_stride, rows_valid, d.I, (const T*)d.r_in, p,
                                      d.col_scale, wave, lane, accA);
  project_tile<T, PB, ALIGNED, MT, U>(g0, d.g_tok_stride, rows_valid, d.O, (const T*)d.r_out, p,
                                      d.row_scale, wave, lane, accG);

  const int r = lane & 15;
  const int q = lane >> 4;
  const bool has_bias = BIAS && d.bias_col != nullptr;
  const bool own_gb = has_bias && d.bias_scale != nullptr;  // bias needs its own projection of g
  if constexpr (BIAS) {
    if (own_gb) {
      f32x4 accB[MT][PB];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int pb = 0; pb < PB; ++pb) accB[mt][pb] = f32x4{0.f, 0.f, 0.f, 0.f};
      project_tile<T, PB, ALIGNED, MT, U>(g0, d.g_tok_stride, rows_valid, d.O, (const T*)d.r_out, p,
                                          d.bias_scale, wave, lane, accB);
      // the same pairwise combination as below, for the bias projection only
      if (wave >= 2) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int pb = 0; pb < PB; ++pb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              sm[2][wave - 2][mt * 16 + q * 4 + i][pb * 16 + r] = (mt * 16 + q * 4 + i < rows_valid) ? accB[mt][pb][i] : 0.f;
      }
      __syncthreads();
      if (wave < 2) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int pb = 0; pb < PB; ++pb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              sm[2][wave][mt * 16 + q * 4 + i][pb * 16 + r] += (mt * 16 + q * 4 + i < rows_valid) ? accB[mt][pb][i] : 0.f;
      }
      __syncthreads();
      for (int e = tid; e < TILE_T * PP; e += COLLECT_THREADS) {
        const int t = e / PP, c = e - t * PP;
        sm[2][0][t][c] += sm[2][1][t][c];
      }
    }
  }

  // ---- combine the 4 K-slices: (w0 + w2) + (w1 + w3), fixed order ----------
  if (wave >= 2) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int pb = 0; pb < PB; ++pb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int t = mt * 16 + q * 4 + i;
          const bool live = t < rows_valid;  // rows past the tile's last token hold garbage on the fast path
          sm[0][wave - 2][t][pb * 16 + r] = live ? accA[mt][pb][i] : 0.f;
          sm[1][wave - 2][t][pb * 16 + r] = live ? accG[mt][pb][i] : 0.f;
        }
  }
  __syncthreads();
  if (wave < 2) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int pb = 0; pb < PB; ++pb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int t = mt * 16 + q * 4 + i;
          const bool live = t < rows_valid;
          sm[0][wave][t][pb * 16 + r] += live ? accA[mt][pb][i] : 0.f;
          sm[1][wave][t][pb * 16 + r] += live ? accG[mt][pb][i] : 0.f;
        }
  }
  __syncthreads();
  for (int e = tid; e < TILE_T * PP; e += COLLECT_THREADS) {
    const int t = e / PP, c = e - t * PP;
    float av = sm[0][0][t][c] + sm[0][1][t][c];
    // without a bias factor the bias shares g': (g'_t) (x) (a'_t + bias_col)
    if (has_bias && !own_gb && c < p) av += d.bias_col[c];
    sm[0][0][t][c] = av;
    sm[1][0][t][c] += sm[1][1][t][c];
  }
  __syncthreads();

  const int pp = p * p;
  if (!PER_TOKEN) {
    // P[i, j] = sum_t g'[t, i] * a'[t, j] (+ gb'[t, i] * bias_col[j]); tokens past rows_valid hold zeros.
    float* dst = args.partials + (((int64_t)m * args.N + n) * args.tiles_per_seq + ts) * pp;
    for (int e = tid; e < pp; e += COLLECT_THREADS) {
      const int i = e / p, j = e - i * p;
      float s = 0.f;
#pragma unroll 8
      for (int t = 0; t < TILE_T; ++t) s = fmaf(sm[1][0][t][i], sm[0][0][t][j], s);
      if constexpr (BIAS) {
        if (own_gb) {
          float sb = 0.f;
          for (int t = 0; t < TILE_T; ++t) sb += sm[2][0][t][i];
          s = fmaf(sb, d.bias_col[j], s);
        }
      }
      dst[e] = s;
    }
  } else {
    const int64_t row0 = args.row_offsets[n] + s0;
    for (int t = wave; t < rows_valid; t += COLLECT_THREADS / WAVE) {
      const int64_t base = (row0 + t) * args.out_row_stride + d.out_col;
      for (int e = lane; e < pp; e += WAVE) {
        const int i = e / p, j = e - i * p;
        float v = sm[1][0][t][i] * sm[0][0][t][j];
        if constexpr (BIAS) {
          if (own_gb) v = fmaf(sm[2][0][t][i], d.bias_col[j], v);
        }
        store_as(args.out, base + e, clampf(v, args.lo, args.hi), args.out_dtype);
      }
    }
  }
}

// ---- persistent variant (p <= 16, aligned operands, no bias) -------------------------------------
// One workgroup per CU walks a contiguous range of (module, tile) items; the host cuts the item list
// into ranges of equal weight, so the launch has no tail.  The scaled projection matrices of the
// current module sit in LDS in MFMA fragment order (k-step s, lane l -> 16 bytes at (s*64 + l)*16),
// staged once per module change instead of being fetched from L2 by every tile.  Each wave owns a
// quarter of the tile's tokens over the whole of K, so nothing has to be combined across waves before
// the token reduction, and that reduction runs on the matrix cores as well: the accumulator registers
// of g' and a' are exactly the A and B operands of v_mfma_f32_16x16x4_f32 (lane (c, q) holds token
// 4q + e, column c), so P += g'^T a' takes four MFMAs per 16 tokens with fp32 products.
struct PersistArgs {
  CollectArgs c;
  const int32_t* wg_first;  // [gridDim.x + 1] first item of each workgroup; item = module * tiles_pm + tile
  int tiles_pm;             // tiles per module = N * tiles_per_seq
  int r_steps;              // k-steps of LDS reserved for projection fragments
  int scratch_bytes;        // LDS between the fragments and the staging rings (exchange / per-token tiles)
  int out_vec8;             // per-token rows: every p x p block starts 16-byte aligned and p is 8 or 16
  const uint4* frag;        // RFG: scaled projection fragments of every module in global memory
  const int64_t* frag_off;  // RFG: [n_modules] first fragment (1 KB) of a module in the table (r_in's, then r_out's)
  const int32_t* order;     // RFG: the items in the order the workgroups take them (wg_first indexes this list), or null
  float* tokproj;           // per-token rows in two steps: [n_modules][N][S][2][16] a', g' of every token, or null
};

// x' = x @ R'^T for this wave's 16*MTW tokens over all of K, R' fragments read from LDS.
// acc[mt][i] belongs to token mt*16 + (lane/16)*4 + i, column lane%16.  Token rows past rows_valid
// re-read a valid row (their accumulator entries are garbage; the caller discards them).
template <typename T, int MTW, int U>
__device__ inline void project_tokens_lds(const T* __restrict__ xrow0, int64_t tok_stride, int rows_valid, int K,
                                          const uint4* __restrict__ rfrag, int lane, f32x4 (&acc)[MTW]) {
  using M = Mma<T>;
  const int r = lane & 15;
  const int q = lane >> 4;
  const T* xrow[MTW];
#pragma unroll
  for (int mt = 0; mt < MTW; ++mt)
    xrow[mt] = xrow0 + (int64_t)min(mt * 16 + r, rows_valid - 1) * tok_stride + q * M::EPL;
  const int nsteps = K / M::KS;

  auto run = [&](int ks0, auto uu_tag) {
    constexpr int UU = decltype(uu_tag)::value;
    uint4 xf[UU][MTW];
    uint4 rf[UU];
#pragma unroll
    for (int u = 0; u < UU; ++u) {
#pragma unroll
      for (int mt = 0; mt < MTW; ++mt) xf[u][mt] = load16_global(xrow[mt] + (ks0 + u) * M::KS);
      rf[u] = rfrag[(ks0 + u) * WAVE + lane];
    }
    // keep every load of the block ahead of the first MFMA: with one wave per SIMD the loads in
    // flight are all that hides the memory latency
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UU; ++u)
#pragma unroll
      for (int mt = 0; mt < MTW; ++mt) M::mma(xf[u][mt], rf[u], acc[mt]);
  };

  int ks0 = 0;
  for (; ks0 + U <= nsteps; ks0 += U) run(ks0, std::integral_constant<int, U>{});
  if constexpr (U > 2) {
    for (; ks0 + 2 <= nsteps; ks0 += 2) run(ks0, std::integral_constant<int, 2>{});
  }
  for (; ks0 < nsteps; ++ks0) run(ks0, std::integral_constant<int, 1>{});
}

__device__ inline int seq_token_limit_uniform(const int32_t* lengths, int n, int S) {
  return lengths ? min(max(load_uniform(lengths + n) - 1, 0), S) : S;
}

// Fills the global fragment table of the RFG variant (nblk blocks of 16 projection rows per k-step, those past
// row p - 1 repeating it): block (m, 0, z) writes the scaled fragments of k-steps
// [z, z + 1) * FRAG_STEPS_PER_WG of module m's r_in, block (m, 1, z) those of its r_out, in the order
// stage_projection gives them in LDS.
constexpr int FRAG_STEPS_PER_WG = 4 * STAGE_B;  // one round of loads per thread

template <typename T>
__global__ __launch_bounds__(COLLECT_THREADS) void frag_prepare_kernel(const bgx_module_desc* __restrict__ mods,
                                                                       const int64_t* __restrict__ frag_off,
                                                                       uint4* __restrict__ frag, int p, int nblk) {
  const bgx_module_desc d = mods[blockIdx.x];
  const int ks0 = blockIdx.z * FRAG_STEPS_PER_WG;
  const int K = blockIdx.y == 0 ? d.I : d.O;
  if (ks0 * Mma<T>::KS >= K) return;
  uint4* dst = frag + frag_off[blockIdx.x] * WAVE;
  for (int blk = 0; blk < nblk; ++blk) {  // blocks of 16 projection rows, interleaved per k-step
    if (blockIdx.y == 0)
      stage_projection<T>((const T*)d.r_in, d.col_scale, d.I, p, dst, threadIdx.x, ks0, ks0 + FRAG_STEPS_PER_WG, blk,
                          nblk, blk * 16);
    else
      stage_projection<T>((const T*)d.r_out, d.row_scale, d.O, p, dst + (size_t)(d.I / Mma<T>::KS) * nblk * WAVE,
                          threadIdx.x, ks0, ks0 + FRAG_STEPS_PER_WG, blk, nblk, blk * 16);
  }
}

// PB = blocks of 16 projection columns (p <= 16 * PB).  More than one only with the fragments in the global table
// (two projections to 32 columns do not fit LDS at the usual widths): a tile then gives PB x PB blocks of P, or,
// per token, a' and g' of 16 * PB columns each for the two-step rows (the only per-token route with PB > 1).
// With RFG the workgroup's waves load each block of table fragments once between them and pass it round through LDS
// (stream_segment_shared: SHARE below) instead of each loading all of it; all four then stream in step, tile after
// tile, and a wave without tokens in a tile streams that tile's first row and discards what it gets.
// BIAS: the launch has modules with a bias column and no bias factor of their own (bias_col without bias_scale):
// their P is sum_t g'_t (x) (a'_t + bias_col), so the column is added to a' of every token before the reduction.
template <typename T, bool PER_TOKEN, int MTW, int U, bool STAGED = false, bool RFG = false, int PB = 1,
          bool BIAS = false>
__global__ __launch_bounds__(COLLECT_THREADS, 1) void collect_persist_kernel(PersistArgs pa) {
  static_assert(!BIAS || (STAGED && PB == 1), "the bias column goes with the streamed kernels at p <= 16");
  static_assert(STAGED || !RFG, "the global fragment table goes with the streamed rows");
  static_assert(PB == 1 || RFG, "wider projections: fragments from the table");
  constexpr bool SHARE = RFG;
  using M = Mma<T>;
  constexpr int WAVE_T = 16 * MTW;      // tokens per wave
  constexpr int TILE_T = 4 * WAVE_T;    // tokens per workgroup
  constexpr int LDP = 16 * PB + 4;  // row of a' or g' in LDS: 16 * PB floats, padded so that rows stay 16-byte aligned
  extern __shared__ __align__(16) unsigned char smem_raw[];
  uint4* rfrag = reinterpret_cast<uint4*>(smem_raw);
  unsigned char* scratch = smem_raw + (size_t)pa.r_steps * WAVE * 16;
  // per-sequence: the P blocks of waves 1..3, double-buffered by tile parity; per-token: a', g' of each wave
  f32x4 (*pred)[3][WAVE] = reinterpret_cast<f32x4 (*)[3][WAVE]>(scratch);
  f32x4 (*pblk)[PB * PB][WAVE] = reinterpret_cast<f32x4 (*)[PB * PB][WAVE]>(scratch);  // PB > 1: [wave][block][lane]
  float (*tok)[2][WAVE_T][LDP] = reinterpret_cast<float (*)[2][WAVE_T][LDP]>(scratch);

  const CollectArgs& args = pa.c;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned char* stage = scratch + pa.scratch_bytes + wave * Stream<MTW>::BYTES_PER_WAVE;  // STAGED only
  const int c = lane & 15;
  const int q = lane >> 4;
  const int p = args.p;
  const int pp = p * p;
  const int item0 = load_uniform(pa.wg_first + blockIdx.x);
  const int item1 = load_uniform(pa.wg_first + blockIdx.x + 1);

  int cur_m = -1;
  int parity = 0;
  // STAGED: the register queue of the wave's input stream, and whether it holds the first block of the
  // tile that comes next
  uint4 v[STAGED ? STREAM_Q : 1][2 * MTW];
  uint4 rq[1][2 * PB];  // (the per-wave fragment queue of stream_segment<RFG>: not used here)
  uint4 rs[2 * PB];  // SHARE: this wave's k-pair of the block of fragments that comes next
  uint4* ring = reinterpret_cast<uint4*>(scratch + pa.scratch_bytes + 4 * Stream<MTW>::BYTES_PER_WAVE);  // SHARE
  int ring_slot = 0;
  bool primed = false;
  // Two-step per-token rows: a tile leaves 16 * MTW tokens x 32 floats per wave, i.e. 8 * MTW registers per lane.
  // They stay in registers until KEEP_TILES tiles have gathered or the range ends, and go to the workspace then:
  // a store shares the in-order completion counter of the stream's loads, so the first wait behind a store also
  // waits for the store's acknowledgement, which under this read load takes several microseconds -- once per
  // tile that was a sixth of the kernel's time; at the end of a range nothing waits behind it.
  // (Deferring wave 0's p x p partial of the per-sequence launches the same way changed nothing: 171.6 us either way.)
  constexpr int KEEP_TILES = PER_TOKEN && PB == 1 ? 8 : 1;  // wider projections: no registers to spare
  f32x4 keepA[KEEP_TILES][MTW * PB], keepG[KEEP_TILES][MTW * PB];
  int64_t keep_at[KEEP_TILES];  // element offset of the tile's first token in tokproj
  int keep_rows[KEEP_TILES];
  int kept = 0;
  auto flush_kept = [&]() {
    if constexpr (PER_TOKEN) {
      // 16-byte piece of a token's 128 * PB bytes: the first 4 * PB are a', the others g'
      constexpr int PIECES = 8 * PB;
      const int part = lane & (PIECES - 1);
#pragma unroll
      for (int j = 0; j < KEEP_TILES; ++j) {
        if (j < kept) {
          // tok[wave] is private to the wave, and a wave's LDS operations complete in order: no workgroup
          // barrier, only the compiler must keep the writes, the reads and the next tile's writes in order
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
            for (int pb = 0; pb < PB; ++pb)
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                tok[wave][0][mt * 16 + q * 4 + i][pb * 16 + c] = keepA[j][mt * PB + pb][i];
                tok[wave][1][mt * 16 + q * 4 + i][pb * 16 + c] = keepG[j][mt * PB + pb][i];
              }
          __builtin_amdgcn_wave_barrier();
          float* dstp = pa.tokproj + keep_at[j];
          constexpr int TOK_PER_PASS = WAVE / PIECES;
#pragma unroll
          for (int k = 0; k < WAVE_T / TOK_PER_PASS; ++k) {
            const int t = k * TOK_PER_PASS + lane / PIECES;
            const float4 val =
                *reinterpret_cast<const float4*>(&tok[wave][part / (4 * PB)][t][(part % (4 * PB)) * 4]);
            if (t < keep_rows[j]) {
              typedef float raw4 __attribute__((ext_vector_type(4)));
              *reinterpret_cast<raw4*>(dstp + t * (32 * PB) + part * 4) = raw4{val.x, val.y, val.z, val.w};
            }
          }
        }
      }
      kept = 0;
    }
  };
  for (int idx = item0; idx < item1; ++idx) {
    // With the fragments in a global table nothing ties a workgroup to consecutive items (no projections staged
    // per module), so the host deals the items out one by one for even loads and passes the resulting list.
    int item = idx;
    if constexpr (RFG) {
      if (pa.order != nullptr) item = load_uniform(pa.order + idx);
    }
    const int m = item / pa.tiles_pm;
    const int tile = item - m * pa.tiles_pm;
    const int n = tile / args.tiles_per_seq;
    const int ts = tile - n * args.tiles_per_seq;
    const int s0 = ts * TILE_T;
    const int s_limit = seq_token_limit_uniform(args.lengths, n, args.S);
    if (s0 >= s_limit) continue;  // whole tile is padding (uniform over the workgroup); nothing ran ahead into it
    const int rows_valid = min(WAVE_T, s_limit - s0 - wave * WAVE_T);  // of this wave; may be <= 0
    // rows the wave streams: its own, or (SHARE, none of its own) the tile's first
    const int rows_eff = SHARE ? max(rows_valid, 1) : rows_valid;

    const bgx_module_desc d = load_uniform(args.mods + m);
    const int nA = d.I / M::KS;
    const uint4* rfA = rfrag;  // fragments of r_in, then of r_out: in LDS, or (RFG) in the global table
    if constexpr (RFG) rfA = pa.frag + load_uniform(pa.frag_off + m) * WAVE;
    const uint4* rfG = rfA + (size_t)nA * PB * WAVE;
    const int64_t t0 = s0 + (SHARE && rows_valid <= 0 ? 0 : wave * WAVE_T);
    const T* a0 = (const T*)d.a + (int64_t)n * d.a_seq_stride + t0 * d.a_tok_stride;
    const T* g0 = (const T*)d.g + (int64_t)n * d.g_seq_stride + t0 * d.g_tok_stride;
    // BIAS: this lane's entry of the bias column, loaded here, ahead of the tile's stream, so that the wait for it
    // further down has none of the stream's loads in front of it; unconditionally (a load behind a branch would
    // make every wait at the join a full drain): a module without the column reads the descriptor table instead
    float bias_v = 0.f;
    if constexpr (BIAS) {
      const float* bp = d.bias_col != nullptr ? d.bias_col : reinterpret_cast<const float*>(args.mods);
      bias_v = bp[min(c, p - 1)];
    }
    if constexpr (STAGED) {
      // a tile nothing ran ahead into (the first of the range, or after padding): its first loads go out
      // before the projections are staged
      if (rows_eff > 0 && !primed) {
        const T* ua[2 * MTW];
        stream_rows<T, MTW>(a0, d.a_tok_stride, rows_eff, lane, ua);
        if constexpr (SHARE)
          stream_prime_shared<T, MTW, PB>(ua, d.I / (2 * M::KS), rfA, lane, wave, v, rs);
        else
          stream_prime<T, MTW, false, PB>(ua, d.I / (2 * M::KS), rfA, lane, v, rq);
        primed = true;
      }
    }
    if (!RFG && m != cur_m) {
      __syncthreads();  // every wave has finished reading the previous module's fragments
      stage_projection<T>((const T*)d.r_in, d.col_scale, d.I, p, rfrag, tid);
      stage_projection<T>((const T*)d.r_out, d.row_scale, d.O, p, rfrag + (size_t)nA * WAVE, tid);
      cur_m = m;
      // Staging has waited for its own loads, but not on every path the compiler sees (its guarded batches):
      // without this explicit "no vector load outstanding", the tile code below would have to assume
      // that staging loads may still be pending behind the stream's and wait for everything.
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), nothing else
      __syncthreads();
    }

    f32x4 accA[MTW * PB];  // [mt * PB + pb]
    f32x4 accG[MTW * PB];
#pragma unroll
    for (int mt = 0; mt < MTW * PB; ++mt) {
      accA[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      accG[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (rows_eff > 0) {
      if constexpr (STAGED) {
        constexpr int RG = 2 * MTW;
        const int nkpA = d.I / (2 * M::KS), nkpG = d.O / (2 * M::KS);
        const T* ua[RG];
        const T* ug[RG];
        const T* un[RG];
        stream_rows<T, MTW>(a0, d.a_tok_stride, rows_eff, lane, ua);
        stream_rows<T, MTW>(g0, d.g_tok_stride, rows_eff, lane, ug);
        if constexpr (SHARE)
          stream_segment_shared<T, MTW, PB>(ua, nkpA, ug, nkpG, rfA, rfG, stage, ring, ring_slot, lane, wave, v, rs, accA);
        else
          stream_segment<T, MTW, false, PB>(ua, nkpA, ug, nkpG, rfA, rfG, stage, lane, v, rq, accA);
        // what follows g: the a rows of the next tile of the range, where this wave has tokens in it
        int nkpN = 0;
        const uint4* rfN = rfG;  // RFG: the next tile's r_in fragments (any readable address when none follows)
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) un[rg] = ug[rg];
        if (idx + 1 < item1) {
          int item2 = idx + 1;
          if constexpr (RFG) {
            if (pa.order != nullptr) item2 = load_uniform(pa.order + idx + 1);
          }
          const int m2 = item2 / pa.tiles_pm;
          const int tile2 = item2 - m2 * pa.tiles_pm;
          const int n2 = tile2 / args.tiles_per_seq;
          const int s02 = (tile2 - n2 * args.tiles_per_seq) * TILE_T;
          const int limit2 = seq_token_limit_uniform(args.lengths, n2, args.S);
          const int rows2 = min(WAVE_T, limit2 - s02 - wave * WAVE_T);
          // SHARE: whenever the tile is not all padding, the waves without tokens in it with its first row
          if (SHARE ? s02 < limit2 : rows2 > 0) {  // rows2 > 0 implies that the tile is not all padding
            const bgx_module_desc* d2 = args.mods + m2;
            const int64_t stride2 = load_uniform(&d2->a_tok_stride);
            const T* a2 = (const T*)load_uniform(&d2->a) + (int64_t)n2 * load_uniform(&d2->a_seq_stride) +
                          (int64_t)(s02 + (rows2 > 0 ? wave * WAVE_T : 0)) * stride2;
            stream_rows<T, MTW>(a2, stride2, max(rows2, 1), lane, un);
            nkpN = load_uniform(&d2->I) / (2 * M::KS);
            if constexpr (RFG) rfN = pa.frag + load_uniform(pa.frag_off + m2) * WAVE;
          }
        }
        if constexpr (SHARE)
          stream_segment_shared<T, MTW, PB>(ug, nkpG, un, nkpN, rfG, rfN, stage, ring, ring_slot, lane, wave, v, rs, accG);
        else
          stream_segment<T, MTW, false, PB>(ug, nkpG, un, nkpN, rfG, rfN, stage, lane, v, rq, accG);
        primed = nkpN > 0;
      } else if constexpr (PB == 1) {
        project_tokens_lds<T, MTW, U>(a0, d.a_tok_stride, rows_valid, d.I, rfA, lane, accA);
        project_tokens_lds<T, MTW, U>(g0, d.g_tok_stride, rows_valid, d.O, rfG, lane, accG);
      }
      if constexpr (BIAS) {
        const float b = d.bias_col != nullptr && c < p ? bias_v : 0.f;
#pragma unroll
        for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) accA[mt][i] += b;
      }
      // token rows past the last valid one hold garbage: zero them in g' (that removes their products)
#pragma unroll
      for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
        for (int pb = 0; pb < PB; ++pb)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (mt * 16 + q * 4 + i >= rows_valid) accG[mt * PB + pb][i] = 0.f;
    } else {
      primed = false;
    }

    if constexpr (!PER_TOKEN) {
      // P[i, j] = sum_t g'[t, i] * a'[t, j] over this wave's tokens, in blocks of 16 x 16; lane (c, q) gets
      // P[16 ib + 4q + e][16 jb + c] of block (ib, jb)
      float* dst = args.partials + (((int64_t)m * args.N + n) * args.tiles_per_seq + ts) * pp;
      if constexpr (PB == 1) {
        f32x4 P = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) P = __builtin_amdgcn_mfma_f32_16x16x4f32(accG[mt][i], accA[mt][i], P, 0, 0, 0);
        if (wave > 0) pred[parity][wave - 1][lane] = P;
        __syncthreads();
        if (wave == 0) {
          const f32x4 p1 = pred[parity][0][lane], p2 = pred[parity][1][lane], p3 = pred[parity][2][lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int i = q * 4 + e;
            if (i < p && c < p) dst[i * p + c] = (P[e] + p1[e]) + (p2[e] + p3[e]);
          }
        }
        parity ^= 1;  // the next tile writes the other buffer, so one barrier per tile is enough
      } else {
        // every wave leaves its PB x PB blocks in LDS as it makes them (none is kept in registers), and the four
        // waves share the sums: wave w adds up blocks w, w + 4, ...
#pragma unroll
        for (int ib = 0; ib < PB; ++ib)
#pragma unroll
          for (int jb = 0; jb < PB; ++jb) {
            f32x4 blk = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
              for (int i = 0; i < 4; ++i)
                blk = __builtin_amdgcn_mfma_f32_16x16x4f32(accG[mt * PB + ib][i], accA[mt * PB + jb][i], blk, 0, 0, 0);
            pblk[wave][ib * PB + jb][lane] = blk;
          }
        __syncthreads();
#pragma unroll
        for (int bb = 0; bb < PB * PB / 4; ++bb) {
          const int b = bb * 4 + wave;
          const int ib = b / PB, jb = b - ib * PB;
          const f32x4 p0 = pblk[0][b][lane], p1 = pblk[1][b][lane], p2 = pblk[2][b][lane], p3 = pblk[3][b][lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int i = ib * 16 + q * 4 + e, j = jb * 16 + c;
            if (i < p && j < p) dst[i * p + j] = (p0[e] + p1[e]) + (p2[e] + p3[e]);
          }
        }
        __syncthreads();  // the next tile's blocks go to the same place
      }
    } else {
      if (PB > 1 || pa.tokproj != nullptr) {
        // two-step rows: the wave's a', g' -- 128 * PB bytes per token -- go to the workspace (later: flush_kept), and
        // token_rows_kernel writes the store rows from them, a whole row at a time
        if (rows_valid > 0) {
#pragma unroll
          for (int j = KEEP_TILES - 1; j > 0; --j) {
#pragma unroll
            for (int mt = 0; mt < MTW * PB; ++mt) {
              keepA[j][mt] = keepA[j - 1][mt];
              keepG[j][mt] = keepG[j - 1][mt];
            }
            keep_at[j] = keep_at[j - 1];
            keep_rows[j] = keep_rows[j - 1];
          }
#pragma unroll
          for (int mt = 0; mt < MTW * PB; ++mt) {
            keepA[0][mt] = accA[mt];
            keepG[0][mt] = accG[mt];
          }
          keep_at[0] = ((((int64_t)m * args.N + n) * args.S) + s0 + wave * WAVE_T) * (32 * PB);
          keep_rows[0] = rows_valid;
          if (++kept == KEEP_TILES) flush_kept();
        }
        continue;
      }
      // tok[wave] is private to the wave, and a wave's LDS operations complete in order: no workgroup
      // barrier, only the compiler must keep the writes, the reads and the next tile's writes in order
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          tok[wave][0][mt * 16 + q * 4 + i][c] = accA[mt][i];
          tok[wave][1][mt * 16 + q * 4 + i][c] = accG[mt][i];
        }
      __builtin_amdgcn_wave_barrier();
      const int64_t row0 = load_uniform(args.row_offsets + n) + s0 + wave * WAVE_T;
      if (pa.out_vec8) {
        // a lane writes 8 consecutive columns of one row i of one token's block: 16 bytes in a 16-bit store
        const int jg = p >> 3;                // 8-column groups per block row: 1 or 2
        const int lt = p == 16 ? 5 : 3;       // log2 of the p * jg lane tasks per token
        auto write_rows = [&](auto dt_tag) {  // one copy of the loop per output dtype, chosen outside it
          constexpr int DT = decltype(dt_tag)::value;
          // a lane keeps its place (i, j0) in the block and walks the tokens in steps of 64 >> lt, so that
          // nothing but two additions depends on the token
          const int rem = lane & ((1 << lt) - 1);
          const int i = rem >> (jg - 1);
          const int j0 = (rem & (jg - 1)) << 3;
          const int step_t = WAVE >> lt;
          int64_t dst = (row0 + (lane >> lt)) * args.out_row_stride + d.out_col + i * p + j0;
          const int64_t dst_step = (int64_t)step_t * args.out_row_stride;
          for (int t = lane >> lt; t < rows_valid; t += step_t, dst += dst_step) {
            const float gv = tok[wave][1][t][i];
            const float4 a_lo = *reinterpret_cast<const float4*>(&tok[wave][0][t][j0]);
            const float4 a_hi = *reinterpret_cast<const float4*>(&tok[wave][0][t][j0 + 4]);
            const float o[8] = {clampf(gv * a_lo.x, args.lo, args.hi), clampf(gv * a_lo.y, args.lo, args.hi),
                                clampf(gv * a_lo.z, args.lo, args.hi), clampf(gv * a_lo.w, args.lo, args.hi),
                                clampf(gv * a_hi.x, args.lo, args.hi), clampf(gv * a_hi.y, args.lo, args.hi),
                                clampf(gv * a_hi.z, args.lo, args.hi), clampf(gv * a_hi.w, args.lo, args.hi)};
            store8_as<DT>(args.out, dst, o);
          }
        };
        if (args.out_dtype == BGX_F32)
          write_rows(std::integral_constant<int, BGX_F32>{});
        else if (args.out_dtype == BGX_F16)
          write_rows(std::integral_constant<int, BGX_F16>{});
        else
          write_rows(std::integral_constant<int, BGX_BF16>{});
      } else
      for (int t = 0; t < rows_valid; ++t) {
        const int64_t base = (row0 + t) * args.out_row_stride + d.out_col;
        for (int e = lane; e < pp; e += WAVE) {
          const int i = e / p, j = e - i * p;
          store_as(args.out, base + e, clampf(tok[wave][1][t][i] * tok[wave][0][t][j], args.lo, args.hi),
                   args.out_dtype);
        }
      }
    }
  }
  flush_kept();
}

// Second step of the two-step per-token rows: one workgroup per token writes that token's whole store row --
// every module's p x p block clamp(g'[i] * a'[j]), the arithmetic of the one-step kernel -- from the 2 * pcols
// floats per module (pcols = 16 for p <= 16, else 32 or 64) the collection kernel left in `tokproj`.  The blocks of a row are written where the descriptors say
// (adjacent blocks make one contiguous stretch: 24 KB for 48 modules at p = 16), a lane stores 8 consecutive
// columns with one 16-byte store, and the projections come out of L2.
template <int DT>
__global__ __launch_bounds__(256) void token_rows_kernel(const bgx_module_desc* __restrict__ mods, int n_modules,
                                                         const float* __restrict__ tokproj,
                                                         const int32_t* __restrict__ lengths,
                                                         const int64_t* __restrict__ row_offsets, int N, int S, int p,
                                                         int pcols, void* out, int64_t out_row_stride, float lo,
                                                         float hi) {
  const int s = blockIdx.x;
  const int n = blockIdx.y;
  if (s >= seq_token_limit(lengths, n, S)) return;
  const int64_t row = row_offsets[n] + s;
  const int jg = p >> 3;                 // 8-column groups per block row (p is a multiple of 8)
  const int tasks_pm = p * jg;           // 16-byte pieces of a module's block
  const int tasks = n_modules * tasks_pm;
  for (int task = threadIdx.x; task < tasks; task += 256) {
    const int m = task / tasks_pm;
    const int rem = task - m * tasks_pm;
    const int i = rem / jg;
    const int j0 = (rem - i * jg) << 3;
    const float* src = tokproj + (((int64_t)m * N + n) * S + s) * (2 * pcols);  // a' (pcols floats), then g'
    const float gv = src[pcols + i];
    const float4 a_lo = *reinterpret_cast<const float4*>(src + j0);
    const float4 a_hi = *reinterpret_cast<const float4*>(src + j0 + 4);
    const float o[8] = {clampf(gv * a_lo.x, lo, hi), clampf(gv * a_lo.y, lo, hi), clampf(gv * a_lo.z, lo, hi),
                        clampf(gv * a_lo.w, lo, hi), clampf(gv * a_hi.x, lo, hi), clampf(gv * a_hi.y, lo, hi),
                        clampf(gv * a_hi.z, lo, hi), clampf(gv * a_hi.w, lo, hi)};
    store8_as<DT>(out, row * out_row_stride + mods[m].out_col + i * p + j0, o);
  }
}

// Adds the per-tile partials of each (module, sequence) in a fixed order (four interleaved running
// sums combined at the end, so that consecutive loads do not wait on each other), clamps, casts and
// writes the module's block of the output row.
__global__ __launch_bounds__(256) void collect_finalize_kernel(
    const bgx_module_desc* __restrict__ mods, const float* __restrict__ partials,
    const int32_t* __restrict__ lengths, const int64_t* __restrict__ out_rows, int N, int S, int p,
    int tiles_per_seq, int tile_tokens, void* out, int64_t out_row_stride, int out_dtype, float lo, float hi) {
  const int n = blockIdx.x;
  const int m = blockIdx.y;
  const int pp = p * p;
  const int s_limit = seq_token_limit(lengths, n, S);
  const int ntiles = (s_limit + tile_tokens - 1) / tile_tokens;
  const float* src = partials + ((int64_t)m * N + n) * tiles_per_seq * pp;
  const int64_t row = out_rows ? out_rows[n] : (int64_t)n;
  const int64_t base = row * out_row_stride + mods[m].out_col;
  for (int e = threadIdx.x; e < pp; e += blockDim.x) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int t = 0;
    for (; t + 4 <= ntiles; t += 4) {
      s0 += src[(int64_t)(t + 0) * pp + e];
      s1 += src[(int64_t)(t + 1) * pp + e];
      s2 += src[(int64_t)(t + 2) * pp + e];
      s3 += src[(int64_t)(t + 3) * pp + e];
    }
    for (; t < ntiles; ++t) s0 += src[(int64_t)t * pp + e];
    store_as(out, base + e, clampf((s0 + s1) + (s2 + s3), lo, hi), out_dtype);
  }
}

// ---- Adafactor factors ---------------------------------------------------------
__global__ __launch_bounds__(256) void adafactor_scales_kernel(const float* __restrict__ row, int O,
                                                               const float* __restrict__ col, int I,
                                                               int dtype, float* row_scale,
                                                               float* col_scale) {
  __shared__ double red[256];
  const int tid = threadIdx.x;
  if (col != nullptr) {
    for (int i = tid; i < I; i += 256)
      col_scale[i] = round_to_dtype(1.0f / sqrtf(col[i] + 1e-30f), dtype);
  }
  if (row != nullptr) {
    // mean(row + eps) accumulated in double so the result does not depend on
    // the reduction tree beyond fp32 rounding of the final mean.
    double s = 0.0;
    for (int o = tid; o < O; o += 256) s += (double)(row[o] + 1e-30f);
    red[tid] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
      if (tid < w) red[tid] += red[tid + w];
      __syncthreads();
    }
    const float mean = (float)(red[0] / (double)O);
    const float sq = sqrtf(mean);
    for (int o = tid; o < O; o += 256)
      row_scale[o] = round_to_dtype(sq * (1.0f / sqrtf(row[o] + 1e-30f)), dtype);
  }
}

// ---- in-place row unit normalisation ----------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void unit_normalize_kernel(T* rows, int64_t n_rows, int64_t D,
                                                             int64_t stride, float eps_sq) {
  __shared__ float red[256];
  const int64_t rowi = blockIdx.x;
  T* x = rows + rowi * stride;
  float s = 0.f;
  for (int64_t d = threadIdx.x; d < D; d += 256) {
    const float v = Elem<T>::load(x + d);
    s = fmaf(v, v, s);
  }
  red[threadIdx.x] = s;
  __syncthreads();
  for (unsigned w = 128; w > 0; w >>= 1) {
    if (threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  // the reference forms rsqrt in the gradient dtype and multiplies there
  const float inv = Elem<T>::round(1.0f / sqrtf(fmaxf(Elem<T>::round(red[0]), eps_sq)));
  for (int64_t d = threadIdx.x; d < D; d += 256) {
    const float v = Elem<T>::load(x + d) * inv;
    if constexpr (sizeof(T) == 4)
      *(float*)(x + d) = v;
    else if constexpr (Elem<T>::code == BGX_F16)
      ((uint16_t*)x)[d] = (uint16_t)f32_to_f16_bits(v);
    else
      ((uint16_t*)x)[d] = (uint16_t)f32_to_bf16_bits(v);
  }
}

// ---- host side ------------------------------------------------------------------------
// Optional event pairs around collect_kernel (benchmark support).  Launches may come from several host
// threads and streams at once (each pair is recorded on its own launch's stream); a launch claims its pair
// under the lock.  Enabling and reading are for the thread that owns the measurement, between launches.
static std::mutex g_timing_lock;
static std::vector<hipEvent_t> g_timing_events;  // start0, stop0, start1, stop1, ...
static int g_timing_used = 0;

int collect_timing_enable(int max_launches) {
  std::lock_guard<std::mutex> hold(g_timing_lock);
  for (hipEvent_t e : g_timing_events) (void)hipEventDestroy(e);
  g_timing_events.clear();
  g_timing_used = 0;
  BGX_REQUIRE(max_launches >= 0, BGX_E_ARG, "collect_timing_enable: max_launches=%d", max_launches);
  for (int i = 0; i < 2 * max_launches; ++i) {
    hipEvent_t e;
    BGX_HIP(hipEventCreate(&e));
    g_timing_events.push_back(e);
  }
  return 0;
}

int collect_timing_read(float* ms_out, int capacity, int* count_out) {
  BGX_REQUIRE(ms_out && count_out && capacity >= 0, BGX_E_ARG, "collect_timing_read: null output");
  std::lock_guard<std::mutex> hold(g_timing_lock);
  const int n = g_timing_used < capacity ? g_timing_used : capacity;
  for (int i = 0; i < n; ++i) {
    BGX_HIP(hipEventSynchronize(g_timing_events[2 * i + 1]));
    BGX_HIP(hipEventElapsedTime(&ms_out[i], g_timing_events[2 * i], g_timing_events[2 * i + 1]));
  }
  *count_out = n;
  return 0;
}

// The event pair of the next timed launch, or false when timing is off or the pairs are used up.
static bool claim_timing_pair(hipEvent_t* start, hipEvent_t* stop) {
  std::lock_guard<std::mutex> hold(g_timing_lock);
  if (2 * (g_timing_used + 1) > (int)g_timing_events.size()) return false;
  *start = g_timing_events[2 * g_timing_used];
  *stop = g_timing_events[2 * g_timing_used + 1];
  ++g_timing_used;
  return true;
}

// ---- host words into device memory without a copy engine ------------------------------------------------
// A launch's descriptor table normally reaches the workspace by hipMemcpyAsync from pageable memory.  For the
// entry point that must not allocate or stage anything, the same bytes travel as kernel arguments instead:
// 3584 bytes per launch, written by the kernel itself.
constexpr int POKE_WORDS = 896;
struct PokeArgs {
  uint32_t words[POKE_WORDS];
};
__global__ void __launch_bounds__(256) poke_kernel(uint32_t* __restrict__ dst, int n, const PokeArgs a) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = a.words[i];
}

static int upload(void* dst, const void* src, size_t bytes, hipStream_t st, bool by_kernel) {
  if (!by_kernel) {
    BGX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, st));
    return 0;
  }
  BGX_REQUIRE(bytes % 4 == 0, BGX_E_ARG, "collect: table of %zu bytes is not a whole number of words", bytes);
  const size_t words = bytes / 4;
  for (size_t w0 = 0; w0 < words; w0 += POKE_WORDS) {
    PokeArgs a;
    const int n = (int)std::min<size_t>(POKE_WORDS, words - w0);
    memcpy(a.words, (const char*)src + w0 * 4, (size_t)n * 4);
    hipLaunchKernelGGL(poke_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (uint32_t*)dst + w0, n, a);
    BGX_HIP(hipGetLastError());
  }
  return 0;
}

static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

constexpr int PERSIST_MAX_WGS = 1024;        // upper bound on the workgroups of the persistent variant
constexpr size_t LDS_PER_WG = 160 * 1024;    // LDS one workgroup may allocate on gfx950

static size_t ranges_offset(int n_modules) { return (size_t)n_modules * sizeof(bgx_module_desc); }
static size_t frag_off_offset(int n_modules) {
  return align_up(ranges_offset(n_modules) + (PERSIST_MAX_WGS + 1) * sizeof(int32_t), 8);
}
// head of the workspace: the descriptor table, the item ranges of the persistent workgroups, and each
// module's position in the global fragment table
static size_t desc_bytes(int n_modules) {
  return align_up(frag_off_offset(n_modules) + (size_t)n_modules * sizeof(int64_t), 256);
}

constexpr int MIN_TILE_T = 64;  // smallest token tile any kernel variant uses: bounds the partials

size_t collect_workspace_bytes(int n_modules, int N, int S, int p) {
  if (n_modules <= 0 || N <= 0 || S <= 0 || p <= 0) return 0;
  const size_t tiles = (size_t)((S + MIN_TILE_T - 1) / MIN_TILE_T);
  return desc_bytes(n_modules) + (size_t)n_modules * N * tiles * p * p * sizeof(float);
}

constexpr int PERSIST_MAX_PB = 4;  // blocks of 16 projection columns the streamed kernel is built for: 1, 2 or 4
static int table_blocks(int p) {
  const int pb = (p + 15) / 16;
  return pb == 3 ? 4 : pb;
}

// Bytes of the global fragment table for these modules (1 KB per k-step of I + O and block of 16 projection
// columns), or 0 when the table cannot be used: a width that is not a multiple of two k-steps, p > 64, a bias column with a factor of its own.
static size_t fragment_table_bytes(const bgx_module_desc* mods, int n_modules, int p, int in_dtype) {
  if (p > 16 * PERSIST_MAX_PB) return 0;
  const int kstep = in_dtype == BGX_F32 ? 16 : 32;
  size_t steps = 0;
  for (int m = 0; m < n_modules; ++m) {
    if (mods[m].I <= 0 || mods[m].O <= 0 || mods[m].I % (2 * kstep) || mods[m].O % (2 * kstep) || mods[m].bias_scale)
      return 0;
    steps += (size_t)(mods[m].I + mods[m].O) / kstep;
  }
  return steps * 1024 * (size_t)table_blocks(p);
}

// The workspace that also holds the fragment table, for launches whose modules are too wide for LDS.
static size_t item_list_bytes(int n_modules, int N, int S) {
  return (size_t)n_modules * (size_t)N * (size_t)((S + 63) / 64) * sizeof(int32_t);
}

// Projected activations and output gradients of every token (a', g': 2 x 16 floats per module and token, 2 x 32 or
// 2 x 64 for p > 16), the intermediate of the two-step per-token rows; 0 where that route does not apply (p other
// than 8, 16 or a multiple of 8 up to 64).
static size_t token_projection_bytes(int n_modules, int N, int S, int p) {
  if (p != 8 && p != 16 && !(p > 16 && p <= 16 * PERSIST_MAX_PB && p % 8 == 0)) return 0;
  return (size_t)n_modules * (size_t)N * (size_t)S * 32 * table_blocks(p) * sizeof(float);
}

// Where the parts of the larger workspace start.
struct WorkspaceLayout {
  size_t frag, order, tokproj, total;
};
static WorkspaceLayout workspace_layout(size_t base, size_t table, int n_modules, int N, int S, int p) {
  WorkspaceLayout l;
  l.frag = align_up(base, 256);
  l.order = align_up(l.frag + table, 256);
  l.tokproj = align_up(l.order + (table ? item_list_bytes(n_modules, N, S) : 0), 256);
  // wider projections reach the two-step rows only through the table
  l.total = l.tokproj + (p > 16 && table == 0 ? 0 : token_projection_bytes(n_modules, N, S, p));
  return l;
}

size_t collect_workspace_bytes_for(const bgx_module_desc* mods, int n_modules, int N, int S, int p, int in_dtype) {
  const size_t base = collect_workspace_bytes(n_modules, N, S, p);
  if (base == 0 || mods == nullptr) return base;
  // behind the minimum: the fragment table, the list of (module, tile) items in the order the workgroups take them
  // (at most one per 64 tokens of a sequence and module; only with a table), the tokens' projections
  return workspace_layout(base, fragment_table_bytes(mods, n_modules, p, in_dtype), n_modules, N, S, p).total;
}

template <typename T, int PB, bool ALIGNED, int MT, int U>
static void launch_collect(bool per_token, bool bias, dim3 grid, hipStream_t st, const CollectArgs& args) {
  const dim3 block(COLLECT_THREADS);
  if (bias) {
    // the rarely used bias variant runs on 64-token tiles whatever MT says, to bound its LDS footprint
    if (per_token)
      hipLaunchKernelGGL((collect_kernel<T, PB, ALIGNED, true, 4, 1, true>), grid, block, 0, st, args);
    else
      hipLaunchKernelGGL((collect_kernel<T, PB, ALIGNED, false, 4, 1, true>), grid, block, 0, st, args);
  } else if (per_token) {
    hipLaunchKernelGGL((collect_kernel<T, PB, ALIGNED, true, MT, U>), grid, block, 0, st, args);
  } else {
    hipLaunchKernelGGL((collect_kernel<T, PB, ALIGNED, false, MT, U>), grid, block, 0, st, args);
  }
}

// tokens per workgroup: 128 for the common case (p <= 16, aligned operands), else 64
// 128-token tiles halve the projection-matrix traffic per token, but a sequence whose length is just past
// a multiple of 128 wastes most of its last tile; fall back to 64-token tiles when that waste exceeds 4 %.
static int tile_tokens_for(int pb, bool aligned, bool bias, int S) {
  if (!(pb == 1 && aligned && !bias)) return 64;
  const int padded = (S + 127) / 128 * 128;
  return (int64_t)padded * 100 <= (int64_t)S * 104 ? 128 : 64;
}

template <typename T>
static void launch_collect_pb(int pb, bool aligned, bool per_token, bool bias, int tile_tokens, dim3 grid,
                              hipStream_t st, const CollectArgs& args) {
  if (pb == 1) {
    if (aligned && tile_tokens == 128) return launch_collect<T, 1, true, 8, 2>(per_token, bias, grid, st, args);
    aligned ? launch_collect<T, 1, true, 4, 2>(per_token, bias, grid, st, args)
            : launch_collect<T, 1, false, 4, 2>(per_token, bias, grid, st, args);
  } else if (pb == 2) {
    aligned ? launch_collect<T, 2, true, 4, 2>(per_token, bias, grid, st, args)
            : launch_collect<T, 2, false, 4, 2>(per_token, bias, grid, st, args);
  } else {
    aligned ? launch_collect<T, 4, true, 4, 1>(per_token, bias, grid, st, args)
            : launch_collect<T, 4, false, 4, 1>(per_token, bias, grid, st, args);
  }
}

constexpr int MAX_DEVICES = 64;

// CUs of the current device (cached per device)
static int compute_units(int* out) {
  static std::atomic<int> cached[MAX_DEVICES];
  int dev = 0;
  BGX_HIP(hipGetDevice(&dev));
  int cus = (dev >= 0 && dev < MAX_DEVICES) ? cached[dev].load(std::memory_order_relaxed) : 0;
  if (cus <= 0) {
    BGX_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (dev >= 0 && dev < MAX_DEVICES) cached[dev].store(cus, std::memory_order_relaxed);
  }
  *out = cus;
  return 0;
}

template <typename T, bool PER_TOKEN, int MTW, int U, bool STAGED, bool RFG, int PB = 1, bool BIAS = false>
static int launch_persist_one(int wgs, size_t lds, hipStream_t st, const PersistArgs& pa) {
  auto kern = collect_persist_kernel<T, PER_TOKEN, MTW, U, STAGED, RFG, PB, BIAS>;
  // the opt-in to more than 64 KB of dynamic LDS is per kernel and per device; do it once for each
  static std::atomic<bool> opted_in[MAX_DEVICES];
  int dev = 0;
  BGX_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= MAX_DEVICES || !opted_in[dev].load(std::memory_order_acquire)) {
    BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_PER_WG));
    if (dev >= 0 && dev < MAX_DEVICES) opted_in[dev].store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(COLLECT_THREADS), lds, st, pa);
  return 0;
}

template <typename T, bool STAGED, bool RFG, bool BIAS = false>
static int launch_persist_s(bool per_token, int tile_tokens, int wgs, size_t lds, hipStream_t st,
                            const PersistArgs& pa) {
  if (tile_tokens == 128)
    return per_token ? launch_persist_one<T, true, 2, 4, STAGED, RFG, 1, BIAS>(wgs, lds, st, pa)
                     : launch_persist_one<T, false, 2, 4, STAGED, RFG, 1, BIAS>(wgs, lds, st, pa);
  return per_token ? launch_persist_one<T, true, 1, 8, STAGED, RFG, 1, BIAS>(wgs, lds, st, pa)
                   : launch_persist_one<T, false, 1, 8, STAGED, RFG, 1, BIAS>(wgs, lds, st, pa);
}

// the variants with the fragments in the global table; pb: blocks of 16 projection columns (more than one: tiles of
// 128 or 256 tokens; per token 128, two-step rows)
template <typename T>
static int launch_persist_table(bool per_token, int pb, int tile_tokens, int wgs, size_t lds, hipStream_t st,
                                const PersistArgs& pa) {
  if (pb == 1) {
    if (tile_tokens == 128)
      return per_token ? launch_persist_one<T, true, 2, 4, true, true, 1>(wgs, lds, st, pa)
                       : launch_persist_one<T, false, 2, 4, true, true, 1>(wgs, lds, st, pa);
    return per_token ? launch_persist_one<T, true, 1, 8, true, true, 1>(wgs, lds, st, pa)
                     : launch_persist_one<T, false, 1, 8, true, true, 1>(wgs, lds, st, pa);
  }
  if (pb == 2) {
    if (per_token) return launch_persist_one<T, true, 2, 4, true, true, 2>(wgs, lds, st, pa);
    return tile_tokens == 256 ? launch_persist_one<T, false, 4, 4, true, true, 2>(wgs, lds, st, pa)
                              : launch_persist_one<T, false, 2, 4, true, true, 2>(wgs, lds, st, pa);
  }
  // four blocks: 128 tokens (with 256 the registers spill 200 bytes)
  return per_token ? launch_persist_one<T, true, 2, 4, true, true, 4>(wgs, lds, st, pa)
                   : launch_persist_one<T, false, 2, 4, true, true, 4>(wgs, lds, st, pa);
}

// staged: streamed token rows; rfg: (staged only) projection fragments from the global table
// bias: modules with a bias column in the launch (streamed variants at p <= 16 only: the caller routes so)
template <typename T>
static int launch_persist(bool staged, bool rfg, bool bias, bool per_token, int pb, int tile_tokens, int wgs,
                          size_t lds, hipStream_t st, const PersistArgs& pa) {
  if (bias)
    return rfg ? launch_persist_s<T, true, true, true>(per_token, tile_tokens, wgs, lds, st, pa)
               : launch_persist_s<T, true, false, true>(per_token, tile_tokens, wgs, lds, st, pa);
  if (rfg) return launch_persist_table<T>(per_token, pb, tile_tokens, wgs, lds, st, pa);
  return staged ? launch_persist_s<T, true, false>(per_token, tile_tokens, wgs, lds, st, pa)
                : launch_persist_s<T, false, false>(per_token, tile_tokens, wgs, lds, st, pa);
}

// LDS beside the projection fragments: the larger of the P exchange buffers and the per-token a', g' tiles
static size_t persist_scratch_bytes(int tile_tokens, int blocks = 1) {
  return std::max((size_t)2 * 3 * WAVE * 16, (size_t)2 * tile_tokens * (16 * blocks + 4) * sizeof(float));
}

int collect_impl(bool per_token, const bgx_module_desc* mods_host, int n_modules, int N, int S,
                 int p, int in_dtype, const int32_t* lengths, const int64_t* rows_or_offsets,
                 void* out, int64_t out_row_stride, int out_dtype, float lo, float hi, void* ws,
                 size_t ws_bytes, void* stream, bool tables_by_kernel) {
  BGX_REQUIRE(mods_host && out && ws, BGX_E_ARG, "collect: null mods/out/workspace");
  BGX_REQUIRE(n_modules > 0 && N > 0 && S > 0, BGX_E_ARG, "collect: n_modules=%d N=%d S=%d", n_modules, N, S);
  BGX_REQUIRE(n_modules <= 65535, BGX_E_SHAPE, "collect: n_modules=%d exceeds 65535", n_modules);
  BGX_REQUIRE(p >= 1 && p <= 64, BGX_E_SHAPE, "collect: projection dim p=%d outside 1..64", p);
  BGX_REQUIRE(in_dtype >= BGX_F32 && in_dtype <= BGX_BF16, BGX_E_DTYPE, "collect: in_dtype=%d", in_dtype);
  BGX_REQUIRE(out_dtype >= BGX_F32 && out_dtype <= BGX_BF16, BGX_E_DTYPE, "collect: out_dtype=%d", out_dtype);
  BGX_REQUIRE(out_row_stride > 0, BGX_E_ARG, "collect: out_row_stride=%lld", (long long)out_row_stride);
  if (per_token)
    BGX_REQUIRE(lengths && rows_or_offsets, BGX_E_ARG, "collect_tok: lengths and row_offsets are required");
  const size_t need = collect_workspace_bytes(n_modules, N, S, p);
  BGX_REQUIRE(ws_bytes >= need, BGX_E_WORKSPACE, "collect: workspace %zu < %zu bytes", ws_bytes, need);
  BGX_REQUIRE(((uintptr_t)ws & 255) == 0, BGX_E_ALIGN, "collect: workspace must be 256-byte aligned");

  const int epl = in_dtype == BGX_F32 ? 4 : 8;
  const int kstep = in_dtype == BGX_F32 ? 16 : 32;
  bool aligned = true;
  bool any_bias = false;     // modules with a bias column ...
  bool scaled_bias = false;  // ... and with a factor of its own on it (a second projection of g: tile kernel only)
  for (int m = 0; m < n_modules; ++m) {
    const bgx_module_desc& d = mods_host[m];
    BGX_REQUIRE(d.a && d.g && d.r_in && d.r_out, BGX_E_ARG, "collect: module %d has a null a/g/r_in/r_out", m);
    BGX_REQUIRE(d.I > 0 && d.O > 0, BGX_E_ARG, "collect: module %d I=%d O=%d", m, d.I, d.O);
    BGX_REQUIRE(d.out_col >= 0 && d.out_col + (int64_t)p * p <= out_row_stride, BGX_E_ARG,
                "collect: module %d columns [%lld, +%d) do not fit a row of %lld", m, (long long)d.out_col,
                p * p, (long long)out_row_stride);
    BGX_REQUIRE(d.bias_col != nullptr || d.bias_scale == nullptr, BGX_E_ARG,
                "collect: module %d has a bias_scale but no bias_col", m);
    any_bias = any_bias || d.bias_col != nullptr;
    scaled_bias = scaled_bias || d.bias_scale != nullptr;
    const bool ok = ((uintptr_t)d.a % 16 == 0) && ((uintptr_t)d.g % 16 == 0) &&
                    ((uintptr_t)d.r_in % 16 == 0) && ((uintptr_t)d.r_out % 16 == 0) &&
                    (d.I % kstep == 0) && (d.O % kstep == 0) && (d.a_seq_stride % epl == 0) &&
                    (d.col_scale == nullptr || (uintptr_t)d.col_scale % 16 == 0) &&
                    (d.row_scale == nullptr || (uintptr_t)d.row_scale % 16 == 0) &&
                    (d.bias_scale == nullptr || (uintptr_t)d.bias_scale % 16 == 0) &&
                    (d.a_tok_stride % epl == 0) && (d.g_seq_stride % epl == 0) &&
                    (d.g_tok_stride % epl == 0);
    aligned = aligned && ok;
  }

  hipStream_t st = (hipStream_t)stream;
  bgx_module_desc* mods_dev = (bgx_module_desc*)ws;
  // Workgroups are dispatched module by module; putting the modules with the most columns first
  // leaves the cheapest tiles for the end of the launch, which shortens its tail.  The order has no
  // effect on the result: every descriptor carries its own output column.
  std::vector<bgx_module_desc> sorted(mods_host, mods_host + n_modules);
  std::stable_sort(sorted.begin(), sorted.end(), [](const bgx_module_desc& x, const bgx_module_desc& y) {
    return (int64_t)x.I + x.O > (int64_t)y.I + y.O;
  });

  CollectArgs args;
  args.mods = mods_dev;
  args.lengths = lengths;
  args.N = N;
  args.S = S;
  args.p = p;
  const int pb = (p + 15) / 16;
  // Projections wider than 16 columns: per-sequence rows go through the streamed kernel with the fragments in the
  // global table, when the caller's workspace has room for it, on tiles of 128 or 256 tokens (a wave then loads
  // as many bytes of fragments as of tokens, or half as many).
  const size_t frag_bytes = fragment_table_bytes(sorted.data(), n_modules, p, in_dtype);
  const WorkspaceLayout lay = workspace_layout(need, frag_bytes, n_modules, N, S, p);
  // Per-token rows take it only in two steps (projections of every token to the workspace, whole rows from there).
  const int64_t out_elem = out_dtype == BGX_F32 ? 4 : 2;
  bool wide_tok = per_token && pb > 1 && p % 8 == 0 && (uintptr_t)out % 16 == 0 &&
                  (out_row_stride * out_elem) % 16 == 0 && lay.total > lay.tokproj && ws_bytes >= lay.total &&
                  N <= 65535 && !switches().collect_two_step_off;
  for (int m = 0; m < n_modules && wide_tok; ++m) wide_tok = (sorted[m].out_col * out_elem) % 16 == 0;
  const bool wide = pb > 1 && pb <= PERSIST_MAX_PB && (!per_token || wide_tok) && aligned && !any_bias &&
                    frag_bytes > 0 && ws_bytes >= lay.frag + frag_bytes && switches().collect_staged &&
                    switches().collect_persist;
  int tile_tokens = tile_tokens_for(pb, aligned, scaled_bias, S);
  if (wide && per_token) tile_tokens = 128;
  if (wide && !per_token) {
    // 256 tokens where the sequence length wastes little of a wave's 64 (measured 208 us against 225 us at p = 32
    // on 4 x 1024 tokens of 48 modules); with four blocks the registers hold a wave's 32 tokens only
    tile_tokens = pb == 2 && (int64_t)((S + 63) / 64 * 64) * 100 <= (int64_t)S * 104 ? 256 : 128;
  }
  args.tiles_per_seq = (S + tile_tokens - 1) / tile_tokens;
  int64_t tiles = (int64_t)N * args.tiles_per_seq;
  BGX_REQUIRE(tiles <= 0x7fffffffLL, BGX_E_SHAPE, "collect: %lld tiles exceed the grid limit", (long long)tiles);

  // The persistent variant needs every module's projection fragments (16 rows x (I + O) elements) to
  // fit in LDS beside its exchange buffers.
  int r_steps = 0;
  for (int m = 0; m < n_modules; ++m) r_steps = std::max(r_steps, (sorted[m].I + sorted[m].O) / kstep);
  const size_t scratch_bytes =
      per_token ? persist_scratch_bytes(tile_tokens, wide ? table_blocks(p) : 1)
                : (wide ? (size_t)4 * WAVE * 16 * table_blocks(p) * table_blocks(p) : (size_t)2 * 3 * WAVE * 16);
  size_t persist_lds = (size_t)r_steps * 1024 + scratch_bytes;
  bool persist = pb == 1 && aligned && !scaled_bias && persist_lds <= LDS_PER_WG &&
                 tiles * n_modules <= 0x7fffffffLL;
  // staging rings for fully coalesced loads: every K a multiple of two k-steps, and 32 KB more of LDS
  const size_t stage_bytes = (size_t)4 * (tile_tokens == 256   ? Stream<4>::BYTES_PER_WAVE
                                          : tile_tokens == 128 ? Stream<2>::BYTES_PER_WAVE
                                                               : Stream<1>::BYTES_PER_WAVE);
  bool staged = persist && persist_lds + stage_bytes <= LDS_PER_WG;
  for (int m = 0; m < n_modules && staged; ++m)
    staged = sorted[m].I % (2 * kstep) == 0 && sorted[m].O % (2 * kstep) == 0;
  staged = staged && switches().collect_staged;
  if (staged) persist_lds += stage_bytes;
  // Modules too wide for LDS: the streamed kernel with the fragments in a global table, when the caller's
  // workspace has room for it (bgx_collect_workspace_bytes_for) -- else the tile kernel.
  const size_t frag_ws_off = lay.frag;
  bool rfg = !persist && (pb == 1 || wide) && aligned && !scaled_bias && tiles * n_modules <= 0x7fffffffLL && frag_bytes > 0 &&
             ws_bytes >= frag_ws_off + frag_bytes;
  rfg = rfg && switches().collect_staged;
  if (rfg) {  // beside the rest: the ring through which the workgroup shares the table's fragments
    persist = staged = true;
    r_steps = 0;
    persist_lds = scratch_bytes + stage_bytes + (size_t)stream_ring_bytes(table_blocks(p));
  }
  // BGX_COLLECT_PERSIST=0 in the environment forces the one-workgroup-per-tile kernel (tests, comparisons)
  persist = persist && switches().collect_persist;
  // a bias column goes with the streamed variants only
  if (any_bias && !staged) persist = false;
  rfg = rfg && persist;
  if (!persist && any_bias && tile_tokens != 64) {  // the tile kernel's bias variant runs on 64-token tiles
    tile_tokens = 64;
    args.tiles_per_seq = (S + tile_tokens - 1) / tile_tokens;
    tiles = (int64_t)N * args.tiles_per_seq;
    BGX_REQUIRE(tiles <= 0x7fffffffLL, BGX_E_SHAPE, "collect: %lld tiles exceed the grid limit", (long long)tiles);
  }

  std::vector<unsigned char> head((size_t)n_modules * sizeof(bgx_module_desc));
  memcpy(head.data(), sorted.data(), head.size());
  // table variant: room behind the table for the item list that lets the workgroups take items out of order
  const size_t order_ws_off = lay.order;
  const bool rfg_order = rfg && ws_bytes >= order_ws_off + (size_t)tiles * n_modules * sizeof(int32_t) &&
                         !switches().collect_lpt_off;
  std::vector<int32_t> order;
  int wgs = 0;
  if (persist) {
    int cus = 0;
    const int rc_cus = compute_units(&cus);
    if (rc_cus != 0) return rc_cus;
    const int64_t items = tiles * n_modules;
    wgs = (int)std::min<int64_t>(std::min(std::max(cus, 1), PERSIST_MAX_WGS), items);
    // Contiguous ranges with the smallest possible maximum cost.  An item costs its k-steps plus a constant
    // for the token reduction; a range also pays for staging the projections of every module it touches
    // (16 rows against the tile's tokens, counted twice because those loads come in dependent rounds).
    std::vector<int32_t> first((size_t)wgs + 1, (int32_t)items);
    constexpr int REDUCE_STEPS = 2;
    std::vector<double> w(n_modules), sw(n_modules);
    double total = 0.0, biggest = 0.0;
    for (int m = 0; m < n_modules; ++m) {
      const double ks = (double)((sorted[m].I + sorted[m].O) / kstep);
      w[m] = ks + REDUCE_STEPS;
      sw[m] = rfg ? 0.0 : ks * 32.0 / (double)tile_tokens;  // nothing is staged when the fragments stay in global memory
      total += (double)tiles * w[m] + sw[m];
      biggest = std::max(biggest, w[m] + sw[m]);
    }
    // ranges filled in order up to `limit`: how many are needed (bounds != nullptr: also where they start)
    auto fill = [&](double limit, int32_t* bounds) {
      int64_t parts = 1;
      double load = 0.0;
      int staged_m = -1;
      for (int m = 0; m < n_modules; ++m) {
        int64_t left = tiles;
        while (left > 0) {
          const double extra = staged_m == m ? 0.0 : sw[m];
          const int64_t fit = (int64_t)std::floor((limit - load - extra) / w[m] + 1e-9);
          if (fit <= 0) {  // load > 0 here, since limit >= biggest
            if (bounds && parts < wgs) bounds[parts] = (int32_t)((int64_t)m * tiles + (tiles - left));
            ++parts;
            load = 0.0;
            staged_m = -1;
            continue;
          }
          const int64_t take = std::min(fit, left);
          load += extra + (double)take * w[m];
          staged_m = m;
          left -= take;
        }
      }
      return parts;
    };
    double lo_l = std::max(biggest, total / (double)wgs), hi_l = total + biggest;
    for (int it = 0; it < 48 && hi_l - lo_l > 1e-3 * lo_l; ++it) {
      const double mid = 0.5 * (lo_l + hi_l);
      if (fill(mid, nullptr) <= wgs) hi_l = mid; else lo_l = mid;
    }
    first[0] = 0;
    fill(hi_l, first.data());
    first[wgs] = (int32_t)items;
    if (rfg_order) {
      // Longest item first to the least loaded workgroup: the modules are sorted by width, so the items come in that
      // order already.  A workgroup's items stay in ascending order (tiles of one module one after the other).
      std::vector<int32_t> owner((size_t)items);
      std::vector<int32_t> count((size_t)wgs, 0);
      typedef std::pair<double, int> Load;
      std::priority_queue<Load, std::vector<Load>, std::greater<Load>> heap;
      for (int g = 0; g < wgs; ++g) heap.push(Load(0.0, g));
      for (int64_t it = 0; it < items; ++it) {
        const Load l = heap.top();
        heap.pop();
        owner[(size_t)it] = l.second;
        ++count[(size_t)l.second];
        heap.push(Load(l.first + w[(size_t)(it / tiles)], l.second));
      }
      for (int g = 0; g < wgs; ++g) first[(size_t)g + 1] = first[(size_t)g] + count[(size_t)g];
      order.resize((size_t)items);
      std::vector<int32_t> next(first.begin(), first.end() - 1);
      for (int64_t it = 0; it < items; ++it) order[(size_t)next[(size_t)owner[(size_t)it]]++] = (int32_t)it;
    }
    head.resize(desc_bytes(n_modules), 0);
    memcpy(head.data() + ranges_offset(n_modules), first.data(), first.size() * sizeof(int32_t));
    if (rfg) {  // where each module's fragments start, in fragments of 1 KB
      std::vector<int64_t> foff((size_t)n_modules);
      int64_t steps = 0;
      for (int m = 0; m < n_modules; ++m) {
        foff[m] = steps;
        steps += (int64_t)(sorted[m].I + sorted[m].O) / kstep * table_blocks(p);
      }
      memcpy(head.data() + frag_off_offset(n_modules), foff.data(), foff.size() * sizeof(int64_t));
    }
  }
  if (const int rc = upload(mods_dev, head.data(), head.size(), st, tables_by_kernel)) return rc;
  if (!order.empty())
    if (const int rc = upload((char*)ws + order_ws_off, order.data(), order.size() * sizeof(int32_t), st,
                              tables_by_kernel))
      return rc;
  uint4* frag_dev = (uint4*)((char*)ws + frag_ws_off);
  const int64_t* frag_off_dev = (const int64_t*)((const char*)ws + frag_off_offset(n_modules));
  if (rfg) {
    int widest = 0;
    for (int m = 0; m < n_modules; ++m) widest = std::max(widest, std::max(sorted[m].I, sorted[m].O) / kstep);
    const dim3 pgrid((unsigned)n_modules, 2, (unsigned)((widest + FRAG_STEPS_PER_WG - 1) / FRAG_STEPS_PER_WG));
    if (in_dtype == BGX_F32)
      hipLaunchKernelGGL(frag_prepare_kernel<float>, pgrid, dim3(COLLECT_THREADS), 0, st, mods_dev, frag_off_dev, frag_dev, p,
                         table_blocks(p));
    else if (in_dtype == BGX_F16)
      hipLaunchKernelGGL(frag_prepare_kernel<f16_t>, pgrid, dim3(COLLECT_THREADS), 0, st, mods_dev, frag_off_dev, frag_dev, p,
                         table_blocks(p));
    else
      hipLaunchKernelGGL(frag_prepare_kernel<bf16_t>, pgrid, dim3(COLLECT_THREADS), 0, st, mods_dev, frag_off_dev, frag_dev, p,
                         table_blocks(p));
    BGX_HIP(hipGetLastError());
  }
  args.partials = (float*)((char*)ws + desc_bytes(n_modules));
  args.row_offsets = per_token ? rows_or_offsets : nullptr;
  args.out = out;
  args.out_row_stride = out_row_stride;
  args.out_dtype = out_dtype;
  args.lo = lo;
  args.hi = hi;

  const dim3 grid((unsigned)tiles, (unsigned)n_modules);
  bool two_step = false;
  hipEvent_t ev_start, ev_stop;
  const bool timed = claim_timing_pair(&ev_start, &ev_stop);
  if (timed) BGX_HIP(hipEventRecord(ev_start, st));
  if (persist) {
    PersistArgs pa;
    pa.c = args;
    pa.wg_first = (const int32_t*)((const char*)ws + ranges_offset(n_modules));
    pa.frag = frag_dev;
    pa.frag_off = frag_off_dev;
    pa.order = order.empty() ? nullptr : (const int32_t*)((const char*)ws + order_ws_off);
    pa.tiles_pm = (int)tiles;
    pa.r_steps = r_steps;
    pa.scratch_bytes = (int)scratch_bytes;
    bool vec8 = per_token && (p == 8 || p == 16 || wide) && (uintptr_t)out % 16 == 0 &&
                (out_row_stride * out_elem) % 16 == 0;
    for (int m = 0; m < n_modules && vec8; ++m) vec8 = (sorted[m].out_col * out_elem) % 16 == 0;
    pa.out_vec8 = vec8 ? 1 : 0;
    // per-token rows in two steps when the blocks can be written 16 bytes at a time and the caller's workspace has
    // room for the tokens' projections (bgx_collect_workspace_bytes_for)
    two_step = vec8 && lay.total > lay.tokproj && ws_bytes >= lay.total && N <= 65535 &&
               !switches().collect_two_step_off;
    pa.tokproj = two_step ? (float*)((char*)ws + lay.tokproj) : nullptr;
    int rc;
    if (in_dtype == BGX_F32)
      rc = launch_persist<float>(staged, rfg, any_bias, per_token, pb, tile_tokens, wgs, persist_lds, st, pa);
    else if (in_dtype == BGX_F16)
      rc = launch_persist<f16_t>(staged, rfg, any_bias, per_token, pb, tile_tokens, wgs, persist_lds, st, pa);
    else
      rc = launch_persist<bf16_t>(staged, rfg, any_bias, per_token, pb, tile_tokens, wgs, persist_lds, st, pa);
    if (rc != 0) return rc;
    note_kernel(FAMILY_COLLECT, rfg ? "collect_persist_table" : staged ? "collect_persist_lds" : "collect_persist_direct");
  } else if (in_dtype == BGX_F32) {
    launch_collect_pb<float>(pb, aligned, per_token, any_bias, tile_tokens, grid, st, args);
  } else if (in_dtype == BGX_F16) {
    launch_collect_pb<f16_t>(pb, aligned, per_token, any_bias, tile_tokens, grid, st, args);
  } else {
    launch_collect_pb<bf16_t>(pb, aligned, per_token, any_bias, tile_tokens, grid, st, args);
  }
  BGX_HIP(hipGetLastError());
  if (!persist) note_kernel(FAMILY_COLLECT, "collect_tile");
  if (two_step) {
    const dim3 tgrid((unsigned)S, (unsigned)N);
    const float* tp = (const float*)((const char*)ws + lay.tokproj);
    if (out_dtype == BGX_F32)
      hipLaunchKernelGGL(token_rows_kernel<BGX_F32>, tgrid, dim3(256), 0, st, mods_dev, n_modules, tp, lengths,
                         rows_or_offsets, N, S, p, 16 * table_blocks(p), out, out_row_stride, lo, hi);
    else if (out_dtype == BGX_F16)
      hipLaunchKernelGGL(token_rows_kernel<BGX_F16>, tgrid, dim3(256), 0, st, mods_dev, n_modules, tp, lengths,
                         rows_or_offsets, N, S, p, 16 * table_blocks(p), out, out_row_stride, lo, hi);
    else
      hipLaunchKernelGGL(token_rows_kernel<BGX_BF16>, tgrid, dim3(256), 0, st, mods_dev, n_modules, tp, lengths,
                         rows_or_offsets, N, S, p, 16 * table_blocks(p), out, out_row_stride, lo, hi);
    BGX_HIP(hipGetLastError());
  }
  if (timed) BGX_HIP(hipEventRecord(ev_stop, st));

  if (!per_token) {
    hipLaunchKernelGGL(collect_finalize_kernel, dim3((unsigned)N, (unsigned)n_modules), dim3(256), 0, st,
                       mods_dev, args.partials, lengths, rows_or_offsets, N, S, p, args.tiles_per_seq, tile_tokens,
                       out, out_row_stride, out_dtype, lo, hi);
    BGX_HIP(hipGetLastError());
  }
  return 0;
}

// ---- the entry point that allocates nothing ------------------------------------------------------------
// Its workspace is this array: one copy per GPU, held from the moment the library is loaded on that GPU until
// the process ends.  `scratch` itself is a host-side stand-in, not a device address: host code only ever uses
// the address hipGetSymbolAddress returns for the device that is current, looked up once per device.
static __device__ __align__(256) unsigned char scratch[BGX_STATIC_SCRATCH_BYTES];
static std::mutex g_scratch_lock;
static void* g_scratch_ptr[MAX_DEVICES];  // per device, nullptr until the first call on it

static int static_scratch(void** out) {
  int dev = 0;
  BGX_HIP(hipGetDevice(&dev));
  BGX_REQUIRE(dev >= 0 && dev < MAX_DEVICES, BGX_E_ARG, "collect_seq_static: device %d outside 0..%d", dev,
              MAX_DEVICES - 1);
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    BGX_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    BGX_REQUIRE(ptr != nullptr && ((uintptr_t)ptr & 255) == 0, BGX_E_ALIGN,
                "collect_seq_static: the scratch array's device address %p is unusable", ptr);
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

int collect_seq_static_impl(const bgx_module_desc* mods_host, int n_modules, int N, int S, int p, int in_dtype,
                            const int32_t* lengths, const int64_t* out_rows, void* out, int64_t out_row_stride,
                            int out_dtype, float lo, float hi, void* stream) {
  BGX_REQUIRE(mods_host != nullptr && n_modules > 0 && N > 0 && S > 0 && p >= 1 && p <= 64, BGX_E_ARG,
              "collect_seq_static: n_modules=%d N=%d S=%d p=%d", n_modules, N, S, p);
  const size_t need = collect_workspace_bytes(n_modules, N, S, p);
  BGX_REQUIRE(need <= (size_t)BGX_STATIC_SCRATCH_BYTES, BGX_E_WORKSPACE,
              "collect_seq_static: %d modules x %d sequences x %d tokens at p=%d need %zu bytes of scratch, the "
              "static array holds %zu; use bgx_collect_seq with a workspace of the caller's",
              n_modules, N, S, p, need, (size_t)BGX_STATIC_SCRATCH_BYTES);
  void* ptr = nullptr;
  if (const int rc = static_scratch(&ptr)) return rc;
  // Every word of the workspace that a launch reads, the same launch has written before (descriptors and item
  // ranges by the table upload, partials by the collection kernel), so nothing needs clearing between calls.
  return collect_impl(false, mods_host, n_modules, N, S, p, in_dtype, lengths, out_rows, out, out_row_stride,
                      out_dtype, lo, hi, ptr, (size_t)BGX_STATIC_SCRATCH_BYTES, stream, /*tables_by_kernel=*/true);
}

int adafactor_scales_impl(const float* row, int O, const float* col, int I, int dtype, float* row_scale,
                          float* col_scale, void* stream) {
  BGX_REQUIRE(dtype >= BGX_F32 && dtype <= BGX_BF16, BGX_E_DTYPE, "adafactor_scales: dtype=%d", dtype);
  BGX_REQUIRE((row == nullptr) == (row_scale == nullptr), BGX_E_ARG, "adafactor_scales: row / row_scale mismatch");
  BGX_REQUIRE((col == nullptr) == (col_scale == nullptr), BGX_E_ARG, "adafactor_scales: col / col_scale mismatch");
  BGX_REQUIRE(row == nullptr || O > 0, BGX_E_ARG, "adafactor_scales: O=%d", O);
  BGX_REQUIRE(col == nullptr || I > 0, BGX_E_ARG, "adafactor_scales: I=%d", I);
  if (row == nullptr && col == nullptr) return 0;
  hipLaunchKernelGGL(adafactor_scales_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, row, O, col, I,
                     dtype, row_scale, col_scale);
  BGX_HIP(hipGetLastError());
  return 0;
}

int unit_normalize_impl(void* rows, int64_t n_rows, int64_t D, int64_t stride, int dtype, void* stream) {
  BGX_REQUIRE(rows != nullptr, BGX_E_ARG, "unit_normalize_rows: null rows");
  BGX_REQUIRE(n_rows >= 0 && D > 0 && stride >= D, BGX_E_ARG, "unit_normalize_rows: n_rows=%lld D=%lld stride=%lld",
              (long long)n_rows, (long long)D, (long long)stride);
  BGX_REQUIRE(n_rows <= 0x7fffffffLL, BGX_E_SHAPE, "unit_normalize_rows: too many rows");
  if (n_rows == 0) return 0;
  // eps of fp32, squared (bergson/builder.py:14)
  const float eps_sq = 1.1920928955078125e-07f * 1.1920928955078125e-07f;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)n_rows), block(256);
  if (dtype == BGX_F32)
    hipLaunchKernelGGL(unit_normalize_kernel<float>, grid, block, 0, st, (float*)rows, n_rows, D, stride, eps_sq);
  else if (dtype == BGX_F16)
    hipLaunchKernelGGL(unit_normalize_kernel<f16_t>, grid, block, 0, st, (f16_t*)rows, n_rows, D, stride, eps_sq);
  else if (dtype == BGX_BF16)
    hipLaunchKernelGGL(unit_normalize_kernel<bf16_t>, grid, block, 0, st, (bf16_t*)rows, n_rows, D, stride, eps_sq);
  else
    BGX_REQUIRE(false, BGX_E_DTYPE, "unit_normalize_rows: dtype=%d", dtype);
  BGX_HIP(hipGetLastError());
  return 0;
}

}  // namespace bgx
