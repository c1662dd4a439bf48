// Gradient-store scan for gfx950 (MI355X): scores every store row against Q
// queries, streaming the store once from HBM.
//
//   scan_gemm_kernel   LDS-tiled MFMA GEMM  scores[n, q] = <store[n], queries[q]>,
//                      with the row sum of squares accumulated from the same
//                      tiles, and a fused epilogue: unit-norm scaling, optional
//                      dense score write, per-row max over queries, and a
//                      per-query threshold filter that appends the few scores
//                      that can still enter the top-k to a candidate list.
//   scan_direct_kernel the same 256 x 256 (or 256 x 128) tile for aligned 16-bit
//                      operands: K tiles loaded straight into LDS, fragment
//                      pipeline across the barrier; the kernel of scans with more
//                      than 64 queries.
//   scan_stream_kernel at most 32 queries over a long store: no tiles, every wave
//                      streams its own rows through a register queue and takes the
//                      queries as MFMA fragments from a table in L2.
//   scan_select_kernel per query: exact top-k of (running top-k U candidates) by
//                      radix select on unique 64-bit keys, sorted; raises the
//                      query's threshold for the next pass.  Long candidate lists
//                      are first cut down by the k-th largest of a sample.
//   scan_finish_kernel decodes keys into (value, row) and the row maxima.
//
// The store is processed in passes of at most `chunk_rows` rows so that the
// candidate lists are bounded (a pass can never append more than chunk_rows
// entries per query) and the thresholds tighten quickly.
//
// Reference op sequence: bergson/score/scorer.py:89-115 (per-module GEMMs,
// sum of squares, division, max over queries) and
// bergson/query/attributor.py:137-167, :229-235 (row normalisation, GEMM,
// torch.topk).

#include <type_traits>
#include <utility>

#include "common.hpp"
#include "direct.hpp"
#include "mma32.hpp"
#include "stream.hpp"

namespace bgx {

// ---- order-preserving float <-> uint32 ------------------------------------------------
__host__ __device__ inline uint32_t f32_ordered(float f) {
  union {
    float f;
    uint32_t u;
  } c;
  c.f = f;
  return (c.u & 0x80000000u) ? ~c.u : (c.u | 0x80000000u);
}
__host__ __device__ inline float ordered_f32(uint32_t o) {
  union {
    float f;
    uint32_t u;
  } c;
  c.u = (o & 0x80000000u) ? (o & 0x7fffffffu) : ~o;
  return c.f;
}
// Unique key: larger score first, then lower row number.
__device__ inline uint64_t make_key(float score, uint32_t row) {
  return ((uint64_t)f32_ordered(score) << 32) | (uint64_t)(0xffffffffu - row);
}

// Entry of a by-row candidate list (a pass without thresholds writes row r's score to entry r): the key, or 0 --
// below every key of a real score, and dropped by the selection -- for a score no later pass would admit either
// (NaN and -inf fail every `score > threshold` test).  A row's fate then does not depend on the pass it falls in.
__device__ inline uint64_t make_key_or_empty(float score, uint32_t row) {
  return score > -INFINITY ? make_key(score, row) : 0ull;
}

constexpr int SCAN_KMAX = 2048;

struct ScanArgs {
  const void* store;
  const void* queries;
  int64_t row0;          // first store row of this pass
  int64_t rows;          // rows in this pass
  int64_t D;
  int64_t store_stride;  // elements
  int Q;
  int row_tiles;         // ceil(rows / BM)
  int q_tiles;           // ceil(Q / BN)
  float query_scale;
  int unit_norm;
  // outputs / state (may be null)
  float* scores;         // [n_rows, Q]
  float* sumsq;          // [n_rows]
  const float* sumsq_in; // [n_rows] row sums of squares from an earlier scan of the same store, or null
  uint32_t* row_max_enc; // [n_rows] ordered-uint encoding
  float* row_sum_part;   // [rows of this pass][n_parts] sum over each wave column's queries, or null
  int n_parts;           // q_tiles * (waves along the queries)
  const float* thr;      // [Q] current k-th best per query
  uint32_t* cand_count;  // [Q]
  uint64_t* cand;        // [Q][cand_cap]
  int64_t cand_cap;
  int first_pass;        // no thresholds yet: row r of the pass is entry r of every query's list (streaming kernel, scan_gemm_kernel)
  int units_per_wave;    // streaming kernel: 16-row units per wave of the grid, the first units_rem waves one more
  int units_rem;
};

// Reduction over the 32 lanes of a half wave with data-parallel-primitive moves (no LDS round trips): a running
// combination over shifts of 1, 2, 4 and 8 lanes inside each row of 16, then the first row's total handed to the
// second.  The total of lanes 0 .. 31 ends up in lane 31, that of lanes 32 .. 63 in lane 63; the other lanes hold
// partial results.  `identity` is what a lane without a source contributes.
template <bool IS_MAX>
__device__ __forceinline__ float reduce_half_wave(float v, float identity) {
  auto op = [](float x, float y) { return IS_MAX ? fmaxf(x, y) : x + y; };
  const int id = __float_as_int(identity);
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(id, __float_as_int(v), 0x111, 0xf, 0xf, false)));  // row_shr:1
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(id, __float_as_int(v), 0x112, 0xf, 0xf, false)));  // row_shr:2
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(id, __float_as_int(v), 0x114, 0xf, 0xf, false)));  // row_shr:4
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(id, __float_as_int(v), 0x118, 0xf, 0xf, false)));  // row_shr:8
  v = op(v, __int_as_float(__builtin_amdgcn_update_dpp(id, __float_as_int(v), 0x142, 0xa, 0xf, false)));  // row_bcast:15
  return v;
}

// Epilogue of a workgroup tile whose waves hold (TM x TN) blocks of 32 x 32 scores in MFMA layout: scale by the
// row multipliers s_inv, then dense scores, row maxima, row-sum partials and the threshold filter.
// One row block (acc_row = the wave's TN blocks of 32 rows x 32 queries; `blk` = which 32 rows of the wave's).
// A lane holds, for 16 rows (e), one score per query block: the products and their maximum / sum over the query
// blocks are a handful of instructions per row, the reductions over the 32 lanes use no LDS, only the lane that
// ends up with a row's result touches memory, all addresses are a per-lane base plus constants, and the
// candidate path (scores above a query's current k-th best: rare once the thresholds have settled) is entered
// only by rows that have one.  thr[j] is +inf for queries past Q.
template <int TN, int WTM, int WTN, int WN, bool FIRST_OK>
__device__ __forceinline__ void scan_block_epilogue(const ScanArgs& args, f32x16 (&acc_row)[TN], const float (&thr)[TN],
                                                    const float* s_inv, int blk, int wm, int wn, int fr, int fh,
                                                    int64_t g_row0, int64_t q_row0, int qt) {
  const int row_b = wm * WTM + blk * 32 + fh * 4;  // tile row of e = 0; e adds (e >> 2) * 8 + (e & 3)
  const int64_t prow_b = g_row0 + row_b;           // pass-local
  const int64_t grow_b = args.row0 + prow_b;
  const int64_t q_b = q_row0 + wn * WTN + fr;      // query of j = 0; j adds 32
  bool q_ok[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) q_ok[j] = q_b + j * 32 < args.Q;
  // how many of the 16 rows exist: rows_here <= 0 none, >= 28 all
  const int64_t rows_here = args.rows - prow_b;
  uint32_t* const rmax_p = args.row_max_enc != nullptr ? args.row_max_enc + grow_b : nullptr;
  float* const rsum_p =
      args.row_sum_part != nullptr ? args.row_sum_part + prow_b * args.n_parts + (qt * WN + wn) : nullptr;
  const bool writer = fr == 31;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 w4 = *reinterpret_cast<const f32x4*>(s_inv + row_b + g * 8);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e = g * 4 + c;
      const int dr = g * 8 + c;  // row offset of this e
      const bool row_ok = dr < rows_here;
      float v[TN];
      float rmax = -INFINITY, rsum = 0.f;
      bool any = false;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        v[j] = acc_row[j][e] * w4[c];
        if (q_ok[j]) {
          rmax = fmaxf(rmax, v[j]);
          rsum += v[j];
        }
        any |= v[j] > thr[j];
      }
      if (args.scores != nullptr && row_ok) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (q_ok[j]) args.scores[(grow_b + dr) * args.Q + q_b + j * 32] = v[j];
      }
      if (FIRST_OK && args.first_pass) {
        // no thresholds yet: every score is a candidate, and row r of the pass is entry r of each query's list
        // (one serialised atomic per score otherwise)
        if (row_ok) {
#pragma unroll
          for (int j = 0; j < TN; ++j)
            if (q_ok[j])
              args.cand[(q_b + j * 32) * args.cand_cap + prow_b + dr] = make_key_or_empty(v[j], (uint32_t)(grow_b + dr));
        }
      } else if (any && row_ok) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (v[j] > thr[j]) {
            const int64_t q = q_b + j * 32;
            const uint32_t pos = atomicAdd(&args.cand_count[q], 1u);
            if ((int64_t)pos < args.cand_cap) args.cand[q * args.cand_cap + pos] = make_key(v[j], (uint32_t)(grow_b + dr));
          }
      }
      if (rmax_p != nullptr) {
        rmax = reduce_half_wave<true>(rmax, -INFINITY);
        if (writer && row_ok) atomicMax(rmax_p + dr, f32_ordered(rmax));
      }
      if (rsum_p != nullptr) {
        rsum = reduce_half_wave<false>(rsum, 0.f);
        if (writer && row_ok) rsum_p[(int64_t)dr * args.n_parts] = rsum;
      }
    }
  }
}

// Sixteen values per lane reduced over the 32 lanes of a half wave at once: at each of four exchanges a lane
// keeps one half of its values and hands the other half to a partner that keeps the opposite half (partners: lane
// ^ 16 through a swizzle, then the mirror images within 16 and within 8 lanes, then lane ^ 2), so the values
// halve while the lanes combined double; a last exchange with lane ^ 1 completes it.  Lane fr ends up with the
// result for value (fr >> 1) & 15 (lanes fr and fr ^ 1 hold the same).  62 instructions for 16 reductions; the
// order of the additions is fixed by the lane numbers.
template <bool IS_MAX>
__device__ __forceinline__ float reduce16_half_wave(const float (&x)[16], int fr) {
  auto op = [](float p, float q) { return IS_MAX ? fmaxf(p, q) : p + q; };
  auto dpp = [](float v, auto ctrl_tag) {
    constexpr int CTRL = decltype(ctrl_tag)::value;
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
  };
  const bool b4 = (fr & 16) != 0, b3 = (fr & 8) != 0, b2 = (fr & 4) != 0, b1 = (fr & 2) != 0;
  float a8[8], a4[4], a2[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float keep = b4 ? x[8 + i] : x[i], send = b4 ? x[i] : x[8 + i];
    a8[i] = op(keep, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(send), 0x401F)));  // lane ^ 16
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float keep = b3 ? a8[4 + i] : a8[i], send = b3 ? a8[i] : a8[4 + i];
    a4[i] = op(keep, dpp(send, std::integral_constant<int, 0x140>{}));  // row_mirror: lane <-> 15 - lane
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float keep = b2 ? a4[2 + i] : a4[i], send = b2 ? a4[i] : a4[2 + i];
    a2[i] = op(keep, dpp(send, std::integral_constant<int, 0x141>{}));  // row_half_mirror: lane <-> 7 - lane
  }
  const float keep = b1 ? a2[1] : a2[0], send = b1 ? a2[0] : a2[1];
  float r = op(keep, dpp(send, std::integral_constant<int, 0x4E>{}));  // quad_perm [2, 3, 0, 1]: lane ^ 2
  r = op(r, dpp(r, std::integral_constant<int, 0xB1>{}));                // quad_perm [1, 0, 3, 2]: lane ^ 1
  return r;
}

// The same for a block whose 32 rows and TN * 32 queries all exist (every block of a scan whose row and query
// counts are multiples of the tile, and all but the edge blocks otherwise): straight-line code -- the products and
// each row's maximum / sum over the lane's query blocks, the sixteen rows reduced over the lanes together, one
// atomic / store instruction in which sixteen lanes write a row each.
// Candidates (scores above their query's current k-th best; a few per thousand scores once the thresholds have
// settled): a lane looks at the sixteen scores of a query block one by one only when the largest of them is above
// the query's threshold, and that code is marked unlikely so that it is laid out behind the function -- stepping
// over it, block after block, otherwise costs more in instruction fetch than the rest of the epilogue.
template <int TN, int WTM, int WTN, int WN>
__device__ __forceinline__ void scan_block_epilogue_full(const ScanArgs& args, f32x16 (&acc_row)[TN],
                                                         const float (&thr)[TN],
                                                         const float* s_inv, int blk, int wm, int wn, int fr, int fh,
                                                         int64_t g_row0, int64_t q_row0, int qt) {
  const int row_b = wm * WTM + blk * 32 + fh * 4;
  const int64_t prow_b = g_row0 + row_b;
  const int64_t grow_b = args.row0 + prow_b;
  const int64_t q_b = q_row0 + wn * WTN + fr;
  float rmax[16], rsum[16];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 w4 = *reinterpret_cast<const f32x4*>(s_inv + row_b + g * 8);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e = g * 4 + c;
      float m = -INFINITY, t = 0.f;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const float v = acc_row[j][e] * w4[c];
        acc_row[j][e] = v;  // kept for the dense scores and the candidate path
        m = fmaxf(m, v);
        t += v;
      }
      rmax[e] = m;
      rsum[e] = t;
    }
  }
  if (args.scores != nullptr) {
#pragma unroll
    for (int e = 0; e < 16; ++e)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        args.scores[(grow_b + (e >> 2) * 8 + (e & 3)) * args.Q + q_b + j * 32] = acc_row[j][e];
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    float cmax = acc_row[j][0];
#pragma unroll
    for (int e = 1; e < 16; ++e) cmax = fmaxf(cmax, acc_row[j][e]);
    if (__builtin_expect(cmax > thr[j], 0)) {
      // the lane's candidates of this block are counted and their places reserved with one atomic: one wait for the
      // wave per query block (an atomic per candidate is one wait per row in which any lane has one -- most of the
      // sixteen while the thresholds are still loose)
      const int64_t q = q_b + j * 32;
      uint64_t* const list = args.cand + q * args.cand_cap;
      uint32_t n = 0;
#pragma unroll
      for (int e = 0; e < 16; ++e) n += acc_row[j][e] > thr[j] ? 1u : 0u;
      uint32_t pos = atomicAdd(args.cand_count + q, n);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float v = acc_row[j][e];
        if (v > thr[j]) {
          if ((int64_t)pos < args.cand_cap) list[pos] = make_key(v, (uint32_t)(grow_b + (e >> 2) * 8 + (e & 3)));
          ++pos;
        }
      }
    }
  }
  // this lane's row after the reductions: value (fr >> 1) & 15
  const int e_mine = (fr >> 1) & 15;
  const int dr_mine = (e_mine >> 2) * 8 + (e_mine & 3);
  const bool writer = (fr & 1) == 0;
  if (args.row_max_enc != nullptr) {
    const float row_max = reduce16_half_wave<true>(rmax, fr);
    if (writer) atomicMax(args.row_max_enc + grow_b + dr_mine, f32_ordered(row_max));
  }
  if (args.row_sum_part != nullptr) {
    const float row_sum = reduce16_half_wave<false>(rsum, fr);
    if (writer) args.row_sum_part[(prow_b + dr_mine) * args.n_parts + (qt * WN + wn)] = row_sum;
  }
}

// The row blocks are taken by a pack expansion, not a loop: their indices are then constants whatever the
// unroller decides, and the accumulators never need an address.  acc[i] is the wave's 32-row block
// (i + block_rot) mod TM.
template <int TM, int TN, int WTM, int WTN, int WN, bool FIRST_OK, int... Is>
__device__ __forceinline__ void scan_tile_epilogue_blocks(const ScanArgs& args, f32x16 (&acc)[TM][TN],
                                                          const float (&thr)[TN], const float* s_inv, int wm, int wn,
                                                          int fr, int fh, int64_t g_row0, int64_t q_row0, int qt,
                                                          int block_rot, std::integer_sequence<int, Is...>) {
  // whether every row and query of this wave's sub-tile exists (the same for all lanes of the wave)
  // (a first pass that writes its candidates by row number takes the general path: it is a few thousand rows)
  const bool full = g_row0 + (wm + 1) * WTM <= args.rows && q_row0 + (wn + 1) * WTN <= args.Q &&
                    !(FIRST_OK && args.first_pass);
  if (full) {
    (scan_block_epilogue_full<TN, WTM, WTN, WN>(args, acc[Is], thr, s_inv, (Is + block_rot) % TM, wm, wn, fr, fh,
                                                g_row0, q_row0, qt),
     ...);
  } else {
    (scan_block_epilogue<TN, WTM, WTN, WN, FIRST_OK>(args, acc[Is], thr, s_inv, (Is + block_rot) % TM, wm, wn, fr, fh,
                                                     g_row0, q_row0, qt),
     ...);
  }
}

template <int TM, int TN, int WTM, int WTN, int WN, bool FIRST_OK = false>
__device__ __forceinline__ void scan_tile_epilogue(const ScanArgs& args, f32x16 (&acc)[TM][TN], const float* s_inv,
                                                   int wm, int wn, int fr, int fh, int64_t g_row0, int64_t q_row0,
                                                   int qt, int block_rot = 0) {
  float thr[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int64_t q = q_row0 + wn * WTN + j * 32 + fr;
    thr[j] = (args.thr != nullptr && q < args.Q) ? args.thr[q] : INFINITY;
  }
  scan_tile_epilogue_blocks<TM, TN, WTM, WTN, WN, FIRST_OK>(args, acc, thr, s_inv, wm, wn, fr, fh, g_row0, q_row0, qt,
                                                            block_rot, std::make_integer_sequence<int, TM>{});
}

// Workgroup tile BM x BN, WM x WN waves, each wave (BM/WM) x (BN/WN) as 32x32 MFMA blocks.
// PF = how many K tiles the global loads run ahead of the LDS stores (one register set per tile in flight);
// STREAM = non-temporal loads of the store rows, for launches with one query tile, where every store line
// is wanted exactly once.
template <typename T, int BM, int BN, int WM, int WN, bool ALIGNED, int PF = 1, bool STREAM = false>
__global__ __launch_bounds__(WM* WN * 64) void scan_gemm_kernel(ScanArgs args) {
  using M = Mma32<T>;
  constexpr int NT = WM * WN * 64;
  constexpr int EPL = M::EPL;
  constexpr int BK = TILE_CHUNKS * EPL;  // elements of K per tile
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int GCH = BM * TILE_CHUNKS / NT;  // store chunks per thread
  constexpr int QCH = BN * TILE_CHUNKS / NT;  // query chunks per thread
  static_assert(BM * TILE_CHUNKS % NT == 0 && BN * TILE_CHUNKS % NT == 0, "loader mapping");
  static_assert(NT % TILE_CHUNKS == 0, "loader mapping");
  constexpr int ROWS_PER_PASS = NT / TILE_CHUNKS;

  extern __shared__ __align__(16) unsigned char smem[];
  // [buf][BM + BN rows][LDS_ROW_BYTES]
  constexpr int BUF_BYTES = (BM + BN) * LDS_ROW_BYTES;
  __shared__ __align__(16) float s_inv[BM];

  // XCD-aware tile order: workgroup b runs on XCD b % 8; the q_tiles
  // workgroups of one row tile share that XCD's L2.
  const int b = blockIdx.x;
  const int xcd = b & 7;
  const int slot = b >> 3;
  const int rt_local = slot / args.q_tiles;
  const int qt = slot - rt_local * args.q_tiles;
  const int rt = rt_local * 8 + xcd;
  if (rt >= args.row_tiles) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  const T* store = (const T*)args.store + args.row0 * args.store_stride;
  const T* queries = (const T*)args.queries;
  const int64_t g_row0 = (int64_t)rt * BM;  // pass-local first row
  const int64_t q_row0 = (int64_t)qt * BN;
  const int64_t D = args.D;

  const int lrow = tid / TILE_CHUNKS;
  const int lcol = tid % TILE_CHUNKS;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  float ss[GCH];
#pragma unroll
  for (int i = 0; i < GCH; ++i) ss[i] = 0.f;

  const int KT = (int)((D + BK - 1) / BK);
  // Streaming variant (one query tile): row tiles start at different K tiles.  All rows of the store are the same number of
  // bytes apart, so workgroups that walk K in step would ask the same few memory channels for every row at
  // once.  The starting tile depends only on the row's position in the store, never on the pass.
  const int k_rot = STREAM ? (int)((((args.row0 + g_row0) / BM) * 5) % KT) : 0;
  uint4 gr[PF][GCH], qr[PF][QCH];  // K tile t travels in register set t % PF
  auto gload = [&](int kt, auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
    int kte = kt + k_rot;
    if (kte >= KT) kte -= KT;
    const int64_t k = (int64_t)kte * BK + lcol * EPL;
#pragma unroll
    for (int i = 0; i < GCH; ++i)
      gr[SET][i] = load_chunk<T, ALIGNED, STREAM>(store, g_row0 + lrow + i * ROWS_PER_PASS, args.rows,
                                                  args.store_stride, k, D);
#pragma unroll
    for (int i = 0; i < QCH; ++i)
      qr[SET][i] = load_chunk<T, ALIGNED>(queries, q_row0 + lrow + i * ROWS_PER_PASS, args.Q, D, k, D);
  };
  auto lstore = [&](int buf, auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
    unsigned char* base = smem + buf * BUF_BYTES;
#pragma unroll
    for (int i = 0; i < GCH; ++i) {
      *reinterpret_cast<uint4*>(base + (lrow + i * ROWS_PER_PASS) * LDS_ROW_BYTES + lcol * 16) = gr[SET][i];
      ss[i] = M::sumsq(gr[SET][i], ss[i]);
    }
#pragma unroll
    for (int i = 0; i < QCH; ++i)
      *reinterpret_cast<uint4*>(base + (BM + lrow + i * ROWS_PER_PASS) * LDS_ROW_BYTES + lcol * 16) = qr[SET][i];
  };

  // Pipeline: while the MFMAs of K tile kt run from LDS buffer kt&1, the registers that hold tile kt+1
  // are written to the other buffer and the global loads of tile kt+1+PF are issued into the register set
  // that has just been emptied; one barrier per tile.
  gload(0, std::integral_constant<int, 0>{});
  lstore(0, std::integral_constant<int, 0>{});
  if (KT > 1) gload(1, std::integral_constant<int, 1 % PF>{});
  if constexpr (PF > 1)
    if (KT > 2) gload(2, std::integral_constant<int, 2 % PF>{});
  static_assert(PF == 1 || PF == 2, "prologue spells out its loads");
  __syncthreads();

  const int fr = lane & 31;
  const int fh = lane >> 5;
  auto mma_step = [&](const unsigned char* gb, const unsigned char* qb, int kk) {
    uint4 af[TM], bf[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const uint4*>(gb + i * 32 * LDS_ROW_BYTES + kk * 32);
#pragma unroll
    for (int j = 0; j < TN; ++j) bf[j] = *reinterpret_cast<const uint4*>(qb + j * 32 * LDS_ROW_BYTES + kk * 32);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) M::mma(af[i], bf[j], acc[i][j]);
  };
  auto k_tile = [&](int kt, auto set_tag) {  // set_tag: the register set of tile kt + 1
    const int buf = kt & 1;
    const unsigned char* gb = smem + buf * BUF_BYTES + (wm * WTM + fr) * LDS_ROW_BYTES + fh * 16;
    const unsigned char* qb = smem + buf * BUF_BYTES + (BM + wn * WTN + fr) * LDS_ROW_BYTES + fh * 16;
    mma_step(gb, qb, 0);
    if (kt + 1 < KT) lstore(buf ^ 1, set_tag);
    if (kt + 1 + PF < KT) gload(kt + 1 + PF, set_tag);
#pragma unroll
    for (int kk = 1; kk < TILE_CHUNKS / 2; ++kk) mma_step(gb, qb, kk);
    __syncthreads();
  };
  if constexpr (PF == 1) {
    for (int kt = 0; kt < KT; ++kt) k_tile(kt, std::integral_constant<int, 0>{});
  } else {
    for (int kt = 0; kt < KT; kt += 2) {
      k_tile(kt, std::integral_constant<int, 1>{});
      if (kt + 1 < KT) k_tile(kt + 1, std::integral_constant<int, 0>{});
    }
  }

  // ---- row sum of squares -> per-row multiplier ------------------------------------
#pragma unroll
  for (int i = 0; i < GCH; ++i) {
    float s = ss[i];
    s += __shfl_xor(s, 1);
    s += __shfl_xor(s, 2);
    s += __shfl_xor(s, 4);
    if (lcol == 0) {
      const int row = lrow + i * ROWS_PER_PASS;
      float w = args.query_scale;
      if (args.unit_norm) w = s > 0.f ? args.query_scale / sqrtf(s) : 0.f;
      s_inv[row] = w;
      const int64_t grow = g_row0 + row;
      if (qt == 0 && args.sumsq != nullptr && grow < args.rows) args.sumsq[args.row0 + grow] = s;
    }
  }
  __syncthreads();

  if (args.first_pass && blockIdx.x == 0)
    for (int q = tid; q < args.Q; q += NT) args.cand_count[q] = (uint32_t)args.rows;
  scan_tile_epilogue<TM, TN, WTM, WTN, WN, true>(args, acc, s_inv, wm, wn, fr, fh, g_row0, q_row0, qt);
}

// ---- many queries, 16-bit stores: tiles loaded straight into LDS ---------------------------------------
// The 256 x 256 tile of the kernel above with 8 waves as 2 x 4, for aligned fp16 / bf16 operands whose D is a
// multiple of 64.  What differs is how the tiles reach LDS and how the fragments leave it:
//  * global_load_lds (16 bytes per lane, 1 KB per wave instruction) writes the K tiles into LDS without passing
//    through registers: no staging registers, no ds_write, and the row sums of squares come from the A fragments
//    each wave reads anyway (the four waves that share 128 rows take a 32-row block each);
//  * rows are 128 bytes, unpadded; chunk c of row r sits at position c ^ (r & 7) ^ ((r >> 3) & 1), which the
//    loader produces by permuting which global chunk each lane fetches: fragment reads are conflict-free;
//  * three A buffers and two B buffers (160 KB): the store rows are fetched two K tiles ahead, the queries
//    (L2-resident) one ahead; the per-tile wait is a vmcnt that leaves the youngest A tile in flight, and the
//    barrier is the bare s_barrier (wg_barrier_lds) -- __syncthreads would wait for every outstanding load;
//  * the fragments are double-buffered in registers and the pipeline runs across the barrier: the reads of
//    step 0 of the next tile are issued right after it, before the MFMAs of the last step of this tile.
constexpr int SD_BM = 256;
constexpr int SD_A_BYTES = SD_BM * SD_ROW;
constexpr int SD_THREADS = 512;
// BN = 256, or 128 for at most 128 queries (one query tile: half the MFMA work of a 256-wide tile that would be
// half empty)
constexpr int sd_lds_bytes(int bn) { return 3 * SD_A_BYTES + 2 * bn * SD_ROW; }

template <typename T, int BN, bool ONE_QT>
__global__ __launch_bounds__(SD_THREADS) void scan_direct_kernel(ScanArgs args) {
  using M = Mma32<T>;
  typedef __attribute__((address_space(1))) const void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
  constexpr int BK = 64;  // elements of K per tile
  constexpr int WN = 4, WTM = 128, WTN = BN / WN, TM = 4, TN = WTN / 32;
  constexpr int NB = BN / 64;  // query-tile load instructions per wave
  constexpr int SD_B_BYTES = BN * SD_ROW;
  static_assert(BN == 256 || BN == 128, "query tile");
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_inv = reinterpret_cast<float*>(smem);  // after the main loop: [SD_BM] row multipliers

  const int b = blockIdx.x;
  const int xcd = b & 7;
  const int slot = b >> 3;
  const int rt_local = slot / args.q_tiles;
  const int qt = slot - rt_local * args.q_tiles;
  const int rt = rt_local * 8 + xcd;
  if (rt >= args.row_tiles) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int64_t g_row0 = (int64_t)rt * SD_BM;  // pass-local first row
  const int64_t q_row0 = (int64_t)qt * BN;
  const int KT = (int)(args.D / BK);

  // loader: instruction i of a wave fills rows i * 64 + wave * 8 .. + 7 of a tile; lane l is position l & 7 of
  // row l >> 3 and fetches the chunk that belongs there.  Rows past the end repeat the last one (their scores
  // are never written).
  const T* aptr[4];
  const T* bptr[NB];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = i * 64 + wave * 8 + (lane >> 3);
    const int ch = (lane & 7) ^ sd_key(r);
    const int64_t grow = min(g_row0 + r, args.rows - 1);
    aptr[i] = (const T*)args.store + (args.row0 + grow) * args.store_stride + ch * 8;
    if (i < NB) {
      const int64_t qrow = min(q_row0 + r, (int64_t)args.Q - 1);
      bptr[i] = (const T*)args.queries + qrow * args.D + ch * 8;
    }
  }
  auto load_a = [&](int kt) {
    unsigned char* dst = smem + (kt % 3) * SD_A_BYTES + wave * 1024;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t)(aptr[i] + (int64_t)kt * BK), (lptr_t)(dst + i * 8192), 16, 0,
                                       ONE_QT ? 2 : 0);  // one query tile: every store line is wanted once (nt)
  };
  auto load_b = [&](int kt) {
    unsigned char* dst = smem + 3 * SD_A_BYTES + (kt & 1) * SD_B_BYTES + wave * 1024;
#pragma unroll
    for (int i = 0; i < NB; ++i)
      __builtin_amdgcn_global_load_lds((gptr_t)(bptr[i] + (int64_t)kt * BK), (lptr_t)(dst + i * 8192), 16, 0, 0);
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  // one partial per 16-byte chunk position of the K tile, as the tile kernel's loader threads keep them: the
  // row norms then come out bit-identical, whichever of the two kernels scores a row
  float ss[4] = {0.f, 0.f, 0.f, 0.f};

  const int fr = lane & 31;
  const int fh = lane >> 5;
  int aoff[TM], boff[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) aoff[i] = (wm * WTM + ((i + wn) & 3) * 32 + fr) * SD_ROW;
#pragma unroll
  for (int j = 0; j < TN; ++j) boff[j] = 3 * SD_A_BYTES + (wn * WTN + j * 32 + fr) * SD_ROW;
  const int key = sd_key(fr);  // rows advance in steps of 32: the key depends on fr alone
  // The four waves that share 128 rows number their 32-row blocks from different starts (block (i + wn) & 3 is
  // wave wn's i-th): each wave's first block is then a different one, and summing its squares is that wave's
  // share of the row norms -- no choice of fragment at run time.

  // The fragment reads are spelled as instructions: the compiler makes an LDS read it can see wait for every
  // outstanding direct-to-LDS load (it cannot tell the buffers apart), which would undo the prefetch.  The
  // waits are explicit too: LDS reads return in order, so "at most TM + TN outstanding" means that the step
  // issued before the latest TM + TN reads has arrived.  (No other LDS or scalar-memory traffic inside the loop.)
  uint4 af[2][TM], bf[2][TN];
  uint32_t chk[4];  // byte offset of this lane's chunk in its row, per k-step of the tile
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) chk[kk] = (uint32_t)(((kk * 2 + fh) ^ key) * 16);
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  auto rd = [&](int kt, auto kk_tag, auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr int KK = decltype(kk_tag)::value;
    const uint32_t ab = lds0 + (uint32_t)(kt % 3) * SD_A_BYTES + chk[KK];
    const uint32_t bb = lds0 + (uint32_t)(kt & 1) * SD_B_BYTES + chk[KK];
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[SET][i] = sd_lds_read16(ab + (uint32_t)aoff[i]);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      bf[SET][j] = sd_lds_read16(bb + (uint32_t)boff[j]);
  };
  auto mm = [&](auto set_tag, auto kk_tag) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr int KK = decltype(kk_tag)::value;
    ss[KK] = M::sumsq(af[SET][0], ss[KK]);  // this wave's share of the row norms: its first 32-row block
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) M::mma(af[SET][i], bf[SET][j], acc[i][j]);
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;

  // prologue: A(0), B(0), then A(1) stays in flight over the first barrier
  load_a(0);
  load_b(0);
  if (KT > 1) {
    load_a(1);
    wg_barrier_lds<4>();
  } else {
    wg_barrier_lds<0>();
  }
  __builtin_amdgcn_sched_barrier(0);
  using K0 = std::integral_constant<int, 0>;
  using K1 = std::integral_constant<int, 1>;
  using K2 = std::integral_constant<int, 2>;
  using K3 = std::integral_constant<int, 3>;
  constexpr int WAIT_LDS_STEP = 0xC07F | ((TM + TN) << 8);  // lgkmcnt(TM + TN), nothing else
  constexpr int WAIT_LDS_0 = 0xC07F;  // lgkmcnt(0), nothing else
  __builtin_amdgcn_sched_barrier(0);
  rd(0, K0{}, S0{});
  __builtin_amdgcn_sched_barrier(0);
  if (1 < KT) load_b(1);
  if (2 < KT) load_a(2);
  for (int kt = 0; kt < KT; ++kt) {
    __builtin_amdgcn_sched_barrier(0);
    rd(kt, K1{}, S1{});
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_STEP);
    __builtin_amdgcn_sched_barrier(0);
    mm(S0{}, K0{});
    __builtin_amdgcn_sched_barrier(0);
    rd(kt, K2{}, S0{});
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_STEP);
    __builtin_amdgcn_sched_barrier(0);
    mm(S1{}, K1{});
    __builtin_amdgcn_sched_barrier(0);
    rd(kt, K3{}, S1{});
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_STEP);
    __builtin_amdgcn_sched_barrier(0);
    mm(S0{}, K2{});
    __builtin_amdgcn_sched_barrier(0);
    // In flight, oldest first: A(kt + 1), then B(kt + 1) and A(kt + 2).  Tile kt + 1 must have landed (this
    // wave's part; the barrier makes that all of it), A(kt + 2) may still fly; the fragment reads above have
    // completed, so after the barrier tile kt's buffers take B(kt + 2) and A(kt + 3).
    if (kt + 2 < KT)
      wg_barrier_lds<4>();
    else
      wg_barrier_lds<0>();
    __builtin_amdgcn_sched_barrier(0);
    if (kt + 1 < KT) rd(kt + 1, K0{}, S0{});
    __builtin_amdgcn_sched_barrier(0);
    mm(S1{}, K3{});  // its fragments arrived before the barrier
    __builtin_amdgcn_sched_barrier(0);
    // the loads go out behind the first MFMAs after the barrier, so that those are not held up by their issue
    if (kt + 2 < KT) load_b(kt + 2);
    if (kt + 3 < KT) load_a(kt + 3);
  }
  __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);

  // ---- row sum of squares -> per-row multiplier (the tile buffers are free now) ----------------------------
  // chunk positions 2 kk (lanes fh = 0) and 2 kk + 1 (fh = 1), added up in the order of the tile kernel's butterfly
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) ss[kk] += __shfl_xor(ss[kk], 32);
  const float ssq = (ss[0] + ss[1]) + (ss[2] + ss[3]);
  wg_barrier_lds<0>();  // every wave is past its last fragment read
  __builtin_amdgcn_sched_barrier(0);
  if (fh == 0) {
    const int row = wm * WTM + wn * 32 + fr;
    float w = args.query_scale;
    if (args.unit_norm) w = ssq > 0.f ? args.query_scale / sqrtf(ssq) : 0.f;
    s_inv[row] = w;
    const int64_t grow = g_row0 + row;
    if (qt == 0 && args.sumsq != nullptr && grow < args.rows) args.sumsq[args.row0 + grow] = ssq;
  }
  __syncthreads();

  scan_tile_epilogue<TM, TN, WTM, WTN, WN>(args, acc, s_inv, wm, wn, fr, fh, g_row0, q_row0, qt, wn);
}

// ---- many queries, many rows: 384 x 256 tiles on four waves ---------------------------------------------------
// With eight waves on a 256 x 256 tile a wave issues 32 MFMAs per K tile, and what it pays per tile beside them --
// 24 fragment reads, the barrier, its share of the loads, the loop -- leaves the matrix pipes half idle.  This
// kernel gives one wave per SIMD all 512 registers (the accumulators overflow into the AccVGPRs) -- four waves as
// 2 x 2, each 192 rows x 128 queries = 6 x 4 blocks of 32 x 32 = 384 accumulator registers -- for a 384 x 256
// tile: 96 MFMAs per wave and K tile against 40 fragment reads, and 1/153.6 byte per flop from L2 instead of
// 1/128.  The tile's two K tiles (2 x 80 KB) fill the LDS; with one wave per SIMD nothing else hides a stall (a
// vector-ALU instruction between two MFMAs costs its whole latency), so every global load and every fragment read
// is placed by hand between two MFMAs of the step before the one that needs it (sched_barrier after each: the
// order below is the order that is executed), and the loads of a tile go out right behind the barrier that
// frees their stage, so that the youngest has most of a tile's time before the wait at the next barrier.
//   LDS layout, swizzle, direct-to-LDS loads, explicit waits, row norms from the fragments: as in
//   scan_direct_kernel, and the scores are the same bits (each is the same sequence of MFMAs over K).
//   The launch covers whole tiles only: rows a multiple of 384 (the host cuts its passes accordingly; what is left
//   goes to the kernel above).
constexpr int SW_BM = 384, SW_BN = 256, SW_THREADS = 256;
constexpr int SW_A_BYTES = SW_BM * SD_ROW, SW_B_BYTES = SW_BN * SD_ROW, SW_STAGE = SW_A_BYTES + SW_B_BYTES;
constexpr int SW_LDS_BYTES = 2 * SW_STAGE;
// Rows of one round of the chip -- 256 workgroups, one per compute unit: 256 / (query tiles) row tiles.  24 576 rows
// at 1024 queries (64 row tiles x 4 query tiles), 98 304 with one query tile.
static int64_t sw_round_rows(int Q) {
  const int q_tiles = (Q + SW_BN - 1) / SW_BN;
  const int row_tiles = 256 / q_tiles;
  return (int64_t)(row_tiles > 0 ? row_tiles : 1) * SW_BM;
}
constexpr int64_t SW_MIN_ROWS = 10240;         // shorter passes leave most of the chip idle whatever the tile

template <int N>
__device__ inline void sw_wait_lds() {  // s_waitcnt lgkmcnt(N), nothing else
  __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));
}

template <typename T, bool NORMS_GIVEN>
__global__ __launch_bounds__(SW_THREADS) void scan_wide_kernel(ScanArgs args) {
  using M = Mma32<T>;
  constexpr int BK = 64;
  constexpr int TM = 6, TN = 4, WTM = 192, WTN = 128, WN = 2;
  constexpr int NA = SW_BM / 32, NB = SW_BN / 32;  // load instructions per wave and K tile: 12 + 8
  constexpr int ACC_TM = 4;                        // row blocks 0 .. 3 accumulate in AccVGPRs (256), 4 and 5 in VGPRs
  extern __shared__ __align__(128) unsigned char smem[];
  float* s_inv = reinterpret_cast<float*>(smem);  // after the main loop: [SW_BM] row multipliers

  const int b = blockIdx.x;
  const int xcd = b & 7;
  const int slot = b >> 3;
  const int rt_local = slot / args.q_tiles;
  const int qt = slot - rt_local * args.q_tiles;
  const int rt = rt_local * 8 + xcd;
  if (rt >= args.row_tiles) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t g_row0 = (int64_t)rt * SW_BM;  // pass-local first row
  const int64_t q_row0 = (int64_t)qt * SW_BN;
  const int KT = (int)(args.D / BK);
  const int fr = lane & 31;
  const int fh = lane >> 5;

  // ---- loader: instruction i of wave w fills rows i * 32 + w * 8 .. + 7 of a tile (1 KB of LDS); lane l is
  // position l & 7 of row l >> 3 and fetches the chunk that belongs there: chunk c of row r sits at position
  // c ^ (r & 7) ^ ((r >> 3) & 1), and (r >> 3) & 1 = w & 1 for every i.  Addresses are a uniform base (the tile,
  // advanced by one K tile per iteration) plus one 32-bit offset per lane and instruction.
  const int lrow = wave * 8 + (lane >> 3);
  const int lch = (lane & 7) ^ (lane >> 3) ^ (wave & 1);
  const uint32_t row_bytes = (uint32_t)(args.store_stride * sizeof(T));
  const uint32_t q_bytes = (uint32_t)(args.D * sizeof(T));
  const uint64_t a_base = (uint64_t)(uintptr_t)args.store + (uint64_t)((args.row0 + g_row0) * args.store_stride) * sizeof(T);
  const uint64_t b_base = (uint64_t)(uintptr_t)args.queries + (uint64_t)(q_row0 * args.D) * sizeof(T);
  const int r_last = (int)min((int64_t)SW_BM, args.rows - g_row0) - 1;  // last valid row of this tile, likewise
  const int q_last = args.Q - 1 - (int)q_row0;  // last valid query row of this tile (rows past it repeat it)
  uint32_t a_voff[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) a_voff[i] = (uint32_t)min(i * 32 + lrow, r_last) * row_bytes + (uint32_t)lch * 16u;
  uint32_t b_voff[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) b_voff[i] = (uint32_t)min(i * 32 + lrow, q_last) * q_bytes + (uint32_t)lch * 16u;
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const uint32_t lds_wave = lds0 + (uint32_t)wave * 1024u;
  // instruction idx (0 .. NA-1: rows of the store; NA .. NA+NB-1: queries) of K tile kt, into stage `stg`
  auto load_one_to = [&](int kt, int stg, int idx) {
    const uint32_t stage = lds_wave + (uint32_t)stg * SW_STAGE;
    const uint64_t koff = (uint64_t)kt * (BK * sizeof(T));
    if (idx < NA)
      sw_load_lds16(a_base + koff, a_voff[idx], stage + (uint32_t)idx * 4096u);
    else
      sw_load_lds16(b_base + koff, b_voff[idx - NA], stage + (uint32_t)(SW_A_BYTES + (idx - NA) * 4096));
  };
  auto load_one = [&](int kt, int idx) { load_one_to(kt, kt & 1, idx); };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  // Row norms: the two waves that share 192 rows take three 32-row blocks each.  Wave wn numbers its blocks from
  // 3 wn (its block i is rows (i + 3 wn) mod 6), so that "the first three" is the same code in both; one partial
  // per 16-byte chunk position of the K tile, as in the other tile kernels: identical bits.
  float ss[3][4];
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) ss[i][kk] = 0.f;

  // fragment addresses: row (wm * 192 + blk * 32 + fr), position ((2 kk + fh) ^ key) with key = sd_key(fr) for
  // every block; (2 kk + fh) ^ key = (2 kk) ^ (fh ^ key), so a k-step is an XOR on the (128-byte aligned) address.
  // The wave's blocks 0 .. 2 start at row block 3 wn, its blocks 3 .. 5 at row block 3 (1 - wn).
  const uint32_t c0 = (uint32_t)((fh ^ sd_key(fr)) * 16);
  const uint32_t a_frag_lo = lds0 + (uint32_t)((wm * WTM + 96 * wn + fr) * SD_ROW) + c0;
  const uint32_t a_frag_hi = lds0 + (uint32_t)((wm * WTM + 96 * (1 - wn) + fr) * SD_ROW) + c0;
  const uint32_t b_frag = lds0 + (uint32_t)(SW_A_BYTES + (wn * WTN + fr) * SD_ROW) + c0;
  // Row fragments have one register set: block i's four MFMAs come one after the other, and the read of the next
  // step's block i goes out right behind them.  Query fragments are used by all six blocks and have two sets.
  uint4 af[TM], bf[2][TN];
  uint32_t ra_lo, ra_hi, rb;  // read addresses of the step that is being read
  auto rd_base = [&](int stage, auto kk_tag) {
    constexpr int KK = decltype(kk_tag)::value;
    const uint32_t st = (uint32_t)stage * SW_STAGE;
    ra_lo = (a_frag_lo + st) ^ (uint32_t)(KK * 32);
    ra_hi = (a_frag_hi + st) ^ (uint32_t)(KK * 32);
    rb = (b_frag + st) ^ (uint32_t)(KK * 32);
  };
  auto rd_a = [&](auto i_tag) {
    constexpr int I = decltype(i_tag)::value;
    af[I] = sw_lds_read16<(I % 3) * 32 * SD_ROW>(I < 3 ? ra_lo : ra_hi);
  };
  auto rd_b = [&](auto set_tag, auto j_tag) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr int J = decltype(j_tag)::value;
    bf[SET][J] = sw_lds_read16<J * 32 * SD_ROW>(rb);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  using I4 = std::integral_constant<int, 4>;
  using I5 = std::integral_constant<int, 5>;

  // One k-step: the 24 MFMAs of step KK from query set SET; behind them, one at a time, the reads of the step
  // that follows (k-step NKK of stage `nstage`, query set 1 - SET) and whatever `side(n)` adds behind MFMA n.
  // LDS reads return in order, so "at most N outstanding" names the read that has arrived.  Issue order within a
  // step: B0 B1 B2 B3 A0 A1 A2 A3 A4 A5 (behind MFMAs 3 4 5 6 8 9 11 15 19 23).
  //   before MFMA 0:  B0..B3, A0 of this step, i.e. all but the last five reads of the step before            -> 5
  //   before MFMA 4:  A1; younger: A2 A3 A4 A5 and this step's B0                                            -> 5
  //   before MFMA 8:  A2; younger: A3 A4 A5 and this step's B0 B1 B2 B3                                      -> 7
  //   before MFMA 12: A3; younger: A4 A5, B0 B1 B2 B3 A0 A1 A2                                              -> 9
  //   before MFMA 16: A4; younger: A5, B0 B1 B2 B3 A0 A1 A2 A3                                              -> 9
  //   before MFMA 20: A5; younger: B0 B1 B2 B3 A0 A1 A2 A3 A4                                               -> 9
  // Row blocks 0 and 1 are refilled only behind MFMAs 8 and 9 so that, just before MFMA 8, the fragments of the
  // three blocks whose norms this wave sums are all in their registers: the twelve steps of the three sums of
  // squares then run as four rounds of three independent instructions.  (Four dependent ones in front of each
  // block's MFMAs wait for one another, and one behind each MFMA costs more still: with one wave per SIMD every
  // switch from the matrix pipe to the vector pipe and back is paid for.)
  // `mid()` runs before the read behind MFMA 3 (the tile change puts its barrier there).  Every step is the same
  // code: the very last one reads a step that does not exist (whatever the other stage holds; never used).
  auto step = [&](auto set_tag, auto kk_tag, auto nkk_tag, int nstage, auto&& mid, auto&& side) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr int KK = decltype(kk_tag)::value;
    using NK = decltype(nkk_tag);
    using NS = std::integral_constant<int, 1 - SET>;
    sw_wait_lds<5>();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (i == 1) { sw_wait_lds<5>(); __builtin_amdgcn_sched_barrier(0); }
      if (i == 2) { sw_wait_lds<7>(); __builtin_amdgcn_sched_barrier(0); }
      if (i >= 3) { sw_wait_lds<9>(); __builtin_amdgcn_sched_barrier(0); }
      if (!NORMS_GIVEN && i == 2) {
        ss[0][KK] = M::template sumsq_part<0>(af[0], ss[0][KK]);
        ss[1][KK] = M::template sumsq_part<0>(af[1], ss[1][KK]);
        ss[2][KK] = M::template sumsq_part<0>(af[2], ss[2][KK]);
        ss[0][KK] = M::template sumsq_part<1>(af[0], ss[0][KK]);
        ss[1][KK] = M::template sumsq_part<1>(af[1], ss[1][KK]);
        ss[2][KK] = M::template sumsq_part<1>(af[2], ss[2][KK]);
        ss[0][KK] = M::template sumsq_part<2>(af[0], ss[0][KK]);
        ss[1][KK] = M::template sumsq_part<2>(af[1], ss[1][KK]);
        ss[2][KK] = M::template sumsq_part<2>(af[2], ss[2][KK]);
        ss[0][KK] = M::template sumsq_part<3>(af[0], ss[0][KK]);
        ss[1][KK] = M::template sumsq_part<3>(af[1], ss[1][KK]);
        ss[2][KK] = M::template sumsq_part<3>(af[2], ss[2][KK]);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = i * TN + j;
        if (i < ACC_TM)
          sw_mfma<T, true>(af[i], bf[SET][j], acc[i][j]);
        else
          sw_mfma<T, false>(af[i], bf[SET][j], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        if (n == 3) mid();
        if (n == 3) { rd_base(nstage, NK{}); rd_b(NS{}, I0{}); }
        if (n == 4) rd_b(NS{}, I1{});
        if (n == 5) rd_b(NS{}, I2{});
        if (n == 6) rd_b(NS{}, I3{});
        if (n == 8) rd_a(I0{});
        if (n == 9) rd_a(I1{});
        if (n == 11) rd_a(I2{});
        if (n == 15) rd_a(I3{});
        if (n == 19) rd_a(I4{});
        if (n == 23) rd_a(I5{});
        side(n);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  using K0 = std::integral_constant<int, 0>;
  using K1 = std::integral_constant<int, 1>;
  using K2 = std::integral_constant<int, 2>;
  using K3 = std::integral_constant<int, 3>;
  auto nothing = [] {};
  auto tile_change = [] {
    wg_barrier_lds<0>();
    __builtin_amdgcn_sched_barrier(0);
  };

  // The 20 loads of a tile go out one behind every third MFMA, starting right behind the barrier that gives up the
  // stage they fill: seven in what is left of the last step of tile t, eight and five in the first two steps of tile
  // t + 1, for tile t + 2.  The barrier that needs them waits for all of this wave's loads, the youngest included, so
  // what counts is how long before it the last one is issued: 58 MFMAs here (it was 14 with one load per four
  // MFMAs spread over the whole period, and the wait for that load showed in every tile).  Issued faster than
  // one per two or three MFMAs the loads hold up the wave at the load instruction -- with one wave per SIMD the
  // MFMAs behind it wait too.
  // There is ONE copy of the tile code and no branch in it: past the end of the row the loads fetch the last K
  // tile again (into a stage nobody reads any more; a few loads per 192 tiles) and the reads take whatever the
  // other stage holds.  One copy on purpose: in every copy the compiler has to find registers for the whole tile
  // without spilling, and a spilled fragment would be stored before its read has arrived -- the first version,
  // with the first and last tiles peeled off, failed exactly so.

  // prologue: tile 0 lands, its step 0 is read, tile 1 begins
#pragma unroll
  for (int idx = 0; idx < NA + NB; ++idx) load_one(0, idx);
  wg_barrier_lds<0>();
  __builtin_amdgcn_sched_barrier(0);
  rd_base(0, K0{});
  rd_b(S0{}, I0{});
  rd_b(S0{}, I1{});
  rd_b(S0{}, I2{});
  rd_b(S0{}, I3{});
  rd_a(I0{});
  rd_a(I1{});
  rd_a(I2{});
  rd_a(I3{});
  rd_a(I4{});
  rd_a(I5{});
  {
    const int k1 = min(1, KT - 1);
#pragma unroll
    for (int idx = 0; idx < 7; ++idx) load_one_to(k1, 1, idx);  // what the last step of a tile issues for the next but one
  }
  __builtin_amdgcn_sched_barrier(0);

  for (int kt = 0; kt < KT; ++kt) {
    const int st = kt & 1;
    const int k1 = min(kt + 1, KT - 1);  // the tile whose loads are finished during this one ...
    const int k2 = min(kt + 2, KT - 1);  // ... and the one whose loads begin behind this tile's barrier
    // (a clamped tile number only changes where the data comes from: the stage is the one tile kt + 1 / kt + 2 would use)
    step(S0{}, K0{}, K1{}, st, nothing, [&](int n) {
      if (n % 3 == 1 && n <= 22) load_one_to(k1, st ^ 1, 7 + n / 3);
    });
    step(S1{}, K1{}, K2{}, st, nothing, [&](int n) {
      if (n % 3 == 1 && n <= 13) load_one_to(k1, st ^ 1, 15 + n / 3);
    });
    step(S0{}, K2{}, K3{}, st, nothing, [](int) {});
    // Last step of the tile.  Its fragments were asked for during the step before; behind its first four MFMAs
    // every read of this stage has to be back (the stage is given up) and tile kt + 1 has to have landed in the
    // other stage: all of this wave's loads and reads done, then the barrier makes that all waves'.  Behind the
    // barrier: step 0 of tile kt + 1 is read, and tile kt + 2 begins to load into the stage just given up.
    step(S1{}, K3{}, K0{}, st ^ 1, tile_change, [&](int n) {
      if (n % 3 == 1 && n >= 4) load_one_to(k2, st, n / 3 - 1);
    });
    // The MFMAs are opaque to the compiler, which therefore adds no wait states before code of its own that reads
    // an accumulator (it may place such code right behind the loop): the last results are given their 20 states
    // here, where it cannot get in between.
    asm volatile("s_nop 15\n\ts_nop 4" ::: "memory");
  }
  sw_wait_lds<0>();

  // ---- row sum of squares -> per-row multiplier (the tile buffers are free now) ----------------------------
  wg_barrier_lds<0>();  // every wave is past its last fragment read
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 3; ++i) {
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) ss[i][kk] += __shfl_xor(ss[i][kk], 32);
    float ssq = (ss[i][0] + ss[i][1]) + (ss[i][2] + ss[i][3]);
    if (fh == 0) {
      const int row = wm * WTM + (wn * 3 + i) * 32 + fr;
      if (NORMS_GIVEN) ssq = g_row0 + row < args.rows ? args.sumsq_in[args.row0 + g_row0 + row] : 0.f;
      float w = args.query_scale;
      if (args.unit_norm) w = ssq > 0.f ? args.query_scale / sqrtf(ssq) : 0.f;
      s_inv[row] = w;
      const int64_t grow = g_row0 + row;
      if (qt == 0 && args.sumsq != nullptr && grow < args.rows) args.sumsq[args.row0 + grow] = ssq;
    }
  }
  __syncthreads();

  scan_tile_epilogue<TM, TN, WTM, WTN, WN>(args, acc, s_inv, wm, wn, fr, fh, g_row0, q_row0, qt, 3 * wn);
}

// ---- few queries: the store streamed once, no tiles in LDS ---------------------------------------
// With at most 32 queries the scan is a matter of reading the store once, and the tile kernel above -- a
// barrier and an LDS round trip of the whole workgroup per 64 columns -- tops out at 5.3 TB/s.  This kernel
// is the collection kernel's input stream pointed at the store: persistent workgroups, each wave streams 64
// rows at a time over all of D with whole-line non-temporal loads through its register queue and its own
// LDS slot, the queries come as MFMA fragments from a table in global memory (built once per scan; every
// wave reads the same table, so it lives in L2), the row norms are summed from the data on its way to LDS.
// With one or two blocks of 16 queries every wave loads the table's fragments for itself and no workgroup barrier
// is anywhere; with three (SHARE) the waves of a workgroup load each fragment once between them and share it through
// LDS (stream_segment_shared: one barrier per four k-pairs, the waves stream in step).  Same box, 10^6 x 12288 fp16:
// 48 queries 4.10 ms shared against 4.32, 32 queries 4.00 either way, 16 queries 4.01 against 3.92 -- the waves then
// wait for each other's selection loops, and there is little to save.  Scores land in 16 x 16 accumulators: lane (c, q4) holds rows 4 q4 + e of
// each 16-row block against query 16 qb + c.
constexpr int SS_MTW = 4;                // 16-row blocks per wave
constexpr int SS_WAVE_ROWS = 16 * SS_MTW;
constexpr int SS_TILE_ROWS = 4 * SS_WAVE_ROWS;
constexpr int SS_MAX_QUERIES = 96;       // up to six blocks of 16 queries (LDS: the fragment ring is 16 KB per block)
// blocks of 16 queries whose scores pass through LDS together on their way to the rows' lanes
constexpr int ss_score_blocks(int qb) { return qb <= 3 ? qb : (qb <= 5 ? 2 : 1); }

template <typename T>
__global__ __launch_bounds__(COLLECT_THREADS) void scan_query_fragments_kernel(const T* __restrict__ queries, int Q,
                                                                               int64_t D, int nblk,
                                                                               uint4* __restrict__ table) {
  const int blk = blockIdx.y;
  const int ks0 = blockIdx.x * 4 * STAGE_B;
  if ((int64_t)ks0 * Mma<T>::KS >= D) return;
  stage_projection<T>(queries + (int64_t)blk * 16 * D, nullptr, (int)D, min(16, Q - blk * 16), table, threadIdx.x, ks0,
                      ks0 + 4 * STAGE_B, blk, nblk);
}

template <typename T, int QB, bool SHARE = (QB >= 3)>
__global__ __launch_bounds__(COLLECT_THREADS, 1) void scan_stream_kernel(ScanArgs args, const uint4* __restrict__ qfrag) {
  using M = Mma<T>;
  using St = Stream<SS_MTW>;
  constexpr int RG = St::RG;
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned char* stage = smem + wave * St::BYTES_PER_WAVE;
  constexpr int EB = ss_score_blocks(QB);
  constexpr int SC_PITCH = 16 * EB + 1;  // floats per row of the wave's score block in LDS (odd: no bank conflicts)
  float* sc = reinterpret_cast<float*>(smem + 4 * St::BYTES_PER_WAVE) + wave * (SS_WAVE_ROWS * SC_PITCH);
  float* wrow = reinterpret_cast<float*>(smem + 4 * St::BYTES_PER_WAVE) + 4 * (SS_WAVE_ROWS * SC_PITCH) +
                wave * SS_WAVE_ROWS;  // row multipliers
  // behind them: the two slots through which the workgroup's waves share the table's fragments
  uint4* ring = reinterpret_cast<uint4*>(smem + 4 * St::BYTES_PER_WAVE + 4 * (SS_WAVE_ROWS * SC_PITCH) * sizeof(float) +
                                         4 * SS_WAVE_ROWS * sizeof(float));
  int ring_slot = 0;
  const int c = lane & 15;
  const int q4 = lane >> 4;
  const int rho = lane >> 3;
  const int sig = lane & 7;

  const T* store = (const T*)args.store + args.row0 * args.store_stride;
  const int nkp = (int)(args.D / (2 * M::KS));
  // Rows are dealt to the waves of the grid in units of 16, as evenly as those allow; a wave walks its
  // stretch 64 rows at a time and its last step may be shorter.
  const int gw = blockIdx.x * 4 + wave;
  const int64_t r_first = ((int64_t)gw * args.units_per_wave + min(gw, args.units_rem)) * 16;
  const int64_t r_last =
      min(args.rows, r_first + ((int64_t)args.units_per_wave + (gw < args.units_rem ? 1 : 0)) * 16);
  // SHARE: the waves of a workgroup stream in step: all take as many steps as its first wave, which has the most
  // rows; a wave whose rows have run out streams the pass's first row and drops the result.
  const int gw0 = SHARE ? blockIdx.x * 4 : gw;
  const int n_steps = (int)((((int64_t)args.units_per_wave + (gw0 < args.units_rem ? 1 : 0)) * 16 + SS_WAVE_ROWS - 1) /
                            SS_WAVE_ROWS);

  if (args.first_pass && blockIdx.x == 0 && tid < args.Q) args.cand_count[tid] = (uint32_t)args.rows;

  // Every wave (SHARE: every workgroup) walks D from its own starting k-pair (a multiple of the queue length) and
  // wraps around: at any moment the waves of the chip then read different parts of the query table, whose 4 KB
  // stretches would otherwise each be wanted by all of them at once.  A step is two segments, [rot, nkp) and [0, rot).
  const int rot = stream_rotation(nkp, SHARE ? (int)blockIdx.x : gw);
  const int nseg = rot > 0 ? 2 : 1;
  constexpr int KP = 2 * M::KS;        // elements of a k-pair
  constexpr int FP = 2 * QB * WAVE;    // table entries of a k-pair

  uint4 v[STREAM_Q][RG];
  uint4 rq[SHARE ? 1 : STREAM_Q][2 * QB];  // per-wave fragment queue
  uint4 rs[2 * QB];                        // SHARE: this wave's k-pair of the next block of fragments
  f32x4 acc[SS_MTW * QB];
  float ssq[RG];
  bool primed = false;
  for (int item = 0; item < n_steps * nseg; ++item) {
    const int step = item / nseg;
    const int sg = item - step * nseg;
    const int64_t prow0 = r_first + (int64_t)step * SS_WAVE_ROWS;  // pass-local first row of this step
    const int rows_valid = (int)min((int64_t)SS_WAVE_ROWS, r_last - prow0);  // <= 0: none left for this wave
    const int64_t srow0 = rows_valid > 0 ? prow0 : 0;  // the rows it streams
    const int srows = max(rows_valid, 1);
    const int k0 = sg == 0 ? rot : 0;
    const int len = nseg == 1 ? nkp : (sg == 0 ? nkp - rot : rot);
    const T* ur[RG];
    const T* un[RG];
    stream_rows<T, SS_MTW>(store + srow0 * args.store_stride + k0 * KP, args.store_stride, srows, lane, ur);
    if (!primed) {
      if constexpr (SHARE)
        stream_prime_shared<T, SS_MTW, QB>(ur, len, qfrag + k0 * FP, lane, wave, v, rs);
      else
        stream_prime<T, SS_MTW, true, QB>(ur, len, qfrag + k0 * FP, lane, v, rq);
    }
    int len_next = 0;
    int k1 = 0;
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) un[rg] = ur[rg];
    if (sg + 1 < nseg) {
      // the same rows from k-pair 0
      stream_rows<T, SS_MTW>(store + srow0 * args.store_stride, args.store_stride, srows, lane, un);
      len_next = rot;
    } else if (step + 1 < n_steps) {
      const int64_t prow1 = prow0 + SS_WAVE_ROWS;
      const int rows1 = (int)min((int64_t)SS_WAVE_ROWS, r_last - prow1);
      k1 = rot;
      stream_rows<T, SS_MTW>(store + (rows1 > 0 ? prow1 : 0) * args.store_stride + k1 * KP, args.store_stride,
                             max(rows1, 1), lane, un);
      len_next = nkp - rot;
    }
    if (sg == 0) {
#pragma unroll
      for (int i = 0; i < SS_MTW * QB; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int rg = 0; rg < RG; ++rg) ssq[rg] = 0.f;
    }
    if constexpr (SHARE)
      stream_segment_shared<T, SS_MTW, QB, true>(ur, len, un, len_next, qfrag + k0 * FP, qfrag + k1 * FP, stage, ring,
                                                 ring_slot, lane, wave, v, rs, acc, ssq);
    else
      stream_segment<T, SS_MTW, true, QB, true>(ur, len, un, len_next, qfrag + k0 * FP, qfrag + k1 * FP, stage, lane, v,
                                                rq, acc, ssq);
    primed = len_next > 0;
    if (sg + 1 < nseg) continue;
    if (rows_valid <= 0) continue;  // nothing of this wave's in the step (no workgroup barrier below)

    // ---- row norms: lane (rho, sig) carried slot sig of row rg * 8 + rho; a row's 8 lanes add up ----
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
      float s = ssq[rg];
      s += __shfl_xor(s, 1);
      s += __shfl_xor(s, 2);
      s += __shfl_xor(s, 4);
      const int row = rg * 8 + rho;
      if (sig == 0) {
        float w = args.query_scale;
        if (args.unit_norm) w = s > 0.f ? args.query_scale / sqrtf(s) : 0.f;
        wrow[row] = w;
        if (args.sumsq != nullptr && row < rows_valid) args.sumsq[args.row0 + prow0 + row] = s;
      }
    }
    __builtin_amdgcn_wave_barrier();

    // ---- scores: through LDS, EB blocks of queries at a time, so that lane l owns row l and walks the queries
    // in a plain loop -------------
    const int row = lane;
    const bool row_ok = row < rows_valid;
    const int64_t prow = prow0 + row;
    const int64_t grow = args.row0 + prow;
    const float w = wrow[row];
    float rmax = -INFINITY;
    float rsum = 0.f;
#pragma unroll
    for (int g0 = 0; g0 < QB; g0 += EB) {
      if (g0 > 0) __builtin_amdgcn_wave_barrier();  // the lanes have read the blocks before
#pragma unroll
      for (int mt = 0; mt < SS_MTW; ++mt)
#pragma unroll
        for (int eb = 0; eb < EB; ++eb)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (g0 + eb < QB)
              sc[(mt * 16 + q4 * 4 + e) * SC_PITCH + eb * 16 + c] = acc[mt * QB + g0 + eb][e];
      __builtin_amdgcn_wave_barrier();
      const int q_end = min(args.Q, (g0 + EB) * 16);
      for (int qi = g0 * 16; qi < q_end; ++qi) {
        const float val = sc[row * SC_PITCH + qi - g0 * 16] * w;
        const float thr = args.thr != nullptr ? args.thr[qi] : INFINITY;
        if (row_ok) {
          rmax = fmaxf(rmax, val);
          rsum += val;  // queries in ascending order: a fixed sum
          if (args.scores != nullptr) args.scores[grow * args.Q + qi] = val;
          if (args.first_pass) {
            args.cand[qi * args.cand_cap + prow] = make_key_or_empty(val, (uint32_t)grow);
          } else if (val > thr) {
            const uint32_t pos = atomicAdd(&args.cand_count[qi], 1u);
            if ((int64_t)pos < args.cand_cap) args.cand[qi * args.cand_cap + pos] = make_key(val, (uint32_t)grow);
          }
        }
      }
    }
    if (row_ok) {
      if (args.row_max_enc != nullptr) atomicMax(&args.row_max_enc[grow], f32_ordered(rmax));
      if (args.row_sum_part != nullptr) args.row_sum_part[prow * args.n_parts] = rsum;
    }
    __builtin_amdgcn_wave_barrier();  // sc and wrow are rewritten by the next tile
  }
}

// ---- per-query exact selection ---------------------------------------------------------------
struct SelectArgs {
  uint64_t* top;         // [Q][k] sorted descending
  uint32_t* top_count;   // [Q]
  uint64_t* cand;        // [Q][cand_cap]
  uint32_t* cand_count;  // [Q]
  float* thr;            // [Q]
  int64_t cand_cap;
  int k;
};

// Threads per query: 1024 behind a pass without thresholds (one candidate per row), 256 behind the others, whose
// lists are a few hundred entries -- the selection is some fifty workgroup barriers, and those cost by the wave.
constexpr int SELECT_THREADS_LONG = 1024, SELECT_THREADS_SHORT = 256;
constexpr uint32_t SELECT_SAMPLE = 4096;                     // > SCAN_KMAX
constexpr uint32_t SELECT_PRESELECT_MIN = 4 * SELECT_SAMPLE;  // shorter lists go to the exact selection directly
constexpr int SELECT_COMPACT_KEYS = 4096;                     // keys per compaction step: 64 (sub-block, wave) pairs

struct SelectShared {
  uint64_t keys[SCAN_KMAX];
  uint32_t hist[256];
  uint32_t part[SELECT_COMPACT_KEYS / 64 + 1];  // compaction: per (sub-block, wave) counts, then offsets
  uint64_t prefix;
  uint32_t rank;
  uint32_t fill;
};

// The rank-th largest (rank from 1, rank <= n) of the n keys elem(0..n-1): radix select, 8 bits per pass from
// the top.  Every thread of the workgroup calls it.
template <int THREADS, typename F>
__device__ uint64_t radix_kth(F elem, uint32_t n, uint32_t rank, SelectShared& sh) {
  const int tid = threadIdx.x;
  if (tid == 0) {
    sh.prefix = 0;
    sh.rank = rank;  // rank inside the current bucket
  }
  __syncthreads();
  for (int shift = 56; shift >= 0; shift -= 8) {
    if (tid < 256) sh.hist[tid] = 0;
    __syncthreads();
    const uint64_t prefix = sh.prefix;
    const uint64_t mask = shift == 56 ? 0ull : (~0ull << (shift + 8));
    for (uint32_t i = tid; i < n; i += THREADS) {
      const uint64_t key = elem(i);
      if ((key & mask) == prefix) atomicAdd(&sh.hist[(uint32_t)(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (tid < 64) {
      // wave 0: lane l owns bins 4l..4l+3; counts of all higher bins through a suffix sum over the lanes
      const uint32_t h0 = sh.hist[4 * tid], h1 = sh.hist[4 * tid + 1], h2 = sh.hist[4 * tid + 2],
                     h3 = sh.hist[4 * tid + 3];
      const uint32_t own = h0 + h1 + h2 + h3;
      uint32_t incl = own;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_down(incl, d);
        if (tid + d < 64) incl += o;
      }
      const uint32_t above = incl - own;
      const uint32_t r = sh.rank;
      if (above < r && r <= incl) {  // true for exactly one lane
        uint32_t rr = r - above;
        int d;
        if (h3 >= rr) {
          d = 3;
        } else if (h3 + h2 >= rr) {
          d = 2;
          rr -= h3;
        } else if (h3 + h2 + h1 >= rr) {
          d = 1;
          rr -= h3 + h2;
        } else {
          d = 0;
          rr -= h3 + h2 + h1;
        }
        sh.rank = rr;
        sh.prefix = prefix | ((uint64_t)(4 * tid + d) << shift);
      }
    }
    __syncthreads();
  }
  const uint64_t kth = sh.prefix;
  __syncthreads();  // the next call resets prefix and rank
  return kth;
}

// Merges each query's candidate list into its running top-k.  A long list (a pass without a threshold
// leaves one entry per row) is first cut down in place: the k-th largest of a strided sample of it is a
// lower bound of the k-th largest overall, and only entries at or above that bound stay.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void scan_select_kernel(SelectArgs a) {
  constexpr int SELECT_THREADS = THREADS;
  constexpr int SELECT_COMPACT_U = SELECT_COMPACT_KEYS / THREADS;
  __shared__ SelectShared sh;

  const int q = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int k = a.k;
  uint64_t* top = a.top + (int64_t)q * k;
  uint64_t* cand = a.cand + (int64_t)q * a.cand_cap;
  const uint32_t ntop = a.top_count[q];
  uint32_t ncand = a.cand_count[q];
  if ((int64_t)ncand > a.cand_cap) ncand = (uint32_t)a.cand_cap;
  if (ncand == 0) return;  // nothing new for this query

  if (ncand >= SELECT_PRESELECT_MIN) {
    const uint32_t step = ncand / SELECT_SAMPLE;
    const uint64_t bound =
        radix_kth<THREADS>([&](uint32_t i) -> uint64_t { return cand[(uint64_t)i * step]; }, SELECT_SAMPLE, (uint32_t)k, sh);
    // order-preserving compaction in place: a step reads SELECT_COMPACT_U * SELECT_THREADS entries, and writes
    // its survivors only after every thread has read, at positions no later step reads from
    constexpr int NW = SELECT_THREADS / 64;
    constexpr uint32_t STEP = SELECT_COMPACT_U * SELECT_THREADS;
    uint32_t w_base = 0;
    for (uint32_t base = 0; base < ncand; base += STEP) {
      uint64_t key[SELECT_COMPACT_U];
      uint32_t lane_off[SELECT_COMPACT_U];
      bool keep[SELECT_COMPACT_U];
#pragma unroll
      for (int j = 0; j < SELECT_COMPACT_U; ++j) {
        const uint32_t i = base + j * SELECT_THREADS + tid;
        key[j] = i < ncand ? cand[i] : 0ull;
      }
#pragma unroll
      for (int j = 0; j < SELECT_COMPACT_U; ++j) {
        const uint32_t i = base + j * SELECT_THREADS + tid;
        keep[j] = i < ncand && key[j] >= bound;
        const uint64_t ballot = __ballot(keep[j]);
        lane_off[j] = __popcll(ballot & ((1ull << lane) - 1ull));
        if (lane == 0) sh.part[j * NW + wave] = __popcll(ballot);
      }
      __syncthreads();
      if (tid < 64) {
        // exclusive prefix over the SELECT_COMPACT_U * NW = 64 counts, in (sub-block, wave) order
        const uint32_t own = sh.part[tid];
        uint32_t incl = own;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const uint32_t o = __shfl_up(incl, d);
          if (tid >= d) incl += o;
        }
        sh.part[tid] = incl - own;
        if (tid == 63) sh.part[64] = incl;
      }
      __syncthreads();
#pragma unroll
      for (int j = 0; j < SELECT_COMPACT_U; ++j)
        if (keep[j]) cand[w_base + sh.part[j * NW + wave] + lane_off[j]] = key[j];
      w_base += sh.part[64];
      __syncthreads();
    }
    __threadfence_block();
    __syncthreads();
    ncand = w_base;
  }
  static_assert(SELECT_COMPACT_U * SELECT_THREADS / 64 == 64 && THREADS >= 256, "the compaction's offsets are one wave's prefix sum");

  const uint32_t total = ntop + ncand;
  auto elem = [&](uint32_t i) -> uint64_t { return i < ntop ? top[i] : cand[i - ntop]; };

  uint64_t kth = 0;  // keep keys >= kth
  if (total > (uint32_t)k) kth = radix_kth<THREADS>(elem, total, (uint32_t)k, sh);

  if (tid == 0) sh.fill = 0;
  __syncthreads();
  for (uint32_t i = tid; i < total; i += SELECT_THREADS) {
    const uint64_t key = elem(i);
    if (key >= kth && key != 0) {  // 0 = an empty entry of a by-row list
      const uint32_t pos = atomicAdd(&sh.fill, 1u);
      if (pos < SCAN_KMAX) sh.keys[pos] = key;
    }
  }
  __syncthreads();
  const uint32_t kept = min(sh.fill, (uint32_t)k);
  // bitonic sort, descending, padded with zeros (below every real key)
  uint32_t n2 = 1;
  while (n2 < kept) n2 <<= 1;
  for (uint32_t i = kept + tid; i < n2; i += SELECT_THREADS) sh.keys[i] = 0;
  __syncthreads();
  for (uint32_t size = 2; size <= n2; size <<= 1) {
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      for (uint32_t i = tid; i < n2 / 2; i += SELECT_THREADS) {
        const uint32_t lo = 2 * i - (i & (stride - 1));
        const uint32_t hi = lo + stride;
        const bool desc = (lo & size) == 0;
        const uint64_t x = sh.keys[lo], y = sh.keys[hi];
        if ((x < y) == desc) {
          sh.keys[lo] = y;
          sh.keys[hi] = x;
        }
      }
      __syncthreads();
    }
  }
  for (uint32_t i = tid; i < kept; i += SELECT_THREADS) top[i] = sh.keys[i];
  if (tid == 0) {
    a.top_count[q] = kept;
    a.cand_count[q] = 0;
    if (kept == (uint32_t)k) a.thr[q] = ordered_f32((uint32_t)(sh.keys[k - 1] >> 32));
  }
}

// ---- selection for k beyond what one workgroup sorts in LDS ------------------------------------------------
constexpr int SCAN_KMAX_LARGE = 65536;
constexpr int SELECT_THREADS_LARGE = 1024;

// dst[dst_base ...] = the keys of src[0, n) that are >= bound, in their order; returns how many.  Every thread of
// the workgroup calls it.  src == dst with dst_base == 0 compacts in place: a step's survivors are written only
// after every thread has read the step, at positions no later step reads from.
template <int THREADS>
__device__ uint32_t compact_keys(const uint64_t* src, uint32_t n, uint64_t bound, uint64_t* dst, uint32_t dst_base,
                                 SelectShared& sh) {
  constexpr int NW = THREADS / 64;
  constexpr int U = SELECT_COMPACT_KEYS / THREADS;
  static_assert(U * NW == 64, "the offsets are one wave's prefix sum");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t w_base = dst_base;
  for (uint32_t base = 0; base < n; base += SELECT_COMPACT_KEYS) {
    uint64_t key[U];
    uint32_t lane_off[U];
    bool keep[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const uint32_t i = base + j * THREADS + tid;
      key[j] = i < n ? src[i] : 0ull;
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const uint32_t i = base + j * THREADS + tid;
      keep[j] = i < n && key[j] >= bound;
      const uint64_t ballot = __ballot(keep[j]);
      lane_off[j] = __popcll(ballot & ((1ull << lane) - 1ull));
      if (lane == 0) sh.part[j * NW + wave] = __popcll(ballot);
    }
    __syncthreads();
    if (tid < 64) {
      const uint32_t own = sh.part[tid];
      uint32_t incl = own;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_up(incl, d);
        if (tid >= d) incl += o;
      }
      sh.part[tid] = incl - own;
      if (tid == 63) sh.part[64] = incl;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < U; ++j)
      if (keep[j]) dst[w_base + sh.part[j * NW + wave] + lane_off[j]] = key[j];
    w_base += sh.part[64];
    __syncthreads();
  }
  __threadfence_block();
  __syncthreads();
  return w_base - dst_base;
}

// scan_select_kernel for k > SCAN_KMAX: the running top-k of a query stays in global memory, unsorted -- after every
// pass it is the k largest keys seen so far (exact: the k-th largest of old entries and candidates by radix
// selection, then both lists cut at it) -- and is sorted once, when the scan is over (scan_sort_top_kernel).
__global__ __launch_bounds__(SELECT_THREADS_LARGE) void scan_select_large_kernel(SelectArgs a, int64_t top_stride) {
  __shared__ SelectShared sh;
  const int q = blockIdx.x;
  const uint32_t k = (uint32_t)a.k;
  uint64_t* top = a.top + (int64_t)q * top_stride;
  uint64_t* cand = a.cand + (int64_t)q * a.cand_cap;
  const uint32_t ntop = a.top_count[q];
  uint32_t ncand = a.cand_count[q];
  if ((int64_t)ncand > a.cand_cap) ncand = (uint32_t)a.cand_cap;
  if (ncand == 0) return;
  const uint32_t total = ntop + ncand;
  auto elem = [&](uint32_t i) -> uint64_t { return i < ntop ? top[i] : cand[i - ntop]; };
  uint64_t kth = 1;  // entry 0 of a by-row list is an empty one
  if (total > k) {
    const uint64_t found = radix_kth<SELECT_THREADS_LARGE>(elem, total, k, sh);
    kth = found > 1 ? found : 1;
  }
  uint32_t kept = compact_keys<SELECT_THREADS_LARGE>(top, ntop, kth, top, 0, sh);
  kept += compact_keys<SELECT_THREADS_LARGE>(cand, ncand, kth, top, kept, sh);
  if (threadIdx.x == 0) {
    a.top_count[q] = kept;
    a.cand_count[q] = 0;
    if (kept == k) a.thr[q] = ordered_f32((uint32_t)(kth >> 32));
  }
}

// Sorts each query's top[0, top_count) in place, descending: bitonic network over the next power of two (the row
// has room for it; padded with zeros, which sort last), one workgroup per query.
__global__ __launch_bounds__(1024) void scan_sort_top_kernel(uint64_t* top, const uint32_t* top_count, int64_t top_stride) {
  uint64_t* keys = top + (int64_t)blockIdx.x * top_stride;
  const uint32_t kept = top_count[blockIdx.x];
  uint32_t n2 = 1;
  while (n2 < kept) n2 <<= 1;
  for (uint32_t i = kept + threadIdx.x; i < n2; i += 1024) keys[i] = 0;
  __threadfence_block();
  __syncthreads();
  for (uint32_t size = 2; size <= n2; size <<= 1) {
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      for (uint32_t i = threadIdx.x; i < n2 / 2; i += 1024) {
        const uint32_t lo = 2 * i - (i & (stride - 1));
        const uint32_t hi = lo + stride;
        const bool desc = (lo & size) == 0;
        const uint64_t x = keys[lo], y = keys[hi];
        if ((x < y) == desc) {
          keys[lo] = y;
          keys[hi] = x;
        }
      }
      __threadfence_block();
      __syncthreads();
    }
  }
}

__global__ void scan_init_kernel(uint32_t* top_count, uint32_t* cand_count, float* thr, int Q, uint32_t* row_max_enc,
                                 int64_t n_rows) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < Q) {
    if (top_count) top_count[i] = 0;
    if (cand_count) cand_count[i] = 0;
    if (thr) thr[i] = -INFINITY;
  }
  if (row_max_enc && i < n_rows) row_max_enc[i] = 0;  // below every encoded float
}

// A query with fewer than k selectable scores (NaN and -inf are never selected) gets (-inf, -1) in the rest.
__global__ void scan_finish_kernel(const uint64_t* top, const uint32_t* top_count, int64_t top_stride, int Q, int k,
                                   int64_t row_base, float* topk_val, int64_t* topk_idx, const uint32_t* row_max_enc,
                                   float* row_max, int64_t n_rows) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (top != nullptr && i < (int64_t)Q * k) {
    const bool filled = (uint32_t)(i % k) < top_count[i / k];
    const uint64_t key = filled ? top[(i / k) * top_stride + i % k] : 0ull;
    topk_val[i] = filled ? ordered_f32((uint32_t)(key >> 32)) : -INFINITY;
    topk_idx[i] = filled ? (int64_t)(0xffffffffu - (uint32_t)key) + row_base : (int64_t)-1;
  }
  if (row_max != nullptr && i < n_rows) row_max[i] = ordered_f32(row_max_enc[i]);
}

// row_mean[row0 + r] = (sum of the row's partial sums, in part order) / Q
__global__ void scan_row_mean_kernel(const float* __restrict__ part, int n_parts, int64_t rows, int64_t row0,
                                     float inv_q, float* __restrict__ row_mean) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  float s = 0.f;
  for (int p = 0; p < n_parts; ++p) s += part[r * n_parts + p];
  row_mean[row0 + r] = s * inv_q;
}

// ---- row sums of squares on their own ---------------------------------------------------------------------
// sumsq[n] = sum_k store[n, k]^2 in exactly the order the tile kernels form it inside a scan: one partial per
// 16-byte position c of a 128-byte K tile, each running over the K tiles in ascending order, the eight partials
// combined as ((c0 + c1) + (c2 + c3)) + ((c4 + c5) + (c6 + c7)).  The values are therefore the bits a scan's own
// `sumsq` output holds (scan_gemm_kernel without its rotated start, scan_direct_kernel, scan_wide_kernel), and a
// scan that is given them (bgx_scan_known_norms) returns the bits of a scan that computed them.
// Eight lanes per row (lane c owns position c: a load instruction reads whole 128-byte lines of eight rows),
// eight K tiles in flight per lane, every row read once with the non-temporal hint: bound by HBM.
template <typename T, bool ALIGNED>
__global__ __launch_bounds__(256) void row_sumsq_kernel(const T* __restrict__ store, int64_t n_rows, int64_t D,
                                                        int64_t stride, float* __restrict__ sumsq) {
  using M = Mma32<T>;
  constexpr int EPL = M::EPL;
  constexpr int BK = TILE_CHUNKS * EPL;  // elements per 128-byte K tile
  constexpr int U = 8;
  const int c = threadIdx.x & 7;
  const int64_t row = (int64_t)blockIdx.x * 32 + (threadIdx.x >> 3);
  const int64_t KT = (D + BK - 1) / BK;
  float s = 0.f;
  for (int64_t kt0 = 0; kt0 < KT; kt0 += U) {
    uint4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      v[u] = load_chunk<T, ALIGNED, ALIGNED>(store, row, n_rows, stride, (kt0 + u) * BK + c * EPL, D);
#pragma unroll
    for (int u = 0; u < U; ++u) s = M::sumsq(v[u], s);  // a chunk past the end is zero and adds nothing
  }
  s += __shfl_xor(s, 1);
  s += __shfl_xor(s, 2);
  s += __shfl_xor(s, 4);
  if (c == 0 && row < n_rows) sumsq[row] = s;
}

// ---- host side --------------------------------------------------------------------------------
constexpr int64_t SCAN_DEFAULT_CHUNK = 65536;
constexpr int64_t SCAN_FIRST_CHUNK = 4096;

static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct ScanLayout {
  size_t top, top_count, cand_count, thr, row_part, cand, total;
};

// Entries of a query's row of the running top-k: k, or beyond SCAN_KMAX the next power of two (the final sort pads
// the row to it).
static int64_t scan_top_stride(int k) {
  if (k <= SCAN_KMAX) return k > 0 ? k : 0;
  int64_t n2 = 1;
  while (n2 < k) n2 <<= 1;
  return n2;
}

static ScanLayout scan_layout(int Q, int k, int64_t chunk_rows) {
  ScanLayout l;
  size_t off = 0;
  l.top = off;
  off += align_up((size_t)Q * (size_t)scan_top_stride(k) * 8, 256);
  l.top_count = off;
  off += align_up((size_t)Q * 4, 256);
  l.cand_count = off;
  off += align_up((size_t)Q * 4, 256);
  l.thr = off;
  off += align_up((size_t)Q * 4, 256);
  l.row_part = off;  // per-pass partial row sums: at most 4 wave columns per 256-query tile
  off += align_up((size_t)chunk_rows * (size_t)((Q + 255) / 256 * 4) * 4, 256);
  l.cand = off;
  off += k > 0 ? align_up((size_t)Q * (size_t)chunk_rows * 8, 256) : 0;
  l.total = off;
  return l;
}

// Rows per pass: the candidate lists hold one entry per (query, row of a pass) in the worst case, so the
// default keeps Q * chunk near 64 Mi entries (512 MB) -- 65536 rows at 1024 queries, more for fewer.
static int64_t effective_chunk(int64_t chunk_rows, int Q) {
  if (chunk_rows > 0) return chunk_rows;
  if (Q > SW_BN / 2) {
    // many queries: whole rounds of the 384 x 256 tile kernel, Q * chunk near 96 Mi entries -- 98 304 rows (four
    // rounds) at 1024 queries, 393 216 (four rounds) at 256
    const int64_t round = sw_round_rows(Q);
    const int64_t c = ((int64_t)96 << 20) / Q / round * round;
    if (c >= round && c >= SCAN_KMAX) return c;  // (a pass is never shorter than the largest k by default)
  }
  int64_t c = ((int64_t)64 << 20) / (Q > 0 ? Q : 1);
  if (c > ((int64_t)1 << 20)) c = (int64_t)1 << 20;
  if (c < SCAN_DEFAULT_CHUNK) c = SCAN_DEFAULT_CHUNK;
  return c / 256 * 256;
}

size_t scan_workspace_bytes(int Q, int k, int64_t chunk_rows) {
  if (Q <= 0 || k < 0) return 0;
  return scan_layout(Q, k, effective_chunk(chunk_rows, Q)).total;
}

// Bytes of the query fragment table of the streaming kernel (1 KB per k-step and block of 16 queries), or 0
// where that kernel does not apply: more than 32 queries, a row length that is no multiple of two k-steps.
static size_t query_table_bytes(int Q, int64_t D, int dtype) {
  if (Q <= 0 || Q > SS_MAX_QUERIES) return 0;
  const int kstep = dtype == BGX_F32 ? 16 : 32;
  if (D <= 0 || D % (2 * kstep) != 0) return 0;
  return (size_t)((Q + 15) / 16) * (size_t)(D / kstep) * 1024;
}

size_t scan_workspace_bytes_for(int Q, int k, int64_t chunk_rows, int64_t D, int dtype) {
  const size_t base = scan_workspace_bytes(Q, k, chunk_rows);
  return align_up(std::max<size_t>(base, 256), 256) + query_table_bytes(Q, D, dtype);
}

template <typename T>
static int launch_stream(const ScanArgs& a, int blocks, const uint4* table, int wgs, hipStream_t st) {
  // stage slots, score blocks (pitch 16 * ss_score_blocks + 1 floats), row multipliers, the fragment ring (three
  // blocks and more)
  const size_t smem = 4 * Stream<SS_MTW>::BYTES_PER_WAVE +
                      4 * SS_WAVE_ROWS * (size_t)(16 * ss_score_blocks(blocks) + 1) * sizeof(float) +
                      4 * SS_WAVE_ROWS * sizeof(float) + (blocks >= 3 ? (size_t)stream_ring_bytes(blocks) : 0);
  auto go = [&](auto kern) -> int {
    BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(kern, dim3((unsigned)wgs), dim3(COLLECT_THREADS), smem, st, a, table);
    return 0;
  };
  const int rc = blocks == 1   ? go(scan_stream_kernel<T, 1>)
                 : blocks == 2 ? go(scan_stream_kernel<T, 2>)
                 : blocks == 3 ? go(scan_stream_kernel<T, 3>)
                 : blocks == 4 ? go(scan_stream_kernel<T, 4>)
                 : blocks == 5 ? go(scan_stream_kernel<T, 5>)
                               : go(scan_stream_kernel<T, 6>);
  if (rc != 0) return rc;
  BGX_HIP(hipGetLastError());
  return 0;
}

template <typename T>
static int launch_query_fragments(const void* queries, int Q, int64_t D, uint4* table, hipStream_t st) {
  const int blocks = (Q + 15) / 16;
  const int64_t steps = D / Mma<T>::KS;
  const dim3 grid((unsigned)((steps + 4 * STAGE_B - 1) / (4 * STAGE_B)), (unsigned)blocks);
  hipLaunchKernelGGL(scan_query_fragments_kernel<T>, grid, dim3(COLLECT_THREADS), 0, st, (const T*)queries, Q, D, blocks,
                     table);
  BGX_HIP(hipGetLastError());
  return 0;
}

template <typename T, int BM, int BN, int WM, int WN, bool ALIGNED, int PF, bool STREAM>
static int launch_gemm_v(const ScanArgs& a, hipStream_t st) {
  constexpr int NT = WM * WN * 64;
  constexpr size_t smem = 2 * (size_t)(BM + BN) * LDS_ROW_BYTES;
  const int row_tiles_pad = (a.row_tiles + 7) / 8 * 8;
  const dim3 grid((unsigned)(row_tiles_pad * a.q_tiles));
  auto kern = scan_gemm_kernel<T, BM, BN, WM, WN, ALIGNED, PF, STREAM>;
  BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
  hipLaunchKernelGGL(kern, grid, dim3(NT), smem, st, a);
  BGX_HIP(hipGetLastError());
  return 0;
}

// PF: see the kernel.  The small-tile variants are bound by HBM latency (a K tile is only 16 KB per
// workgroup), so they run two tiles ahead, and stream the store past the caches when no other workgroup
// will want the same rows.
template <typename T, int BM, int BN, int WM, int WN, int PF = 1>
static int launch_gemm(const ScanArgs& a, bool aligned, hipStream_t st) {
  if (!aligned) return launch_gemm_v<T, BM, BN, WM, WN, false, PF, false>(a, st);
  if (PF > 1 && a.q_tiles == 1) return launch_gemm_v<T, BM, BN, WM, WN, true, PF, true>(a, st);
  return launch_gemm_v<T, BM, BN, WM, WN, true, PF, false>(a, st);
}

// Whether passes of this scan can run on the 384 x 256 tile kernel (whole rounds of it; see scan_wide_kernel).
static bool wide_scan_ok(int dtype, bool aligned, int64_t D, int64_t stride, int Q) {
  return dtype != BGX_F32 && aligned && D % 64 == 0 && Q > SW_BN / 2 && !switches().scan_wide_off &&
         stride * 2 * (SW_BM + 8) < ((int64_t)1 << 32) && D * 2 * (SW_BN + 8) < ((int64_t)1 << 32);
}

template <typename T>
static int launch_gemm_t(ScanArgs& a, bool aligned, hipStream_t st) {
  // large tiles when there is enough work to fill the chip with them
  const int64_t big_tiles = ((a.rows + 255) / 256) * ((a.Q + 255) / 256);
  // (a pass the 384 x 256 tiles take is theirs even when it is less than a round of the chip: the last 12 864 rows
  // of a million, 136 workgroups, take 0.62 ms there and 0.77 ms on the 128 x 64 tiles)
  bool wide_pass = false;
  if constexpr (sizeof(T) == 2)
    wide_pass = wide_scan_ok(Elem<T>::code, aligned, a.D, a.store_stride, a.Q) && a.rows >= SW_MIN_ROWS;
  if (a.Q > 64 && a.rows >= 256 && (big_tiles >= 256 || wide_pass)) {
    // 8 waves, each 128 x 64: two waves per SIMD hide each other's LDS and barrier stalls
    constexpr int BM = 256, BN = 256;
    a.row_tiles = (int)((a.rows + BM - 1) / BM);
    a.q_tiles = (a.Q + BN - 1) / BN;
    a.n_parts = a.q_tiles * 4;
    if constexpr (sizeof(T) == 2) {
      if (wide_pass) {
        a.row_tiles = (int)((a.rows + SW_BM - 1) / SW_BM);
        const int row_tiles_pad = (a.row_tiles + 7) / 8 * 8;
        a.q_tiles = (a.Q + SW_BN - 1) / SW_BN;
        a.n_parts = a.q_tiles * 2;
        auto kern = a.sumsq_in != nullptr ? scan_wide_kernel<T, true> : scan_wide_kernel<T, false>;
        BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SW_LDS_BYTES));
        hipLaunchKernelGGL(kern, dim3((unsigned)(row_tiles_pad * a.q_tiles)), dim3(SW_THREADS), SW_LDS_BYTES, st, a);
        BGX_HIP(hipGetLastError());
        note_kernel(FAMILY_SCAN, a.sumsq_in != nullptr ? "scan_wide_known_norms" : "scan_wide");
        return 0;
      }
      // aligned 16-bit operands, D a multiple of the K tile: tiles loaded straight into LDS
      if (aligned && a.D % 64 == 0 && !switches().scan_direct_off) {
        const int row_tiles_pad = (a.row_tiles + 7) / 8 * 8;
        auto launch = [&](auto kern, int bn, unsigned wgs) -> int {
          BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, sd_lds_bytes(bn)));
          hipLaunchKernelGGL(kern, dim3(wgs), dim3(SD_THREADS), sd_lds_bytes(bn), st, a);
          return 0;
        };
        int rc;
        if (a.Q <= 128) {
          a.q_tiles = 1;
          a.n_parts = 4;
          rc = launch(scan_direct_kernel<T, 128, true>, 128, (unsigned)row_tiles_pad);
        } else if (a.q_tiles == 1) {
          rc = launch(scan_direct_kernel<T, 256, true>, 256, (unsigned)row_tiles_pad);
        } else {
          rc = launch(scan_direct_kernel<T, 256, false>, 256, (unsigned)(row_tiles_pad * a.q_tiles));
        }
        if (rc != 0) return rc;
        BGX_HIP(hipGetLastError());
        note_kernel(FAMILY_SCAN, "scan_direct");
        return 0;
      }
    }
    note_kernel(FAMILY_SCAN, "scan_gemm");
    return launch_gemm<T, BM, BN, 2, 4>(a, aligned, st);
  } else if (a.Q > 32) {
    note_kernel(FAMILY_SCAN, "scan_gemm");
    constexpr int BM = 128, BN = 64;
    a.row_tiles = (int)((a.rows + BM - 1) / BM);
    a.q_tiles = (a.Q + BN - 1) / BN;
    a.n_parts = a.q_tiles;
    return launch_gemm<T, BM, BN, 4, 1, 2>(a, aligned, st);
  } else {
    note_kernel(FAMILY_SCAN, "scan_gemm");
    constexpr int BM = 128, BN = 32;
    a.row_tiles = (int)((a.rows + BM - 1) / BM);
    a.q_tiles = (a.Q + BN - 1) / BN;
    a.n_parts = a.q_tiles;
    return launch_gemm<T, BM, BN, 4, 1, 2>(a, aligned, st);
  }
}

// scores[n, q] = <rows[n], queries[q]> for every (n, q): the GEMM alone, no norms, no selection.
int gemm_scores(const void* rows, int64_t n_rows, int64_t D, int64_t stride, int dtype, const void* queries, int Q,
                float* scores, hipStream_t st) {
  ScanArgs a;
  a.store = rows;
  a.queries = queries;
  a.row0 = 0;
  a.rows = n_rows;
  a.D = D;
  a.store_stride = stride;
  a.Q = Q;
  a.row_tiles = 0;
  a.q_tiles = 0;
  a.query_scale = 1.0f;
  a.unit_norm = 0;
  a.scores = scores;
  a.sumsq = nullptr;
  a.sumsq_in = nullptr;
  a.row_max_enc = nullptr;
  a.row_sum_part = nullptr;
  a.n_parts = 0;
  a.thr = nullptr;
  a.cand_count = nullptr;
  a.cand = nullptr;
  a.cand_cap = 0;
  a.first_pass = 0;
  a.units_per_wave = 0;
  a.units_rem = 0;
  const int epl = dtype == BGX_F32 ? 4 : 8;
  const bool aligned = ((uintptr_t)rows % 16 == 0) && ((uintptr_t)queries % 16 == 0) && (D % epl == 0) &&
                       (stride % epl == 0);
  if (dtype == BGX_F16) return launch_gemm_t<f16_t>(a, aligned, st);
  if (dtype == BGX_BF16) return launch_gemm_t<bf16_t>(a, aligned, st);
  return launch_gemm_t<float>(a, aligned, st);
}

int scan_impl(const void* store, int64_t n_rows, int64_t D, int64_t stride, int dtype, const void* queries, int Q,
              float query_scale, int unit_norm, int k, int64_t row_base, float* topk_val, int64_t* topk_idx,
              float* row_max, float* row_mean, float* scores, float* sumsq, const float* sumsq_in, void* ws,
              size_t ws_bytes, int64_t chunk_rows, void* stream) {
  BGX_REQUIRE(store && queries, BGX_E_ARG, "scan: null store/queries");
  BGX_REQUIRE(n_rows > 0 && D > 0 && Q > 0 && stride >= D, BGX_E_ARG, "scan: n_rows=%lld D=%lld Q=%d stride=%lld",
              (long long)n_rows, (long long)D, Q, (long long)stride);
  BGX_REQUIRE(dtype >= BGX_F32 && dtype <= BGX_BF16, BGX_E_DTYPE, "scan: dtype=%d", dtype);
  BGX_REQUIRE(row_base >= 0 && n_rows + row_base <= 0xffffffffLL, BGX_E_SHAPE,
              "scan: row numbers must fit 32 bits (n_rows=%lld row_base=%lld)", (long long)n_rows, (long long)row_base);
  const bool want_topk = topk_val != nullptr || topk_idx != nullptr;
  if (want_topk) {
    BGX_REQUIRE(topk_val && topk_idx, BGX_E_ARG, "scan: topk_val and topk_idx go together");
    BGX_REQUIRE(k >= 1 && k <= SCAN_KMAX_LARGE && k <= n_rows, BGX_E_SHAPE, "scan: k=%d outside 1..min(%d, n_rows=%lld)",
                k, SCAN_KMAX_LARGE, (long long)n_rows);
  } else {
    k = 0;
  }
  const int64_t chunk = effective_chunk(chunk_rows, Q);
  const ScanLayout lay = scan_layout(Q, k, chunk);
  const int64_t top_stride = scan_top_stride(k);
  const bool need_init = want_topk || row_max != nullptr;
  if (want_topk || row_mean != nullptr) {
    BGX_REQUIRE(ws != nullptr, BGX_E_WORKSPACE, "scan: workspace required for top-k and row means");
    BGX_REQUIRE(((uintptr_t)ws & 255) == 0, BGX_E_ALIGN, "scan: workspace must be 256-byte aligned");
    BGX_REQUIRE(ws_bytes >= lay.total, BGX_E_WORKSPACE, "scan: workspace %zu < %zu bytes", ws_bytes, lay.total);
  }
  hipStream_t st = (hipStream_t)stream;
  char* w = (char*)ws;
  uint64_t* top = want_topk ? (uint64_t*)(w + lay.top) : nullptr;
  uint32_t* top_count = want_topk ? (uint32_t*)(w + lay.top_count) : nullptr;
  uint32_t* cand_count = want_topk ? (uint32_t*)(w + lay.cand_count) : nullptr;
  float* thr = want_topk ? (float*)(w + lay.thr) : nullptr;
  uint64_t* cand = want_topk ? (uint64_t*)(w + lay.cand) : nullptr;
  float* row_part = row_mean != nullptr ? (float*)(w + lay.row_part) : nullptr;
  // the row maxima are accumulated in place in an order-preserving integer
  // encoding and decoded by the finish kernel
  uint32_t* row_max_enc = (uint32_t*)row_max;

  if (need_init) {
    const int64_t n_init = (row_max ? n_rows : 0) > Q ? n_rows : Q;
    hipLaunchKernelGGL(scan_init_kernel, dim3((unsigned)((n_init + 255) / 256)), dim3(256), 0, st, top_count,
                       cand_count, thr, Q, row_max_enc, row_max ? n_rows : 0);
    BGX_HIP(hipGetLastError());
  }

  const size_t esz = dtype_size(dtype);
  const int epl = dtype == BGX_F32 ? 4 : 8;
  const bool aligned = ((uintptr_t)store % 16 == 0) && ((uintptr_t)queries % 16 == 0) && (D % epl == 0) &&
                       (stride % epl == 0);
  (void)esz;

  // Few queries and a pass large enough to give every CU several tiles: the streaming kernel, if the
  // workspace has room for its query fragment table (bgx_scan_workspace_bytes_for).
  const size_t table_bytes = query_table_bytes(Q, D, dtype);
  const size_t table_off = align_up(std::max<size_t>(lay.total, 256), 256);
  int cus = 0;
  {
    int dev = 0;
    BGX_HIP(hipGetDevice(&dev));
    BGX_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  }
  const bool stream_ok = table_bytes > 0 && aligned && ws != nullptr && ((uintptr_t)ws & 255) == 0 &&
                         ws_bytes >= table_off + table_bytes && !switches().scan_stream_off;
  // With top-k the streaming scan opens with one tile per workgroup and no thresholds (the select kernel
  // cuts that pass's one-entry-per-row lists down); every later pass is as long as the workspace allows.
  const int64_t stream_first = (int64_t)std::max(cus, 1) * SS_TILE_ROWS;
  const int64_t stream_min_rows = 2 * stream_first;
  const bool stream_scan = stream_ok && n_rows >= stream_min_rows && chunk >= stream_first;
  uint4* qtable = stream_ok ? (uint4*)((char*)ws + table_off) : nullptr;
  bool table_built = false;

  int64_t done = 0;
  int64_t longest_pass = 0;
  const char* main_kernel = "";
  while (done < n_rows) {
    int64_t rows = n_rows - done;
    if (want_topk) {
      // the first pass has no threshold yet and keeps every score (the selection behind it then sorts one entry per
      // row and query), so that pass stays small and later passes grow fourfold
      int64_t lim = done == 0 ? SCAN_FIRST_CHUNK : done * 4;
      // with the wide tile kernel the second pass is a whole round already (thresholds from 4096 rows let
      // through k / 4096 of the scores: a few hundred candidates per query)
      if (done > 0 && lim < sw_round_rows(Q) && wide_scan_ok(dtype, aligned, D, stride, Q)) lim = sw_round_rows(Q);
      if (stream_scan) lim = done == 0 ? stream_first : chunk;
      if (lim < k) lim = k;
      if (lim > chunk) lim = chunk;
      if (rows > lim) rows = lim;
    }
    if (row_part != nullptr && rows > chunk) rows = chunk;  // the partial sums of one pass fit the workspace
    // many queries: long passes are cut to whole rounds of the 384 x 256 tile kernel (the end of the store makes
    // one last, shorter pass)
    if (rows >= sw_round_rows(Q) && wide_scan_ok(dtype, aligned, D, stride, Q)) rows = rows / sw_round_rows(Q) * sw_round_rows(Q);
    ScanArgs a;
    a.store = store;
    a.queries = queries;
    a.row0 = done;
    a.rows = rows;
    a.D = D;
    a.store_stride = stride;
    a.Q = Q;
    a.row_tiles = 0;
    a.q_tiles = 0;
    a.query_scale = query_scale;
    a.unit_norm = unit_norm;
    a.scores = scores;
    a.sumsq = sumsq;
    a.sumsq_in = sumsq_in;
    a.row_max_enc = row_max_enc;
    a.row_sum_part = row_part;
    a.n_parts = 0;
    a.thr = thr;
    a.cand_count = cand_count;
    a.cand = cand;
    a.cand_cap = chunk;
    a.first_pass = 0;
    a.units_per_wave = 0;
    a.units_rem = 0;
    int rc;
    if (stream_scan && rows >= 16 * SS_TILE_ROWS) {
      a.first_pass = want_topk && done == 0;
      if (!table_built) {
        rc = dtype == BGX_F16    ? launch_query_fragments<f16_t>(queries, Q, D, qtable, st)
             : dtype == BGX_BF16 ? launch_query_fragments<bf16_t>(queries, Q, D, qtable, st)
                                 : launch_query_fragments<float>(queries, Q, D, qtable, st);
        if (rc != 0) return rc;
        table_built = true;
      }
      a.row_tiles = (int)((rows + SS_TILE_ROWS - 1) / SS_TILE_ROWS);
      a.q_tiles = 1;
      a.n_parts = 1;
      const int wgs = (int)std::min<int64_t>(std::max(cus, 1), a.row_tiles);
      const int64_t units = (rows + 15) / 16;
      a.units_per_wave = (int)(units / (4 * wgs));
      a.units_rem = (int)(units % (4 * wgs));
      const int blocks = (Q + 15) / 16;
      rc = dtype == BGX_F16    ? launch_stream<f16_t>(a, blocks, qtable, wgs, st)
           : dtype == BGX_BF16 ? launch_stream<bf16_t>(a, blocks, qtable, wgs, st)
                               : launch_stream<float>(a, blocks, qtable, wgs, st);
      note_kernel(FAMILY_SCAN, "scan_stream");
    } else {
      // (honoured by scan_gemm_kernel, which takes the short first pass; the other tile kernels let every score of
      // a pass without thresholds through their candidate filter instead, with the same result)
      a.first_pass = want_topk && done == 0;
      rc = dtype == BGX_F16    ? launch_gemm_t<f16_t>(a, aligned, st)
           : dtype == BGX_BF16 ? launch_gemm_t<bf16_t>(a, aligned, st)
                               : launch_gemm_t<float>(a, aligned, st);
    }
    if (rc != 0) return rc;
    if (rows > longest_pass) {  // the scan is named after the kernel of its longest pass
      longest_pass = rows;
      main_kernel = noted_kernel(FAMILY_SCAN);
    }
    if (row_part != nullptr) {
      hipLaunchKernelGGL(scan_row_mean_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, st, row_part,
                         a.n_parts, rows, done, 1.0f / (float)Q, row_mean);
      BGX_HIP(hipGetLastError());
    }
    if (want_topk) {
      SelectArgs s;
      s.top = top;
      s.top_count = top_count;
      s.cand = cand;
      s.cand_count = cand_count;
      s.thr = thr;
      s.cand_cap = chunk;
      s.k = k;
      if (k > SCAN_KMAX)
        hipLaunchKernelGGL(scan_select_large_kernel, dim3((unsigned)Q), dim3(SELECT_THREADS_LARGE), 0, st, s, top_stride);
      else if (a.first_pass)
        hipLaunchKernelGGL(scan_select_kernel<SELECT_THREADS_LONG>, dim3((unsigned)Q), dim3(SELECT_THREADS_LONG), 0, st, s);
      else
        hipLaunchKernelGGL(scan_select_kernel<SELECT_THREADS_SHORT>, dim3((unsigned)Q), dim3(SELECT_THREADS_SHORT), 0, st, s);
      BGX_HIP(hipGetLastError());
    }
    done += rows;
  }
  note_kernel(FAMILY_SCAN, main_kernel);
  if (want_topk && k > SCAN_KMAX) {
    hipLaunchKernelGGL(scan_sort_top_kernel, dim3((unsigned)Q), dim3(1024), 0, st, top, (const uint32_t*)top_count,
                       top_stride);
    BGX_HIP(hipGetLastError());
  }

  if (need_init) {
    const int64_t n_fin = ((int64_t)Q * k > (row_max ? n_rows : 0)) ? (int64_t)Q * k : n_rows;
    hipLaunchKernelGGL(scan_finish_kernel, dim3((unsigned)((n_fin + 255) / 256)), dim3(256), 0, st,
                       (const uint64_t*)top, (const uint32_t*)top_count, top_stride, Q, k, row_base, topk_val, topk_idx,
                       (const uint32_t*)row_max_enc, row_max, row_max ? n_rows : 0);
    BGX_HIP(hipGetLastError());
  }
  return 0;
}

int row_sumsq_impl(const void* store, int64_t n_rows, int64_t D, int64_t stride, int dtype, float* sumsq, void* stream) {
  BGX_REQUIRE(store && sumsq, BGX_E_ARG, "row_sumsq: null store/sumsq");
  BGX_REQUIRE(n_rows > 0 && D > 0 && stride >= D, BGX_E_ARG, "row_sumsq: n_rows=%lld D=%lld stride=%lld",
              (long long)n_rows, (long long)D, (long long)stride);
  BGX_REQUIRE(dtype >= BGX_F32 && dtype <= BGX_BF16, BGX_E_DTYPE, "row_sumsq: dtype=%d", dtype);
  BGX_REQUIRE((n_rows + 31) / 32 <= 0x7fffffffLL, BGX_E_SHAPE, "row_sumsq: too many rows");
  const int epl = dtype == BGX_F32 ? 4 : 8;
  const bool aligned = ((uintptr_t)store % 16 == 0) && (D % epl == 0) && (stride % epl == 0);
  const dim3 grid((unsigned)((n_rows + 31) / 32)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define BGX_ROW_SUMSQ(T_)                                                                                        \
  if (aligned)                                                                                                   \
    hipLaunchKernelGGL((row_sumsq_kernel<T_, true>), grid, block, 0, st, (const T_*)store, n_rows, D, stride, sumsq); \
  else                                                                                                           \
    hipLaunchKernelGGL((row_sumsq_kernel<T_, false>), grid, block, 0, st, (const T_*)store, n_rows, D, stride, sumsq);
  if (dtype == BGX_F16) {
    BGX_ROW_SUMSQ(f16_t)
  } else if (dtype == BGX_BF16) {
    BGX_ROW_SUMSQ(bf16_t)
  } else {
    BGX_ROW_SUMSQ(float)
  }
#undef BGX_ROW_SUMSQ
  BGX_HIP(hipGetLastError());
  return 0;
}

}  // namespace bgx
