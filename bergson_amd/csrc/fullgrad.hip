// Weight-shaped (unprojected) gradients: projection_dim 0 / None, and the input of the global projection.
//
// Reference: bergson/collector/collector.py:609-644 (Adam), :646-700 (Adafactor), :701-742 (no
// normaliser) with p = None; bergson/gradients.py:300-349, :380-400 (normalisers).
//
// Per sequence the gradient is g^T a [O, I] (the reference's `g.mT @ a`): wgrad_seq_kernel runs that GEMM
// over the tokens and everything after it -- normalisation, the bias column, clamp to the store dtype's
// range, cast, and the scatter into the rows of the store.  fullgrad_seq_kernel is the second half alone,
// for a caller that has formed the product with a GEMM of its own.
// Per token the gradient is the outer product g_t (x) a_t; fullgrad_tok_kernel forms it, normalises it
// and writes it straight to the token's row.  Both are bound by the bytes they write.

#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "mma32.hpp"

namespace bgx {

// sum[n, o] = sum_s g[n, s, o]   (the un-normalised bias gradient of a sequence)
__global__ __launch_bounds__(256) void token_sum_kernel(const void* __restrict__ g, int64_t seq_stride,
                                                        int64_t tok_stride, int S, int O, int dtype,
                                                        float* __restrict__ sum) {
  const int n = blockIdx.y;
  const int o = blockIdx.x * blockDim.x + threadIdx.x;
  if (o >= O) return;
  const int64_t base = (int64_t)n * seq_stride + o;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  int s = 0;
  for (; s + 4 <= S; s += 4) {
    s0 += load_as(g, base + (int64_t)(s + 0) * tok_stride, dtype);
    s1 += load_as(g, base + (int64_t)(s + 1) * tok_stride, dtype);
    s2 += load_as(g, base + (int64_t)(s + 2) * tok_stride, dtype);
    s3 += load_as(g, base + (int64_t)(s + 3) * tok_stride, dtype);
  }
  for (; s < S; ++s) s0 += load_as(g, base + (int64_t)s * tok_stride, dtype);
  sum[(int64_t)n * O + o] = (s0 + s1) + (s2 + s3);
}

struct FullArgs {
  int O, I, Iw;  // Iw = I + 1 when the bias column is written
  int dtype;
  const float* row_scale;   // [O] or NULL   Adafactor row factor (already sqrt(mean) * rsqrt)
  const float* col_scale;   // [I] or NULL   Adafactor column factor
  const float* adam_v;      // [O, I] or NULL  Adam second moments of the weight
  const float* bias_scale;  // [O] or NULL   factor of the bias gradient (NULL = 1)
  void* out;
  int64_t out_row_stride, out_col;
  int out_dtype;
  float lo, hi;
};

__device__ inline float normalise_weight(const FullArgs& a, float v, int o, int i) {
  if (a.adam_v != nullptr) return v / (sqrtf(a.adam_v[(int64_t)o * a.I + i]) + 1e-8f);
  if (a.row_scale != nullptr) v *= a.row_scale[o];
  if (a.col_scale != nullptr) v *= a.col_scale[i];
  return v;
}

// out[row(n), out_col + o * Iw + i] = clamp(normalise(P[n, o, i]));  column I = bias_sum[n, o] * bias_scale[o]
__global__ __launch_bounds__(256) void fullgrad_seq_kernel(FullArgs a, const void* __restrict__ P,
                                                           const float* __restrict__ bias_sum,
                                                           const int64_t* __restrict__ out_rows) {
  const int n = blockIdx.y;
  const int64_t row = out_rows ? out_rows[n] : (int64_t)n;
  const int64_t dst0 = row * a.out_row_stride + a.out_col;
  const int64_t per_seq = (int64_t)a.O * a.Iw;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < per_seq; e += (int64_t)gridDim.x * blockDim.x) {
    const int o = (int)(e / a.Iw);
    const int i = (int)(e - (int64_t)o * a.Iw);
    float v;
    if (i < a.I) {
      v = normalise_weight(a, load_as(P, ((int64_t)n * a.O + o) * a.I + i, a.dtype), o, i);
    } else {
      v = bias_sum[(int64_t)n * a.O + o];
      if (a.bias_scale != nullptr) v *= a.bias_scale[o];
    }
    // the reference holds the normalised gradient in the model dtype before it clamps and casts
    v = round_to_dtype(v, a.dtype);
    store_as(a.out, dst0 + e, clampf(v, a.lo, a.hi), a.out_dtype);
  }
}

// one workgroup per (token, slab of output features): out[row(t), out_col + o * Iw + i] = g[o] * a[i], normalised
constexpr int TOK_SLAB = 8;  // output features per workgroup step
__global__ __launch_bounds__(256) void fullgrad_tok_kernel(FullArgs a, const void* __restrict__ act,
                                                           const void* __restrict__ g, int64_t a_seq_stride,
                                                           int64_t a_tok_stride, int64_t g_seq_stride,
                                                           int64_t g_tok_stride, int S,
                                                           const int32_t* __restrict__ lengths,
                                                           const int64_t* __restrict__ row_offsets) {
  const int n = blockIdx.y;
  const int s = blockIdx.x;
  if (s >= lengths[n] - 1) return;
  const int64_t dst0 = (row_offsets[n] + s) * a.out_row_stride + a.out_col;
  const int64_t abase = (int64_t)n * a_seq_stride + (int64_t)s * a_tok_stride;
  const int64_t gbase = (int64_t)n * g_seq_stride + (int64_t)s * g_tok_stride;
  for (int o0 = blockIdx.z * TOK_SLAB; o0 < a.O; o0 += gridDim.z * TOK_SLAB) {
    const int on = min(TOK_SLAB, a.O - o0);
    for (int e = threadIdx.x; e < on * a.Iw; e += blockDim.x) {
      const int oo = e / a.Iw;
      const int i = e - oo * a.Iw;
      const int o = o0 + oo;
      const float gv = load_as(g, gbase + o, a.dtype);
      float v;
      if (i < a.I) {
        // product formed in the model dtype as in the reference (g.unsqueeze(-1) * a.unsqueeze(-2))
        if (a.adam_v != nullptr) {
          v = round_to_dtype(gv * load_as(act, abase + i, a.dtype), a.dtype);
          v = v / (sqrtf(a.adam_v[(int64_t)o * a.I + i]) + 1e-8f);
        } else {
          float gs = gv, as = load_as(act, abase + i, a.dtype);
          if (a.row_scale != nullptr) gs = round_to_dtype(gs * a.row_scale[o], a.dtype);
          if (a.col_scale != nullptr) as = round_to_dtype(as * a.col_scale[i], a.dtype);
          v = gs * as;
        }
      } else {
        v = gv;
        if (a.bias_scale != nullptr) v *= a.bias_scale[o];
      }
      v = round_to_dtype(v, a.dtype);
      store_as(a.out, dst0 + (int64_t)o * a.Iw + i, clampf(v, a.lo, a.hi), a.out_dtype);
    }
  }
}

// ---- per-sequence gradient with the GEMM over tokens fused ---------------------------------------------------
// out[row(n), out_col + o * Iw + i] = clamp(normalise(sum_s g[n, s, o] * a[n, s, i])) in one kernel: the
// reference's `g.mT @ a` (collector.py:623, :684, :735) and everything after it.  Both operands are stored token
// by token, i.e. with the contraction index as the slow one, which is the wrong way round for the MFMA operands (a
// lane wants 8 consecutive tokens of one feature).  Tiles of BK tokens x 64 features go to LDS as they are; for
// 16-bit types the fragments come out of LDS through the transposing read ds_read_b64_tr_b16: within each group of
// 16 lanes, lane 4 q + c receives, as element e, element c of what lane q + 4 e of the group read.  A lane that
// reads 4 consecutive features at (token k0 + s / 4, feature m0 + 4 (s % 4)), s = its place in the group, therefore
// ends up with 4 consecutive tokens of feature m0 + s; two such reads are a K = 8 half of a 32 x 32 x 16 operand.
// fp32 operands use the 32 x 32 x 2 MFMA, whose operands are one value per lane and need no transposition.
// A workgroup of four waves (2 x 2 blocks of 32 x 32) owns 64 x 64 of one sequence's [O, I] -- small tiles, so that
// the few-sequence batches of small modules still spread over the chip and several workgroups share a CU; the K
// loop runs over the sequence's tokens (those below lengths[n] - 1 when lengths are given), two LDS stages, global
// loads of the next stage in flight during the MFMAs.  The results leave through LDS so that a lane stores 8
// consecutive values.  Rounding points are those of the two-step path: the sum is rounded to the model dtype (the
// GEMM's output), normalised, rounded again, clamped, cast.
struct WgradIn {
  const void* act;
  const void* g;
  int64_t a_seq_stride, a_tok_stride, g_seq_stride, g_tok_stride;
  int S;
  const int32_t* lengths;   // NULL: all S tokens
  const int64_t* out_rows;  // NULL: row n
  int aligned;              // whole 16-byte pieces of both operands can be loaded at once
  int tiles_i;
};

// The projected variant (PROJECT): the tile does not leave as weight-shaped values.  Its normalised values, rounded
// to the model dtype as the reference's are (collector.py:623-634), are projected from both sides inside the
// workgroup -- Z = L[:, tile's output features] Q_tile R[:, tile's input features]^T, three small MFMA products through
// LDS -- and the p x p result goes to partial[sequence][tile]; wgrad_project_sum_kernel adds a sequence's tiles in a
// fixed order, clamps, casts and writes the row.  Nothing of size [N, O, I] is written or read back.
struct WgradProject {
  const void* left;    // [p, O]   model dtype
  const void* right;   // [p, right_stride]: columns 0 .. I - 1
  const float* bias_col;  // [p] or NULL: the right projection's column for the bias gradient
  int64_t right_stride;
  int p;
  int left_whole, right_whole;  // rows of left / right can be loaded in whole 16-byte pieces
  float* partial;      // [N][tiles][p * p]
};

constexpr int WG_OUT_PITCH_PAD = 4;  // floats added to a row of the staged result tile

// TB: 32 x 32 blocks per wave and side -- the tile is 64 TB square on 2 x 2 waves.
template <typename T, int TB>
struct WgradTile {
  static constexpr bool F32 = sizeof(T) == 4;
  static constexpr int BT = 64 * TB;                     // tile edge
  static constexpr int BK = F32 ? 32 : 64;               // tokens per stage
  static constexpr int VEC = 16 / (int)sizeof(T);        // elements per 16-byte piece
  static constexpr int PITCH = BT * (int)sizeof(T);      // bytes per token row of a tile
  static constexpr int OPERAND = BK * PITCH;             // 8 KB (TB = 1), 16 KB (TB = 2)
  static constexpr int STAGE = 2 * OPERAND;              // g tile, then a tile
  static constexpr int NCH = BK * (BT / VEC) / 256;      // 16-byte pieces per thread, operand and stage
  static constexpr int OUT_PITCH = BT + WG_OUT_PITCH_PAD;
  // byte offset of element (token k, feature c) inside an operand tile.  16-bit: a transposing read of half a
  // wave touches 64 bytes of each of four consecutive token rows, which must fall into different banks: with
  // 128-byte rows (TB = 1) consecutive rows are half the banks apart already and the two 64-byte halves of a row
  // swap on every second pair of rows; with 256-byte rows (TB = 2) every row starts at bank 0 and the four 64-byte
  // units of row k are permuted by k mod 4.  fp32: odd token rows are shifted by half the banks, for the two rows a
  // K = 2 operand reads.
  __device__ static int off(int k, int c) {
    if constexpr (F32) {
      return k * PITCH + ((c ^ ((k & 1) << 5)) << 2);
    } else {
      const int b = c * 2;
      const int perm = TB == 1 ? ((k >> 1) & 1) : (k & 3);
      return k * PITCH + (((b >> 6) ^ perm) << 6) + (b & 63);
    }
  }
};

typedef short s16x4 __attribute__((__vector_size__(4 * sizeof(short))));

__device__ inline uint2 lds_read_tr16(const unsigned char* p) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(uintptr_t)(uint32_t)(uintptr_t)p);
  return __builtin_bit_cast(uint2, v);
}

// Two tile sizes.  A 64 x 64 tile (one 32 x 32 block per wave) asks the L2s for 16 KB per 0.52 MFLOP, and on
// Pythia-sized modules that is what bounds it (~300 TFLOP/s at ~10 TB/s from the L2s); 128 x 128 (2 x 2 blocks per
// wave) asks for half as much per flop and half as much of LDS per MFMA.  The small tile keeps the few-sequence
// batches of small modules spread over the chip.
// WHOLE: both operands can be loaded in whole 16-byte pieces (aligned rows, widths of whole pieces).  The loads are
// then unconditional -- a piece past the end of the sequence or of the row is fetched from a clamped address and
// zeroed afterwards -- so that the compiler sees straight-line code and lets the two register sets' loads stay in
// flight past each other (around conditional loads it waits for all of them).
template <typename T, int TB, bool PROJECT, bool WHOLE>
__global__ __launch_bounds__(256, 2) void wgrad_seq_kernel(FullArgs a, WgradIn in, WgradProject pj) {
  using L = WgradTile<T, TB>;
  constexpr int BT = L::BT, BK = L::BK, VEC = L::VEC, NCH = L::NCH, OUT_PITCH = L::OUT_PITCH;
  constexpr int CPR = BT / VEC;  // 16-byte pieces per tile row
  constexpr int WT = 32 * TB;    // rows / columns of a wave's part of the tile
  // the result leaves through LDS 64 rows at a time (block row i of the two wave rows), the bias partial sums behind
  static_assert(2 * L::STAGE >= (64 * OUT_PITCH + 256) * 4, "the staged result rows reuse the operand stages");
  __shared__ __align__(16) unsigned char smem[2 * L::STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int fr = lane & 31, fh = lane >> 5;
  const int n = blockIdx.y;
  const int o0 = (blockIdx.x / in.tiles_i) * BT, i0 = (blockIdx.x % in.tiles_i) * BT;
  int Sn = in.S;
  if (in.lengths != nullptr) Sn = max(0, min(in.S, in.lengths[n] - 1));
  const int KT = (Sn + BK - 1) / BK;
  const bool with_bias = a.Iw > a.I && i0 == 0;

  const T* gp = (const T*)in.g + (int64_t)n * in.g_seq_stride;
  const T* ap = (const T*)in.act + (int64_t)n * in.a_seq_stride;

  // ---- loader: piece c of a stage is 16 bytes of token row c / CPR
  // two register sets: a stage is asked for three iterations before it is computed on and written to LDS two
  // iterations later, so that its loads have two iterations' time to arrive
  uint4 gv[2][NCH], av[2][NCH];
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  // what does not change from stage to stage is worked out once per thread: piece j is token row p_row[j] of a
  // stage, its columns start at p_gcol[j] / p_acol[j] (clamped into the row for the unconditional loads of WHOLE)
  int p_row[NCH], p_gcol[NCH], p_acol[NCH], p_lds[NCH];
  bool p_gok[NCH], p_aok[NCH];
#pragma unroll
  for (int j = 0; j < NCH; ++j) {
    const int c = tid + 256 * j;
    p_row[j] = c / CPR;
    const int col = (c % CPR) * VEC;
    p_gok[j] = o0 + col < a.O;
    p_aok[j] = i0 + col < a.I;
    p_gcol[j] = WHOLE ? min(o0 + col, a.O - VEC) : o0 + col;
    p_acol[j] = WHOLE ? min(i0 + col, a.I - VEC) : i0 + col;
    p_lds[j] = L::off(c / CPR, col);
  }
  auto fetch = [&](const T* base, int64_t tok_stride, int width, int col, bool col_ok, int s) -> uint4 {
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if constexpr (WHOLE) {
      // (what lies outside is zeroed when the piece is written to LDS, not here: touching the value now would
      // mean waiting for it now)
      v = load16_global(base + (int64_t)min(s, Sn - 1) * tok_stride + col);
    } else if (s < Sn && col_ok) {
      const T* src = base + (int64_t)s * tok_stride + col;
      if (in.aligned && col + VEC <= width) {
        v = load16_global(src);
      } else {
        struct {
          T e[VEC];
        } tmp;
#pragma unroll
        for (int e = 0; e < VEC; ++e) tmp.e[e] = col + e < width ? src[e] : T{};
        v = __builtin_bit_cast(uint4, tmp);
      }
    }
    return v;
  };
  int set_kt[2] = {0, 0};  // the stage each register set holds
  auto load_stage = [&](int kt, auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
    set_kt[SET] = kt;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int sj = kt * BK + p_row[j];
      gv[SET][j] = fetch(gp, in.g_tok_stride, a.O, p_gcol[j], p_gok[j], sj);
      av[SET][j] = fetch(ap, in.a_tok_stride, a.I, p_acol[j], p_aok[j], sj);
    }
  };
  auto store_stage = [&](int st, auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
    unsigned char* base = smem + st * L::STAGE;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      uint4 gw = gv[SET][j], aw = av[SET][j];
      if constexpr (WHOLE) {
        const bool row_ok = set_kt[SET] * BK + p_row[j] < Sn;
        const bool g_ok = row_ok && p_gok[j], a_ok = row_ok && p_aok[j];
        gw = make_uint4(g_ok ? gw.x : 0u, g_ok ? gw.y : 0u, g_ok ? gw.z : 0u, g_ok ? gw.w : 0u);
        aw = make_uint4(a_ok ? aw.x : 0u, a_ok ? aw.y : 0u, a_ok ? aw.z : 0u, a_ok ? aw.w : 0u);
      }
      *reinterpret_cast<uint4*>(base + p_lds[j]) = gw;
      *reinterpret_cast<uint4*>(base + L::OPERAND + p_lds[j]) = aw;
    }
  };

  f32x16 acc[TB][TB];
#pragma unroll
  for (int i = 0; i < TB; ++i)
#pragma unroll
    for (int j = 0; j < TB; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  float bias_part = 0.f;
  constexpr int PARTS = 256 / BT;  // threads per output feature for the bias sum
  const int b_col = tid % BT, b_part = tid / BT;

  // place of this lane's transposing reads: token (lane % 16) / 4 of its K = 4 group, features 4 (lane % 4) .. + 3 of
  // the 16 its group of lanes covers
  const int rk = 8 * fh + ((lane & 15) >> 2);
  const int rc = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  int g_rd[TB], a_rd[TB];
#pragma unroll
  for (int i = 0; i < TB; ++i) {
    g_rd[i] = L::off(rk, wm * WT + i * 32 + rc);
    a_rd[i] = L::off(rk, wn * WT + i * 32 + rc);
  }
  auto compute = [&](int st) {
    const unsigned char* gt = smem + st * L::STAGE;
    const unsigned char* at = gt + L::OPERAND;
    if constexpr (L::F32) {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        float gf[TB], af[TB];
#pragma unroll
        for (int i = 0; i < TB; ++i) gf[i] = *reinterpret_cast<const float*>(gt + L::off(kk + fh, wm * WT + i * 32 + fr));
#pragma unroll
        for (int j = 0; j < TB; ++j) af[j] = *reinterpret_cast<const float*>(at + L::off(kk + fh, wn * WT + j * 32 + fr));
#pragma unroll
        for (int i = 0; i < TB; ++i)
#pragma unroll
          for (int j = 0; j < TB; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(gf[i], af[j], acc[i][j], 0, 0, 0);
      }
    } else {
      // (token rows ks + rk and ks + rk + 4 of a k-step permute their 64-byte units like row rk does, whatever ks:
      // a read's address is the lane's address in row rk plus a constant)
#pragma unroll
      for (int ks = 0; ks < BK; ks += 16) {
        uint4 gf[TB], af[TB];
#pragma unroll
        for (int i = 0; i < TB; ++i) {
          const uint2 g0 = lds_read_tr16(gt + g_rd[i] + ks * L::PITCH);
          const uint2 g1 = lds_read_tr16(gt + g_rd[i] + (ks + 4) * L::PITCH);
          gf[i] = make_uint4(g0.x, g0.y, g1.x, g1.y);
        }
#pragma unroll
        for (int j = 0; j < TB; ++j) {
          const uint2 a0 = lds_read_tr16(at + a_rd[j] + ks * L::PITCH);
          const uint2 a1 = lds_read_tr16(at + a_rd[j] + (ks + 4) * L::PITCH);
          af[j] = make_uint4(a0.x, a0.y, a1.x, a1.y);
        }
#pragma unroll
        for (int i = 0; i < TB; ++i)
#pragma unroll
          for (int j = 0; j < TB; ++j) Mma32<T>::mma(gf[i], af[j], acc[i][j]);
      }
    }
    if (with_bias) {
      for (int k = b_part; k < BK; k += PARTS)
        bias_part += Elem<T>::load(reinterpret_cast<const T*>(gt + L::off(k, b_col)));
    }
  };

  if (KT > 0) {
    load_stage(0, Set0{});
    store_stage(0, Set0{});
  }
  if (WHOLE ? KT > 0 : KT > 1) load_stage(1, Set0{});
  if (WHOLE ? KT > 0 : KT > 2) load_stage(2, Set1{});
  // (projected variant) this lane's fragments of L and R for the tile's k-steps: asked for now, used behind the K
  // loop
  constexpr int KSTEPS = BT / 16;
  uint4 lf[PROJECT ? KSTEPS : 1], rf[PROJECT ? KSTEPS : 1];
  if constexpr (PROJECT) {
    const T* left = (const T*)pj.left;
    const T* right = (const T*)pj.right;
#pragma unroll
    for (int q = 0; q < KSTEPS; ++q) {
      lf[q] = pj.left_whole ? load_chunk<T, true>(left, fr, pj.p, a.O, o0 + q * 16 + 8 * fh, a.O)
                            : load_chunk<T, false>(left, fr, pj.p, a.O, o0 + q * 16 + 8 * fh, a.O);
      rf[q] = pj.right_whole ? load_chunk<T, true>(right, fr, pj.p, pj.right_stride, i0 + q * 16 + 8 * fh, a.I)
                             : load_chunk<T, false>(right, fr, pj.p, pj.right_stride, i0 + q * 16 + 8 * fh, a.I);
    }
  }
  __syncthreads();
  // iteration kt: stage kt + 1 (asked for two iterations ago) goes to the LDS stage that iteration kt - 1 read, its
  // register set takes stage kt + 3, then the MFMAs of stage kt
  if constexpr (WHOLE) {
    // no branch inside: a stage past the end of the sequence is fetched from its last row and written as zeros (so
    // that an odd number of stages runs as the next even one), and the compiler can count the loads in flight
    for (int kt = 0; kt < KT; kt += 2) {
      store_stage(1, Set0{});
      load_stage(kt + 3, Set0{});
      compute(0);
      __syncthreads();
      store_stage(0, Set1{});
      load_stage(kt + 4, Set1{});
      compute(1);
      __syncthreads();
    }
  } else {
    for (int kt = 0; kt < KT; kt += 2) {
      if (kt + 1 < KT) store_stage(1, Set0{});
      if (kt + 3 < KT) load_stage(kt + 3, Set0{});
      compute(0);
      __syncthreads();
      if (kt + 1 < KT) {
        if (kt + 2 < KT) store_stage(0, Set1{});
        if (kt + 4 < KT) load_stage(kt + 4, Set1{});
        compute(1);
        __syncthreads();
      }
    }
  }

  if constexpr (PROJECT) {
    static_assert(!L::F32, "the projected epilogue multiplies on the 16-bit matrix instructions");
    // LDS: the normalised tile, transposed -- Qt[i][o], rows of BT output features: a lane of the K loop's
    // accumulators holds one input feature and runs of four consecutive output features, which are one 8-byte write
    // each this way round, and the first product's operand (32 input features x 16 output features per k-step) is a
    // plain 16-byte read; behind it the bias partial sums, the bias values, L b, and the two halves of W[j'][i]
    constexpr int Q_PITCH = BT * 2 + 16;  // bytes per row: BT values and 16 bytes against bank conflicts
    constexpr int QT_BYTES = BT * Q_PITCH;
    unsigned char* qt = smem;
    float* red = reinterpret_cast<float*>(smem + QT_BYTES);  // [PARTS][BT]
    float* bvec = red + 256;                                  // [BT]
    float* wb = bvec + BT;                                    // [32]
    unsigned char* w_hi = reinterpret_cast<unsigned char*>(wb + 32);
    unsigned char* w_lo = w_hi + 32 * Q_PITCH;
    static_assert(QT_BYTES + (256 + BT + 32) * 4 + 2 * 32 * Q_PITCH <= 2 * L::STAGE, "projected epilogue in LDS");
    auto pack2 = [](float x, float y) -> uint32_t {
      return std::is_same<T, bf16_t>::value ? f32x2_to_bf16x2_bits(x, y) : f32x2_to_f16x2_bits(x, y);
    };
    auto unpack_lo = [](uint32_t w) -> float {
      return std::is_same<T, bf16_t>::value ? bf16_bits_to_f32(w & 0xffffu) : f16_bits_to_f32(w & 0xffffu);
    };
    auto unpack_hi = [](uint32_t w) -> float {
      return std::is_same<T, bf16_t>::value ? bf16_bits_to_f32(w >> 16) : f16_bits_to_f32(w >> 16);
    };
#pragma unroll
    for (int i = 0; i < TB; ++i)
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        const int il = wn * WT + j * 32 + fr, ii = i0 + il;
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          const int ol = wm * WT + i * 32 + 8 * gq + 4 * fh;  // four consecutive output features from here
          float v[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int o = o0 + ol + c;
            v[c] = 0.f;
            if (o < a.O && ii < a.I)
              v[c] = round_to_dtype(normalise_weight(a, round_to_dtype(acc[i][j][gq * 4 + c], a.dtype), o, ii), a.dtype);
          }
          *reinterpret_cast<uint2*>(qt + il * Q_PITCH + ol * 2) = make_uint2(pack2(v[0], v[1]), pack2(v[2], v[3]));
        }
      }
    if (with_bias) red[b_part * BT + b_col] = bias_part;
    __syncthreads();
    const T* left = (const T*)pj.left;
    if (wave < 2 * TB) {
      // Wt[i, j'] = sum_o Qt[i][o] L[j', o0 + o] for the wave's 32 input features
      f32x16 w;
#pragma unroll
      for (int e = 0; e < 16; ++e) w[e] = 0.f;
      const unsigned char* q_rd = qt + (wave * 32 + fr) * Q_PITCH + 8 * fh * 2;
#pragma unroll
      for (int ks = 0; ks < BT; ks += 16)
        Mma32<T>::mma(*reinterpret_cast<const uint4*>(q_rd + ks * 2), lf[ks / 16], w);
      // W = hi + lo in the model dtype (the second product then sees W to twice the dtype's precision), written as
      // W[j'][i]: this lane is j' = fr and holds runs of four consecutive input features
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const int il = wave * 32 + 8 * gq + 4 * fh;
        const uint32_t h01 = pack2(w[gq * 4 + 0], w[gq * 4 + 1]), h23 = pack2(w[gq * 4 + 2], w[gq * 4 + 3]);
        const uint32_t l01 = pack2(w[gq * 4 + 0] - unpack_lo(h01), w[gq * 4 + 1] - unpack_hi(h01));
        const uint32_t l23 = pack2(w[gq * 4 + 2] - unpack_lo(h23), w[gq * 4 + 3] - unpack_hi(h23));
        *reinterpret_cast<uint2*>(w_hi + fr * Q_PITCH + il * 2) = make_uint2(h01, h23);
        *reinterpret_cast<uint2*>(w_lo + fr * Q_PITCH + il * 2) = make_uint2(l01, l23);
      }
    }
    if (with_bias && tid < BT) {
      // the tile's bias gradients: summed over the tokens, scaled, rounded to the model dtype
      float t = 0.f;
#pragma unroll
      for (int q = 0; q < PARTS; ++q) t += red[q * BT + tid];
      const int o = o0 + tid;
      if (a.bias_scale != nullptr && o < a.O) t *= a.bias_scale[o];
      bvec[tid] = o < a.O ? round_to_dtype(t, a.dtype) : 0.f;
    }
    __syncthreads();
    f32x16 z;
#pragma unroll
    for (int e = 0; e < 16; ++e) z[e] = 0.f;
    if (wave == 0) {
      // Z[j', j] = sum_i W[j', i] R[j, i0 + i]
#pragma unroll
      for (int ks = 0; ks < BT; ks += 16) {
        const uint4 hi4 = *reinterpret_cast<const uint4*>(w_hi + fr * Q_PITCH + (ks + 8 * fh) * 2);
        const uint4 lo4 = *reinterpret_cast<const uint4*>(w_lo + fr * Q_PITCH + (ks + 8 * fh) * 2);
        Mma32<T>::mma(hi4, rf[ks / 16], z);
        Mma32<T>::mma(lo4, rf[ks / 16], z);
      }
    } else if (with_bias && wave == 1 && lane < 32) {
      // (L b)[j'] over the tile's output features
      float t = 0.f;
      if (lane < pj.p)
        for (int o = 0; o < BT && o0 + o < a.O; ++o) t += Elem<T>::load(left + (int64_t)lane * a.O + o0 + o) * bvec[o];
      wb[lane] = t;
    }
    if (with_bias) __syncthreads();
    if (wave == 0) {
      const int tiles = (int)gridDim.x;
      float* dst = pj.partial + ((int64_t)n * tiles + blockIdx.x) * pj.p * pj.p;
      const int j = fr;
      float rb = 0.f;
      if (with_bias && j < pj.p) rb = pj.bias_col[j];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int jl = 8 * (e >> 2) + 4 * fh + (e & 3);
        if (jl < pj.p && j < pj.p) dst[jl * pj.p + j] = z[e] + (with_bias ? wb[jl] * rb : 0.f);
      }
    }
    return;
  }
  // ---- epilogue: normalise in place, stage 64 rows of the tile in LDS at a time (the operand stages are done
  // with: the loop ends on a barrier) -- block row i of both wave rows -- then every lane stores 8 consecutive
  // values of a row
  const int64_t row = in.out_rows ? in.out_rows[n] : (int64_t)n;
  const int64_t dst0 = row * a.out_row_stride + a.out_col;
  float* tile = reinterpret_cast<float*>(smem);
  float* red = tile + 64 * OUT_PITCH;  // the bias partial sums, behind the staged rows
  if (with_bias) red[b_part * BT + b_col] = bias_part;
  const int es = (int)dtype_size(a.out_dtype);
  // rows of the tile start on 16-byte boundaries of the output when the row pitch and the tile's first element do
  const bool rows_aligned = ((uintptr_t)a.out + (uintptr_t)(dst0 + (int64_t)o0 * a.Iw + i0) * es) % 16 == 0 &&
                            ((int64_t)a.Iw * es) % 16 == 0;
#pragma unroll
  for (int i = 0; i < TB; ++i) {
    if (i > 0) __syncthreads();  // the rows staged before have been stored
    // acc[i][j][e]: output feature o0 + WT wm + 32 i + 8 (e / 4) + 4 fh + e % 4, input feature i0 + WT wn + 32 j + fr
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const int il = wn * WT + j * 32 + fr, ii = i0 + il;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int sl = wm * 32 + 8 * (e >> 2) + 4 * fh + (e & 3);  // staged row
        const int o = o0 + wm * WT + i * 32 + (sl - wm * 32);
        float v = 0.f;
        if (o < a.O && ii < a.I) {
          v = round_to_dtype(acc[i][j][e], a.dtype);
          v = clampf(round_to_dtype(normalise_weight(a, v, o, ii), a.dtype), a.lo, a.hi);
        }
        tile[sl * OUT_PITCH + il] = v;
      }
    }
    __syncthreads();
    constexpr int PIECES = 64 * (BT / 8) / 256;  // 8-value pieces per thread
#pragma unroll
    for (int q = 0; q < PIECES; ++q) {
      const int piece = tid + 256 * q;
      const int sl = piece / (BT / 8), il = (piece % (BT / 8)) * 8;
      const int o = o0 + (sl >> 5) * WT + i * 32 + (sl & 31), ii = i0 + il;
      if (o >= a.O || ii >= a.I) continue;
      float v[8];
      const f32x4 lo4 = *reinterpret_cast<const f32x4*>(tile + sl * OUT_PITCH + il);
      const f32x4 hi4 = *reinterpret_cast<const f32x4*>(tile + sl * OUT_PITCH + il + 4);
      v[0] = lo4[0], v[1] = lo4[1], v[2] = lo4[2], v[3] = lo4[3];
      v[4] = hi4[0], v[5] = hi4[1], v[6] = hi4[2], v[7] = hi4[3];
      const int64_t dst = dst0 + (int64_t)o * a.Iw + ii;
      if (rows_aligned && ii + 8 <= a.I) {
        if (a.out_dtype == BGX_F32)
          store8_as<BGX_F32>(a.out, dst, v);
        else if (a.out_dtype == BGX_F16)
          store8_as<BGX_F16>(a.out, dst, v);
        else
          store8_as<BGX_BF16>(a.out, dst, v);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (ii + e < a.I) store_as(a.out, dst + e, v[e], a.out_dtype);
      }
    }
  }
  if (with_bias && b_part == 0 && o0 + b_col < a.O) {
    float bias_total = 0.f;
#pragma unroll
    for (int q = 0; q < PARTS; ++q) bias_total += red[q * BT + b_col];
    const int o = o0 + b_col;
    if (a.bias_scale != nullptr) bias_total *= a.bias_scale[o];
    bias_total = round_to_dtype(bias_total, a.dtype);
    store_as(a.out, dst0 + (int64_t)o * a.Iw + a.I, clampf(bias_total, a.lo, a.hi), a.out_dtype);
  }
}

// ---- the global projection: acc[m, j] += sum_k rows[m, k] * proj[j, k] ---------------------------------------
// projection_target = "global" (collector.py:364-390): every module's flattened gradient [rows, W] times its
// block [P, W] of the one projection matrix, summed into a [rows, P] fp32 accumulator.  Both operands have few
// rows and a very long contraction (W = O * I: 10^5 .. 10^7), so the work is split along k: a workgroup takes 32
// rows, up to 64 columns of the result and one slab of k; its four waves take every fourth k-step of the slab, so
// that together they read whole 128-byte lines, with fragments loaded straight from global memory (both operands
// have the contraction index as the fast one, which is what the MFMA operands want).  The waves' sums are added in
// a fixed order through LDS and written to partial[slab][m][j]; project_reduce_kernel adds the slabs in order, so
// the result does not depend on which workgroup finishes first.
struct ProjArgs {
  const void* rows;
  const void* proj;
  int64_t M, W, row_stride;
  int P;
  int64_t slab_len;  // elements of k per workgroup, a multiple of four k-steps
  int n_slabs;
  float* partial;    // [n_slabs, M, P]
};

constexpr int PROJ_PB = 2;  // 32-column blocks of the result per workgroup

template <typename T, bool ALIGNED>
__global__ __launch_bounds__(256) void project_rows_kernel(ProjArgs a) {
  using M32 = Mma32<T>;
  constexpr int EPL = M32::EPL, KS = 2 * EPL;
  __shared__ float red[3][PROJ_PB][16][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int fr = lane & 31, fh = lane >> 5;
  const int slab = blockIdx.x;
  const int64_t m0 = (int64_t)blockIdx.y * 32;
  const int j0 = blockIdx.z * (32 * PROJ_PB);
  const int64_t k_begin = (int64_t)slab * a.slab_len;
  const int64_t k_end = min(a.W, k_begin + a.slab_len);

  const T* arow = (const T*)a.rows + min(m0 + fr, a.M - 1) * a.row_stride;
  const T* prow[PROJ_PB];
#pragma unroll
  for (int b = 0; b < PROJ_PB; ++b) prow[b] = (const T*)a.proj + (int64_t)min(j0 + b * 32 + fr, a.P - 1) * a.W;

  auto frag = [&](const T* row, int64_t k) -> uint4 {
    if (ALIGNED) return k < k_end ? load16_global(row + k) : make_uint4(0u, 0u, 0u, 0u);
    struct {
      T e[EPL];
    } tmp;
#pragma unroll
    for (int e = 0; e < EPL; ++e) tmp.e[e] = k + e < k_end ? row[k + e] : T{};
    return __builtin_bit_cast(uint4, tmp);
  };

  f32x16 acc[PROJ_PB];
#pragma unroll
  for (int b = 0; b < PROJ_PB; ++b)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[b][e] = 0.f;
  const bool second = j0 + 32 < a.P;  // the second block of columns exists
  // four k-steps of this wave per round, their loads issued together
  constexpr int UN = 4;
  for (int64_t k = k_begin + wave * KS; k < k_end; k += UN * 4 * KS) {
    uint4 af[UN], b0[UN], b1[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int64_t ka = k + (int64_t)u * 4 * KS + EPL * fh;
      af[u] = frag(arow, ka);
      b0[u] = frag(prow[0], ka);
      b1[u] = second ? frag(prow[1], ka) : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      M32::mma(af[u], b0[u], acc[0]);
      if (second) M32::mma(af[u], b1[u], acc[1]);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int b = 0; b < PROJ_PB; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) red[wave - 1][b][e][lane] = acc[b][e];
  }
  __syncthreads();
  if (wave == 0) {
    // acc[b][e] = row m0 + 8 (e / 4) + 4 fh + e % 4, column j0 + 32 b + fr
#pragma unroll
    for (int b = 0; b < PROJ_PB; ++b) {
      const int j = j0 + b * 32 + fr;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t m = m0 + 8 * (e >> 2) + 4 * fh + (e & 3);
        if (m < a.M && j < a.P)
          a.partial[((int64_t)slab * a.M + m) * a.P + j] =
              ((acc[b][e] + red[0][b][e][lane]) + red[1][b][e][lane]) + red[2][b][e][lane];
      }
    }
  }
}

// acc[m, j] += sum over the slabs, in an order that depends on the shape alone.  Few results: one wave per
// result, lane l adds slabs l, l + 64, ... and the lanes' sums meet in a butterfly; many results: one thread each.
__global__ __launch_bounds__(256) void project_reduce_kernel(const float* __restrict__ partial, int n_slabs, int64_t M,
                                                             int P, float* __restrict__ acc, int64_t acc_stride,
                                                             int by_wave) {
  const int64_t total = M * P;
  if (by_wave) {
    const int64_t e = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (e >= total) return;
    const int lane = threadIdx.x & 63;
    float s = 0.f;
    for (int t = lane; t < n_slabs; t += 64) s += partial[(int64_t)t * total + e];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d);
    if (lane == 0) {
      const int64_t m = e / P;
      acc[m * acc_stride + (e - m * P)] += s;
    }
  } else {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= total) return;
    float s = 0.f;
    for (int t = 0; t < n_slabs; ++t) s += partial[(int64_t)t * total + e];
    const int64_t m = e / P;
    acc[m * acc_stride + (e - m * P)] += s;
  }
}

static bool dtype_ok(int dt) { return dt >= BGX_F32 && dt <= BGX_BF16; }

int token_sum_impl(const void* g, int64_t g_seq_stride, int64_t g_tok_stride, int N, int S, int O, int dtype,
                   float* sum, void* stream) {
  BGX_REQUIRE(g && sum, BGX_E_ARG, "token_sum: null pointer");
  BGX_REQUIRE(N > 0 && S > 0 && O > 0 && N <= 65535, BGX_E_SHAPE, "token_sum: N=%d S=%d O=%d", N, S, O);
  BGX_REQUIRE(dtype_ok(dtype), BGX_E_DTYPE, "token_sum: dtype=%d", dtype);
  hipLaunchKernelGGL(token_sum_kernel, dim3((unsigned)((O + 255) / 256), (unsigned)N), dim3(256), 0,
                     (hipStream_t)stream, g, g_seq_stride, g_tok_stride, S, O, dtype, sum);
  BGX_HIP(hipGetLastError());
  return 0;
}

static int fill_args(FullArgs& fa, const char* what, int O, int I, int dtype, const float* row_scale,
                     const float* col_scale, const float* adam_v, int collect_bias, const float* bias_scale, void* out,
                     int64_t out_row_stride, int64_t out_col, int out_dtype, float lo, float hi) {
  BGX_REQUIRE(out != nullptr, BGX_E_ARG, "%s: null out", what);
  BGX_REQUIRE(O > 0 && I > 0, BGX_E_SHAPE, "%s: O=%d I=%d", what, O, I);
  BGX_REQUIRE(dtype_ok(dtype) && dtype_ok(out_dtype), BGX_E_DTYPE, "%s: dtype=%d out_dtype=%d", what, dtype, out_dtype);
  BGX_REQUIRE(adam_v == nullptr || (row_scale == nullptr && col_scale == nullptr), BGX_E_ARG,
              "%s: Adam moments and Adafactor factors are exclusive", what);
  fa.O = O;
  fa.I = I;
  fa.Iw = I + (collect_bias ? 1 : 0);
  BGX_REQUIRE(out_col >= 0 && out_col + (int64_t)O * fa.Iw <= out_row_stride, BGX_E_ARG,
              "%s: columns [%lld, +%lld) do not fit a row of %lld", what, (long long)out_col,
              (long long)O * fa.Iw, (long long)out_row_stride);
  fa.dtype = dtype;
  fa.row_scale = row_scale;
  fa.col_scale = col_scale;
  fa.adam_v = adam_v;
  fa.bias_scale = bias_scale;
  fa.out = out;
  fa.out_row_stride = out_row_stride;
  fa.out_col = out_col;
  fa.out_dtype = out_dtype;
  fa.lo = lo;
  fa.hi = hi;
  return 0;
}

int fullgrad_seq_impl(const void* P, int N, int O, int I, int dtype, const float* row_scale, const float* col_scale,
                      const float* adam_v, const float* bias_sum, const float* bias_scale, const int64_t* out_rows,
                      void* out, int64_t out_row_stride, int64_t out_col, int out_dtype, float lo, float hi,
                      void* stream) {
  BGX_REQUIRE(P != nullptr, BGX_E_ARG, "fullgrad_seq: null P");
  BGX_REQUIRE(N > 0 && N <= 65535, BGX_E_SHAPE, "fullgrad_seq: N=%d", N);
  FullArgs fa;
  const int rc = fill_args(fa, "fullgrad_seq", O, I, dtype, row_scale, col_scale, adam_v, bias_sum != nullptr,
                           bias_scale, out, out_row_stride, out_col, out_dtype, lo, hi);
  if (rc != 0) return rc;
  const int64_t per_seq = (int64_t)O * fa.Iw;
  const unsigned gx = (unsigned)std::min<int64_t>((per_seq + 1023) / 1024, 4096);
  hipLaunchKernelGGL(fullgrad_seq_kernel, dim3(gx, (unsigned)N), dim3(256), 0, (hipStream_t)stream, fa, P, bias_sum,
                     out_rows);
  BGX_HIP(hipGetLastError());
  return 0;
}

// Tile edge of a launch: 128 for long sequences of modules with enough tiles of that size for two rounds of the chip
// (two workgroups to a CU).  With fewer the last, partly filled round costs more than the larger tile saves, and
// with short sequences its longer epilogue does: by the tracer, 4 x 1024 tokens of a 1024 x 4096 module (1024 large
// tiles) take 110 us against 123 us on the small tiles, of a 768 x 3072 module (576 large tiles, 1.1 rounds) 88 us
// against 73.
static int wgrad_tile_edge(int O, int I, int N, int S) {
  const int64_t big = (int64_t)((O + 127) / 128) * ((I + 127) / 128);
  return O >= 128 && I >= 128 && S >= 512 && big * N >= 1024 && !switches().wgrad_big_off ? 128 : 64;
}

template <typename T, bool PROJECT>
static int64_t launch_wgrad(const FullArgs& fa, WgradIn in, const WgradProject& pj, int N, hipStream_t st) {
  const int bt = wgrad_tile_edge(fa.O, fa.I, N, in.S);
  in.tiles_i = (fa.I + bt - 1) / bt;
  const int64_t tiles = (int64_t)((fa.O + bt - 1) / bt) * in.tiles_i;
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool whole = in.aligned && fa.O % VEC == 0 && fa.I % VEC == 0;
  const dim3 grid((unsigned)tiles, (unsigned)N), block(256);
  if (bt == 128 && whole)
    hipLaunchKernelGGL((wgrad_seq_kernel<T, 2, PROJECT, true>), grid, block, 0, st, fa, in, pj);
  else if (bt == 128)
    hipLaunchKernelGGL((wgrad_seq_kernel<T, 2, PROJECT, false>), grid, block, 0, st, fa, in, pj);
  else if (whole)
    hipLaunchKernelGGL((wgrad_seq_kernel<T, 1, PROJECT, true>), grid, block, 0, st, fa, in, pj);
  else
    hipLaunchKernelGGL((wgrad_seq_kernel<T, 1, PROJECT, false>), grid, block, 0, st, fa, in, pj);
  note_kernel(FAMILY_FULLGRAD, PROJECT ? (bt == 128 ? "wgrad_seq_projected_128" : "wgrad_seq_projected_64")
                                       : (bt == 128 ? "wgrad_seq_128" : "wgrad_seq_64"));
  return tiles;
}

// Adds a sequence's tiles in two steps, each in an order that depends on the shape alone.  A workgroup takes 64
// values e and one group of consecutive tiles; four threads per value each add every fourth tile of the group and
// meet in LDS.  Step 1 (groups > 1): sums[n][group][e] = sum of the group's tiles of partial[n].  Step 2 (one group):
// out[row(n), out_col + e] = clamp(sum), cast.
constexpr int WG_SUM_GROUP = 16;  // tiles per group in step 1
__global__ __launch_bounds__(256) void wgrad_project_sum_kernel(const float* __restrict__ src, int tiles, int pp,
                                                                int per_group, float* __restrict__ sums,
                                                                const int64_t* __restrict__ out_rows, void* out,
                                                                int64_t out_row_stride, int64_t out_col, int out_dtype,
                                                                float lo, float hi) {
  __shared__ float red[4][64];
  const int n = blockIdx.y, grp = blockIdx.z, groups = gridDim.z;
  const int el = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int e = blockIdx.x * 64 + el;
  const int t0 = grp * per_group, t1 = min(tiles, t0 + per_group);
  float s = 0.f;
  if (e < pp) {
    const float* base = src + (int64_t)n * tiles * pp + e;
    for (int t = t0 + q; t < t1; t += 4) s += base[(int64_t)t * pp];
  }
  red[q][el] = s;
  __syncthreads();
  if (q != 0 || e >= pp) return;
  const float total = (red[0][el] + red[1][el]) + (red[2][el] + red[3][el]);
  if (sums != nullptr) {
    sums[((int64_t)n * groups + grp) * pp + e] = total;
  } else {
    const int64_t row = out_rows ? out_rows[n] : (int64_t)n;
    store_as(out, row * out_row_stride + out_col + e, clampf(total, lo, hi), out_dtype);
  }
}

static int64_t wgrad_sum_groups(int64_t tiles) { return (tiles + WG_SUM_GROUP - 1) / WG_SUM_GROUP; }

size_t collect_seq_weight_workspace_bytes(int N, int I, int O, int p) {
  if (N <= 0 || I <= 0 || O <= 0 || p <= 0) return 0;
  // (sized for 64 x 64 tiles; a launch on 128 x 128 tiles uses a quarter)
  const size_t tiles = (size_t)((O + 63) / 64) * (size_t)((I + 63) / 64);
  // the tiles' contributions, and behind them the sums of groups of tiles
  return ((size_t)N * (tiles + (size_t)wgrad_sum_groups((int64_t)tiles)) * (size_t)p * p * 4 + 255) / 256 * 256;
}

// Per-sequence rows of a module whose normaliser acts on the weight-shaped gradient (Adam's second moments, or
// Adafactor's factors): out[row(n), out_col : + p * p] = clamp(L normalise(g[n]^T a[n] [| bias]) R^T)
// (collector.py:609-644 with a projection, per sequence).  16-bit models, p <= 32.
int collect_seq_weight_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride,
                            int64_t g_seq_stride, int64_t g_tok_stride, int N, int S, int I, int O, int p, int dtype,
                            const float* row_scale, const float* col_scale, const float* adam_v, const void* left,
                            const void* right, int64_t right_stride, const float* bias_col, const float* bias_scale,
                            const int32_t* lengths, const int64_t* out_rows, void* out, int64_t out_row_stride,
                            int64_t out_col, int out_dtype, float lo, float hi, void* ws, size_t ws_bytes,
                            void* stream) {
  const int collect_bias = bias_col != nullptr;
  BGX_REQUIRE(a && g && left && right && out, BGX_E_ARG, "collect_seq_weight: null pointer");
  BGX_REQUIRE(N > 0 && S > 0 && N <= 65535 && I > 0 && O > 0, BGX_E_SHAPE, "collect_seq_weight: N=%d S=%d I=%d O=%d", N,
              S, I, O);
  BGX_REQUIRE(p >= 1 && p <= 32, BGX_E_SHAPE, "collect_seq_weight: p=%d outside 1..32", p);
  BGX_REQUIRE(dtype == BGX_F16 || dtype == BGX_BF16, BGX_E_DTYPE, "collect_seq_weight: dtype=%d (16-bit models only)",
              dtype);
  BGX_REQUIRE(dtype_ok(out_dtype), BGX_E_DTYPE, "collect_seq_weight: out_dtype=%d", out_dtype);
  BGX_REQUIRE(a_tok_stride >= I && g_tok_stride >= O && a_seq_stride >= 0 && g_seq_stride >= 0 &&
                  right_stride >= I,
              BGX_E_ARG, "collect_seq_weight: strides a (%lld, %lld) g (%lld, %lld) right %lld", (long long)a_seq_stride,
              (long long)a_tok_stride, (long long)g_seq_stride, (long long)g_tok_stride, (long long)right_stride);
  BGX_REQUIRE(adam_v == nullptr || (row_scale == nullptr && col_scale == nullptr), BGX_E_ARG,
              "collect_seq_weight: Adam moments and Adafactor factors are exclusive");
  BGX_REQUIRE(out_col >= 0 && out_col + (int64_t)p * p <= out_row_stride, BGX_E_ARG,
              "collect_seq_weight: columns [%lld, +%d) do not fit a row of %lld", (long long)out_col, p * p,
              (long long)out_row_stride);
  const size_t need = collect_seq_weight_workspace_bytes(N, I, O, p);
  BGX_REQUIRE(ws != nullptr && ((uintptr_t)ws & 255) == 0 && ws_bytes >= need, BGX_E_WORKSPACE,
              "collect_seq_weight: workspace %zu < %zu bytes (or not 256-byte aligned)", ws_bytes, need);
  BGX_REQUIRE((int64_t)((O + 63) / 64) * ((I + 63) / 64) <= 0x7fffffff, BGX_E_SHAPE, "collect_seq_weight: O=%d I=%d", O,
              I);
  FullArgs fa;
  fa.O = O;
  fa.I = I;
  fa.Iw = I + (collect_bias ? 1 : 0);
  fa.dtype = dtype;
  fa.row_scale = row_scale;
  fa.col_scale = col_scale;
  fa.adam_v = adam_v;
  fa.bias_scale = bias_scale;
  fa.out = nullptr;
  fa.out_row_stride = 0;
  fa.out_col = 0;
  fa.out_dtype = out_dtype;
  fa.lo = lo;
  fa.hi = hi;
  WgradIn in;
  in.act = a;
  in.g = g;
  in.a_seq_stride = a_seq_stride;
  in.a_tok_stride = a_tok_stride;
  in.g_seq_stride = g_seq_stride;
  in.g_tok_stride = g_tok_stride;
  in.S = S;
  in.lengths = lengths;
  in.out_rows = nullptr;
  const int64_t es = 2;
  auto whole = [&](const void* q, int64_t s0, int64_t s1) {
    return ((uintptr_t)q % 16 == 0) && (s0 * es) % 16 == 0 && (s1 * es) % 16 == 0;
  };
  in.aligned = whole(a, a_seq_stride, a_tok_stride) && whole(g, g_seq_stride, g_tok_stride);
  in.tiles_i = 0;
  WgradProject pj;
  pj.left = left;
  pj.right = right;
  pj.bias_col = bias_col;
  pj.right_stride = right_stride;
  pj.p = p;
  pj.partial = (float*)ws;
  // whole 16-byte pieces: aligned rows, and a width of whole pieces (a piece never straddles the end of a row)
  pj.left_whole = (uintptr_t)left % 16 == 0 && O % 8 == 0;
  pj.right_whole = (uintptr_t)right % 16 == 0 && right_stride % 8 == 0 && I % 8 == 0;
  hipStream_t st = (hipStream_t)stream;
  const int64_t n_tiles = dtype == BGX_F16 ? launch_wgrad<f16_t, true>(fa, in, pj, N, st)
                                           : launch_wgrad<bf16_t, true>(fa, in, pj, N, st);
  BGX_HIP(hipGetLastError());
  const int pp = p * p;
  const int groups = (int)wgrad_sum_groups(n_tiles);
  float* sums = (float*)ws + (size_t)N * (size_t)n_tiles * pp;
  const unsigned ex = (unsigned)((pp + 63) / 64);
  if (groups > 1) {
    BGX_REQUIRE(groups <= 65535, BGX_E_SHAPE, "collect_seq_weight: O=%d I=%d", O, I);
    hipLaunchKernelGGL(wgrad_project_sum_kernel, dim3(ex, (unsigned)N, (unsigned)groups), dim3(256), 0, st,
                       (const float*)ws, (int)n_tiles, pp, WG_SUM_GROUP, sums, nullptr, nullptr, 0, 0, out_dtype, lo, hi);
    hipLaunchKernelGGL(wgrad_project_sum_kernel, dim3(ex, (unsigned)N, 1u), dim3(256), 0, st, (const float*)sums, groups,
                       pp, groups, nullptr, out_rows, out, out_row_stride, out_col, out_dtype, lo, hi);
  } else {
    hipLaunchKernelGGL(wgrad_project_sum_kernel, dim3(ex, (unsigned)N, 1u), dim3(256), 0, st, (const float*)ws,
                       (int)n_tiles, pp, (int)n_tiles, nullptr, out_rows, out, out_row_stride, out_col, out_dtype, lo, hi);
  }
  BGX_HIP(hipGetLastError());
  return 0;
}

int fullgrad_seq_gemm_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride,
                           int64_t g_seq_stride, int64_t g_tok_stride, int N, int S, int I, int O, int dtype,
                           const float* row_scale, const float* col_scale, const float* adam_v, int collect_bias,
                           const float* bias_scale, const int32_t* lengths, const int64_t* out_rows, void* out,
                           int64_t out_row_stride, int64_t out_col, int out_dtype, float lo, float hi, void* stream) {
  BGX_REQUIRE(a && g, BGX_E_ARG, "fullgrad_seq_gemm: null pointer");
  BGX_REQUIRE(N > 0 && S > 0 && N <= 65535, BGX_E_SHAPE, "fullgrad_seq_gemm: N=%d S=%d", N, S);
  BGX_REQUIRE(a_tok_stride >= I && g_tok_stride >= O && a_seq_stride >= 0 && g_seq_stride >= 0, BGX_E_ARG,
              "fullgrad_seq_gemm: strides a (%lld, %lld) g (%lld, %lld)", (long long)a_seq_stride,
              (long long)a_tok_stride, (long long)g_seq_stride, (long long)g_tok_stride);
  FullArgs fa;
  const int rc = fill_args(fa, "fullgrad_seq_gemm", O, I, dtype, row_scale, col_scale, adam_v, collect_bias,
                           bias_scale, out, out_row_stride, out_col, out_dtype, lo, hi);
  if (rc != 0) return rc;
  BGX_REQUIRE(((int64_t)((O + 63) / 64)) * ((I + 63) / 64) <= 0x7fffffff, BGX_E_SHAPE,
              "fullgrad_seq_gemm: O=%d I=%d", O, I);
  WgradIn in;
  in.act = a;
  in.g = g;
  in.a_seq_stride = a_seq_stride;
  in.a_tok_stride = a_tok_stride;
  in.g_seq_stride = g_seq_stride;
  in.g_tok_stride = g_tok_stride;
  in.S = S;
  in.lengths = lengths;
  in.out_rows = out_rows;
  const int64_t es = (int64_t)dtype_size(dtype);
  auto whole = [&](const void* p, int64_t s0, int64_t s1) {
    return ((uintptr_t)p % 16 == 0) && (s0 * es) % 16 == 0 && (s1 * es) % 16 == 0;
  };
  in.aligned = whole(a, a_seq_stride, a_tok_stride) && whole(g, g_seq_stride, g_tok_stride);
  in.tiles_i = 0;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == BGX_F32)
    launch_wgrad<float, false>(fa, in, WgradProject{}, N, st);
  else if (dtype == BGX_F16)
    launch_wgrad<f16_t, false>(fa, in, WgradProject{}, N, st);
  else
    launch_wgrad<bf16_t, false>(fa, in, WgradProject{}, N, st);
  BGX_HIP(hipGetLastError());
  return 0;
}

// how the contraction is cut: enough workgroups to fill the chip, slabs of whole groups of four k-steps
static void project_plan(int64_t M, int64_t W, int P, int dtype, int64_t* slab_len, int* n_slabs) {
  const int64_t ks4 = 4 * (dtype == BGX_F32 ? 8 : 16);
  const int64_t tiles = ((M + 31) / 32) * ((P + 32 * PROJ_PB - 1) / (32 * PROJ_PB));
  int64_t want = std::max<int64_t>(1, 1024 / tiles);
  const int64_t max_slabs = std::max<int64_t>(1, W / (16 * ks4));
  want = std::min(std::min(want, max_slabs), (int64_t)4096);
  int64_t len = (W + want - 1) / want;
  len = (len + ks4 - 1) / ks4 * ks4;
  *slab_len = len;
  *n_slabs = (int)((W + len - 1) / len);
}

size_t project_rows_workspace_bytes(int64_t M, int64_t W, int P, int dtype) {
  if (M <= 0 || W <= 0 || P <= 0) return 0;
  int64_t len;
  int n;
  project_plan(M, W, P, dtype, &len, &n);
  return (size_t)n * (size_t)M * (size_t)P * sizeof(float);
}

int project_rows_impl(const void* rows, int64_t M, int64_t W, int64_t row_stride, int dtype, const void* proj, int P,
                      float* acc, int64_t acc_stride, void* ws, size_t ws_bytes, void* stream) {
  BGX_REQUIRE(rows && proj && acc, BGX_E_ARG, "project_rows: null pointer");
  BGX_REQUIRE(M > 0 && W > 0 && P > 0 && row_stride >= W && acc_stride >= P, BGX_E_SHAPE,
              "project_rows: M=%lld W=%lld P=%d strides %lld %lld", (long long)M, (long long)W, P,
              (long long)row_stride, (long long)acc_stride);
  BGX_REQUIRE(dtype_ok(dtype), BGX_E_DTYPE, "project_rows: dtype=%d", dtype);
  BGX_REQUIRE((M + 31) / 32 <= 65535 && (P + 32 * PROJ_PB - 1) / (32 * PROJ_PB) <= 65535, BGX_E_SHAPE,
              "project_rows: M=%lld P=%d", (long long)M, P);
  ProjArgs pa;
  project_plan(M, W, P, dtype, &pa.slab_len, &pa.n_slabs);
  const size_t need = (size_t)pa.n_slabs * (size_t)M * (size_t)P * sizeof(float);
  BGX_REQUIRE(ws != nullptr && ws_bytes >= need, BGX_E_WORKSPACE, "project_rows: workspace of %zu bytes, need %zu",
              ws_bytes, need);
  pa.rows = rows;
  pa.proj = proj;
  pa.M = M;
  pa.W = W;
  pa.row_stride = row_stride;
  pa.P = P;
  pa.partial = (float*)ws;
  const int64_t es = (int64_t)dtype_size(dtype);
  const bool aligned = (uintptr_t)rows % 16 == 0 && (uintptr_t)proj % 16 == 0 && (row_stride * es) % 16 == 0 &&
                       (W * es) % 16 == 0;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)pa.n_slabs, (unsigned)((M + 31) / 32), (unsigned)((P + 32 * PROJ_PB - 1) / (32 * PROJ_PB)));
#define BGX_PROJ_LAUNCH(T)                                                                         \
  do {                                                                                             \
    if (aligned)                                                                                   \
      hipLaunchKernelGGL((project_rows_kernel<T, true>), grid, dim3(256), 0, st, pa);              \
    else                                                                                           \
      hipLaunchKernelGGL((project_rows_kernel<T, false>), grid, dim3(256), 0, st, pa);             \
  } while (0)
  if (dtype == BGX_F32)
    BGX_PROJ_LAUNCH(float);
  else if (dtype == BGX_F16)
    BGX_PROJ_LAUNCH(f16_t);
  else
    BGX_PROJ_LAUNCH(bf16_t);
#undef BGX_PROJ_LAUNCH
  BGX_HIP(hipGetLastError());
  const int64_t total = M * P;
  const int by_wave = total < 16384 ? 1 : 0;
  const int64_t blocks = by_wave ? (total + 3) / 4 : (total + 255) / 256;
  hipLaunchKernelGGL(project_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, st, pa.partial, pa.n_slabs, M, P, acc,
                     acc_stride, by_wave);
  BGX_HIP(hipGetLastError());
  return 0;
}

int fullgrad_tok_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride, int64_t g_seq_stride,
                      int64_t g_tok_stride, int N, int S, int I, int O, int dtype, const float* row_scale,
                      const float* col_scale, const float* adam_v, int collect_bias, const float* bias_scale,
                      const int32_t* lengths, const int64_t* row_offsets, void* out, int64_t out_row_stride,
                      int64_t out_col, int out_dtype, float lo, float hi, void* stream) {
  BGX_REQUIRE(a && g && lengths && row_offsets, BGX_E_ARG, "fullgrad_tok: null pointer");
  BGX_REQUIRE(N > 0 && S > 0 && N <= 65535, BGX_E_SHAPE, "fullgrad_tok: N=%d S=%d", N, S);
  FullArgs fa;
  const int rc = fill_args(fa, "fullgrad_tok", O, I, dtype, row_scale, col_scale, adam_v, collect_bias, bias_scale,
                           out, out_row_stride, out_col, out_dtype, lo, hi);
  if (rc != 0) return rc;
  // enough slabs per token to fill the GPU when there are few tokens
  const int64_t tokens = (int64_t)N * S;
  int gz = (int)std::min<int64_t>((O + TOK_SLAB - 1) / TOK_SLAB, std::max<int64_t>(1, 4096 / tokens));
  gz = std::min(gz, 65535);
  hipLaunchKernelGGL(fullgrad_tok_kernel, dim3((unsigned)S, (unsigned)N, (unsigned)gz), dim3(256), 0,
                     (hipStream_t)stream, fa, a, g, a_seq_stride, a_tok_stride, g_seq_stride, g_tok_stride, S, lengths,
                     row_offsets);
  BGX_HIP(hipGetLastError());
  return 0;
}

}  // namespace bgx
