// Adam second-moment normalisation on the collection path.
//
// The reference forms, per sequence or per token, the full weight-shaped gradient, divides it by
// sqrt(v) + 1e-8 and projects it from both sides (bergson/collector/collector.py:609-644,
// bergson/gradients.py:380-388).  Per token t that is
//     P_t[i, j] = sum_o L[i, o] g_t[o] * H_t[o, j],
//     H_t[o, j] = sum_k a_t[k] * C[(j, o), k],      C[(j, o), k] = R[j, k] / (sqrt(v[o, k]) + 1e-8)
// so nothing weight-shaped is formed per token: H is one GEMM of the activations against a table C that
// depends on the module only (built once by adam_table_kernel), and P_t is a small contraction of H_t with
// L and g_t.  The per-sequence gradient is the sum of its tokens' P_t (the normalisation is linear).
//
// This build materialises H for a chunk of tokens at a time (GEMM on the scan kernel's main loop), stored
// per token as [j][o] so that the contraction over o reads it contiguously, and contracts it on the matrix
// cores (adam_contract_mfma_kernel): P_t = L Z_t with Z_t[o, j] = g_t[o] H_t[o, j], L as the A operand shared
// by the tokens of a wave, Z_t formed in registers as the B operand.  H is O*p values per token, which makes
// the path HBM-heavy for large modules; fusing the contraction into the GEMM is the planned next step.

#include <stdlib.h>

#include <algorithm>

#include <type_traits>

#include "common.hpp"
#include "direct.hpp"
#include "mma16.hpp"
#include "mma32.hpp"

namespace bgx {

int gemm_scores(const void* rows, int64_t n_rows, int64_t D, int64_t stride, int dtype, const void* queries, int Q,
                float* scores, hipStream_t st);

// The table's shape.  16-bit models with p <= 32 run on the fused kernels, which want whole 256-feature chunks of
// O and whole 64-element K tiles of I: their table is padded with zero rows up to O_pad and zero columns up to
// I_pad, and when the bias gradient is collected the bias is one more input feature -- column I of the table holds
// bias_col[j] * bias_scale[o], and the activations get a column of ones there (see adam_pad_kernel), so that
//   sum_o L[i,o] g_t[o] (H_t[o,j] + 1 * bias_col[j] bias_scale[o]) = P_t[i,j] + (sum_o L[i,o] g_t[o] bias_scale[o]) bias_col[j],
// which is the bias column of the reference's [grad | bias_grad] projection (collector.py:626-644).  Zero rows and
// columns add exact zeros.  Other models (fp32, p > 32) keep the plain [p * O, I] table and take the bias as two
// vectors.
struct AdamDims {
  int O_pad, I_pad;
  bool padded;     // the table is not the plain [p * O, I] one
  bool bias_in_k;  // the bias travels as input feature I
};
static AdamDims adam_dims(int O, int I, int p, int dtype, bool bias) {
  AdamDims d{O, I, false, false};
  if (dtype == BGX_F32 || p > 32) return d;
  d.O_pad = (O + 255) / 256 * 256;
  d.I_pad = (I + (bias ? 1 : 0) + 63) / 64 * 64;
  d.bias_in_k = bias;
  d.padded = d.O_pad != O || d.I_pad != I;
  return d;
}

// table[(j * O_pad + o) * I_pad + k] = round_T(R[j, k] / (sqrt(v[o, k]) + 1e-8)) for o < O, k < I;
// round_T(bias_col[j] * bias_scale[o]) at k = I when the bias is collected; 0 elsewhere
template <typename T>
__global__ __launch_bounds__(256) void adam_table_kernel(const T* __restrict__ r_in, const float* __restrict__ v,
                                                         const float* __restrict__ bias_col,
                                                         const float* __restrict__ bias_scale, int O, int I, int O_pad,
                                                         int I_pad, int p, T* __restrict__ table) {
  const int64_t total = (int64_t)O_pad * p * I_pad;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int k = (int)(idx % I_pad);
    const int64_t jo = idx / I_pad;
    const int o = (int)(jo % O_pad);
    const int j = (int)(jo / O_pad);
    float val = 0.f;
    if (o < O && k < I) {
      const float w = 1.0f / (sqrtf(v[(int64_t)o * I + k]) + 1e-8f);
      val = Elem<T>::load(r_in + (int64_t)j * I + k) * w;
    } else if (o < O && k == I && bias_col != nullptr) {
      val = bias_col[j] * bias_scale[o];
    }
    if constexpr (sizeof(T) == 4)
      *(float*)(table + idx) = val;
    else if constexpr (Elem<T>::code == BGX_F16)
      ((uint16_t*)table)[idx] = (uint16_t)f32_to_f16_bits(val);
    else
      ((uint16_t*)table)[idx] = (uint16_t)f32_to_bf16_bits(val);
  }
}

// dst[t, c] = src[t, c] for c < cols, `one_at` gets 1 (the bias's input feature; -1 = none), the rest 0:
// [N, S, cols] rows of any stride into a contiguous [N * S, cols_pad] copy.  16-bit elements.
__global__ __launch_bounds__(256) void adam_pad_kernel(const uint16_t* __restrict__ src, int64_t seq_stride,
                                                       int64_t tok_stride, int S, int cols, uint16_t* __restrict__ dst,
                                                       int cols_pad, int one_at, uint16_t one, int64_t total) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(idx % cols_pad);
    const int64_t t = idx / cols_pad;
    uint16_t val = 0;
    if (c < cols)
      val = src[(t / S) * seq_stride + (t % S) * tok_stride + c];
    else if (c == one_at)
      val = one;
    dst[idx] = val;
  }
}

struct ContractArgs {
  const float* H;        // [chunk_tokens][p][O]
  const void* g;         // [N, S, O]
  const void* r_out;     // [p, O]
  int64_t g_seq_stride, g_tok_stride;
  int64_t t0;            // first flattened token of the chunk
  int chunk_tokens;
  int S, O, p;
  const int32_t* lengths;
  // per-token output
  const int64_t* row_offsets;
  void* out;
  int64_t out_row_stride, out_col;
  int out_dtype;
  float lo, hi;
  // per-sequence: per-token fp32 rows of the chunk
  float* ptok;           // [chunk_tokens, p * p]
  // bias column (both NULL when the bias is not collected)
  const float* bias_col;    // [p]  column I of the [p, I+1] right projection
  const float* bias_scale;  // [O]  1 / (sqrt(bias_avg_sq) + 1e-8)
};

constexpr int CONTRACT_OC = 32;  // output features staged per step

// Generic fallback (any O, any alignment): one workgroup per token of the chunk,
// P_t[i, j] = sum_o L[i, o] g_t[o] H_t[o, j] on the vector ALUs.
template <typename T, bool PER_TOKEN>
__global__ __launch_bounds__(256) void adam_contract_kernel(ContractArgs a) {
  __shared__ float s_lg[CONTRACT_OC][65];  // [o][i]  L[i, o] * g_t[o]
  __shared__ float s_h[CONTRACT_OC][65];   // [o][j]
  __shared__ float s_bs[CONTRACT_OC];      // bias factor of the staged output features
  const int tl = blockIdx.x;
  const int64_t t = a.t0 + tl;
  const int n = (int)(t / a.S);
  const int s = (int)(t - (int64_t)n * a.S);
  const int p = a.p, pp = p * p;
  bool valid = true;
  if (a.lengths != nullptr) valid = s < a.lengths[n] - 1;
  if (PER_TOKEN && !valid) return;
  const int tid = threadIdx.x;
  float acc[16];   // p*p <= 4096 outputs over 256 threads
  float accb[16];  // sum_o L[i, o] g[o] bias_scale[o] of each output's row i
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    acc[c] = 0.f;
    accb[c] = 0.f;
  }
  if (valid) {
    const T* g = (const T*)a.g + (int64_t)n * a.g_seq_stride + (int64_t)s * a.g_tok_stride;
    const T* L = (const T*)a.r_out;
    const float* H = a.H + (int64_t)tl * a.O * p;
    for (int o0 = 0; o0 < a.O; o0 += CONTRACT_OC) {
      const int oc = min(CONTRACT_OC, a.O - o0);
      __syncthreads();
      for (int e = tid; e < oc * p; e += 256) {
        const int oo = e / p, x = e - oo * p;
        s_lg[oo][x] = Elem<T>::load(L + (int64_t)x * a.O + o0 + oo) * Elem<T>::load(g + o0 + oo);
        s_h[oo][x] = H[(int64_t)x * a.O + o0 + oo];
      }
      if (a.bias_col != nullptr && tid < oc) s_bs[tid] = a.bias_scale[o0 + tid];
      __syncthreads();
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        const int e = tid + c * 256;
        if (e < pp) {
          const int i = e / p, j = e - i * p;
          float sum = acc[c];
          for (int oo = 0; oo < oc; ++oo) sum = fmaf(s_lg[oo][i], s_h[oo][j], sum);
          acc[c] = sum;
          if (a.bias_col != nullptr) {
            float sb = accb[c];
            for (int oo = 0; oo < oc; ++oo) sb = fmaf(s_lg[oo][i], s_bs[oo], sb);
            accb[c] = sb;
          }
        }
      }
    }
  }
  if (a.bias_col != nullptr) {
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const int e = tid + c * 256;
      if (e < pp) acc[c] = fmaf(accb[c], a.bias_col[e % p], acc[c]);
    }
  }
  if (PER_TOKEN) {
    const int64_t base = (a.row_offsets[n] + s) * a.out_row_stride + a.out_col;
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const int e = tid + c * 256;
      if (e < pp) store_as(a.out, base + e, clampf(acc[c], a.lo, a.hi), a.out_dtype);
    }
  } else {
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const int e = tid + c * 256;
      if (e < pp) a.ptok[(int64_t)tl * pp + e] = acc[c];
    }
  }
}

// The same contraction on the matrix cores.  A wave owns TT tokens of the chunk; per k-step (KS output
// features) it loads the fragments of L once and, for every token, builds the B operand
// Z_t[o, j] = g_t[o] * H_t[j][o] in registers (rounded to the model dtype, as the reference's normalised
// gradient is) and accumulates P_t[16 it .. , 16 jt ..] += L[., o-slice] Z_t[o-slice, .].
// Needs O % KS == 0 and 16-byte aligned g rows and L; PT = ceil(p / 16).
template <typename T, bool PER_TOKEN, bool BIAS, int PT, int TT>
__global__ __launch_bounds__(256) void adam_contract_mfma_kernel(ContractArgs a) {
  using M = Mma<T>;
  constexpr int HV = M::EPL / 4;  // 16-byte loads of fp32 values per fragment
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = lane & 15;
  const int q = lane >> 4;
  const int p = a.p, O = a.O, pp = p * p;
  const int64_t tl0 = ((int64_t)blockIdx.x * 4 + wave) * TT;  // first chunk-local token of this wave
  if (tl0 >= a.chunk_tokens) return;

  const T* grow[TT];
  const float* hrow[TT];
  bool valid[TT];
  int64_t out_base[TT];
#pragma unroll
  for (int u = 0; u < TT; ++u) {
    const bool in_chunk = tl0 + u < a.chunk_tokens;
    const int64_t tl = in_chunk ? tl0 + u : a.chunk_tokens - 1;
    const int64_t t = a.t0 + tl;
    const int n = (int)(t / a.S);
    const int s = (int)(t - (int64_t)n * a.S);
    valid[u] = in_chunk && (a.lengths == nullptr || s < a.lengths[n] - 1);
    grow[u] = (const T*)a.g + (int64_t)n * a.g_seq_stride + (int64_t)s * a.g_tok_stride + q * M::EPL;
    hrow[u] = a.H + tl * (int64_t)O * p + q * M::EPL;
    out_base[u] = PER_TOKEN ? (a.row_offsets[n] + s) * a.out_row_stride + a.out_col : tl * pp;
  }
  const T* lrow[PT];
  int64_t hcol[PT];
#pragma unroll
  for (int t = 0; t < PT; ++t) {
    const int r = min(t * 16 + c, p - 1);  // rows / columns past p repeat the last one and are not stored
    lrow[t] = (const T*)a.r_out + (int64_t)r * O + q * M::EPL;
    hcol[t] = (int64_t)r * O;
  }

  f32x4 acc[TT][PT][PT];
  f32x4 accb[BIAS ? TT : 1][PT];
#pragma unroll
  for (int u = 0; u < TT; ++u)
#pragma unroll
    for (int it = 0; it < PT; ++it) {
      if (BIAS) accb[u][it] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int jt = 0; jt < PT; ++jt) acc[u][it][jt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  const int nsteps = O / M::KS;
  for (int ks = 0; ks < nsteps; ++ks) {
    const int k0 = ks * M::KS;
    uint4 af[PT];
#pragma unroll
    for (int it = 0; it < PT; ++it) af[it] = load16_global(lrow[it] + k0);
    float bs[M::EPL];
    if (BIAS) {
#pragma unroll
      for (int h = 0; h < HV; ++h) {
        const uint4 v = load16_global(a.bias_scale + k0 + q * M::EPL + 4 * h);
        bs[4 * h] = __uint_as_float(v.x);
        bs[4 * h + 1] = __uint_as_float(v.y);
        bs[4 * h + 2] = __uint_as_float(v.z);
        bs[4 * h + 3] = __uint_as_float(v.w);
      }
    }
#pragma unroll
    for (int u = 0; u < TT; ++u) {
      const uint4 gv = load16_global(grow[u] + k0);
      if (BIAS) {
        uint4 bfb = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int e = 0; e < M::EPL; ++e) M::set(bfb, e, M::get(gv, e) * bs[e]);
#pragma unroll
        for (int it = 0; it < PT; ++it) M::mma(af[it], bfb, accb[u][it]);
      }
#pragma unroll
      for (int jt = 0; jt < PT; ++jt) {
        uint4 bf = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int h = 0; h < HV; ++h) {
          const uint4 hv = load16_global(hrow[u] + hcol[jt] + k0 + 4 * h);
          M::set(bf, 4 * h, M::get(gv, 4 * h) * __uint_as_float(hv.x));
          M::set(bf, 4 * h + 1, M::get(gv, 4 * h + 1) * __uint_as_float(hv.y));
          M::set(bf, 4 * h + 2, M::get(gv, 4 * h + 2) * __uint_as_float(hv.z));
          M::set(bf, 4 * h + 3, M::get(gv, 4 * h + 3) * __uint_as_float(hv.w));
        }
#pragma unroll
        for (int it = 0; it < PT; ++it) M::mma(af[it], bf, acc[u][it][jt]);
      }
    }
  }

  // acc[u][it][jt][e] = P_t[16 it + 4 q + e][16 jt + c]
#pragma unroll
  for (int u = 0; u < TT; ++u) {
    if (tl0 + u >= a.chunk_tokens) continue;
    if (PER_TOKEN && !valid[u]) continue;
#pragma unroll
    for (int it = 0; it < PT; ++it)
#pragma unroll
      for (int jt = 0; jt < PT; ++jt) {
        const int j = jt * 16 + c;
        const float bc = (BIAS && j < p) ? a.bias_col[j] : 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = it * 16 + q * 4 + e;
          if (i < p && j < p) {
            float v = acc[u][it][jt][e];
            if (BIAS) v = fmaf(accb[u][it][e], bc, v);
            if (PER_TOKEN)
              store_as(a.out, out_base[u] + i * p + j, clampf(v, a.lo, a.hi), a.out_dtype);
            else
              a.ptok[out_base[u] + i * p + j] = valid[u] ? v : 0.f;
          }
        }
      }
  }
}

// ---- fused path: H never leaves the CU ------------------------------------------------------------
// Workgroup (token tile of 256, column j of P) walks the output features in chunks of 256:
//   1. the tile GEMM of the store scan (256 x 256, K = I): acc[t, o] = sum_k a[t, k] * table[(j, o), k],
//   2. acc goes to LDS in the model dtype (the tile buffers are free by then),
//   3. second MFMA pass, one wave per 32 tokens: pacc[t, i] += sum_o (acc[t, o] * g[t, o]) * L[i, o], the
//      A operand read back from LDS and scaled by 16 bytes of the token's g row, the B operand 16 bytes
//      of L's row i,
// and finally writes ptok[t][i * p + j].  Needs a 16-bit model dtype, O % 256 == 0, I % 64 == 0,
// p <= 32, aligned rows, no bias column; everything else takes the two-kernel path above.
struct FusedArgs {
  const void* a;  // activations of the chunk, [tokens, I]
  int64_t a_tok_stride;
  const void* table;  // [(p * O), I]
  const void* g;
  int64_t g_seq_stride, g_tok_stride;
  const void* r_out;  // [p, O]
  int64_t t0;         // first flattened token of the chunk
  int tokens;
  int S, I, O, p;
  const int32_t* lengths;
  float* ptok;  // [tokens][p * p]
  int ttx;      // token tiles per group of 32 workgroups that share an XCD; 0 = plain workgroup order
};

// two fp32 values rounded to nearest-even in T, packed low | high << 16 (the hardware's packed conversion
// for bf16: the software rounding of f32_to_bf16_bits costs six vector instructions per value, and a
// workgroup converts 65 536 values per chunk of output features)
template <typename T>
__device__ inline uint32_t pack2_bits(float lo, float hi) {
  if constexpr (Elem<T>::code == BGX_F16) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 r = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, r);
  } else {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, b2));
  }
}

constexpr int FUSED_TILE = 256;

// (x0 * g.lo, x1 * g.hi) rounded to T, packed like `g2` (two T values).  fp16 rounds x to T first: the packed
// half multiply then gives the once-rounded exact product in one instruction; bf16 multiplies in fp32.
template <typename T>
__device__ inline uint32_t scaled_pair_bits(float x0, float x1, uint32_t g2) {
  if constexpr (Elem<T>::code == BGX_F16) {
    typedef _Float16 hv __attribute__((ext_vector_type(2)));
    const uint32_t h2 = pack2_bits<T>(x0, x1);
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(hv, h2) * __builtin_bit_cast(hv, g2));
  } else {
    const float b0 = __uint_as_float(g2 << 16), b1 = __uint_as_float(g2 & 0xffff0000u);
    return pack2_bits<T>(x0 * b0, x1 * b1);
  }
}

// ---- fused path, tiles loaded straight into LDS ------------------------------------------------------------
// A workgroup owns (256 tokens, column j of P) and walks the output features in chunks of 256.  Per chunk it runs a
// 256 x 256 tile GEMM over K = I (H[t, o] = sum_k a[t, k] table[(j, o), k]) on the store scan's direct-to-LDS
// pipeline (direct.hpp), and a second MFMA pass adds pacc[t, i] += sum_o (H[t, o] g[t, o]) L[i, o] straight from
// the accumulators: the GEMM blocks are accumulated transposed (the table's fragment as the A operand), so lane
// (fr, fh) holds token fr of a block and its 16 accumulators are rows q*8 + fh*4 + c (q, c = 0..3) of the block's 32
// table rows; the loader puts table row fh*16 + q*4 + c at that place of the LDS tile, which makes those 16
// accumulators 16 consecutive output features, fh*16 + e.  A k-step of the second pass takes e = 8s .. 8s+7, one
// 16-byte piece of the token's g row and of a row of L per lane (the order of k inside an MFMA is free as long as
// both operands use the same one).  H never leaves the registers, and the K tiles of all chunks form one pipeline.
// Which (token tile, column j) a workgroup takes: workgroup b runs on XCD b % 8, and the 32 that an XCD runs at a
// time share operands through its L2 -- `ttx` token tiles x 32 / ttx columns (chosen by the host); in the plain
// order every XCD would walk the whole table.  The workgroup writes its column of the per-token p x p blocks to
// `ptok` (fp32 [tokens][p * p]); rows past `tokens` and positions from a sequence's last token on are left zero.
//  * the second pass is fed from LDS as well:
//  * eight waves as 4 x 2: a wave owns 64 tokens against 128 table rows of the chunk (2 x 4 blocks of 32 x 32,
//    128 accumulators), so that a K tile costs the workgroup 192 KB of fragment reads -- with 8 x 1 (every wave
//    reading all 256 table rows) it was 288 KB, and together with the 64 KB the loads write that is more LDS time
//    than the tile has MFMA time; the two waves that share tokens add their sums once, at the end;
//  * one ring of tiles -- three row buffers, two operand buffers, 160 KB -- carries two kinds of tile: the K tiles
//    of a chunk (256 tokens x 64 of I against 256 table rows x 64), and behind them four slices of the chunk's g
//    values (256 tokens x 2 x 32 output features: 32 from each half of the chunk, so that every wave has work on
//    every slice; in a row buffer) with the matching slice of L
//    (p rows x 64 features, in the operand buffer, which a g slice does not otherwise need).  The g values used to
//    be fetched by the lanes that needed them, 32 bytes of 32 different lines per load instruction, and came
//    through the L1 up to four times: with the path from L2 into the CU as the bound, a quarter of the kernel;
//  * a g slice is four MFMAs per wave (H of one 32-feature block for two token blocks, scaled by g in registers,
//    against L), its operands read from LDS with the K tiles' swizzle; nothing of the second pass touches global
//    memory, and its loads travel two tiles ahead like all others;
//  * loads are uniform base + 32-bit lane offset (sw_load_lds16), fragment reads and waits are spelled out as in
//    scan_direct_kernel.
constexpr int FD_A_BYTES = FUSED_TILE * SD_ROW, FD_B_BYTES = FUSED_TILE * SD_ROW;
constexpr int FD_LDS_BYTES = 3 * FD_A_BYTES + 2 * FD_B_BYTES;
constexpr int FD_GSLICES = 4;  // slices of 64 output features per chunk of 256

template <typename T>
__global__ __launch_bounds__(512) void adam_fused_direct_kernel(FusedArgs a) {
  using M = Mma32<T>;
  static_assert(sizeof(T) == 2, "the fused Adam kernel is for 16-bit model dtypes");
  constexpr int BM = FUSED_TILE, BN = FUSED_TILE, BK = 64;
  constexpr int TM = 2, TN = 4;  // eight waves as 4 x 2: 64 tokens (two blocks) x 128 table rows (four blocks) per wave
  extern __shared__ __align__(128) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int fr = lane & 31;
  const int fh = lane >> 5;
  int tt = blockIdx.x, j = blockIdx.y;
  if (a.ttx > 0) {
    const int b = blockIdx.x + gridDim.x * blockIdx.y;
    const int xcd = b & 7, slot = b >> 3;
    const int jx = 32 / a.ttx, n_super_tt = gridDim.x / a.ttx;
    const int super = (slot >> 5) * 8 + xcd, within = slot & 31;
    tt = (super % n_super_tt) * a.ttx + within % a.ttx;
    j = (super / n_super_tt) * jx + within / a.ttx;
  }
  const int t_row0 = tt * BM;  // chunk-local first token of the tile
  const int p = a.p, O = a.O, pp = p * p;
  const int rows_here = a.tokens - t_row0;  // valid tokens of this tile (may exceed BM)
  const int KT = a.I / BK;
  const int n_chunks = O / BN;
  const int per_chunk = KT + FD_GSLICES;
  const int total = per_chunk * n_chunks;

  // ---- loader: instruction i of wave w fills rows i * 64 + w * 8 .. + 7 of a 256-row tile; lane l is position
  // l & 7 of row l >> 3 and fetches chunk (l & 7) ^ sd_key(row).  Rows past the end repeat the last one.
  const uint32_t a_row_bytes = (uint32_t)(a.a_tok_stride * sizeof(T));
  const uint32_t g_row_bytes = (uint32_t)(a.g_tok_stride * sizeof(T));
  const uint32_t t_row_bytes = (uint32_t)(a.I * sizeof(T));
  const uint32_t l_row_bytes = (uint32_t)(O * sizeof(T));
  uint32_t voff_a[4], voff_g[4], voff_t[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = i * 64 + wave * 8 + (lane >> 3);
    const uint32_t ch = (uint32_t)((lane & 7) ^ sd_key(r)) * 16u;
    const uint32_t rc = (uint32_t)min(r, rows_here - 1);
    voff_a[i] = rc * a_row_bytes + ch;
    // a g slice takes 32 features from each half of the chunk (see g_slice): chunks 0 .. 3 of an LDS row are
    // features 32 s .. of the chunk, chunks 4 .. 7 features 128 + 32 s ..
    voff_g[i] = rc * g_row_bytes + (ch < 64u ? ch : ch + 192u);
    // table row that goes to LDS row r: bits (q1 q0 h c1 c0) -> (h q1 q0 c1 c0) within each block of 32, so that a
    // lane's 16 accumulators of a block are 16 consecutive output features (see adam_fused_kernel)
    const int pr = (r & ~31) | ((r & 4) << 2) | ((r & 24) >> 1) | (r & 3);
    voff_t[i] = (uint32_t)pr * t_row_bytes + ch;
  }
  // L slice: rows 0 .. 31 of the operand buffer, loaded by waves 0 .. 3 (8 rows each); rows past p repeat row p - 1
  const uint32_t ch_l = (uint32_t)((lane & 7) ^ sd_key(wave * 8 + (lane >> 3))) * 16u;
  const uint32_t voff_l =
      (uint32_t)min((wave & 3) * 8 + (lane >> 3), p - 1) * l_row_bytes + (ch_l < 64u ? ch_l : ch_l + 192u);
  const uint64_t act_base = (uint64_t)(uintptr_t)a.a + (uint64_t)t_row0 * a_row_bytes;
  const uint64_t g_base = (uint64_t)(uintptr_t)a.g + (uint64_t)(a.t0 + t_row0) * g_row_bytes;
  const uint64_t tab_base = (uint64_t)(uintptr_t)a.table + (uint64_t)j * O * t_row_bytes;
  const uint64_t l_base = (uint64_t)(uintptr_t)a.r_out;
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const uint32_t lds_wave = lds0 + (uint32_t)wave * 1024u;
  // tile t of the sequence: chunk t / per_chunk, position t % per_chunk (< KT: K tile, else g slice)
  int ld_a_pos = 0, ld_a_chunk = 0, ld_b_pos = 0, ld_b_chunk = 0;  // the two loaders' own places in the sequence
  auto load_a = [&](int t) {
    const uint32_t dst = lds_wave + (uint32_t)(t % 3) * FD_A_BYTES;
    if (ld_a_pos < KT) {
      const uint64_t base = act_base + (uint64_t)ld_a_pos * (BK * sizeof(T));
#pragma unroll
      for (int i = 0; i < 4; ++i) sw_load_lds16(base, voff_a[i], dst + (uint32_t)i * 8192u);
    } else {
      const uint64_t base = g_base + ((uint64_t)ld_a_chunk * BN + (uint64_t)(ld_a_pos - KT) * 32) * sizeof(T);
#pragma unroll
      for (int i = 0; i < 4; ++i) sw_load_lds16(base, voff_g[i], dst + (uint32_t)i * 8192u);
    }
    if (++ld_a_pos == per_chunk) {
      ld_a_pos = 0;
      ++ld_a_chunk;
    }
  };
  auto load_b = [&](int t) {
    const uint32_t dst = lds_wave + (uint32_t)(3 * FD_A_BYTES) + (uint32_t)(t & 1) * FD_B_BYTES;
    const bool is_k = ld_b_pos < KT;
    const uint64_t base =
        is_k ? tab_base + (uint64_t)ld_b_chunk * BN * t_row_bytes + (uint64_t)ld_b_pos * (BK * sizeof(T))
             : l_base + ((uint64_t)ld_b_chunk * BN + (uint64_t)(ld_b_pos - KT) * 32) * sizeof(T);
    // an L slice is 32 rows: instruction 0 of waves 0 .. 3 (the other waves fetch the same rows again into rows
    // 32 .. 63 of the buffer, which nothing reads: every wave then issues the same number of loads, and
    // "all but the youngest four" means the same thing to all of them)
    if (is_k) {
#pragma unroll
      for (int i = 0; i < 4; ++i) sw_load_lds16(base, voff_t[i], dst + (uint32_t)i * 8192u);
    } else {
      sw_load_lds16(base, voff_l, dst);
    }
    if (++ld_b_pos == per_chunk) {
      ld_b_pos = 0;
      ++ld_b_chunk;
    }
  };

  f32x16 pacc[TM];
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) pacc[i][e] = 0.f;
#pragma unroll
    for (int jj = 0; jj < TN; ++jj)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][jj][e] = 0.f;
  }

  // fragment reads per k-step: the wave's 64 token rows (two fragments) and its 128 table rows (four)
  const uint32_t key = (uint32_t)sd_key(fr);  // rows advance in steps of 32: the key depends on fr alone
  const uint32_t a_frag = lds0 + (uint32_t)((wm * 64 + fr) * SD_ROW);
  const uint32_t b_frag = lds0 + (uint32_t)(3 * FD_A_BYTES + (wn * 128 + fr) * SD_ROW);
  uint4 af[2][TM], bf[2][TN];
  auto rd = [&](int t, auto kk_tag, auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr int KK = decltype(kk_tag)::value;
    const uint32_t chk = (((uint32_t)(KK * 2 + fh)) ^ key) * 16u;
    const uint32_t ab = a_frag + (uint32_t)(t % 3) * FD_A_BYTES + chk;
    const uint32_t bb = b_frag + (uint32_t)(t & 1) * FD_B_BYTES + chk;
    af[SET][0] = sw_lds_read16<0 * 32 * SD_ROW>(ab);
    af[SET][1] = sw_lds_read16<1 * 32 * SD_ROW>(ab);
    bf[SET][0] = sw_lds_read16<0 * 32 * SD_ROW>(bb);
    bf[SET][1] = sw_lds_read16<1 * 32 * SD_ROW>(bb);
    bf[SET][2] = sw_lds_read16<2 * 32 * SD_ROW>(bb);
    bf[SET][3] = sw_lds_read16<3 * 32 * SD_ROW>(bb);
  };
  auto mm = [&](auto set_tag) {
    constexpr int SET = decltype(set_tag)::value;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int jj = 0; jj < TN; ++jj)
        M::mma(bf[SET][jj], af[SET][i], acc[i][jj]);  // transposed block: rows = output features
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  using K0 = std::integral_constant<int, 0>;
  using K1 = std::integral_constant<int, 1>;
  using K2 = std::integral_constant<int, 2>;
  using K3 = std::integral_constant<int, 3>;
  constexpr int WAIT_LDS_STEP = 0xC07F | ((TM + TN) << 8);  // lgkmcnt(6): the step issued before the latest six reads
  constexpr int WAIT_LDS_0 = 0xC07F;

  // prologue: tile 0 lands, its step 0 is read; tile 1's operands and tile 2's rows are under way
  load_a(0);
  load_b(0);
  if (total > 1) {
    load_a(1);
    wg_barrier_lds<4>();
  } else {
    wg_barrier_lds<0>();
  }
  __builtin_amdgcn_sched_barrier(0);
  rd(0, K0{}, S0{});
  __builtin_amdgcn_sched_barrier(0);
  if (1 < total) load_b(1);
  if (2 < total) load_a(2);

  auto tile_end_barrier = [&](int t) {
    // In flight, oldest first: rows(t + 1), then operands(t + 1) and rows(t + 2).  Tile t + 1 must have landed
    // (this wave's part; the barrier makes that all of it), rows(t + 2) -- always the youngest four loads of a
    // wave -- may still fly; this tile's reads have completed, so its buffers can take operands(t + 2) and
    // rows(t + 3) behind the barrier.
    if (t + 2 < total)
      wg_barrier_lds<4>();
    else
      wg_barrier_lds<0>();
    __builtin_amdgcn_sched_barrier(0);
  };
  // one g slice: pacc[t, i] += sum over its features of (H[t, o] * g[t, o]) * L[i, o].  Slice S is features
  // 32 S .. 32 S + 31 of both halves of the chunk, i.e. accumulator block S of every wave, so that all eight waves
  // work on every slice; the half of wave column wn sits in chunks 4 wn .. 4 wn + 3 of the LDS rows.  Lane (fr, fh)
  // holds token fr and features fh * 16 + e of the block, and takes them eight at a time (sp = 0, 1): chunk
  // 4 wn + 2 fh + sp of the token's row of g, and the same chunk of row fr of L.
  auto g_slice = [&](int t, auto s_tag) {
    constexpr int S = decltype(s_tag)::value;
    const uint32_t gb = a_frag + (uint32_t)(t % 3) * FD_A_BYTES;
    const uint32_t lb = lds0 + (uint32_t)(3 * FD_A_BYTES + fr * SD_ROW) + (uint32_t)(t & 1) * FD_B_BYTES;
    uint4 gq[TM][2], lq[2];
#pragma unroll
    for (int sp = 0; sp < 2; ++sp) {
      const uint32_t chk = (((uint32_t)(4 * wn + fh * 2 + sp)) ^ key) * 16u;
      lq[sp] = sd_lds_read16(lb + chk);
      gq[0][sp] = sw_lds_read16<0 * 32 * SD_ROW>(gb + chk);
      gq[1][sp] = sw_lds_read16<1 * 32 * SD_ROW>(gb + chk);
    }
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int sp = 0; sp < 2; ++sp) {
        const f32x16& h = acc[i][S];
        uint4 zf;
        zf.x = scaled_pair_bits<T>(h[8 * sp + 0], h[8 * sp + 1], gq[i][sp].x);
        zf.y = scaled_pair_bits<T>(h[8 * sp + 2], h[8 * sp + 3], gq[i][sp].y);
        zf.z = scaled_pair_bits<T>(h[8 * sp + 4], h[8 * sp + 5], gq[i][sp].z);
        zf.w = scaled_pair_bits<T>(h[8 * sp + 6], h[8 * sp + 7], gq[i][sp].w);
        M::mma(zf, lq[sp], pacc[i]);
      }
    __builtin_amdgcn_sched_barrier(0);
  };

  int t = 0;
  for (int c = 0; c < n_chunks; ++c) {
    // ---- the chunk's K tiles: four k-steps each, fragments double-buffered, the pipeline runs across the barrier
    for (int kt = 0; kt < KT; ++kt, ++t) {
      __builtin_amdgcn_sched_barrier(0);
      rd(t, K1{}, S1{});
      __builtin_amdgcn_s_waitcnt(WAIT_LDS_STEP);
      __builtin_amdgcn_sched_barrier(0);
      mm(S0{});
      __builtin_amdgcn_sched_barrier(0);
      rd(t, K2{}, S0{});
      __builtin_amdgcn_s_waitcnt(WAIT_LDS_STEP);
      __builtin_amdgcn_sched_barrier(0);
      mm(S1{});
      __builtin_amdgcn_sched_barrier(0);
      rd(t, K3{}, S1{});
      __builtin_amdgcn_s_waitcnt(WAIT_LDS_STEP);
      __builtin_amdgcn_sched_barrier(0);
      mm(S0{});
      __builtin_amdgcn_sched_barrier(0);
      tile_end_barrier(t);
      if (kt + 1 < KT) rd(t + 1, K0{}, S0{});
      __builtin_amdgcn_sched_barrier(0);
      mm(S1{});  // its fragments arrived before the barrier
      __builtin_amdgcn_sched_barrier(0);
      // the loads go out behind the first MFMAs after the barrier, so that those are not held up by their issue
      if (t + 2 < total) load_b(t + 2);
      if (t + 3 < total) load_a(t + 3);
    }
    // ---- the chunk's four g slices
    g_slice(t, std::integral_constant<int, 0>{});
    tile_end_barrier(t);
    load_b(t + 2);
    load_a(t + 3);
    ++t;
    g_slice(t, std::integral_constant<int, 1>{});
    tile_end_barrier(t);
    if (t + 2 < total) load_b(t + 2);
    if (t + 3 < total) load_a(t + 3);
    ++t;
    g_slice(t, std::integral_constant<int, 2>{});
    tile_end_barrier(t);
    if (t + 2 < total) load_b(t + 2);
    if (t + 3 < total) load_a(t + 3);
    ++t;
    g_slice(t, std::integral_constant<int, 3>{});
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int jj = 0; jj < TN; ++jj)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][jj][e] = 0.f;
    __builtin_amdgcn_sched_barrier(0);
    tile_end_barrier(t);
    if (c + 1 < n_chunks) rd(t + 1, K0{}, S0{});
    __builtin_amdgcn_sched_barrier(0);
    if (t + 2 < total) load_b(t + 2);
    if (t + 3 < total) load_a(t + 3);
    ++t;
  }
  __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);

  // the two waves that share 64 tokens add their halves of the sum over the output features, in a fixed order,
  // through the tile buffers (every wave is past its last fragment read behind the barrier)
  float* red = reinterpret_cast<float*>(smem);
  wg_barrier_lds<0>();
  __builtin_amdgcn_sched_barrier(0);
  if (wn == 1) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) red[((wm * TM + i) * 16 + e) * 64 + lane] = pacc[i][e];
  }
  __syncthreads();
  if (wn == 0) {
    // pacc[i][e] = P[token (e>>2)*8 + fh*4 + (e&3) of block i of this wave's 64][row fr], column j
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int tl = t_row0 + wm * 64 + i * 32 + (e >> 2) * 8 + fh * 4 + (e & 3);
        if (tl < a.tokens && fr < p) {
          bool valid = true;
          if (a.lengths != nullptr) {
            const int64_t t = a.t0 + tl;
            const int n = (int)(t / a.S);
            valid = (int)(t - (int64_t)n * a.S) < a.lengths[n] - 1;
          }
          const float v = pacc[i][e] + red[((wm * TM + i) * 16 + e) * 64 + lane];
          a.ptok[(int64_t)tl * pp + fr * p + j] = valid ? v : 0.f;
        }
      }
  }
}

// ---- fused path, one wave per SIMD ----------------------------------------------------------------------------
// adam_fused_direct_kernel's computation and tile ring on four waves instead of eight.  With eight waves on a
// 256 x 256 tile every wave reads 2 + 4 fragments per k-step, 192 KB per K tile and workgroup, and the loads
// write another 64 KB: 2048 cycles of LDS time beside the 2048 cycles the tile's MFMAs take.  Four waves as 2 x 2
// own 128 tokens x 128 table rows each (4 x 4 blocks of 32 x 32) and read 4 + 4 fragments per k-step, 128 KB per
// tile.  The 256 accumulators of a wave are the AccVGPRs (MFMAs written as instructions, as in the store scan's
// wide-tile kernel), pacc and everything else the ordinary registers; one wave per SIMD means nothing hides a
// stall, so fragment reads and loads are placed by hand between the MFMAs:
//  * a K tile is four k-steps of 16 MFMAs; the 8 fragment reads of the next step follow MFMAs 0 .. 7 of a step
//    (into the other register set), and every step ends with a wait for them -- no read is in flight across a
//    step boundary;
//  * tile t's part of the load stream is "stage t": the 8 loads of operands(t + 2) and the 8 of rows(t + 3).
//    Four of them go out behind the barrier of tile t, which sits after the fourth MFMA of its last k-step and
//    frees the buffers they write; the other twelve are spread over tile t + 1, before its barrier.  That barrier
//    waits for all but the youngest eight loads (rows(t + 3)), so operands(t + 2) and rows(t + 2) have landed;
//  * every load instruction is a uniform 64-bit base + one per-lane offset that is the same for all eight
//    instructions of a tile (instruction i fetches rows 32 i + 8 wave + lane / 8, and 32 rows on, the swizzle key
//    and the permuted table row repeat): the kernel takes whole token tiles only;
//  * past the end of the sequence the stream goes on fetching the last tile into the buffers whose turn it is
//    (which nothing reads any more), so that the wait counts mean the same in every tile;
//  * the first k-step of a chunk's first tile accumulates onto a literal zero, which saves clearing 256
//    accumulators per chunk.
// Token tile x column mapping (ttx), the second pass's operand layout and the ptok layout are the direct kernel's.
constexpr int FW_THREADS = 256;

template <typename T>
__device__ inline void fw_mfma_zero(const uint4& a, const uint4& b, f32x16& c) {
  typedef uint32_t raw4 __attribute__((ext_vector_type(4)));
  const raw4 av = {a.x, a.y, a.z, a.w}, bv = {b.x, b.y, b.z, b.w};
  if constexpr (std::is_same<T, f16_t>::value)
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=a"(c) : "v"(av), "v"(bv));
  else
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(av), "v"(bv));
}

template <typename T>
__device__ inline void fw_mfma_after_valu(const uint4& a, const uint4& b, f32x16& c) {
  typedef uint32_t raw4 __attribute__((ext_vector_type(4)));
  const raw4 av = {a.x, a.y, a.z, a.w}, bv = {b.x, b.y, b.z, b.w};
  if constexpr (std::is_same<T, f16_t>::value)
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "v"(bv));
  else
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "v"(bv));
}

template <int... Is, typename F>
__device__ inline void fw_static_for(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}

template <typename T>
__global__ __launch_bounds__(FW_THREADS) void adam_fused_wide_kernel(FusedArgs a) {
  static_assert(sizeof(T) == 2, "the fused Adam kernel is for 16-bit model dtypes");
  constexpr int BM = FUSED_TILE, BN = FUSED_TILE, BK = 64;
  constexpr int TM = 4, TN = 4;
  extern __shared__ __align__(128) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int fr = lane & 31;
  const int fh = lane >> 5;
  int tt = blockIdx.x, j = blockIdx.y;
  if (a.ttx > 0) {
    const int b = blockIdx.x + gridDim.x * blockIdx.y;
    const int xcd = b & 7, slot = b >> 3;
    const int jx = 32 / a.ttx, n_super_tt = gridDim.x / a.ttx;
    const int super = (slot >> 5) * 8 + xcd, within = slot & 31;
    tt = (super % n_super_tt) * a.ttx + within % a.ttx;
    j = (super / n_super_tt) * jx + within / a.ttx;
  }
  const int t_row0 = tt * BM;
  const int p = a.p, O = a.O, pp = p * p;
  const int KT = a.I / BK;  // at least 4 (host)
  const int n_chunks = O / BN;

  // ---- the load stream
  const uint32_t a_row_bytes = (uint32_t)(a.a_tok_stride * sizeof(T));
  const uint32_t g_row_bytes = (uint32_t)(a.g_tok_stride * sizeof(T));
  const uint32_t t_row_bytes = (uint32_t)(a.I * sizeof(T));
  const uint32_t l_row_bytes = (uint32_t)(O * sizeof(T));
  const int rbase = wave * 8 + (lane >> 3);  // row of the first of a tile's eight load instructions
  const uint32_t ch = (uint32_t)((lane & 7) ^ sd_key(rbase)) * 16u;
  const uint32_t gch = ch < 64u ? ch : ch + 192u;  // a g / L slice is 32 features from each half of the chunk
  const uint32_t v_act = (uint32_t)rbase * a_row_bytes + ch;
  const uint32_t v_g = (uint32_t)rbase * g_row_bytes + gch;
  // table row that goes to LDS row r: bits (q1 q0 h c1 c0) -> (h q1 q0 c1 c0) within each block of 32
  const uint32_t v_tab = (uint32_t)(((rbase & 4) << 2) | ((rbase & 24) >> 1) | (rbase & 3)) * t_row_bytes + ch;
  const uint32_t v_l = (uint32_t)min(rbase, p - 1) * l_row_bytes + gch;
  const uint64_t act_base = (uint64_t)(uintptr_t)a.a + (uint64_t)t_row0 * a_row_bytes;
  const uint64_t g_base = (uint64_t)(uintptr_t)a.g + (uint64_t)(a.t0 + t_row0) * g_row_bytes;
  const uint64_t tab_base = (uint64_t)(uintptr_t)a.table + (uint64_t)j * O * t_row_bytes;
  const uint64_t l_base = (uint64_t)(uintptr_t)a.r_out;
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const uint32_t lds_wave = lds0 + (uint32_t)wave * 1024u;

  // one tile's eight loads: base + i * step for the lanes' common offset, to dst + i * 4096.  Which tile a stage
  // fetches follows from the place in the chunk, which is fixed where the stage is set up (set_* below), so a
  // descriptor is a handful of scalar additions.
  struct Desc {
    uint64_t base;
    uint32_t step, dst, voff;
  };
  Desc db, da;  // the stage under way: operands, then rows
  uint32_t a_off = 0, b_off = 0;  // byte offsets of the current tile's buffers within their rings; the stage set up in
                                  // tile t writes the buffers tile t has just left
  const uint32_t k_step_tab = 32u * t_row_bytes, k_step_act = 32u * a_row_bytes, k_step_g = 32u * g_row_bytes;
  auto set_b_k = [&](int chunk, int pos) {  // K tile `pos` of the table rows of `chunk`
    db.base = tab_base + (uint64_t)chunk * BN * t_row_bytes + (uint64_t)pos * (BK * sizeof(T));
    db.step = k_step_tab;
    db.voff = v_tab;
    db.dst = lds_wave + (uint32_t)(3 * FD_A_BYTES) + b_off;
  };
  auto set_b_l = [&](int chunk, int sl) {  // slice `sl` of L: 32 rows, one load instruction (issue() skips the other seven)
    db.base = l_base + ((uint64_t)chunk * BN + (uint64_t)sl * 32) * sizeof(T);
    db.step = 0u;
    db.voff = v_l;
    db.dst = lds_wave + (uint32_t)(3 * FD_A_BYTES) + b_off;
  };
  auto set_a_k = [&](int pos) {
    da.base = act_base + (uint64_t)pos * (BK * sizeof(T));
    da.step = k_step_act;
    da.voff = v_act;
    da.dst = lds_wave + a_off;
  };
  auto set_a_g = [&](int chunk, int sl) {
    da.base = g_base + ((uint64_t)chunk * BN + (uint64_t)sl * 32) * sizeof(T);
    da.step = k_step_g;
    da.voff = v_g;
    da.dst = lds_wave + a_off;
  };
  // load n of the stage: 0 .. 7 operands (an L slice has load 0 only: B_IS_L), 8 .. 15 rows
  auto issue = [&](auto n_tag, auto b_is_l_tag) {
    constexpr int N = decltype(n_tag)::value;
    constexpr bool B_IS_L = decltype(b_is_l_tag)::value;
    if constexpr (N < 8) {
      if constexpr (!B_IS_L || N == 0)
        sw_load_lds16(db.base + (uint64_t)N * db.step, db.voff, db.dst + (uint32_t)N * 4096u);
    } else
      sw_load_lds16(da.base + (uint64_t)(N - 8) * da.step, da.voff, da.dst + (uint32_t)(N - 8) * 4096u);
  };

  f32x16 pacc[TM];
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) pacc[i][e] = 0.f;

  // ---- fragment reads: the wave's 128 token rows and its 128 table rows, four fragments each per k-step
  const uint32_t key = (uint32_t)sd_key(fr);
  const uint32_t a_frag = lds0 + (uint32_t)((wm * 128 + fr) * SD_ROW);
  const uint32_t b_frag = lds0 + (uint32_t)(3 * FD_A_BYTES + (wn * 128 + fr) * SD_ROW);
  uint32_t chk[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) chk[kk] = (((uint32_t)(kk * 2 + fh)) ^ key) * 16u;
  uint4 af[2][TM], bf[2][TN];
  // read n of a k-step's eight, in the order the MFMAs want them
  auto rd_one = [&](uint32_t ab, uint32_t bb, auto set_tag, auto n_tag) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr int N = decltype(n_tag)::value;
    if constexpr (N == 0) bf[SET][0] = sw_lds_read16<0 * 32 * SD_ROW>(bb);
    if constexpr (N == 1) af[SET][0] = sw_lds_read16<0 * 32 * SD_ROW>(ab);
    if constexpr (N == 2) bf[SET][1] = sw_lds_read16<1 * 32 * SD_ROW>(bb);
    if constexpr (N == 3) bf[SET][2] = sw_lds_read16<2 * 32 * SD_ROW>(bb);
    if constexpr (N == 4) bf[SET][3] = sw_lds_read16<3 * 32 * SD_ROW>(bb);
    if constexpr (N == 5) af[SET][1] = sw_lds_read16<1 * 32 * SD_ROW>(ab);
    if constexpr (N == 6) af[SET][2] = sw_lds_read16<2 * 32 * SD_ROW>(ab);
    if constexpr (N == 7) af[SET][3] = sw_lds_read16<3 * 32 * SD_ROW>(ab);
  };
  // MFMA n of a k-step: token block n / 4 against table block n % 4, transposed (rows = output features)
  auto mfma_one = [&](auto set_tag, auto n_tag, auto zero_tag) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr int N = decltype(n_tag)::value;
    if constexpr (decltype(zero_tag)::value)
      fw_mfma_zero<T>(bf[SET][N % 4], af[SET][N / 4], acc[N / 4][N % 4]);
    else
      sw_mfma<T, true>(bf[SET][N % 4], af[SET][N / 4], acc[N / 4][N % 4]);
  };
  using I16 = std::make_integer_sequence<int, 16>;
  using I8 = std::make_integer_sequence<int, 8>;
  using I4 = std::make_integer_sequence<int, 4>;
  using TrueT = std::true_type;
  using FalseT = std::false_type;
  constexpr int WAIT_LDS_0 = 0xC07F;
  auto next_offsets = [&](uint32_t& an, uint32_t& bn) {
    an = a_off + FD_A_BYTES;
    if (an == 3u * FD_A_BYTES) an = 0;
    bn = b_off ^ (uint32_t)FD_B_BYTES;
  };
  // the tile's barrier: everything but the youngest eight loads (rows of the tile after next) has landed, for every
  // wave; behind it this tile's buffers take the first loads of the next stage
  auto tile_barrier = [&](auto&& set_stage) {
    asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    set_stage();
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- one K tile.  FIRST: the chunk's first (accumulate onto zero); LAST: the chunk's last (a g slice follows, which
  // reads its own operands); prevl / newl: the operands of the stage under way / of the stage set up here are a slice of L
  auto k_tile = [&](auto first_tag, auto last_tag, auto prevl, auto newl, auto&& set_stage) {
    constexpr bool FIRST = decltype(first_tag)::value, LAST = decltype(last_tag)::value;
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    // k-steps 0 .. 2: MFMAs of the step, reads of the next one behind MFMAs 0 .. 7, four loads behind 8, 10, 12, 14
    auto step = [&](auto cur_tag, auto nxt_tag, auto kk_tag, auto zero_tag) {
      constexpr int KK = decltype(kk_tag)::value;  // the step that is read
      const uint32_t ab = a_frag + a_off + chk[KK], bb = b_frag + b_off + chk[KK];
      __builtin_amdgcn_sched_barrier(0);
      fw_static_for(I16{}, [&](auto n) {
        constexpr int N = decltype(n)::value;
        mfma_one(cur_tag, n, zero_tag);
        if constexpr (N < 8) rd_one(ab, bb, nxt_tag, n);
        if constexpr (N >= 8 && N % 2 == 0) issue(std::integral_constant<int, 4 * KK + (N - 8) / 2>{}, prevl);
        __builtin_amdgcn_sched_barrier(0);
      });
      __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);
      __builtin_amdgcn_sched_barrier(0);
    };
    step(S0{}, S1{}, std::integral_constant<int, 1>{}, std::integral_constant<bool, FIRST>{});
    step(S1{}, S0{}, std::integral_constant<int, 2>{}, FalseT{});
    step(S0{}, S1{}, std::integral_constant<int, 3>{}, FalseT{});
    // k-step 3: the barrier behind the fourth MFMA, then the next tile's first reads and the next stage's first loads
    uint32_t an, bn;
    next_offsets(an, bn);
    const uint32_t ab = a_frag + an + chk[0], bb = b_frag + bn + chk[0];
    __builtin_amdgcn_sched_barrier(0);
    fw_static_for(I16{}, [&](auto n) {
      constexpr int N = decltype(n)::value;
      mfma_one(S1{}, n, FalseT{});
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (N == 3) tile_barrier(set_stage);
      if constexpr (!LAST && N >= 4 && N < 12) rd_one(ab, bb, S0{}, std::integral_constant<int, N - 4>{});
      if constexpr (N >= 12) issue(std::integral_constant<int, N - 12>{}, newl);
      __builtin_amdgcn_sched_barrier(0);
    });
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);
    a_off = an;
    b_off = bn;
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- one g slice: pacc[t, i] += sum over its features of (H[t, o] * g[t, o]) * L[i, o].  Slice S is features
  // 32 S .. 32 S + 31 of both halves of the chunk, i.e. accumulator block S of every wave; the half of wave column wn
  // sits in chunks 4 wn .. 4 wn + 3 of the LDS rows.  Lane (fr, fh) holds token fr and features fh * 16 + e of the block
  // and takes them eight at a time (sp = 0, 1): chunk 4 wn + 2 fh + sp of the token's row of g and of row fr of L.
  auto g_slice = [&](auto s_tag, auto prevl, auto newl, auto&& set_stage) {
    constexpr int S = decltype(s_tag)::value;
    const uint32_t gb = a_frag + a_off;
    const uint32_t lb = lds0 + (uint32_t)(3 * FD_A_BYTES + fr * SD_ROW) + b_off;
    uint4 gq[TM][2], lq[2];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sp = 0; sp < 2; ++sp) {
      const uint32_t c16 = (((uint32_t)(4 * wn + fh * 2 + sp)) ^ key) * 16u;
      lq[sp] = sd_lds_read16(lb + c16);
      gq[0][sp] = sw_lds_read16<0 * 32 * SD_ROW>(gb + c16);
      gq[1][sp] = sw_lds_read16<1 * 32 * SD_ROW>(gb + c16);
      gq[2][sp] = sw_lds_read16<2 * 32 * SD_ROW>(gb + c16);
      gq[3][sp] = sw_lds_read16<3 * 32 * SD_ROW>(gb + c16);
    }
    issue(std::integral_constant<int, 4>{}, prevl);
    issue(std::integral_constant<int, 5>{}, prevl);
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);
    uint32_t an, bn;
    next_offsets(an, bn);
    const uint32_t ab = a_frag + an + chk[0], bb = b_frag + bn + chk[0];  // the K tile behind slice 3
    __builtin_amdgcn_sched_barrier(0);
    fw_static_for(I8{}, [&](auto n) {
      constexpr int N = decltype(n)::value;
      constexpr int sp = N / 4, i = N % 4;
      const f32x16& h = acc[i][S];
      uint4 zf;
      zf.x = scaled_pair_bits<T>(h[8 * sp + 0], h[8 * sp + 1], gq[i][sp].x);
      zf.y = scaled_pair_bits<T>(h[8 * sp + 2], h[8 * sp + 3], gq[i][sp].y);
      zf.z = scaled_pair_bits<T>(h[8 * sp + 4], h[8 * sp + 5], gq[i][sp].z);
      zf.w = scaled_pair_bits<T>(h[8 * sp + 6], h[8 * sp + 7], gq[i][sp].w);
      // pacc stays in the ordinary registers (left to the compiler it wanders between the two files, 16 moves a
      // time), so this MFMA is an instruction too -- and it reads what vector instructions have just written, which
      // the hardware does not interlock: two wait states in front of it (the compiler puts as many before its own)
      fw_mfma_after_valu<T>(zf, lq[sp], pacc[i]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (N < 5) {  // the rest of the stage under way goes out before the barrier ...
        issue(std::integral_constant<int, 6 + 2 * N>{}, prevl);
        issue(std::integral_constant<int, 7 + 2 * N>{}, prevl);
      }
      if constexpr (N == 5) {
        // ... which sits here: the slice's operands were read at its start, the rest of it works from registers.  Behind
        // it the first reads of the K tile that follows slice 3 (after the last chunk: of buffers that hold nothing
        // anyone uses) and the next stage's first loads
        tile_barrier(set_stage);
        if constexpr (S == 3) fw_static_for(I8{}, [&](auto r) { rd_one(ab, bb, std::integral_constant<int, 0>{}, r); });
      }
      if constexpr (N >= 6) {
        issue(std::integral_constant<int, 2 * (N - 6)>{}, newl);
        issue(std::integral_constant<int, 2 * (N - 6) + 1>{}, newl);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    a_off = an;
    b_off = bn;
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: rows(0), operands(0), rows(1), then the first four loads of stage -1 = operands(1), rows(2)
  set_a_k(0);
  fw_static_for(I8{}, [&](auto n) { issue(std::integral_constant<int, 8 + decltype(n)::value>{}, FalseT{}); });
  set_b_k(0, 0);
  fw_static_for(I8{}, [&](auto n) { issue(n, FalseT{}); });
  a_off = FD_A_BYTES;
  set_a_k(1);
  fw_static_for(I8{}, [&](auto n) { issue(std::integral_constant<int, 8 + decltype(n)::value>{}, FalseT{}); });
  a_off = 2 * FD_A_BYTES;
  b_off = FD_B_BYTES;
  set_b_k(0, 1);
  set_a_k(2);
  fw_static_for(I4{}, [&](auto n) { issue(n, FalseT{}); });
  a_off = 0;
  b_off = 0;
  asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");  // tile 0 has landed
  __builtin_amdgcn_sched_barrier(0);
  {
    const uint32_t ab = a_frag + chk[0], bb = b_frag + chk[0];
    fw_static_for(I8{}, [&](auto n) { rd_one(ab, bb, std::integral_constant<int, 0>{}, n); });
    __builtin_amdgcn_s_waitcnt(WAIT_LDS_0);
  }
  __builtin_amdgcn_sched_barrier(0);

  // A chunk is KT >= 4 K tiles and four g slices; the stage set up in the tile at place q fetches operands(q + 2) and
  // rows(q + 3), and after the last chunk the stream fetches the last chunk's first tiles again, into buffers that
  // nothing reads any more.
  for (int c = 0; c < n_chunks; ++c) {
    const int cn = c + 1 < n_chunks ? c + 1 : c;
    k_tile(TrueT{}, FalseT{}, FalseT{}, FalseT{}, [&]() {
      set_b_k(c, 2);
      set_a_k(3);
    });
    for (int q = 1; q <= KT - 4; ++q)
      k_tile(FalseT{}, FalseT{}, FalseT{}, FalseT{}, [&]() {
        set_b_k(c, q + 2);
        set_a_k(q + 3);
      });
    k_tile(FalseT{}, FalseT{}, FalseT{}, FalseT{}, [&]() {
      set_b_k(c, KT - 1);
      set_a_g(c, 0);
    });
    k_tile(FalseT{}, FalseT{}, FalseT{}, TrueT{}, [&]() {
      set_b_l(c, 0);
      set_a_g(c, 1);
    });
    k_tile(FalseT{}, TrueT{}, TrueT{}, TrueT{}, [&]() {
      set_b_l(c, 1);
      set_a_g(c, 2);
    });
    // the MFMAs above are instructions the compiler does not see through: their results are read (by instructions
    // it places) no sooner than the last one has left the pipe
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    g_slice(std::integral_constant<int, 0>{}, TrueT{}, TrueT{}, [&]() {
      set_b_l(c, 2);
      set_a_g(c, 3);
    });
    g_slice(std::integral_constant<int, 1>{}, TrueT{}, TrueT{}, [&]() {
      set_b_l(c, 3);
      set_a_k(0);
    });
    g_slice(std::integral_constant<int, 2>{}, TrueT{}, FalseT{}, [&]() {
      set_b_k(cn, 0);
      set_a_k(1);
    });
    g_slice(std::integral_constant<int, 3>{}, FalseT{}, FalseT{}, [&]() {
      set_b_k(cn, 1);
      set_a_k(2);
    });
  }

  // the two waves that share 128 tokens add their halves of the sum over the output features, in a fixed order,
  // through the tile buffers (behind the barrier every load has landed and every wave is past its last read)
  float* red = reinterpret_cast<float*>(smem);
  asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");  // pacc's last MFMA has left the pipe before anything the compiler places reads it
  wg_barrier_lds<0>();
  __builtin_amdgcn_sched_barrier(0);
  if (wn == 1) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) red[((wm * TM + i) * 16 + e) * 64 + lane] = pacc[i][e];
  }
  __syncthreads();
  if (wn == 0) {
    // pacc[i][e] = P[token (e>>2)*8 + fh*4 + (e&3) of block i of this wave's 128][row fr], column j
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int tl = t_row0 + wm * 128 + i * 32 + (e >> 2) * 8 + fh * 4 + (e & 3);
        if (tl < a.tokens && fr < p) {
          bool valid = true;
          if (a.lengths != nullptr) {
            const int64_t t = a.t0 + tl;
            const int n = (int)(t / a.S);
            valid = (int)(t - (int64_t)n * a.S) < a.lengths[n] - 1;
          }
          const float v = pacc[i][e] + red[((wm * TM + i) * 16 + e) * 64 + lane];
          a.ptok[(int64_t)tl * pp + fr * p + j] = valid ? v : 0.f;
        }
      }
  }
}

// per-token rows from ptok: clamp, cast, scatter to the rows of the valid tokens
__global__ __launch_bounds__(256) void adam_tok_finalize_kernel(const float* __restrict__ ptok, int64_t t0, int tokens,
                                                                int S, int pp, const int32_t* __restrict__ lengths,
                                                                const int64_t* __restrict__ row_offsets, void* out,
                                                                int64_t out_row_stride, int64_t out_col, int out_dtype,
                                                                float lo, float hi) {
  const int tl = blockIdx.x;
  const int64_t t = t0 + tl;
  const int n = (int)(t / S);
  const int s = (int)(t - (int64_t)n * S);
  if (s >= lengths[n] - 1) return;
  const int64_t base = (row_offsets[n] + s) * out_row_stride + out_col;
  for (int e = threadIdx.x; e < pp; e += blockDim.x)
    store_as(out, base + e, clampf(ptok[(int64_t)tl * pp + e], lo, hi), out_dtype);
}

constexpr int SEQ_SLICES = 32;

// part[n - n_first, slice, e] = sum over one slice of the chunk's tokens of sequence n, in token order.
__global__ __launch_bounds__(256) void adam_seq_slice_kernel(const float* __restrict__ ptok, float* __restrict__ part,
                                                             int64_t t0, int chunk_tokens, int S, int pp, int n_first) {
  const int n = n_first + blockIdx.x;
  const int sl = blockIdx.y;
  const int64_t lo = (int64_t)n * S > t0 ? (int64_t)n * S : t0;
  const int64_t hi_seq = (int64_t)(n + 1) * S;
  const int64_t hi = hi_seq < t0 + chunk_tokens ? hi_seq : t0 + chunk_tokens;
  const int64_t per = (hi - lo + SEQ_SLICES - 1) / SEQ_SLICES;
  const int64_t a = lo + sl * per;
  const int64_t b = a + per < hi ? a + per : hi;
  for (int e = threadIdx.x; e < pp; e += blockDim.x) {
    float s = 0.f;
    for (int64_t t = a; t < b; ++t) s += ptok[(t - t0) * pp + e];
    part[((int64_t)blockIdx.x * SEQ_SLICES + sl) * pp + e] = s;
  }
}

// acc[n, e] += the slices of sequence n, in slice order.
__global__ __launch_bounds__(256) void adam_seq_sum_kernel(const float* __restrict__ part, float* __restrict__ acc, int pp,
                                                           int n_first) {
  const int n = n_first + blockIdx.x;
  for (int e = threadIdx.x; e < pp; e += blockDim.x) {
    float s = acc[(int64_t)n * pp + e];
    for (int sl = 0; sl < SEQ_SLICES; ++sl) s += part[((int64_t)blockIdx.x * SEQ_SLICES + sl) * pp + e];
    acc[(int64_t)n * pp + e] = s;
  }
}

__global__ __launch_bounds__(256) void adam_seq_finalize_kernel(const float* __restrict__ acc,
                                                                const int64_t* __restrict__ out_rows, int pp,
                                                                void* out, int64_t out_row_stride, int64_t out_col,
                                                                int out_dtype, float lo, float hi) {
  const int n = blockIdx.x;
  const int64_t row = out_rows ? out_rows[n] : (int64_t)n;
  for (int e = threadIdx.x; e < pp; e += blockDim.x)
    store_as(out, row * out_row_stride + out_col + e, clampf(acc[(int64_t)n * pp + e], lo, hi), out_dtype);
}

__global__ void adam_zero_kernel(float* x, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = 0.f;
}

// ---- host ---------------------------------------------------------------------------------------
static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

size_t adam_table_bytes(int O, int I, int p, int dtype, int with_bias) {
  if (O <= 0 || I <= 0 || p <= 0) return 0;
  const AdamDims d = adam_dims(O, I, p, dtype, with_bias != 0);
  return (size_t)d.O_pad * p * d.I_pad * dtype_size(dtype);
}

int adam_prepare_impl(const void* r_in, const float* v, const float* bias_col, const float* bias_scale, int O, int I,
                      int p, int dtype, void* table, void* stream) {
  BGX_REQUIRE(r_in && v && table, BGX_E_ARG, "adam_prepare: null pointer");
  BGX_REQUIRE((bias_col == nullptr) == (bias_scale == nullptr), BGX_E_ARG,
              "adam_prepare: bias_col and bias_scale go together");
  BGX_REQUIRE(O > 0 && I > 0 && p >= 1 && p <= 64, BGX_E_SHAPE, "adam_prepare: O=%d I=%d p=%d", O, I, p);
  BGX_REQUIRE(dtype >= BGX_F32 && dtype <= BGX_BF16, BGX_E_DTYPE, "adam_prepare: dtype=%d", dtype);
  hipStream_t st = (hipStream_t)stream;
  const AdamDims d = adam_dims(O, I, p, dtype, bias_col != nullptr);
  const int64_t total = (int64_t)d.O_pad * p * d.I_pad;
  const unsigned blocks = (unsigned)((total + 255) / 256 > 65536 * 16 ? 65536 * 16 : (total + 255) / 256);
  // (a table that is not padded leaves the bias to bgx_collect_adam's vectors)
  const float* bc = d.bias_in_k ? bias_col : nullptr;
  const float* bs = d.bias_in_k ? bias_scale : nullptr;
  if (dtype == BGX_F32)
    hipLaunchKernelGGL(adam_table_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float*)r_in, v, bc, bs, O, I,
                       d.O_pad, d.I_pad, p, (float*)table);
  else if (dtype == BGX_F16)
    hipLaunchKernelGGL(adam_table_kernel<f16_t>, dim3(blocks), dim3(256), 0, st, (const f16_t*)r_in, v, bc, bs, O, I,
                       d.O_pad, d.I_pad, p, (f16_t*)table);
  else
    hipLaunchKernelGGL(adam_table_kernel<bf16_t>, dim3(blocks), dim3(256), 0, st, (const bf16_t*)r_in, v, bc, bs, O, I,
                       d.O_pad, d.I_pad, p, (bf16_t*)table);
  BGX_HIP(hipGetLastError());
  return 0;
}

static int64_t adam_chunk(int64_t T, int O, int p, int64_t chunk_tokens) {
  if (chunk_tokens <= 0) {
    // keep H (fp32, O*p per token) near 512 MB
    chunk_tokens = ((int64_t)512 << 20) / ((int64_t)O * p * 4);
    chunk_tokens = chunk_tokens / 256 * 256;
    if (chunk_tokens < 256) chunk_tokens = 256;
  }
  return chunk_tokens < T ? chunk_tokens : T;
}

// [H or the fused kernels' per-token results][per-token results][per-sequence sums][slice sums], then the padded
// copies of a, g and r_out where the table is padded (see adam_dims)
struct AdamWorkspace {
  size_t ptok, acc, part, a_pad, g_pad, l_pad, total;
};
static AdamWorkspace adam_workspace(int N, int S, int I, int O, int p, int dtype, bool bias, int64_t chunk_tokens) {
  const AdamDims d = adam_dims(O, I, p, dtype, bias);
  const int64_t T = (int64_t)N * S;
  const int64_t tc = adam_chunk(T, d.O_pad, p, chunk_tokens);
  const size_t esz = dtype_size(dtype);
  AdamWorkspace w;
  w.ptok = align_up((size_t)tc * d.O_pad * p * 4, 256);
  w.acc = w.ptok + align_up((size_t)tc * p * p * 4, 256);
  w.part = w.acc + align_up((size_t)N * p * p * 4, 256);
  w.a_pad = w.part + align_up((size_t)N * SEQ_SLICES * p * p * 4, 256);
  const bool family = dtype != BGX_F32 && p <= 32;  // room for the copies whatever the operands turn out to look like
  w.g_pad = w.a_pad + (family ? align_up((size_t)T * d.I_pad * esz, 256) : 0);
  w.l_pad = w.g_pad + (family ? align_up((size_t)T * d.O_pad * esz, 256) : 0);
  w.total = w.l_pad + (family ? align_up((size_t)p * d.O_pad * esz, 256) : 0);
  return w;
}

size_t collect_adam_workspace_bytes(int N, int S, int I, int O, int p, int dtype, int with_bias, int64_t chunk_tokens) {
  if (N <= 0 || S <= 0 || I <= 0 || O <= 0 || p <= 0) return 0;
  return adam_workspace(N, S, I, O, p, dtype, with_bias != 0, chunk_tokens).total;
}

int collect_adam_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride, int64_t g_seq_stride,
                      int64_t g_tok_stride, int N, int S, int I, int O, int p, int dtype, const void* table,
                      const void* r_out, const float* bias_col, const float* bias_scale, int per_token,
                      const int32_t* lengths, const int64_t* rows, void* out, int64_t out_row_stride, int64_t out_col,
                      int out_dtype, float lo, float hi, void* ws, size_t ws_bytes, int64_t chunk_tokens,
                      void* stream) {
  BGX_REQUIRE(a && g && table && r_out && out && ws, BGX_E_ARG, "collect_adam: null pointer");
  BGX_REQUIRE((bias_col == nullptr) == (bias_scale == nullptr), BGX_E_ARG,
              "collect_adam: bias_col and bias_scale go together");
  BGX_REQUIRE(N > 0 && S > 0 && I > 0 && O > 0, BGX_E_ARG, "collect_adam: N=%d S=%d I=%d O=%d", N, S, I, O);
  BGX_REQUIRE(p >= 1 && p <= 64, BGX_E_SHAPE, "collect_adam: p=%d outside 1..64", p);
  BGX_REQUIRE(dtype >= BGX_F32 && dtype <= BGX_BF16 && out_dtype >= BGX_F32 && out_dtype <= BGX_BF16, BGX_E_DTYPE,
              "collect_adam: dtype=%d out_dtype=%d", dtype, out_dtype);
  BGX_REQUIRE(a_seq_stride == (int64_t)S * a_tok_stride, BGX_E_ALIGN,
              "collect_adam: activations must be uniformly strided over the flattened tokens");
  BGX_REQUIRE((int64_t)O * p <= 0x7fffffffLL, BGX_E_SHAPE, "collect_adam: O*p too large");
  BGX_REQUIRE(out_col >= 0 && out_col + (int64_t)p * p <= out_row_stride, BGX_E_ARG, "collect_adam: columns do not fit");
  if (per_token) BGX_REQUIRE(lengths && rows, BGX_E_ARG, "collect_adam: per-token mode needs lengths and row_offsets");
  const AdamWorkspace lay = adam_workspace(N, S, I, O, p, dtype, bias_col != nullptr, chunk_tokens);
  BGX_REQUIRE(ws_bytes >= lay.total, BGX_E_WORKSPACE, "collect_adam: workspace %zu < %zu bytes", ws_bytes, lay.total);
  BGX_REQUIRE(((uintptr_t)ws & 255) == 0, BGX_E_ALIGN, "collect_adam: workspace must be 256-byte aligned");

  hipStream_t st = (hipStream_t)stream;
  const int64_t T = (int64_t)N * S;
  const int pp = p * p;
  char* w = (char*)ws;
  const size_t esz = dtype_size(dtype);

  // A padded table (16-bit models, p <= 32; see adam_dims): the operands are brought to its shape -- contiguous
  // copies of a with I_pad columns (a one in column I when the bias travels there), of g and r_out with O_pad
  // columns -- and everything below runs on the padded shapes.  One pass over a and g, against p * O * I
  // multiply-adds per token in the kernel proper.
  const AdamDims dm = adam_dims(O, I, p, dtype, bias_col != nullptr);
  const bool family = dtype != BGX_F32 && p <= 32;  // the fused kernels' shapes (adam_dims pads to them)
  // the fused kernels load whole 16-byte pieces with 32-bit offsets from rows that are uniformly strided over the
  // flattened tokens: operands that are not like that (an odd view of a wider tensor) are copied as well
  const bool a_odd = family && ((uintptr_t)a % 16 != 0 || a_tok_stride % 8 != 0);
  const bool g_odd = family && ((uintptr_t)g % 16 != 0 || g_tok_stride % 8 != 0 ||
                                (N > 1 && g_seq_stride != (int64_t)S * g_tok_stride));
  if (dm.padded || a_odd || g_odd) {
    const uint16_t one = dtype == BGX_F16 ? 0x3C00 : 0x3F80;
    auto pad = [&](const void* src, int64_t seq_stride, int64_t tok_stride, int rows_s, int64_t rows, int cols,
                   void* dst, int cols_pad, int one_at) {
      const int64_t total = rows * cols_pad;
      const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 65536 * 4);
      hipLaunchKernelGGL(adam_pad_kernel, dim3(blocks), dim3(256), 0, st, (const uint16_t*)src, seq_stride, tok_stride,
                         rows_s, cols, (uint16_t*)dst, cols_pad, one_at, one, total);
    };
    if (dm.I_pad != I || a_odd) {
      void* a_pad = w + lay.a_pad;
      pad(a, a_seq_stride, a_tok_stride, S, T, I, a_pad, dm.I_pad, dm.bias_in_k ? I : -1);
      a = a_pad;
      a_tok_stride = dm.I_pad;
      a_seq_stride = (int64_t)S * dm.I_pad;
    }
    if (dm.O_pad != O || g_odd) {
      void* g_pad = w + lay.g_pad;
      pad(g, g_seq_stride, g_tok_stride, S, T, O, g_pad, dm.O_pad, -1);
      g = g_pad;
      g_tok_stride = dm.O_pad;
      g_seq_stride = (int64_t)S * dm.O_pad;
    }
    if (dm.O_pad != O) {
      void* l_pad = w + lay.l_pad;
      pad(r_out, 0, O, p, p, O, l_pad, dm.O_pad, -1);
      r_out = l_pad;
    }
    BGX_HIP(hipGetLastError());
    I = dm.I_pad;
    O = dm.O_pad;
    if (dm.bias_in_k) bias_col = bias_scale = nullptr;  // folded into the table
  }
  const int64_t tc = adam_chunk(T, O, p, chunk_tokens);
  float* H = (float*)w;
  float* ptok = (float*)(w + lay.ptok);
  float* acc = (float*)(w + lay.acc);
  float* part = (float*)(w + lay.part);

  if (!per_token) {
    const int64_t nacc = (int64_t)N * pp;
    hipLaunchKernelGGL(adam_zero_kernel, dim3((unsigned)((nacc + 255) / 256)), dim3(256), 0, st, acc, nacc);
    BGX_HIP(hipGetLastError());
  }
  // ---- fused path ------------------------------------------------------------------------------
  // (after the padding above O is a multiple of the 256-feature chunk, I of the 64-element K tile, the bias is in
  // the table and a, g are aligned and uniformly strided; what is left to check are the 32-bit offsets)
  const bool fused = family && O % FUSED_TILE == 0 && I % 64 == 0 && bias_col == nullptr &&
                     (uintptr_t)r_out % 16 == 0 && (uintptr_t)table % 16 == 0 &&
                     (int64_t)FUSED_TILE * a_tok_stride * 2 < ((int64_t)1 << 32) &&
                     (int64_t)FUSED_TILE * g_tok_stride * 2 < ((int64_t)1 << 32) &&
                     (int64_t)FUSED_TILE * I * 2 < ((int64_t)1 << 32) && (int64_t)p * O * 2 < ((int64_t)1 << 32) &&
                     !switches().adam_fused_off;
  if (fused) {
    // no H: the region reserved for it holds the per-token fp32 results, so a chunk can be much larger
    // (tc * O / p tokens; O >= 256 and p <= 32 make that at least 8 tc, so a batch smaller than one tile is
    // a single pass of T tokens -- the kernel bounds partial tiles by `tokens`)
    const int64_t cap = (int64_t)((size_t)tc * O * p * 4 / ((size_t)pp * 4));
    int64_t fc = cap >= T ? T : cap / FUSED_TILE * FUSED_TILE;
    if (fc <= 0) fc = cap;
    float* ptok_f = (float*)w;
    for (int64_t t0 = 0; t0 < T; t0 += fc) {
      const int64_t rows_c = T - t0 < fc ? T - t0 : fc;
      FusedArgs f;
      f.a = (const char*)a + (size_t)t0 * a_tok_stride * esz;
      f.a_tok_stride = a_tok_stride;
      f.table = table;
      f.g = g;
      f.g_seq_stride = g_seq_stride;
      f.g_tok_stride = g_tok_stride;
      f.r_out = r_out;
      f.t0 = t0;
      f.tokens = (int)rows_c;
      f.S = S;
      f.I = I;
      f.O = O;
      f.p = p;
      f.lengths = lengths;
      f.ptok = ptok_f;
      const dim3 grid((unsigned)((rows_c + FUSED_TILE - 1) / FUSED_TILE), (unsigned)p);
      // 4 token tiles x 8 columns per XCD at a time fetched least through the L2s on every module shape of
      // the benchmark layer (1.3 GB against 1.9 for the plain order on 1024 x 3072; 16 x 2 fetched 2.2: the
      // token tiles' activations then no longer stay in a 4 MB L2); 8 x 4 is next
      int ttx = 0;
      if ((grid.x * grid.y) % 256 == 0) {
        const int prefer[3] = {4, 8, 2};
        for (int c : prefer)
          if (grid.x % c == 0 && p % (32 / c) == 0) {
            ttx = c;
            break;
          }
        if (switches().adam_ttx >= 0) {
          const int v = switches().adam_ttx;
          if (v == 0 || ((v == 2 || v == 4 || v == 8 || v == 16) && grid.x % v == 0 && p % (32 / v) == 0)) ttx = v;
        }
      }
      f.ttx = ttx;
      // one wave per SIMD: whole token tiles, at least four K tiles per chunk; else eight waves
      const bool wide = !switches().adam_wide_off && rows_c % FUSED_TILE == 0 && I >= 256;
      if (wide) {
        if (dtype == BGX_F16) {
          auto kern = adam_fused_wide_kernel<f16_t>;
          BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, FD_LDS_BYTES));
          hipLaunchKernelGGL(kern, grid, dim3(FW_THREADS), FD_LDS_BYTES, st, f);
        } else {
          auto kern = adam_fused_wide_kernel<bf16_t>;
          BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, FD_LDS_BYTES));
          hipLaunchKernelGGL(kern, grid, dim3(FW_THREADS), FD_LDS_BYTES, st, f);
        }
      } else if (dtype == BGX_F16) {
        auto kern = adam_fused_direct_kernel<f16_t>;
        BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, FD_LDS_BYTES));
        hipLaunchKernelGGL(kern, grid, dim3(512), FD_LDS_BYTES, st, f);
      } else {
        auto kern = adam_fused_direct_kernel<bf16_t>;
        BGX_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, FD_LDS_BYTES));
        hipLaunchKernelGGL(kern, grid, dim3(512), FD_LDS_BYTES, st, f);
      }
      BGX_HIP(hipGetLastError());
      note_kernel(FAMILY_ADAM, wide ? "adam_fused_wide" : "adam_fused_direct");
      if (per_token) {
        hipLaunchKernelGGL(adam_tok_finalize_kernel, dim3((unsigned)rows_c), dim3(256), 0, st, ptok_f, t0, (int)rows_c,
                           S, pp, lengths, rows, out, out_row_stride, out_col, out_dtype, lo, hi);
      } else {
        const int n_first = (int)(t0 / S);
        const int n_last = (int)((t0 + rows_c - 1) / S);
        const unsigned nseq = (unsigned)(n_last - n_first + 1);
        hipLaunchKernelGGL(adam_seq_slice_kernel, dim3(nseq, SEQ_SLICES), dim3(256), 0, st, ptok_f, part, t0,
                           (int)rows_c, S, pp, n_first);
        hipLaunchKernelGGL(adam_seq_sum_kernel, dim3(nseq), dim3(256), 0, st, part, acc, pp, n_first);
      }
      BGX_HIP(hipGetLastError());
    }
    if (!per_token) {
      hipLaunchKernelGGL(adam_seq_finalize_kernel, dim3((unsigned)N), dim3(256), 0, st, acc, rows, pp, out,
                         out_row_stride, out_col, out_dtype, lo, hi);
      BGX_HIP(hipGetLastError());
    }
    return 0;
  }

  note_kernel(FAMILY_ADAM, "adam_two_kernel");
  for (int64_t t0 = 0; t0 < T; t0 += tc) {
    const int64_t rows_c = T - t0 < tc ? T - t0 : tc;
    const char* a_chunk = (const char*)a + (size_t)t0 * a_tok_stride * esz;
    // fp32 H: every store instruction of the GEMM epilogue then covers whole 128-byte lines (16-bit
    // scores made that kernel three times slower)
    const int rc = gemm_scores(a_chunk, rows_c, I, a_tok_stride, dtype, table, O * p, H, st);
    if (rc != 0) return rc;
    ContractArgs c;
    c.H = H;
    c.g = g;
    c.r_out = r_out;
    c.g_seq_stride = g_seq_stride;
    c.g_tok_stride = g_tok_stride;
    c.t0 = t0;
    c.chunk_tokens = (int)rows_c;
    c.S = S;
    c.O = O;
    c.p = p;
    c.lengths = lengths;
    c.row_offsets = per_token ? rows : nullptr;
    c.out = out;
    c.out_row_stride = out_row_stride;
    c.out_col = out_col;
    c.out_dtype = out_dtype;
    c.lo = lo;
    c.hi = hi;
    c.ptok = ptok;
    c.bias_col = bias_col;
    c.bias_scale = bias_scale;
    const int kstep = dtype == BGX_F32 ? 16 : 32;
    const int epl = dtype == BGX_F32 ? 4 : 8;
    const bool mfma_ok = O % kstep == 0 && (uintptr_t)g % 16 == 0 && (uintptr_t)r_out % 16 == 0 &&
                         g_seq_stride % epl == 0 && g_tok_stride % epl == 0 &&
                         (bias_scale == nullptr || (uintptr_t)bias_scale % 16 == 0);
    const bool bias = bias_col != nullptr;
    const dim3 block(256);
    if (mfma_ok) {
      const int pt = p <= 16 ? 1 : (p <= 32 ? 2 : 4);
      // tokens per wave: L's fragments are shared by them, but a chunk is only a few thousand tokens and
      // every wave of the chip needs some
      const int tt = pt == 4 ? 1 : 2;
      const dim3 grid((unsigned)((rows_c + 4 * tt - 1) / (4 * tt)));
#define BGX_CONTRACT_M(T_, PT_, TT_)                                                                         \
  if (per_token && bias)                                                                                     \
    hipLaunchKernelGGL((adam_contract_mfma_kernel<T_, true, true, PT_, TT_>), grid, block, 0, st, c);       \
  else if (per_token)                                                                                        \
    hipLaunchKernelGGL((adam_contract_mfma_kernel<T_, true, false, PT_, TT_>), grid, block, 0, st, c);      \
  else if (bias)                                                                                             \
    hipLaunchKernelGGL((adam_contract_mfma_kernel<T_, false, true, PT_, TT_>), grid, block, 0, st, c);      \
  else                                                                                                       \
    hipLaunchKernelGGL((adam_contract_mfma_kernel<T_, false, false, PT_, TT_>), grid, block, 0, st, c);
#define BGX_CONTRACT_P(T_)              \
  if (pt == 1) {                        \
    BGX_CONTRACT_M(T_, 1, 2)            \
  } else if (pt == 2) {                 \
    BGX_CONTRACT_M(T_, 2, 2)            \
  } else {                              \
    BGX_CONTRACT_M(T_, 4, 1)            \
  }
      if (dtype == BGX_F32) {
        BGX_CONTRACT_P(float)
      } else if (dtype == BGX_F16) {
        BGX_CONTRACT_P(f16_t)
      } else {
        BGX_CONTRACT_P(bf16_t)
      }
#undef BGX_CONTRACT_P
#undef BGX_CONTRACT_M
    } else {
      const dim3 grid((unsigned)rows_c);
#define BGX_CONTRACT(T_)                                                                         \
  if (per_token)                                                                                 \
    hipLaunchKernelGGL((adam_contract_kernel<T_, true>), grid, block, 0, st, c);                 \
  else                                                                                           \
    hipLaunchKernelGGL((adam_contract_kernel<T_, false>), grid, block, 0, st, c);
      if (dtype == BGX_F32) {
        BGX_CONTRACT(float)
      } else if (dtype == BGX_F16) {
        BGX_CONTRACT(f16_t)
      } else {
        BGX_CONTRACT(bf16_t)
      }
#undef BGX_CONTRACT
    }
    BGX_HIP(hipGetLastError());
    if (!per_token) {
      const int n_first = (int)(t0 / S);
      const int n_last = (int)((t0 + rows_c - 1) / S);
      const unsigned nseq = (unsigned)(n_last - n_first + 1);
      hipLaunchKernelGGL(adam_seq_slice_kernel, dim3(nseq, SEQ_SLICES), dim3(256), 0, st, ptok, part, t0, (int)rows_c, S,
                         pp, n_first);
      hipLaunchKernelGGL(adam_seq_sum_kernel, dim3(nseq), dim3(256), 0, st, part, acc, pp, n_first);
      BGX_HIP(hipGetLastError());
    }
  }
  if (!per_token) {
    hipLaunchKernelGGL(adam_seq_finalize_kernel, dim3((unsigned)N), dim3(256), 0, st, acc, rows, pp, out,
                       out_row_stride, out_col, out_dtype, lo, hi);
    BGX_HIP(hipGetLastError());
  }
  return 0;
}

}  // namespace bgx
