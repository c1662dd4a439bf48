// Weight-shaped (unprojected) gradients: projection_dim 0 / None, and the input of the global projection.
//
// Reference: bergson/collector/collector.py:609-644 (Adam), :646-700 (Adafactor), :701-742 (no
// normaliser) with p = None; bergson/gradients.py:300-349, :380-400 (normalisers).
//
// Per sequence the gradient g^T a [O, I] is a plain batched GEMM that the caller runs with its BLAS
// (the reference's `g.mT @ a`); fullgrad_seq_kernel is everything after it: normalisation, the bias
// column, clamp to the store dtype's range, cast, and the scatter into the rows of the store.
// Per token the gradient is the outer product g_t (x) a_t; fullgrad_tok_kernel forms it, normalises it
// and writes it straight to the token's row.  Both are bound by the bytes they write.

#include <algorithm>

#include "common.hpp"

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
