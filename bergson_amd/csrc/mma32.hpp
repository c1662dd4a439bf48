// 32x32 MFMA steps and the LDS tile geometry shared by the store-scan GEMM and the fused Adam kernel.
#pragma once

#include "common.hpp"

namespace bgx {

// ---- element traits for the 32x32 MFMA tiles ------------------------------------
// One "substep" consumes a 16-byte fragment per lane for A and for B:
// lane (r = lane%32, h = lane/32) holds EPL consecutive k starting at h*EPL.
template <typename T>
struct Mma32;

template <>
struct Mma32<f16_t> {
  static constexpr int EPL = 8;
  __device__ static void mma(const uint4& a, const uint4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                               0, 0, 0);
  }
  __device__ static float sumsq(const uint4& v, float s) {
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.x), __builtin_bit_cast(h2, v.x), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.y), __builtin_bit_cast(h2, v.y), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.z), __builtin_bit_cast(h2, v.z), s, false);
    s = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.w), __builtin_bit_cast(h2, v.w), s, false);
    return s;
  }
  // the E-th of sumsq's four steps (the four in order give the same bits)
  template <int E>
  __device__ static float sumsq_part(const uint4& v, float s) {
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    const uint32_t w = E == 0 ? v.x : E == 1 ? v.y : E == 2 ? v.z : v.w;
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w), __builtin_bit_cast(h2, w), s, false);
  }
};

template <>
struct Mma32<bf16_t> {
  static constexpr int EPL = 8;
  __device__ static void mma(const uint4& a, const uint4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                c, 0, 0, 0);
  }
  __device__ static float sumsq(const uint4& v, float s) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float lo = __uint_as_float(w[i] << 16);
      const float hi = __uint_as_float(w[i] & 0xffff0000u);
      s = fmaf(lo, lo, s);
      s = fmaf(hi, hi, s);
    }
    return s;
  }
  template <int E>
  __device__ static float sumsq_part(const uint4& v, float s) {
    const uint32_t w = E == 0 ? v.x : E == 1 ? v.y : E == 2 ? v.z : v.w;
    const float lo = __uint_as_float(w << 16);
    const float hi = __uint_as_float(w & 0xffff0000u);
    s = fmaf(lo, lo, s);
    return fmaf(hi, hi, s);
  }
};

template <>
struct Mma32<float> {
  static constexpr int EPL = 4;
  // four K=2 MFMAs; MFMA e consumes element e of both halves of the wave.
  __device__ static void mma(const uint4& a, const uint4& b, f32x16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
  __device__ static float sumsq(const uint4& v, float s) {
    const float x = __uint_as_float(v.x), y = __uint_as_float(v.y), z = __uint_as_float(v.z),
                w = __uint_as_float(v.w);
    s = fmaf(x, x, s);
    s = fmaf(y, y, s);
    s = fmaf(z, z, s);
    s = fmaf(w, w, s);
    return s;
  }
};

// LDS tile rows: BK elements of K (128 bytes) plus 16 bytes of padding against bank conflicts.
constexpr int TILE_ROW_BYTES = 128;
constexpr int TILE_CHUNKS = TILE_ROW_BYTES / 16;
constexpr int LDS_ROW_BYTES = TILE_ROW_BYTES + 16;

// 16 bytes of row `row` of a [n_rows, K] matrix starting at element k; zero outside the matrix.
// STREAM: the data is read once by the launch and every load instruction consumes whole 128-byte lines
// (non-temporal hint; aligned rows only).
template <typename T, bool ALIGNED, bool STREAM = false>
__device__ inline uint4 load_chunk(const T* __restrict__ base, int64_t row, int64_t n_rows, int64_t stride,
                                   int64_t k, int64_t K) {
  constexpr int EPL = Mma32<T>::EPL;
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (row >= n_rows || k >= K) return v;
  const T* p = base + row * stride + k;
  if (ALIGNED) {
    if constexpr (STREAM)
      v = load16_global_stream(p);
    else
      v = *reinterpret_cast<const uint4*>(p);
  } else {
    if constexpr (sizeof(T) == 4) {
      uint32_t* w = &v.x;
      for (int e = 0; e < EPL; ++e)
        if (k + e < K) w[e] = *reinterpret_cast<const uint32_t*>(p + e);
    } else {
      uint32_t* w = &v.x;
      for (int e = 0; e < EPL; ++e)
        if (k + e < K) {
          const uint32_t b = *reinterpret_cast<const uint16_t*>(p + e);
          w[e >> 1] |= (e & 1) ? (b << 16) : b;
        }
    }
  }
  return v;
}

}  // namespace bgx
