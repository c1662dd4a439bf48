// 16x16 MFMA steps shared by the collection and Adam kernels.
#pragma once

#include "common.hpp"

namespace bgx {

// ---- MFMA step per element type ---------------------------------------------
// A "k-step" of one wave covers KS consecutive k; lane (r = lane%16, q = lane/16)
// holds EPL consecutive elements starting at k0 + q*EPL of row r (16 bytes).
template <typename T>
struct Mma;

template <>
struct Mma<bf16_t> {
  static constexpr int EPL = 8;
  static constexpr int KS = 32;
  __device__ static void mma(const uint4& a, const uint4& b, f32x4& c) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  __device__ static float get(const uint4& v, int e) {
    const uint32_t w = (&v.x)[e >> 1];
    return bf16_bits_to_f32((e & 1) ? (w >> 16) : (w & 0xffffu));
  }
  __device__ static void set(uint4& v, int e, float f) {
    uint32_t& w = (&v.x)[e >> 1];
    const uint32_t b = f32_to_bf16_bits(f);
    w = (e & 1) ? ((w & 0x0000ffffu) | (b << 16)) : ((w & 0xffff0000u) | b);
  }
};

template <>
struct Mma<f16_t> {
  static constexpr int EPL = 8;
  static constexpr int KS = 32;
  __device__ static void mma(const uint4& a, const uint4& b, f32x4& c) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                               __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  __device__ static float get(const uint4& v, int e) {
    const uint32_t w = (&v.x)[e >> 1];
    return f16_bits_to_f32((e & 1) ? (w >> 16) : (w & 0xffffu));
  }
  __device__ static void set(uint4& v, int e, float f) {
    uint32_t& w = (&v.x)[e >> 1];
    const uint32_t b = f32_to_f16_bits(f);
    w = (e & 1) ? ((w & 0x0000ffffu) | (b << 16)) : ((w & 0xffff0000u) | b);
  }
};

template <>
struct Mma<float> {
  static constexpr int EPL = 4;
  static constexpr int KS = 16;
  // four K=4 MFMAs; MFMA e consumes element e of every lane, i.e. the k set
  // {k0 + 4q + e : q = 0..3}; A and B use the same assignment so the sum over
  // k is complete.
  __device__ static void mma(const uint4& a, const uint4& b, f32x4& c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
  }
  __device__ static float get(const uint4& v, int e) { return __uint_as_float((&v.x)[e]); }
  __device__ static void set(uint4& v, int e, float f) { (&v.x)[e] = __float_as_uint(f); }
};

}  // namespace bgx
