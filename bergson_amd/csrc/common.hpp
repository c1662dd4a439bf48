// Shared device/host helpers of the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "bergson_amd.h"

namespace bgx {

// ---- host-side error plumbing (defined in capi.hip) -----------------------
void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define BGX_HIP(call)                                  \
  do {                                                 \
    hipError_t e__ = (call);                           \
    if (e__ != hipSuccess) return hip_fail(e__, #call); \
  } while (0)

#define BGX_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) {                   \
      set_error(__VA_ARGS__);        \
      return (code);                 \
    }                                \
  } while (0)

// ---- diagnostic switches (defined in capi.hip) --------------------------------
// BGX_* environment variables that force a kernel variant, for tests and comparisons.  They are read once,
// on first use, into an immutable record; bgx_reload_switches() publishes a fresh one.
struct Switches {
  bool adam_fused_off = false;    // BGX_ADAM_FUSED_OFF set
  bool adam_wide_off = false;     // BGX_ADAM_WIDE_OFF set: eight waves of 64 x 128 where four of 128 x 128 would run
  int adam_ttx = -1;              // BGX_ADAM_TTX (token tiles per XCD group), -1 = unset
  bool collect_staged = true;     // BGX_COLLECT_STAGED != "0"
  bool collect_persist = true;    // BGX_COLLECT_PERSIST != "0"
  bool collect_lpt_off = false;   // BGX_COLLECT_LPT_OFF set
  bool collect_two_step_off = false;  // BGX_COLLECT_TWO_STEP_OFF set: per-token rows written by the collection kernel itself
  bool scan_direct_off = false;   // BGX_SCAN_DIRECT_OFF set
  bool scan_stream_off = false;   // BGX_SCAN_STREAM_OFF set
  bool scan_wide_off = false;     // BGX_SCAN_WIDE_OFF set
  bool wgrad_big_off = false;     // BGX_WGRAD_BIG_OFF set: per-sequence weight gradients on 64 x 64 tiles only
};
const Switches& switches();

// ---- which kernel ran (defined in capi.hip) -------------------------------------
// Every entry point with more than one kernel behind it notes the name of the main kernel it enqueued, per
// calling thread and family; bgx_last_kernel() reads it back.  Tests use it to assert a route without
// forcing one through the switches above.
enum KernelFamily { FAMILY_COLLECT = 0, FAMILY_ADAM = 1, FAMILY_SCAN = 2, FAMILY_FULLGRAD = 3, FAMILY_COUNT = 4 };
void note_kernel(int family, const char* name);
const char* noted_kernel(int family);

// ---- vector types for the MFMA builtins -----------------------------------
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

// Element tags: the kernels are templated on these; the 16-bit types are
// carried as raw bits and only converted through the helpers below.
struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  uint16_t bits;
};

constexpr int WAVE = 64;

// 16-byte load from device memory.  Pointers that come out of a descriptor table carry no address
// space, and the compiler then falls back to generic ("flat") loads, which it cannot keep in flight
// next to LDS traffic; this tells it the pointer is a plain global one.
// The same with the non-temporal hint, for data that is read exactly once: it does not displace what the
// caches hold, so the dirty lines earlier kernels left behind are not written back under this kernel.
// Only for access patterns in which one load instruction consumes whole 128-byte lines -- a line that is
// not retained is fetched again by the next instruction that touches its other half.
__device__ inline uint4 load16_global_stream(const void* p) {
  typedef uint32_t raw4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(1))) const raw4* global_ptr;
  const raw4 v = __builtin_nontemporal_load((global_ptr)(uintptr_t)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ inline uint4 load16_global(const void* p) {
  typedef uint32_t raw4 __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(1))) const raw4* global_ptr;
  const raw4 v = *(global_ptr)(uintptr_t)p;
  return make_uint4(v.x, v.y, v.z, v.w);
}

__host__ __device__ inline size_t dtype_size(int dt) {
  return dt == BGX_F32 ? 4 : 2;
}

// ---- scalar conversions ----------------------------------------------------
__device__ inline float bf16_bits_to_f32(uint32_t b) {
  return __uint_as_float(b << 16);
}
// round-to-nearest-even, NaN kept quiet: the hardware conversion (v_cvt_pk_bf16_f32)
__device__ inline uint32_t f32_to_bf16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}
// two values at once, the first in the low half
__device__ inline uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  typedef float f2 __attribute__((ext_vector_type(2)));
  const f2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, b2));
}
__device__ inline uint32_t f32x2_to_f16x2_bits(float lo, float hi) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 r = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, r);
}
__device__ inline float f16_bits_to_f32(uint32_t b) {
  union {
    uint16_t u;
    _Float16 h;
  } c;
  c.u = (uint16_t)b;
  return (float)c.h;
}
__device__ inline uint32_t f32_to_f16_bits(float f) {
  union {
    uint16_t u;
    _Float16 h;
  } c;
  c.h = (_Float16)f;
  return c.u;
}

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static constexpr int code = BGX_F32;
  __device__ static float load(const float* p) { return *p; }
  __device__ static float round(float x) { return x; }
};
template <>
struct Elem<bf16_t> {
  static constexpr int code = BGX_BF16;
  __device__ static float load(const bf16_t* p) { return bf16_bits_to_f32(p->bits); }
  __device__ static float round(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }
};
template <>
struct Elem<f16_t> {
  static constexpr int code = BGX_F16;
  __device__ static float load(const f16_t* p) { return f16_bits_to_f32(p->bits); }
  __device__ static float round(float x) { return f16_bits_to_f32(f32_to_f16_bits(x)); }
};

// value rounded to the representable set of dtype `dt`
__device__ inline float round_to_dtype(float x, int dt) {
  if (dt == BGX_BF16) return Elem<bf16_t>::round(x);
  if (dt == BGX_F16) return Elem<f16_t>::round(x);
  return x;
}

// store one value as dtype `dt` at element index idx of base
__device__ inline void store_as(void* base, int64_t idx, float v, int dt) {
  if (dt == BGX_F32) {
    ((float*)base)[idx] = v;
  } else if (dt == BGX_F16) {
    ((uint16_t*)base)[idx] = (uint16_t)f32_to_f16_bits(v);
  } else {
    ((uint16_t*)base)[idx] = (uint16_t)f32_to_bf16_bits(v);
  }
}

// eight consecutive values at once; base + idx must be 16-byte aligned in the output dtype DT
template <int DT>
__device__ inline void store8_as(void* base, int64_t idx, const float (&v)[8]) {
  if constexpr (DT == BGX_F32) {
    typedef float raw4 __attribute__((ext_vector_type(4)));
    raw4* dst = reinterpret_cast<raw4*>((float*)base + idx);
    __builtin_nontemporal_store(raw4{v[0], v[1], v[2], v[3]}, dst);
    __builtin_nontemporal_store(raw4{v[4], v[5], v[6], v[7]}, dst + 1);
  } else {
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      w[k] = DT == BGX_F16 ? f32x2_to_f16x2_bits(v[2 * k], v[2 * k + 1]) : f32x2_to_bf16x2_bits(v[2 * k], v[2 * k + 1]);
    typedef uint32_t raw4 __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(raw4{w[0], w[1], w[2], w[3]}, reinterpret_cast<raw4*>((uint16_t*)base + idx));
  }
}

__device__ inline float load_as(const void* base, int64_t idx, int dt) {
  if (dt == BGX_F32) return ((const float*)base)[idx];
  if (dt == BGX_F16) return f16_bits_to_f32(((const uint16_t*)base)[idx]);
  return bf16_bits_to_f32(((const uint16_t*)base)[idx]);
}

__device__ inline float clampf(float v, float lo, float hi) {
  // lo <= hi; the median of the three is the clamped value (one instruction), and NaN propagates like
  // torch.clamp (the median instruction alone would turn it into lo)
  const float r = __builtin_amdgcn_fmed3f(v, lo, hi);
  return v != v ? v : r;
}

}  // namespace bgx
