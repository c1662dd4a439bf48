// Tiles loaded straight from global memory into LDS, and fragments read back from them by hand: the pieces
// shared by the store scan's tile kernels and the fused Adam kernel.
//
// LDS tile rows are 128 bytes (64 elements of a 16-bit type), unpadded; 16-byte chunk c of row r sits at position
// c ^ sd_key(r), which the loader produces by choosing which global chunk each lane fetches (a load instruction
// fills 8 whole rows: lane l is position l & 7 of row l >> 3) and which makes the fragment reads of 32
// consecutive rows conflict-free.
#pragma once

#include <type_traits>

#include "common.hpp"

namespace bgx {

constexpr int SD_ROW = 128;

__device__ inline int sd_key(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// Workgroup barrier without a fence (a fence would wait for every load in flight): waits for this wave's LDS
// traffic, and for all but the youngest VM_LEFT of its vector-memory operations, then s_barrier.  The memory
// clobber keeps the compiler from moving memory accesses across it.
template <int VM_LEFT>
__device__ inline void wg_barrier_lds() {
  static_assert(VM_LEFT == 0 || VM_LEFT == 4 || VM_LEFT == 8, "spelled-out wait counts");
  if constexpr (VM_LEFT == 0)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  else if constexpr (VM_LEFT == 4)
    asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  else
    asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 16 bytes from LDS byte address `addr`; the caller waits (lgkmcnt) before it uses the value
__device__ inline uint4 sd_lds_read16(uint32_t addr) {
  uint4 v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
  return v;
}

template <int OFF>
__device__ inline uint4 sw_lds_read16(uint32_t addr) {
  uint4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
  return v;
}

// 16 bytes per lane from global memory (uniform 64-bit base + one 32-bit offset per lane) straight to LDS at
// byte address `lds` + 16 * lane.  Spelled out so that a load is four instructions (M0, the wait state it needs,
// the load, and at most one add for the offset) -- the builtin went through 64-bit vector address arithmetic.
__device__ inline void sw_load_lds16(uint64_t base, uint32_t voff, uint32_t lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(base), "s"(lds)
               : "memory", "m0");
}

// One 32 x 32 x 16 MFMA with the accumulator block pinned to the AccVGPRs (IN_ACC) or to the ordinary VGPRs.
// Written as instructions: in kernels whose accumulators fill most of the register file (one wave per SIMD) the
// register allocator has no slack, and left to itself it shuffles blocks between the two files and spills.  (Volatile: the statements
// execute in the order they are written, which is the hand-made schedule.)
template <typename T, bool IN_ACC>
__device__ inline void sw_mfma(const uint4& a, const uint4& b, f32x16& c) {
  typedef uint32_t raw4 __attribute__((ext_vector_type(4)));
  const raw4 av = {a.x, a.y, a.z, a.w}, bv = {b.x, b.y, b.z, b.w};
  if constexpr (std::is_same<T, f16_t>::value) {
    if constexpr (IN_ACC)
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(bv));
    else
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "v"(bv));
  } else {
    if constexpr (IN_ACC)
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(bv));
    else
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(av), "v"(bv));
  }
}

}  // namespace bgx
