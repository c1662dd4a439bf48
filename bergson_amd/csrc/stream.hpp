// The streaming input path shared by the collection and the few-queries scan kernels: projection fragments
// in MFMA order, and token (store) rows streamed from HBM with whole-line non-temporal loads through a
// register queue and a wave-private LDS slot.
#pragma once

#include <type_traits>

#include "common.hpp"
#include "mma16.hpp"
#include "mma32.hpp"

namespace bgx {

constexpr int COLLECT_THREADS = 256;  // the workgroup size these helpers are written for (4 waves)
constexpr int STAGE_B = 6;            // fragments a thread keeps in flight while staging a projection

// k-steps [ks0, ks1) of the matrix; the whole of it by default.  The fragment of k-step ks goes to
// dst[(ks * nblk + blk) * 64 + lane]: nblk matrices of 16 rows interleaved per k-step (one by default).  The 16
// rows are rows row0 .. row0 + 15 of R, those past the last (p - 1) repeating it.
template <typename T>
__device__ inline void stage_projection(const T* __restrict__ R, const float* __restrict__ scale, int K, int p,
                                        uint4* __restrict__ dst, int tid, int ks0 = 0, int ks1 = -1, int blk = 0,
                                        int nblk = 1, int row0 = 0) {
  using M = Mma<T>;
  const int nfrag = (ks1 < 0 ? K / M::KS : min(ks1, K / M::KS)) * WAVE;
  constexpr int B = STAGE_B;  // fragments per thread in flight
  for (int f0 = ks0 * WAVE + tid; f0 < nfrag; f0 += COLLECT_THREADS * B) {
    uint4 v[B];
    uint4 s4[B][M::EPL / 4];
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int f = min(f0 + b * COLLECT_THREADS, nfrag - 1);
      const int ks = f >> 6, l = f & 63;
      const int r = l & 15, q = l >> 4;
      const int k0 = ks * M::KS + q * M::EPL;
      v[b] = load16_global(R + (int64_t)min(row0 + r, p - 1) * K + k0);
      if (scale != nullptr) {
#pragma unroll
        for (int e = 0; e < M::EPL / 4; ++e) s4[b][e] = load16_global(scale + k0 + 4 * e);
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int f = f0 + b * COLLECT_THREADS;
      if (scale != nullptr) {
#pragma unroll
        for (int e = 0; e < M::EPL; ++e)
          M::set(v[b], e, M::get(v[b], e) * __uint_as_float((&s4[b][e >> 2].x)[e & 3]));
      }
      if (f < nfrag) dst[((f >> 6) * nblk + blk) * WAVE + (f & 63)] = v[b];
    }
  }
}


// The same projection with the token rows streamed through registers and a wave-private LDS slot, so
// that the global loads are fully coalesced: a load instruction covers 8 token rows x 128 bytes (8 lanes
// per row) instead of 16 rows x 64 bytes, which is worth ~12 % of bandwidth by itself and -- because whole
// lines are consumed at once -- allows the non-temporal hint (+13 %, and no write-back of other kernels'
// dirty lines under this kernel).
//
// Unit = 8 rows x 128 bytes = one k-pair (two k-steps) of 8 tokens, written to LDS as it was loaded
// (lane l -> 16 bytes at l*16: row l/8, slot l%8).  Slot s of row rho of row group rg holds chunk
// s ^ rho ^ (rg & 1) of the pair, which makes the fragment reads (16 token rows x one chunk per lane
// group) conflict-free.  Needs K % (2 * KS) == 0.
//
// A wave's input is one stream of k-pairs: a of its tile, g of its tile, a of its next tile, ...  The
// stream is cut into blocks of up to STREAM_Q k-pairs (a block does not cross a segment), and the wave keeps
// exactly one block ahead in registers: while k-pair j of a block goes to LDS and through the MFMAs,
// k-pair j of the next block is already being loaded into the registers it leaves.  The loads therefore
// never drain between the blocks, the segments or the tiles of a workgroup's range.
constexpr int STREAM_Q = 4;

// A load from memory that nothing writes while the kernel runs, at an address that is the same in every
// lane: goes through the scalar unit, and so stays out of the vector memory queue (whose in-order
// completion would otherwise tie a wait for this value to every stream load issued before it).
template <typename V>
__device__ inline V load_uniform(const V* p) {
  static_assert(sizeof(V) % 4 == 0 && alignof(V) >= 4, "dword granularity");
#if defined(__HIP_DEVICE_COMPILE__)
  typedef __attribute__((address_space(4))) const uint32_t* const_ptr;
  const const_ptr src = (const_ptr)(uintptr_t)p;
  union {
    V v;
    uint32_t w[sizeof(V) / 4];
  } u;
#pragma unroll
  for (size_t i = 0; i < sizeof(V) / 4; ++i) u.w[i] = src[i];
  return u.v;
#else
  return *p;  // the host pass only parses device functions
#endif
}

template <int MTW>
struct Stream {
  static constexpr int RG = 2 * MTW;            // row groups of 8 tokens
  static constexpr int SLOT_BYTES = RG * 1024;  // one k-pair of the wave's tokens
  static constexpr int NSLOT = 1;
  static constexpr int BYTES_PER_WAVE = NSLOT * SLOT_BYTES;
};

// per-lane row pointers of a segment (at its first k-pair)
template <typename T, int MTW>
__device__ inline void stream_rows(const T* base, int64_t tok_stride, int rows_valid, int lane,
                                   const T* (&urow)[2 * MTW]) {
  const int rho = lane >> 3;
  const int sig = lane & 7;
#pragma unroll
  for (int rg = 0; rg < 2 * MTW; ++rg)
    urow[rg] = base + (int64_t)min(rg * 8 + rho, rows_valid - 1) * tok_stride + (sig ^ rho ^ (rg & 1)) * Mma<T>::EPL;
}

// The k-pair at which wave `gw` of the grid starts a segment of nkp k-pairs whose fragments come from a table in
// global memory (it then wraps around): a multiple of the queue length, 0 where the segment is too short.  Every
// wave of a launch reads the same table; walking it in step, all of them ask for the same 4 KB stretch at once
// and those requests queue at the one L2 channel that holds it.
__device__ inline int stream_rotation(int nkp, int gw) {
  const int nblk = nkp / STREAM_Q;
  return nblk >= 2 ? (int)(((unsigned)gw * 7u) % (unsigned)nblk) * STREAM_Q : 0;
}

// Every block issues exactly STREAM_Q * RG loads, in k-pair order, whatever its length: a k-pair that does
// not exist is replaced by a repeat of the block's first one, which is never used.  With that the number of
// loads between the issue of a k-pair and its use is the same on every path through the code, so the
// wait counts the compiler derives are exact (one that differed between two paths would have to be taken
// at its worst case, a full drain).  For module widths that are multiples of STREAM_Q k-pairs the only
// such repeats are at the end of a wave's last tile.
//
// With RFG the fragments do not sit in LDS but in a table in global memory, in the same fragment order (the
// few-queries scan's query table; the collection kernel uses stream_segment_shared below for its projection
// table); they then travel through the same queue: two 1 KB fragment loads per k-pair and block of columns behind
// the wave's 2 * MTW row loads.  They are ordinary cached loads -- every wave reads the same table.
//
// QB = fragment blocks of 16 columns per k-step (1 for a projection to p <= 16; the few-queries scan uses one
// block per 16 queries): acc[mt * QB + qb], table fragment ((k-step) * QB + qb).  SUMSQ also accumulates, per
// lane, the squares of the 16 bytes it carries of each row group (the caller adds up a row's 8 lanes).
//
// loads the first block of a segment (only where nothing ran ahead of it)
template <typename T, int MTW, bool RFG, int QB = 1>
__device__ inline void stream_prime(const T* const (&urow)[2 * MTW], int nkp, const uint4* __restrict__ rf, int lane,
                                    uint4 (&v)[STREAM_Q][2 * MTW], uint4 (&rq)[RFG ? STREAM_Q : 1][2 * QB]) {
#pragma unroll
  for (int j = 0; j < STREAM_Q; ++j) {
    const int jj = j < nkp ? j : 0;
#pragma unroll
    for (int rg = 0; rg < 2 * MTW; ++rg) v[j][rg] = load16_global_stream(urow[rg] + jj * 2 * Mma<T>::KS);
    if constexpr (RFG) {
#pragma unroll
      for (int s = 0; s < 2 * QB; ++s) rq[j][s] = load16_global(rf + (jj * 2 * QB + s) * WAVE + lane);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
}

// Consumes one segment (nkp k-pairs of the rows `cur`, whose first block is in v) into acc, and loads
// behind it: the later blocks of the segment, then the first block of the segment `nxt` (nkp_next = 0:
// nothing follows; nxt must still point at readable rows).  rf: the segment's fragments (LDS, or with RFG
// the global table, whose first block is in rq); rf_next: with RFG the next segment's fragments.
template <typename T, int MTW, bool RFG, int QB = 1, bool SUMSQ = false>
__device__ inline void stream_segment(const T* const (&cur)[2 * MTW], int nkp, const T* const (&nxt)[2 * MTW],
                                      int nkp_next, const uint4* __restrict__ rf, const uint4* __restrict__ rf_next,
                                      unsigned char* __restrict__ stage, int lane, uint4 (&v)[STREAM_Q][2 * MTW],
                                      uint4 (&rq)[RFG ? STREAM_Q : 1][2 * QB], f32x4 (&acc)[MTW * QB],
                                      float* __restrict__ ssq = nullptr) {
  using M = Mma<T>;
  using St = Stream<MTW>;
  constexpr int RG = St::RG;
  constexpr int Q = STREAM_Q;
  const int r = lane & 15;
  const int q = lane >> 4;
  int foff[MTW][2];  // fragment of 16-row block mt, k-step s of the pair, inside a slot
#pragma unroll
  for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
    for (int s = 0; s < 2; ++s)
      foff[mt][s] = (mt * 2 + (r >> 3)) * 1024 + (r & 7) * 128 + (((s * 4 + q) ^ (r & 7) ^ (r >> 3)) << 4);

  for (int kp0 = 0; kp0 < nkp; kp0 += Q) {
    const int len = min(Q, nkp - kp0);
    const bool last = kp0 + Q >= nkp;
    const int len_next = last ? min(Q, nkp_next) : min(Q, nkp - kp0 - Q);
    const T* nptr[RG];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) nptr[rg] = last ? nxt[rg] : cur[rg] + (kp0 + Q) * 2 * M::KS;
    const uint4* nrf = last ? rf_next : rf + (kp0 + Q) * 2 * QB * WAVE;  // RFG only

    auto step = [&](auto j_tag) {
      constexpr int j = decltype(j_tag)::value;
      unsigned char* slot = stage + (j % St::NSLOT) * St::SLOT_BYTES;
      if (j < len) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
          *reinterpret_cast<uint4*>(slot + rg * 1024 + lane * 16) = v[j][rg];
          if constexpr (SUMSQ) ssq[rg] = Mma32<T>::sumsq(v[j][rg], ssq[rg]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      const int jj = j < len_next ? j : 0;
      auto refill = [&]() {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) v[j][rg] = load16_global_stream(nptr[rg] + jj * 2 * M::KS);
        if constexpr (RFG) {
#pragma unroll
          for (int s = 0; s < 2 * QB; ++s) rq[j][s] = load16_global(nrf + (jj * 2 * QB + s) * WAVE + lane);
        }
      };
      // LDS fragments: the refill goes out before the MFMAs.  Table fragments: after them -- rq[j] is
      // still needed by this step's MFMAs, and a refill issued earlier would have to land in other
      // registers, which the loop could only hand over with moves that wait for the loads.
      if constexpr (!RFG) {
        refill();
        __builtin_amdgcn_sched_barrier(0);
      }
      if (j < len) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          uint4 rfv[QB];
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) {
            if constexpr (RFG)
              rfv[qb] = rq[j][s * QB + qb];
            else
              rfv[qb] = rf[(((kp0 + j) * 2 + s) * QB + qb) * WAVE + lane];
          }
#pragma unroll
          for (int mt = 0; mt < MTW; ++mt) {
            const uint4 xf = *reinterpret_cast<const uint4*>(slot + foff[mt][s]);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) M::mma(xf, rfv[qb], acc[mt * QB + qb]);
          }
        }
      }
      if constexpr (RFG) {
        __builtin_amdgcn_sched_barrier(0);
        refill();
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // one code path for full and partial blocks: a second, unguarded copy of the steps would meet this one
    // at a join, where the queue registers of the two have to be reconciled by moves that wait for the loads
    step(std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 1>{});
    step(std::integral_constant<int, 2>{});
    step(std::integral_constant<int, 3>{});
  }
}
static_assert(STREAM_Q == 4, "stream_segment spells out its four steps");

// ---- table fragments shared by the workgroup --------------------------------------------------------------------
// With the fragments in the global table each wave of stream_segment<RFG> loads every fragment for itself: 2 * QB KB
// per k-pair and wave beside its 2 * MTW KB of rows.  Those loads hit in the L2s, but they pass through the compute
// unit's one vector memory pipeline behind the rows' misses, and what they cost is its time (about 21 cycles per
// 1 KB load, added to a step whose rows take HBM's time: four waves at QB = 4 spend 670 of a step's 2170 cycles on
// them).  Here the four waves of a workgroup -- which walk the same k-pairs of the same module at the same time --
// load each fragment once: of a block of STREAM_Q = 4 k-pairs wave w fetches k-pair w (2 * QB loads into rs, one
// block ahead like the rows), writes it to one of two LDS slots at the start of the block, and after a barrier
// every wave reads the block's fragments from there.  One barrier per block: the slot written for block b + 1 was
// last read during block b - 1, which every wave has left when it has passed the barrier of block b.
// Every wave of the workgroup must call these with the same nkp / nkp_next sequence (the barrier); a wave without
// rows of its own passes rows that are safe to read and discards what it accumulates.
constexpr int stream_ring_bytes(int qb) { return 2 * STREAM_Q * 2 * qb * WAVE * 16; }

// bare barrier: the LDS writes of this wave are done, the global loads in flight stay in flight
__device__ inline void stream_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <typename T, int MTW, int QB>
__device__ inline void stream_prime_shared(const T* const (&urow)[2 * MTW], int nkp, const uint4* __restrict__ rf,
                                           int lane, int wave, uint4 (&v)[STREAM_Q][2 * MTW], uint4 (&rs)[2 * QB]) {
  // the fragments first, as in a block of the segment: on every path into a block its fragment loads then have
  // exactly the block's STREAM_Q * 2 * MTW row loads behind them, and the wait in front of the ring write is that count
  const int wj = wave < nkp ? wave : 0;
#pragma unroll
  for (int s = 0; s < 2 * QB; ++s) rs[s] = load16_global(rf + (wj * 2 * QB + s) * WAVE + lane);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < STREAM_Q; ++j) {
    const int jj = j < nkp ? j : 0;
#pragma unroll
    for (int rg = 0; rg < 2 * MTW; ++rg) v[j][rg] = load16_global_stream(urow[rg] + jj * 2 * Mma<T>::KS);
  }
  __builtin_amdgcn_sched_barrier(0);
}

// ring: the two LDS slots (stream_ring_bytes); ring_slot: which of them the block that comes next uses (kept by the
// caller across segments)
template <typename T, int MTW, int QB, bool SUMSQ = false>
__device__ inline void stream_segment_shared(const T* const (&cur)[2 * MTW], int nkp, const T* const (&nxt)[2 * MTW],
                                             int nkp_next, const uint4* __restrict__ rf,
                                             const uint4* __restrict__ rf_next, unsigned char* __restrict__ stage,
                                             uint4* __restrict__ ring, int& ring_slot, int lane, int wave,
                                             uint4 (&v)[STREAM_Q][2 * MTW], uint4 (&rs)[2 * QB],
                                             f32x4 (&acc)[MTW * QB], float* __restrict__ ssq = nullptr) {
  using M = Mma<T>;
  using St = Stream<MTW>;
  constexpr int RG = St::RG;
  constexpr int Q = STREAM_Q;
  constexpr int SLOT = Q * 2 * QB * WAVE;  // uint4 entries of a ring slot
  const int r = lane & 15;
  const int q = lane >> 4;
  int foff[MTW][2];  // fragment of 16-row block mt, k-step s of the pair, inside a slot
#pragma unroll
  for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
    for (int s = 0; s < 2; ++s)
      foff[mt][s] = (mt * 2 + (r >> 3)) * 1024 + (r & 7) * 128 + (((s * 4 + q) ^ (r & 7) ^ (r >> 3)) << 4);

  for (int kp0 = 0; kp0 < nkp; kp0 += Q) {
    const int len = min(Q, nkp - kp0);
    const bool last = kp0 + Q >= nkp;
    const int len_next = last ? min(Q, nkp_next) : min(Q, nkp - kp0 - Q);
    const T* nptr[RG];
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) nptr[rg] = last ? nxt[rg] : cur[rg] + (kp0 + Q) * 2 * M::KS;
    const uint4* nrf = last ? rf_next : rf + (kp0 + Q) * 2 * QB * WAVE;

    // this wave's k-pair of the block goes to the ring; behind the barrier the whole block is there
    uint4* slotf = ring + ring_slot * SLOT;
#pragma unroll
    for (int s = 0; s < 2 * QB; ++s) slotf[(wave * 2 * QB + s) * WAVE + lane] = rs[s];
    stream_barrier();
    __builtin_amdgcn_sched_barrier(0);
    {  // its k-pair of the block that follows (k-pair 0 again where that block is shorter: never used)
      const int wj = wave < len_next ? wave : 0;
#pragma unroll
      for (int s = 0; s < 2 * QB; ++s) rs[s] = load16_global(nrf + (wj * 2 * QB + s) * WAVE + lane);
    }
    __builtin_amdgcn_sched_barrier(0);

    auto step = [&](auto j_tag) {
      constexpr int j = decltype(j_tag)::value;
      if (j < len) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) {
          *reinterpret_cast<uint4*>(stage + rg * 1024 + lane * 16) = v[j][rg];
          if constexpr (SUMSQ) ssq[rg] = Mma32<T>::sumsq(v[j][rg], ssq[rg]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      const int jj = j < len_next ? j : 0;
#pragma unroll
      for (int rg = 0; rg < RG; ++rg) v[j][rg] = load16_global_stream(nptr[rg] + jj * 2 * M::KS);
      __builtin_amdgcn_sched_barrier(0);
      if (j < len) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          uint4 rfv[QB];
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) rfv[qb] = slotf[((j * 2 + s) * QB + qb) * WAVE + lane];
#pragma unroll
          for (int mt = 0; mt < MTW; ++mt) {
            const uint4 xf = *reinterpret_cast<const uint4*>(stage + foff[mt][s]);
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) M::mma(xf, rfv[qb], acc[mt * QB + qb]);
          }
        }
      }
    };
    step(std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 1>{});
    step(std::integral_constant<int, 2>{});
    step(std::integral_constant<int, 3>{});
    ring_slot ^= 1;
  }
}


}  // namespace bgx
