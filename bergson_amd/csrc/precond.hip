// Dense per-module preconditioner on the gradient rows.
//
//   bgx_block_gemm:       out[n, c0 : c0+d] = fp32(in[n, c0 : c0+d]) @ H        (H [d, d] fp32, one per module)
//   bgx_gram_accumulate:  H += fp32(rows[:, c0 : c0+d])^T @ fp32(rows[:, c0 : c0+d])
//
// i.e. DensePreconditioner.apply (bergson/hessians/preconditioner.py:77-92, the per-module `g @ H^p` that
// bergson/builder.py:17-32 and bergson/query/attributor.py:138-145, :195-200 call, and the batched form in
// bergson/score/score.py:111-135) and the autocorrelation Gram accumulation of
// bergson/collector/in_memory_collector.py:149-154 (`hessians[name].addmm_(P.mT, P)` on `P.float()`).
//
// Both are fp32 GEMMs on v_mfma_f32_16x16x4_f32 (the reference computes them in fp32, and the parity bar for
// fp32 is 1e-5).  One workgroup (4 waves, 2 x 2) owns a 128 x 128 output tile of one module and walks K in
// chunks of 16 through double-buffered LDS tiles kept k-major, [k][row] and [k][col] with a row pitch of
// 144 floats: a lane (r = lane % 16, q = lane / 16) reads element [k0 + q][r0 + r], and 144 % 64 = 16 puts the
// 64 lanes of such a read on 64 different banks.  For the apply the A tile is transposed on its way into
// LDS; for the Gram both operands are the same row-major [n][column] block, which already is k-major.
// Every output tile has one owner and the accumulation order is fixed: no atomics, results are
// reproducible run to run.
#include <algorithm>
#include <vector>

#include "common.hpp"

namespace bgx {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int PG_TILE = 128;   // output tile edge
constexpr int PG_KC = 16;      // K chunk
constexpr int PG_PITCH = 144;  // floats per k row of an LDS tile
constexpr int PG_THREADS = 256;

struct BlockDev {
  float* h;         // [dim, dim] fp32
  int64_t col0;     // first column of the module in a row
  int32_t dim;
  int32_t aligned;  // rows of this block can be read with 16-byte loads
};

struct PrecondArgs {
  const void* in;
  int64_t in_stride;
  int in_dtype;
  void* out;
  int64_t out_stride;
  int out_dtype;
  int64_t rows;
  const BlockDev* blocks;
};

// fp32 value of element `idx` of a row in dtype DT
template <int DT>
__device__ inline float elem_as_f32(const void* base, int64_t idx) {
  if constexpr (DT == BGX_F32) return ((const float*)base)[idx];
  if constexpr (DT == BGX_F16) return f16_bits_to_f32(((const uint16_t*)base)[idx]);
  return bf16_bits_to_f32(((const uint16_t*)base)[idx]);
}

// Four consecutive elements starting at column k of row `row` (zero outside rows x dim) as fp32.
template <int DT>
__device__ inline void load4(const void* base, int64_t stride, int64_t row, int64_t n_rows, int64_t col0, int k,
                             int dim, bool aligned, float (&v)[4]) {
  v[0] = v[1] = v[2] = v[3] = 0.f;
  if (row >= n_rows || k >= dim) return;
  const int64_t idx = row * stride + col0 + k;
  if (aligned && k + 4 <= dim) {
    if constexpr (DT == BGX_F32) {
      const float4 x = *reinterpret_cast<const float4*>((const float*)base + idx);
      v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
    } else {
      const uint2 x = *reinterpret_cast<const uint2*>((const uint16_t*)base + idx);
      const uint32_t w[2] = {x.x, x.y};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t b = (w[e >> 1] >> ((e & 1) * 16)) & 0xffffu;
        v[e] = DT == BGX_F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (k + e < dim) v[e] = elem_as_f32<DT>(base, idx + e);
  }
}

// One K chunk from LDS: acc[i][j] += A^T[k][wm*64 + 16 i + r]^T B[k][wn*64 + 16 j + c]
__device__ inline void mma_chunk(const float* __restrict__ at, const float* __restrict__ bt, int lane, int wm, int wn,
                                 f32x4 (&acc)[4][4]) {
  const int r = lane & 15;
  const int q = lane >> 4;
#pragma unroll
  for (int k0 = 0; k0 < PG_KC; k0 += 4) {
    float a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = at[(k0 + q) * PG_PITCH + wm * 64 + i * 16 + r];
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = bt[(k0 + q) * PG_PITCH + wn * 64 + j * 16 + r];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc[i][j], 0, 0, 0);
  }
}

// GRAM = false: out tile = in rows x H.   grid (row tiles, column tiles, blocks)
// GRAM = true:  H tile += in^T in.        grid (tiles of i, tiles of j, blocks); K runs over the rows
template <int DT, bool GRAM>
__global__ __launch_bounds__(PG_THREADS) void precond_kernel(PrecondArgs args) {
  __shared__ __align__(16) float lds[2][2][PG_KC * PG_PITCH];  // [buffer][A^T / B]
  const BlockDev blk = args.blocks[blockIdx.z];
  const int dim = blk.dim;
  const int64_t m0 = (int64_t)blockIdx.x * PG_TILE;  // first output row (GRAM: first i)
  const int n0 = blockIdx.y * PG_TILE;               // first output column
  if (n0 >= dim || (GRAM && m0 >= dim)) return;
  const int64_t K = GRAM ? args.rows : dim;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const bool aligned = blk.aligned != 0;
  const bool h_aligned = (dim & 3) == 0 && ((uintptr_t)blk.h & 15) == 0;

  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // staging registers: U groups of 4 floats per operand and thread
  constexpr int U = PG_KC / 8;
  constexpr int KG = PG_KC / 4;  // groups of 4 k per row of the A tile
  float ra[U][4], rb[U][4];
  auto gload = [&](int64_t kc) {
    if constexpr (GRAM) {
      // A^T[k][i] = in[kc + k][c0 + m0 + i], B[k][j] = in[kc + k][c0 + n0 + j]: KC rows x 32 groups of 4 columns
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int x = tid + u * PG_THREADS;
        const int k = x >> 5, c4 = (x & 31) * 4;
        load4<DT>(args.in, args.in_stride, kc + k, args.rows, blk.col0, (int)m0 + c4, dim, aligned, ra[u]);
        load4<DT>(args.in, args.in_stride, kc + k, args.rows, blk.col0, n0 + c4, dim, aligned, rb[u]);
      }
    } else {
      // A[row][k]: 128 rows x KG groups of 4 k;  B[k][col] = H[kc + k][n0 + col]: KC k x 32 groups of 4 columns
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int x = tid + u * PG_THREADS;
        const int row = x / KG, k4 = (x % KG) * 4;
        load4<DT>(args.in, args.in_stride, m0 + row, args.rows, blk.col0, (int)kc + k4, dim, aligned, ra[u]);
        const int k = x >> 5, c4 = (x & 31) * 4;
        load4<BGX_F32>(blk.h, dim, kc + k, dim, 0, n0 + c4, dim, h_aligned, rb[u]);
      }
    }
  };
  auto lstore = [&](int buf) {
    float* at = lds[buf][0];
    float* bt = lds[buf][1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int x = tid + u * PG_THREADS;
      if constexpr (GRAM) {
        const int k = x >> 5, c4 = (x & 31) * 4;
        *reinterpret_cast<float4*>(at + k * PG_PITCH + c4) = make_float4(ra[u][0], ra[u][1], ra[u][2], ra[u][3]);
        *reinterpret_cast<float4*>(bt + k * PG_PITCH + c4) = make_float4(rb[u][0], rb[u][1], rb[u][2], rb[u][3]);
      } else {
        const int row = x / KG, k4 = (x % KG) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) at[(k4 + e) * PG_PITCH + row] = ra[u][e];
        const int k = x >> 5, c4 = (x & 31) * 4;
        *reinterpret_cast<float4*>(bt + k * PG_PITCH + c4) = make_float4(rb[u][0], rb[u][1], rb[u][2], rb[u][3]);
      }
    }
  };

  const int64_t chunks = (K + PG_KC - 1) / PG_KC;
  gload(0);
  lstore(0);
  __syncthreads();
  for (int64_t ch = 0; ch < chunks; ++ch) {
    const int buf = (int)(ch & 1);
    if (ch + 1 < chunks) gload((ch + 1) * PG_KC);
    mma_chunk(lds[buf][0], lds[buf][1], lane, wm, wn, acc);
    if (ch + 1 < chunks) lstore(buf ^ 1);
    __syncthreads();
  }

  // lane (c, q) holds rows 4q + e, column c of each 16 x 16 tile
  const int c = lane & 15;
  const int q = lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + wn * 64 + j * 16 + c;
      if (col >= dim) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int64_t row = m0 + wm * 64 + i * 16 + q * 4 + e;
        if constexpr (GRAM) {
          if (row < dim) blk.h[row * dim + col] += acc[i][j][e];
        } else {
          if (row < args.rows) store_as(args.out, row * args.out_stride + blk.col0 + col, acc[i][j][e], args.out_dtype);
        }
      }
    }
}

size_t precond_workspace_bytes(int n_blocks) { return (size_t)std::max(n_blocks, 1) * sizeof(BlockDev); }

static int precond_impl(bool gram, const void* in, int in_dtype, int64_t in_stride, void* out, int out_dtype,
                        int64_t out_stride, int64_t rows, const bgx_block_desc* blocks, int n_blocks, void* ws,
                        size_t ws_bytes, void* stream) {
  BGX_REQUIRE(in && blocks && ws, BGX_E_ARG, "precond: null rows/blocks/workspace");
  BGX_REQUIRE(n_blocks > 0 && rows >= 0, BGX_E_ARG, "precond: n_blocks=%d rows=%lld", n_blocks, (long long)rows);
  BGX_REQUIRE(in_dtype == BGX_F32 || in_dtype == BGX_F16 || in_dtype == BGX_BF16, BGX_E_ARG, "precond: in_dtype=%d",
              in_dtype);
  BGX_REQUIRE(ws_bytes >= precond_workspace_bytes(n_blocks), BGX_E_ARG, "precond: workspace too small");
  if (!gram) {
    BGX_REQUIRE(out && out != in, BGX_E_ARG, "block_gemm: out must be a buffer of its own");
    BGX_REQUIRE(out_dtype == BGX_F32 || out_dtype == BGX_F16 || out_dtype == BGX_BF16, BGX_E_ARG,
                "block_gemm: out_dtype=%d", out_dtype);
  }
  if (rows == 0) return 0;
  const int64_t elem = in_dtype == BGX_F32 ? 4 : 2;
  std::vector<BlockDev> dev((size_t)n_blocks);
  int max_dim = 0;
  for (int b = 0; b < n_blocks; ++b) {
    BGX_REQUIRE(blocks[b].h_dev && blocks[b].dim > 0 && blocks[b].col0 >= 0, BGX_E_ARG, "precond: block %d", b);
    dev[b].h = blocks[b].h_dev;
    dev[b].col0 = blocks[b].col0;
    dev[b].dim = blocks[b].dim;
    // four elements per load: 16 bytes of fp32, 8 bytes of a 16-bit type
    const int64_t unit = 4 * elem;
    dev[b].aligned = (uintptr_t)in % unit == 0 && (in_stride * elem) % unit == 0 && (blocks[b].col0 * elem) % unit == 0 &&
                     blocks[b].dim % 4 == 0;
    max_dim = std::max(max_dim, blocks[b].dim);
  }
  hipStream_t st = (hipStream_t)stream;
  BGX_HIP(hipMemcpyAsync(ws, dev.data(), dev.size() * sizeof(BlockDev), hipMemcpyHostToDevice, st));
  PrecondArgs args;
  args.in = in;
  args.in_stride = in_stride;
  args.in_dtype = in_dtype;
  args.out = out;
  args.out_stride = out_stride;
  args.out_dtype = out_dtype;
  args.rows = rows;
  args.blocks = (const BlockDev*)ws;
  const unsigned col_tiles = (unsigned)((max_dim + PG_TILE - 1) / PG_TILE);
  const int64_t row_tiles = gram ? col_tiles : (rows + PG_TILE - 1) / PG_TILE;
  BGX_REQUIRE(row_tiles <= 0x7fffffffLL && col_tiles <= 65535u && n_blocks <= 65535, BGX_E_ARG, "precond: grid too large");
  const dim3 grid((unsigned)row_tiles, col_tiles, (unsigned)n_blocks);
  if (gram) {
    if (in_dtype == BGX_F32)
      hipLaunchKernelGGL((precond_kernel<BGX_F32, true>), grid, dim3(PG_THREADS), 0, st, args);
    else if (in_dtype == BGX_F16)
      hipLaunchKernelGGL((precond_kernel<BGX_F16, true>), grid, dim3(PG_THREADS), 0, st, args);
    else
      hipLaunchKernelGGL((precond_kernel<BGX_BF16, true>), grid, dim3(PG_THREADS), 0, st, args);
  } else {
    if (in_dtype == BGX_F32)
      hipLaunchKernelGGL((precond_kernel<BGX_F32, false>), grid, dim3(PG_THREADS), 0, st, args);
    else if (in_dtype == BGX_F16)
      hipLaunchKernelGGL((precond_kernel<BGX_F16, false>), grid, dim3(PG_THREADS), 0, st, args);
    else
      hipLaunchKernelGGL((precond_kernel<BGX_BF16, false>), grid, dim3(PG_THREADS), 0, st, args);
  }
  BGX_HIP(hipGetLastError());
  return 0;
}

int block_gemm_impl(const void* in, int in_dtype, int64_t in_stride, void* out, int out_dtype, int64_t out_stride,
                    int64_t rows, const bgx_block_desc* blocks, int n_blocks, void* ws, size_t ws_bytes,
                    void* stream) {
  return precond_impl(false, in, in_dtype, in_stride, out, out_dtype, out_stride, rows, blocks, n_blocks, ws, ws_bytes,
                      stream);
}

int gram_accumulate_impl(const void* rows_dev, int dtype, int64_t stride, int64_t rows, const bgx_block_desc* blocks,
                         int n_blocks, void* ws, size_t ws_bytes, void* stream) {
  return precond_impl(true, rows_dev, dtype, stride, nullptr, BGX_F32, 0, rows, blocks, n_blocks, ws, ws_bytes, stream);
}

}  // namespace bgx
