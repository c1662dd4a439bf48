/*
 * bergson_amd.h -- C ABI of the MI355X (gfx950) hot path for projected
 * per-example gradient collection and gradient-store scoring.
 *
 * The reference (EleutherAI/bergson) is pure Python on PyTorch: it has no FFI
 * of its own.  Every entry point below replaces a *sequence of PyTorch ops*
 * that the reference issues from module hooks or from its scorer; the comment
 * on each entry point names that sequence as bergson/<file>:<lines>.
 *
 * Conventions
 *   - every function returns 0 on success, a positive hipError_t when a HIP
 *     call failed, or a negative BGX_E_* code when an argument was rejected
 *     before anything was enqueued.  bgx_last_error() gives the message of
 *     the last failure on the calling thread.
 *   - all pointers named *_dev are device pointers owned by the caller; the
 *     library allocates no device memory and never synchronises the host: all
 *     work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 *     null stream).  Entry points that take a host table (mods_host,
 *     blocks_host) copy it to the workspace with hipMemcpyAsync;
 *     bgx_collect_seq_static does not even do that.
 *   - "rows" are store rows; "tokens" are (sequence, position) pairs.
 *   - dtypes are BGX_F32 / BGX_F16 / BGX_BF16.
 */
#ifndef BERGSON_AMD_H
#define BERGSON_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BGX_ABI_VERSION 12

enum bgx_dtype { BGX_F32 = 0, BGX_F16 = 1, BGX_BF16 = 2 };

enum bgx_error {
  BGX_E_ARG = -1,       /* null / negative / inconsistent argument          */
  BGX_E_DTYPE = -2,     /* dtype code not supported by this entry point     */
  BGX_E_SHAPE = -3,     /* shape outside what the kernels are built for     */
  BGX_E_WORKSPACE = -4, /* workspace smaller than bgx_*_workspace_bytes()   */
  BGX_E_ALIGN = -5      /* pointer / stride alignment requirement violated  */
};

/* One hooked module (nn.Linear / Conv1D) of one batch.
 *   a      [N, S, I]  module input   (bergson/collector/collector.py:453-458)
 *   g      [N, S, O]  grad wrt module output (collector.py:460-472)
 * both in the model dtype, last dimension contiguous, element strides given.
 *   r_in   [p, I] row-major, model dtype: the "right" projection without its
 *          bias column (collector.py:336-362, :1029-1063)
 *   r_out  [p, O] row-major: the "left" projection
 *   col_scale [I] fp32 or NULL: Adafactor input-side factor
 *          rsqrt(col + 1e-30) already rounded to the model dtype
 *          (collector.py:532-535)
 *   row_scale [O] fp32 or NULL: Adafactor output-side factor
 *          sqrt(mean(row+1e-30)) * rsqrt(row+1e-30), rounded likewise
 *          (collector.py:655-658)
 *   bias_col [p] fp32 or NULL: column I of the [p, I+1] right projection when
 *          the bias gradient is collected (collector.py:552-590)
 *   bias_scale [O] fp32 or NULL: factor applied to g for the bias column only
 *          (rsqrt(bias_avg_sq + 1e-8), gradients.py:339-349); NULL = 1
 *   out_col  first column of this module's p*p block in an output row
 *          (bergson/data.py:380-389)
 */
typedef struct bgx_module_desc {
  const void* a;
  const void* g;
  const void* r_in;
  const void* r_out;
  const float* col_scale;
  const float* row_scale;
  const float* bias_col;
  const float* bias_scale;
  int64_t a_seq_stride;
  int64_t a_tok_stride;
  int64_t g_seq_stride;
  int64_t g_tok_stride;
  int64_t out_col;
  int32_t I;
  int32_t O;
} bgx_module_desc;

int bgx_abi_version(void);
const char* bgx_last_error(void);

/* Diagnostics (no counterpart in the reference).  A handful of BGX_*
 * environment variables force a kernel variant, so that tests can compare the
 * variants (BGX_COLLECT_PERSIST=0, BGX_COLLECT_STAGED=0, BGX_COLLECT_LPT_OFF, BGX_COLLECT_TWO_STEP_OFF,
 * BGX_ADAM_FUSED_OFF, BGX_ADAM_WIDE_OFF, BGX_ADAM_TTX=n, BGX_SCAN_DIRECT_OFF,
 * BGX_SCAN_STREAM_OFF, BGX_SCAN_WIDE_OFF, BGX_WGRAD_BIG_OFF).  The library reads them once, on its
 * first launch;
 * bgx_reload_switches() reads them again.  Launches that are being issued from
 * other threads at that moment see either the old or the new settings. */
int bgx_reload_switches(void);

/* Diagnostics (no counterpart in the reference).  Name of the main kernel the
 * calling thread's last launch of a family enqueued ("" before the first):
 * family 0 = bgx_collect_seq/_tok/_static ("collect_persist_lds",
 * "collect_persist_table", "collect_persist_direct", "collect_tile"),
 * 1 = bgx_collect_adam ("adam_fused_wide", "adam_fused_direct",
 * "adam_two_kernel"), 2 = bgx_scan* (the kernel of the
 * longest pass: "scan_wide", "scan_wide_known_norms", "scan_direct", "scan_stream",
 * "scan_gemm"), 3 = bgx_fullgrad_* / bgx_project_rows.  The pointer is to a
 * string literal. */
const char* bgx_last_kernel(int32_t family);

/* Adafactor factors of one module, computed once per module.
 * Replaces collector.py:532-535 and :655-658 (closed form in
 * bergson/gradients.py:300-337, eps = 1e-30):
 *   col_scale[i] = round_dtype(rsqrt(col[i] + 1e-30))
 *   row_scale[o] = round_dtype(sqrt(mean(row + 1e-30)) * rsqrt(row[o] + 1e-30))
 * row/col are fp32 device vectors; outputs are fp32 vectors holding values
 * representable in `dtype`.  Either pair may be NULL/0 to skip it. */
int bgx_adafactor_scales(const float* row_dev, int32_t O, const float* col_dev,
                         int32_t I, int32_t dtype, float* row_scale_dev,
                         float* col_scale_dev, void* stream);

/* Bytes of device workspace bgx_collect_seq / bgx_collect_tok need.
 * bgx_collect_workspace_bytes is the minimum for any modules of that count.
 * bgx_collect_workspace_bytes_for looks at the modules (only I, O and
 * bias_scale of each descriptor are read) and adds room for (i) a table of pre-scaled
 * projection fragments, 32 bytes per input and output feature (64 for
 * 16 < p <= 32, 128 for 32 < p <= 64), and the list of work items behind it
 * (4 bytes per module and 64 tokens): with it, modules too wide for their
 * projections to be kept on chip (Llama-3-8B's 4096 x 14336) and launches
 * at p > 16 still run through the streamed persistent kernel;
 * without it such launches use the one-workgroup-per-tile kernel, which is a
 * third to a half slower; (ii) at p = 8 or 16 (and, with the table, at any
 * multiple of 8 up to 64: 256 or 512 bytes per module and token),
 * the projected activations and output gradients of every token (128 bytes
 * per module and token): with it bgx_collect_tok writes its rows in two steps
 * -- the collection kernel leaves those projections in the workspace and a
 * second kernel writes each token's store row whole -- instead of scattering
 * one 2 p^2-byte block per module and token from the collection kernel itself
 * (same values).  Both sizes are accepted by the collect entry points. */
size_t bgx_collect_workspace_bytes(int32_t n_modules, int32_t N, int32_t S,
                                   int32_t p);
size_t bgx_collect_workspace_bytes_for(const bgx_module_desc* mods_host,
                                       int32_t n_modules, int32_t N, int32_t S,
                                       int32_t p, int32_t in_dtype);

/* Per-sequence projected gradients of n_modules modules of one batch in ONE
 * launch (plus a small deterministic reduction launch).
 * Replaces, per module: the forward-hook scale + `a @ R_in^T`
 * (collector.py:518-543), the backward-hook scale + `g @ R_out^T`, the token
 * reduction `g'.mT @ a'`, `flatten(1).clamp_(lo, hi)` and the cast to the
 * store dtype (collector.py:646-742; gradient_collectors.py:96-112), and the
 * concatenation of modules into one row (bergson/builder.py:17-32).
 *   out[row(n), mods[m].out_col + i*p + j] =
 *       cast(clamp(sum_s g'[n,s,i] * a'[n,s,j]))
 *   row(n) = out_rows_dev ? out_rows_dev[n] : n
 * mods_host is a HOST array; it is copied into the workspace on `stream`
 * (pageable memory is staged before return; pinned memory must stay valid
 * until the stream reaches the copy).
 * lengths_dev [N] int32 or NULL: document lengths; positions s >= len-1 carry
 * an exactly-zero g (right padding, causal model, labels -100;
 * bergson/data.py:800-804) and are skipped.
 * p in 1..64. */
int bgx_collect_seq(const bgx_module_desc* mods_host, int32_t n_modules,
                    int32_t N, int32_t S, int32_t p, int32_t in_dtype,
                    const int32_t* lengths_dev, const int64_t* out_rows_dev,
                    void* out_dev, int64_t out_row_stride, int32_t out_dtype,
                    float clamp_lo, float clamp_hi, void* workspace_dev,
                    size_t workspace_bytes, void* stream);

/* bgx_collect_seq for callers that cannot allocate device memory or hand over a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  Same arguments and
 * results as bgx_collect_seq, minus the workspace: the descriptor table, the
 * work-item ranges and the per-tile partial sums live in an array of
 * BGX_STATIC_SCRATCH_BYTES that is part of the library's device image (one copy
 * per GPU, held until the process ends), and the tables reach it as kernel
 * arguments rather than through a host-to-device copy.  The call allocates
 * nothing and frees nothing.  A launch whose bgx_collect_workspace_bytes() is
 * larger than the array is rejected with BGX_E_WORKSPACE before anything is
 * enqueued (16 MiB holds 48 modules x 4096 tokens at p = 16 five times over;
 * modules too wide for on-chip projections run through the per-tile kernel
 * unless their fragment table fits as well).  All calls on one GPU share the
 * array: calls that may overlap on a GPU (different streams, different
 * threads) race; calls on one stream are ordered by the stream.
 * `stream` must belong to the device that is current in the calling thread
 * (the array's address is taken for the current device).  The first call on a
 * device looks that address up, reads the device's compute-unit count and
 * opts the kernels into their LDS size; a caller that records the call into
 * a HIP graph makes one call outside the capture first. */
#define BGX_STATIC_SCRATCH_BYTES (16u << 20)
int bgx_collect_seq_static(const bgx_module_desc* mods_host, int32_t n_modules,
                           int32_t N, int32_t S, int32_t p, int32_t in_dtype,
                           const int32_t* lengths_dev,
                           const int64_t* out_rows_dev, void* out_dev,
                           int64_t out_row_stride, int32_t out_dtype,
                           float clamp_lo, float clamp_hi, void* stream);

/* Per-token variant (attribute_tokens): no token reduction; row
 * row_offsets_dev[n] + s of `out` receives flatten(g'[n,s] (x) a'[n,s]) for
 * s < lengths_dev[n] - 1.  Replaces collector.py:660-683 / :730-736 (the
 * [N,S,p,p] product and the boolean-mask gather) and the ragged scatter of
 * bergson/builder.py:174-188.  lengths_dev and row_offsets_dev are required. */
int bgx_collect_tok(const bgx_module_desc* mods_host, int32_t n_modules,
                    int32_t N, int32_t S, int32_t p, int32_t in_dtype,
                    const int32_t* lengths_dev, const int64_t* row_offsets_dev,
                    void* out_dev, int64_t out_row_stride, int32_t out_dtype,
                    float clamp_lo, float clamp_hi, void* workspace_dev,
                    size_t workspace_bytes, void* stream);

/* ---- Adam second-moment normaliser on the collection path ---------------
 * Replaces bergson/collector/collector.py:609-644 with
 * bergson/gradients.py:380-388 (grad / (sqrt(weight_avg_sq) + 1e-8), eps
 * outside the root) and the double-sided projection of collector.py:545-550.
 *
 * bgx_adam_prepare builds, once per module, the table
 *   table[(j*O + o), k] = round_dtype(r_in[j, k] / (sqrt(weight_avg_sq[o, k]) + 1e-8))
 * of bgx_adam_table_bytes(O, I, p, dtype, with_bias) bytes.
 * bgx_collect_adam then computes, for one module of one batch,
 *   P_t[i, j] = sum_o r_out[i, o] g_t[o] * sum_k a_t[k] table[(j*O + o), k]
 * per token t and writes either every valid token's row (per_token != 0:
 * row row_offsets[n] + s, s < lengths[n] - 1) or the sum over each sequence
 * (per_token == 0: row rows[n], or n when rows is NULL), clamped and cast.
 * bias_col_dev [p] / bias_scale_dev [O] (both or neither, the same to both
 * calls): when the bias gradient is collected, column I of the [p, I+1] right
 * projection and 1 / (sqrt(bias_avg_sq) + 1e-8) (gradients.py:390-400); they
 * add (sum_o r_out[i, o] g_t[o] bias_scale[o]) * bias_col[j] to P_t[i, j].
 * For 16-bit models with p <= 32 -- the ones the fused kernels take -- the table
 * is laid out for those kernels whatever the module's widths: O is padded to a
 * multiple of 256 and I (+ 1 with the bias, which then travels as one more
 * input feature: table column I = bias_col[j] * bias_scale[o], against a
 * column of ones in the activations) to a multiple of 64, with zeros; the
 * call pads a, g and r_out to match in its workspace.  Zero rows and columns
 * add exact zeros, so the result is that of the unpadded sums.
 * a must be uniformly strided over the flattened tokens
 * (a_seq_stride == S * a_tok_stride).  chunk_tokens = 0 picks the number of
 * tokens per internal pass. */
size_t bgx_adam_table_bytes(int32_t O, int32_t I, int32_t p, int32_t dtype,
                            int32_t with_bias);
int bgx_adam_prepare(const void* r_in_dev, const float* weight_avg_sq_dev,
                     const float* bias_col_dev, const float* bias_scale_dev,
                     int32_t O, int32_t I, int32_t p, int32_t dtype,
                     void* table_dev, void* stream);
size_t bgx_collect_adam_workspace_bytes(int32_t N, int32_t S, int32_t I,
                                        int32_t O, int32_t p, int32_t dtype,
                                        int32_t with_bias,
                                        int64_t chunk_tokens);
int bgx_collect_adam(const void* a_dev, const void* g_dev,
                     int64_t a_seq_stride, int64_t a_tok_stride,
                     int64_t g_seq_stride, int64_t g_tok_stride, int32_t N,
                     int32_t S, int32_t I, int32_t O, int32_t p, int32_t dtype,
                     const void* table_dev, const void* r_out_dev,
                     const float* bias_col_dev, const float* bias_scale_dev,
                     int32_t per_token, const int32_t* lengths_dev,
                     const int64_t* rows_dev, void* out_dev,
                     int64_t out_row_stride, int64_t out_col,
                     int32_t out_dtype, float clamp_lo, float clamp_hi,
                     void* workspace_dev, size_t workspace_bytes,
                     int64_t chunk_tokens, void* stream);

/* ---- weight-shaped (unprojected) gradients --------------------------------
 * projection_dim 0 / None, and the input of projection_target = "global":
 * bergson/collector/collector.py:609-742 with p = None.  Normalisers as in
 * bergson/gradients.py: Adafactor factors row_scale [O] / col_scale [I] (from
 * bgx_adafactor_scales), or Adam second moments adam_v [O, I]
 * (grad / (sqrt(v) + 1e-8), gradients.py:380-388); the two are exclusive, all
 * NULL = no normaliser.  With the bias gradient collected every row of the
 * gradient has I + 1 entries, the last being the bias gradient times
 * bias_scale [O] (NULL = 1): rsqrt(bias_avg_sq + 1e-8) for Adafactor
 * (gradients.py:339-349), 1 / (sqrt(bias_avg_sq) + 1e-8) for Adam (:390-400).
 *
 * bgx_token_sum: sum_dev[n, o] = sum_s g[n, s, o] (fp32), the bias gradient of
 *   a sequence before its factor (collector.py:612-615, :650-653, :704-707).
 * bgx_fullgrad_seq: P_dev [N, O, I] (contiguous, dtype) is the batched GEMM
 *   g^T a that the caller ran with its BLAS (`g.mT @ a`, collector.py:623,
 *   :684, :735).  Writes out[row(n), out_col + o*(I+b) + i] =
 *   cast(clamp(normalise(P[n, o, i]))), row(n) = out_rows[n] (n when NULL);
 *   bias_sum_dev [N, O] non-NULL adds the bias column (b = 1).
 * bgx_fullgrad_seq_gemm: the same rows straight from a [N, S, I] and
 *   g [N, S, O] (strides in elements, innermost contiguous): the GEMM over the
 *   tokens of a sequence (`g.mT @ a`, collector.py:623, :684, :735; only
 *   tokens s < lengths[n] - 1 when lengths_dev is given) on the matrix cores
 *   with normalisation, bias column (collect_bias != 0: sum_s g[n, s, o] *
 *   bias_scale[o]), clamp, cast and scatter fused behind it, so the [N, O, I]
 *   product never reaches memory.  Same rounding points as BLAS GEMM +
 *   bgx_fullgrad_seq: the sum is rounded to `dtype` before it is normalised.
 * bgx_fullgrad_tok: per token s < lengths[n] - 1 writes row
 *   row_offsets[n] + s with out_col + o*(I+b) + i = normalise(g[o] * a[i])
 *   (collector.py:620-632, :668-683, :730-734), bias column g[o] *
 *   bias_scale[o] when collect_bias != 0. */
int bgx_token_sum(const void* g_dev, int64_t g_seq_stride, int64_t g_tok_stride,
                  int32_t N, int32_t S, int32_t O, int32_t dtype,
                  float* sum_dev, void* stream);
int bgx_fullgrad_seq(const void* P_dev, int32_t N, int32_t O, int32_t I,
                     int32_t dtype, const float* row_scale_dev,
                     const float* col_scale_dev, const float* adam_v_dev,
                     const float* bias_sum_dev, const float* bias_scale_dev,
                     const int64_t* out_rows_dev, void* out_dev,
                     int64_t out_row_stride, int64_t out_col,
                     int32_t out_dtype, float clamp_lo, float clamp_hi,
                     void* stream);
int bgx_fullgrad_seq_gemm(const void* a_dev, const void* g_dev,
                          int64_t a_seq_stride, int64_t a_tok_stride,
                          int64_t g_seq_stride, int64_t g_tok_stride,
                          int32_t N, int32_t S, int32_t I, int32_t O,
                          int32_t dtype, const float* row_scale_dev,
                          const float* col_scale_dev, const float* adam_v_dev,
                          int32_t collect_bias, const float* bias_scale_dev,
                          const int32_t* lengths_dev,
                          const int64_t* out_rows_dev, void* out_dev,
                          int64_t out_row_stride, int64_t out_col,
                          int32_t out_dtype, float clamp_lo, float clamp_hi,
                          void* stream);
/* bgx_collect_seq_weight: per-sequence rows of one module whose normaliser acts
 * on the weight-shaped gradient -- Adam's second moments (adam_v_dev), or
 * Adafactor's factors -- with a projection:
 *   out[row(n), out_col : out_col + p*p] =
 *       clamp(L normalise(g[n]^T a[n] [| bias gradient]) R^T)
 * i.e. the reference's per-sequence branch of _compute_gradient with an Adam
 * normaliser (bergson/collector/collector.py:609-644 with
 * reduce over the tokens; bergson/gradients.py:380-400): `g.mT @ a` over the
 * tokens s < lengths[n] - 1, rounded to the model dtype, divided by
 * sqrt(v) + 1e-8, the bias column appended, projected by L = left_dev [p, O]
 * and R = right_dev [p, right_stride] (columns 0 .. I-1) with bias_col_dev [p]
 * (fp32, or NULL when the bias is not collected) as the column that multiplies
 * the bias gradient sum_s g[n, s, :] * bias_scale_dev (NULL = 1).  One launch forms the product over
 * the tokens on 64 x 64 tiles and projects each tile where it is; nothing
 * weight-shaped reaches memory.  The tiles' p x p contributions meet in the
 * workspace (bgx_collect_seq_weight_workspace_bytes, 256-byte aligned) and are
 * added in a fixed order.  16-bit models (BGX_F16 / BGX_BF16), p <= 32; other
 * cases go through bgx_fullgrad_seq_gemm and bgx_collect_seq. */
size_t bgx_collect_seq_weight_workspace_bytes(int32_t N, int32_t I, int32_t O,
                                              int32_t p);
int bgx_collect_seq_weight(const void* a_dev, const void* g_dev,
                           int64_t a_seq_stride, int64_t a_tok_stride,
                           int64_t g_seq_stride, int64_t g_tok_stride,
                           int32_t N, int32_t S, int32_t I, int32_t O,
                           int32_t p, int32_t dtype,
                           const float* row_scale_dev,
                           const float* col_scale_dev,
                           const float* adam_v_dev, const void* left_dev,
                           const void* right_dev, int64_t right_stride,
                           const float* bias_col_dev,
                           const float* bias_scale_dev,
                           const int32_t* lengths_dev,
                           const int64_t* out_rows_dev, void* out_dev,
                           int64_t out_row_stride, int64_t out_col,
                           int32_t out_dtype, float clamp_lo, float clamp_hi,
                           void* workspace_dev, size_t workspace_bytes,
                           void* stream);
/* The global projection (projection_target = "global",
 * collector.py:364-390: `grad.flatten(1) @ proj.T` per module, summed over
 * the modules): acc_dev[m, j] += sum_k rows_dev[m, k] * proj_dev[j, k] for
 * m < n_rows, j < P, k < width.  rows_dev [n_rows, width] (row stride in
 * elements) is what bgx_fullgrad_seq_gemm / bgx_fullgrad_tok wrote for one
 * module, proj_dev [P, width] (contiguous) the module's block of the projection
 * matrix, both in `dtype`; acc_dev is fp32 and is added to, so a caller zeroes
 * it once and calls this per module.  The contraction is split into slabs
 * whose sums are added in a fixed order (workspace: partial sums). */
size_t bgx_project_rows_workspace_bytes(int64_t n_rows, int64_t width,
                                        int32_t P, int32_t dtype);
int bgx_project_rows(const void* rows_dev, int64_t n_rows, int64_t width,
                     int64_t row_stride, int32_t dtype, const void* proj_dev,
                     int32_t P, float* acc_dev, int64_t acc_stride,
                     void* workspace_dev, size_t workspace_bytes, void* stream);
int bgx_fullgrad_tok(const void* a_dev, const void* g_dev,
                     int64_t a_seq_stride, int64_t a_tok_stride,
                     int64_t g_seq_stride, int64_t g_tok_stride, int32_t N,
                     int32_t S, int32_t I, int32_t O, int32_t dtype,
                     const float* row_scale_dev, const float* col_scale_dev,
                     const float* adam_v_dev, int32_t collect_bias,
                     const float* bias_scale_dev, const int32_t* lengths_dev,
                     const int64_t* row_offsets_dev, void* out_dev,
                     int64_t out_row_stride, int64_t out_col,
                     int32_t out_dtype, float clamp_lo, float clamp_hi,
                     void* stream);

/* Benchmark support (no counterpart in the reference): while enabled, every
 * bgx_collect_seq / bgx_collect_tok call records a HIP event pair immediately
 * around its collect_kernel launch, on the launch stream, so that the kernel's
 * own duration can be read without a profiler.
 *   bgx_collect_timing_enable(n)  n > 0: start recording, at most n launches;
 *                                 n = 0: stop and release the events
 *   bgx_collect_timing_read(ms, capacity, &count): waits for the recorded
 *       events and writes each launch's kernel time in milliseconds.
 * Launches from several threads and streams may be in flight while recording is
 * on (each claims its pair under a lock and records it on its own stream);
 * enable and read belong to one thread, between launches. */
int bgx_collect_timing_enable(int32_t max_launches);
int bgx_collect_timing_read(float* ms_out, int32_t capacity, int32_t* count_out);

/* In-place unit normalisation of rows: g * rsqrt(max(sum g^2, eps_fp32^2)),
 * replaces bergson/builder.py:14,:28-30.  rows_dev [n_rows, D], row stride in
 * elements. */
int bgx_unit_normalize_rows(void* rows_dev, int64_t n_rows, int64_t D,
                            int64_t row_stride, int32_t dtype, void* stream);

/* ---- gradient-store scoring ------------------------------------------- */

/* Bytes of device workspace bgx_scan needs for Q queries, top-k of k and at
 * most chunk_rows store rows per internal pass (0 = library default). */
size_t bgx_scan_workspace_bytes(int32_t Q, int32_t k, int64_t chunk_rows);
/* The same plus room for a table of the queries as matrix-core fragments
 * (1 KB per block of 16 queries and k-step: 32 elements of D at 16 bits, 16 at
 * fp32): with it, scans with at most 96 queries over at least 512 rows per
 * compute unit, D a multiple of two k-steps, stream the store with the
 * few-queries kernel; without it they use the tiled kernel.  A workspace is then needed
 * even when neither top-k nor row means are asked for.  bgx_scan accepts
 * either size. */
size_t bgx_scan_workspace_bytes_for(int32_t Q, int32_t k, int64_t chunk_rows,
                                    int64_t D, int32_t dtype);

/* Scores n_rows store rows [n_rows, D] (row stride in elements) against Q
 * queries [Q, D] of the same dtype, streaming the store once.
 *   score[n, q] = query_scale * <store[n], queries[q]> * w[n]
 *   w[n] = unit_norm ? (sumsq[n] > 0 ? 1/sqrt(sumsq[n]) : 0) : 1
 * which is the index-side normalisation of bergson/score/scorer.py:89-115
 * (scores / clamp_min(sqrt(sum g^2), 1e-12)) and of
 * bergson/query/attributor.py:137-167 (g / ||g||, nan -> 0); queries are
 * normalised by the caller as the reference does before scoring
 * (attributor.py:202-206, bergson/process_grads.py:156-164).
 * Outputs, each optional (NULL to skip):
 *   topk_val_dev [Q, k] fp32, topk_idx_dev [Q, k] int64: per query the k
 *     largest scores in descending order, ties broken by lower row index
 *     (torch.topk, attributor.py:229-235); requires k <= n_rows, k <= 65536
 *     (up to 2048 the running top-k of a query is kept sorted on chip; beyond,
 *     it lives in the workspace and is sorted once at the end).
 *     Scores that are NaN or -inf are never selected, whichever pass or
 *     kernel meets them (torch.topk would rank NaN first); a query with
 *     fewer than k selectable scores gets (-inf, -1) in its last entries
 *   row_max_dev [n_rows] fp32: max over queries (score_mode "nearest",
 *     scorer.py:111-113)
 *   row_mean_dev [n_rows] fp32: mean over queries, summed in a fixed order.
 *     By linearity this is the score against the mean of the queries, which
 *     is how the reference obtains it (aggregation "mean",
 *     bergson/process_grads.py:166-182, then scorer.py:89-115); needs the
 *     workspace
 *   scores_dev [n_rows, Q] fp32 row-major: every score (scorer.py:89-115)
 *   sumsq_dev [n_rows] fp32: sum of squares of each row
 * row_base is added to the row numbers reported in topk_idx_dev. */
int bgx_scan(const void* store_dev, int64_t n_rows, int64_t D,
             int64_t store_row_stride, int32_t dtype, const void* queries_dev,
             int32_t Q, float query_scale, int32_t unit_norm, int32_t k,
             int64_t row_base, float* topk_val_dev, int64_t* topk_idx_dev,
             float* row_max_dev, float* row_mean_dev, float* scores_dev,
             float* sumsq_dev, void* workspace_dev, size_t workspace_bytes,
             int64_t chunk_rows, void* stream);

/* Sums of squares of the rows of a store, in one pass over it (bound by HBM):
 * the index-side half of bergson/query/attributor.py:137-167, which
 * normalises an index once when it is loaded.  row_sumsq_dev [n_rows] fp32
 * receives exactly the values a bgx_scan of the same rows writes to its
 * sumsq_dev (same order of additions), so a scan given them
 * (bgx_scan_known_norms) returns the bits of a scan that formed them. */
int bgx_row_sumsq(const void* store_dev, int64_t n_rows, int64_t D,
                  int64_t store_row_stride, int32_t dtype, float* row_sumsq_dev,
                  void* stream);

/* bgx_scan for a store whose row sums of squares are known: row_sumsq_dev
 * [n_rows] is the sumsq_dev output of an earlier bgx_scan of the same rows, or of bgx_row_sumsq.
 * The reference normalises an index once, when it loads it
 * (query/attributor.py:137-167), and scores it many times; this is the same
 * economy -- kernels that would otherwise sum the squares of every row in
 * their inner loop leave that out and take the multiplier from the array
 * (the 384 x 256 tile kernel for more than 128 queries; the other kernels
 * compute the sums as before, which gives the same values).  Everything else
 * as bgx_scan; there is no sumsq output. */
int bgx_scan_known_norms(const void* store_dev, int64_t n_rows, int64_t D,
                         int64_t store_row_stride, int32_t dtype,
                         const void* queries_dev, int32_t Q, float query_scale,
                         int32_t unit_norm, int32_t k, int64_t row_base,
                         const float* row_sumsq_dev, float* topk_val_dev,
                         int64_t* topk_idx_dev, float* row_max_dev,
                         float* row_mean_dev, float* scores_dev,
                         void* workspace_dev, size_t workspace_bytes,
                         int64_t chunk_rows, void* stream);

/* ---- dense per-module preconditioner --------------------------------------
 * One fp32 matrix h_dev [dim, dim] (row-major) per module; the module's values
 * are columns col0 .. col0 + dim of a gradient row.
 *
 * bgx_block_gemm: out[n, col0 + j] = sum_i fp32(in[n, col0 + i]) * h[i, j] for
 *   every block, rows n < n_rows; fp32 accumulation, cast to out_dtype.  This
 *   is DensePreconditioner.apply, `g @ H^p` per module
 *   (bergson/hessians/preconditioner.py:77-92), as called by
 *   bergson/builder.py:17-32 and bergson/query/attributor.py:138-145,
 *   :195-200, and the batched `torch.bmm` of the split transform in
 *   bergson/score/score.py:111-135.  out_dev must not alias in_dev; columns of
 *   a row that belong to no block are left untouched in out_dev.
 * bgx_gram_accumulate: h[i, j] += sum_n fp32(rows[n, col0 + i]) *
 *   fp32(rows[n, col0 + j]) -- the autocorrelation Gram of
 *   bergson/collector/in_memory_collector.py:149-154
 *   (`hessians[name].addmm_(P.mT, P)` on `P.float()`).  Calls on one stream
 *   accumulate in call order; every element has one writer (no atomics).
 * blocks_host is read during the call; workspace_dev holds
 * bgx_precond_workspace_bytes(n_blocks) bytes. */
typedef struct bgx_block_desc {
  float* h_dev;
  int64_t col0;
  int32_t dim;
  int32_t reserved;
} bgx_block_desc;

size_t bgx_precond_workspace_bytes(int32_t n_blocks);
int bgx_block_gemm(const void* in_dev, int32_t in_dtype, int64_t in_row_stride,
                   void* out_dev, int32_t out_dtype, int64_t out_row_stride,
                   int64_t n_rows, const bgx_block_desc* blocks_host,
                   int32_t n_blocks, void* workspace_dev,
                   size_t workspace_bytes, void* stream);
int bgx_gram_accumulate(const void* rows_dev, int32_t dtype, int64_t row_stride,
                        int64_t n_rows, const bgx_block_desc* blocks_host,
                        int32_t n_blocks, void* workspace_dev,
                        size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BERGSON_AMD_H */
