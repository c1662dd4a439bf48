// extern "C" entry points of libbergson_amd.so (declared in include/bergson_amd.h).
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include <atomic>

#include "common.hpp"

namespace bgx {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
  set_error("%s failed: %s (%d)", what, hipGetErrorString(e), (int)e);
  return (int)e;
}

static thread_local const char* g_last_kernel[FAMILY_COUNT] = {"", "", "", ""};

void note_kernel(int family, const char* name) {
  if (family >= 0 && family < FAMILY_COUNT) g_last_kernel[family] = name;
}

const char* noted_kernel(int family) {
  return family >= 0 && family < FAMILY_COUNT ? g_last_kernel[family] : "";
}

static const Switches* read_switches() {
  Switches* s = new Switches;
  auto off = [](const char* name) {
    const char* e = getenv(name);
    return e != nullptr && e[0] == '0';
  };
  s->adam_fused_off = getenv("BGX_ADAM_FUSED_OFF") != nullptr;
  s->adam_wide_off = getenv("BGX_ADAM_WIDE_OFF") != nullptr;
  if (const char* e = getenv("BGX_ADAM_TTX")) s->adam_ttx = atoi(e);
  s->collect_staged = !off("BGX_COLLECT_STAGED");
  s->collect_persist = !off("BGX_COLLECT_PERSIST");
  s->collect_lpt_off = getenv("BGX_COLLECT_LPT_OFF") != nullptr;
  s->collect_two_step_off = getenv("BGX_COLLECT_TWO_STEP_OFF") != nullptr;
  s->scan_direct_off = getenv("BGX_SCAN_DIRECT_OFF") != nullptr;
  s->scan_stream_off = getenv("BGX_SCAN_STREAM_OFF") != nullptr;
  s->scan_wide_off = getenv("BGX_SCAN_WIDE_OFF") != nullptr;
  s->wgrad_big_off = getenv("BGX_WGRAD_BIG_OFF") != nullptr;
  return s;
}

// The current record.  A superseded record is never freed (a launch on another thread may still be reading
// it; a record is a few bytes and reloading is something only tests do).
static std::atomic<const Switches*> g_switches{nullptr};

const Switches& switches() {
  const Switches* s = g_switches.load(std::memory_order_acquire);
  if (s == nullptr) {
    const Switches* fresh = read_switches();
    if (g_switches.compare_exchange_strong(s, fresh, std::memory_order_acq_rel))
      s = fresh;
    else
      delete fresh;
  }
  return *s;
}

void reload_switches() { g_switches.store(read_switches(), std::memory_order_release); }

size_t collect_workspace_bytes(int n_modules, int N, int S, int p);
size_t collect_workspace_bytes_for(const bgx_module_desc* mods, int n_modules, int N, int S, int p, int in_dtype);
int collect_impl(bool per_token, const bgx_module_desc* mods_host, int n_modules, int N, int S, int p, int in_dtype,
                 const int32_t* lengths, const int64_t* rows_or_offsets, void* out, int64_t out_row_stride,
                 int out_dtype, float lo, float hi, void* ws, size_t ws_bytes, void* stream,
                 bool tables_by_kernel = false);
int collect_seq_static_impl(const bgx_module_desc* mods_host, int n_modules, int N, int S, int p, int in_dtype,
                            const int32_t* lengths, const int64_t* out_rows, void* out, int64_t out_row_stride,
                            int out_dtype, float lo, float hi, void* stream);
int adafactor_scales_impl(const float* row, int O, const float* col, int I, int dtype, float* row_scale,
                          float* col_scale, void* stream);
size_t adam_table_bytes(int O, int I, int p, int dtype, int with_bias);
int adam_prepare_impl(const void* r_in, const float* v, const float* bias_col, const float* bias_scale, int O, int I,
                      int p, int dtype, void* table, void* stream);
size_t collect_adam_workspace_bytes(int N, int S, int I, int O, int p, int dtype, int with_bias, int64_t chunk_tokens);
int collect_adam_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride, int64_t g_seq_stride,
                      int64_t g_tok_stride, int N, int S, int I, int O, int p, int dtype, const void* table,
                      const void* r_out, const float* bias_col, const float* bias_scale, int per_token,
                      const int32_t* lengths, const int64_t* rows, void* out, int64_t out_row_stride, int64_t out_col,
                      int out_dtype, float lo, float hi, void* ws, size_t ws_bytes, int64_t chunk_tokens,
                      void* stream);
int token_sum_impl(const void* g, int64_t g_seq_stride, int64_t g_tok_stride, int N, int S, int O, int dtype,
                   float* sum, void* stream);
int fullgrad_seq_impl(const void* P, int N, int O, int I, int dtype, const float* row_scale, const float* col_scale,
                      const float* adam_v, const float* bias_sum, const float* bias_scale, const int64_t* out_rows,
                      void* out, int64_t out_row_stride, int64_t out_col, int out_dtype, float lo, float hi,
                      void* stream);
int fullgrad_tok_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride, int64_t g_seq_stride,
                      int64_t g_tok_stride, int N, int S, int I, int O, int dtype, const float* row_scale,
                      const float* col_scale, const float* adam_v, int collect_bias, const float* bias_scale,
                      const int32_t* lengths, const int64_t* row_offsets, void* out, int64_t out_row_stride,
                      int64_t out_col, int out_dtype, float lo, float hi, void* stream);
int fullgrad_seq_gemm_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride,
                           int64_t g_seq_stride, int64_t g_tok_stride, int N, int S, int I, int O, int dtype,
                           const float* row_scale, const float* col_scale, const float* adam_v, int collect_bias,
                           const float* bias_scale, const int32_t* lengths, const int64_t* out_rows, void* out,
                           int64_t out_row_stride, int64_t out_col, int out_dtype, float lo, float hi, void* stream);
size_t collect_seq_weight_workspace_bytes(int N, int I, int O, int p);
int collect_seq_weight_impl(const void* a, const void* g, int64_t a_seq_stride, int64_t a_tok_stride,
                            int64_t g_seq_stride, int64_t g_tok_stride, int N, int S, int I, int O, int p, int dtype,
                            const float* row_scale, const float* col_scale, const float* adam_v, const void* left,
                            const void* right, int64_t right_stride, const float* bias_col, const float* bias_scale,
                            const int32_t* lengths, const int64_t* out_rows, void* out, int64_t out_row_stride,
                            int64_t out_col, int out_dtype, float lo, float hi, void* ws, size_t ws_bytes,
                            void* stream);
size_t project_rows_workspace_bytes(int64_t M, int64_t W, int P, int dtype);
int project_rows_impl(const void* rows, int64_t M, int64_t W, int64_t row_stride, int dtype, const void* proj, int P,
                      float* acc, int64_t acc_stride, void* ws, size_t ws_bytes, void* stream);
int collect_timing_enable(int max_launches);
int collect_timing_read(float* ms_out, int capacity, int* count_out);
int unit_normalize_impl(void* rows, int64_t n_rows, int64_t D, int64_t stride, int dtype, void* stream);
size_t scan_workspace_bytes(int Q, int k, int64_t chunk_rows);
size_t scan_workspace_bytes_for(int Q, int k, int64_t chunk_rows, int64_t D, int dtype);
int scan_impl(const void* store, int64_t n_rows, int64_t D, int64_t stride, int dtype, const void* queries, int Q,
              float query_scale, int unit_norm, int k, int64_t row_base, float* topk_val, int64_t* topk_idx,
              float* row_max, float* row_mean, float* scores, float* sumsq, const float* sumsq_in, void* ws,
              size_t ws_bytes, int64_t chunk_rows, void* stream);
int row_sumsq_impl(const void* store, int64_t n_rows, int64_t D, int64_t stride, int dtype, float* sumsq, void* stream);
size_t precond_workspace_bytes(int n_blocks);
int block_gemm_impl(const void* in, int in_dtype, int64_t in_stride, void* out, int out_dtype, int64_t out_stride,
                    int64_t rows, const bgx_block_desc* blocks, int n_blocks, void* ws, size_t ws_bytes,
                    void* stream);
int gram_accumulate_impl(const void* rows_dev, int dtype, int64_t stride, int64_t rows, const bgx_block_desc* blocks,
                         int n_blocks, void* ws, size_t ws_bytes, void* stream);

}  // namespace bgx

extern "C" {

size_t bgx_precond_workspace_bytes(int32_t n_blocks) { return bgx::precond_workspace_bytes(n_blocks); }

int bgx_block_gemm(const void* in_dev, int32_t in_dtype, int64_t in_row_stride, void* out_dev, int32_t out_dtype,
                   int64_t out_row_stride, int64_t n_rows, const bgx_block_desc* blocks_host, int32_t n_blocks,
                   void* workspace_dev, size_t workspace_bytes, void* stream) {
  return bgx::block_gemm_impl(in_dev, in_dtype, in_row_stride, out_dev, out_dtype, out_row_stride, n_rows, blocks_host,
                              n_blocks, workspace_dev, workspace_bytes, stream);
}

int bgx_gram_accumulate(const void* rows_dev, int32_t dtype, int64_t row_stride, int64_t n_rows,
                        const bgx_block_desc* blocks_host, int32_t n_blocks, void* workspace_dev,
                        size_t workspace_bytes, void* stream) {
  return bgx::gram_accumulate_impl(rows_dev, dtype, row_stride, n_rows, blocks_host, n_blocks, workspace_dev,
                                   workspace_bytes, stream);
}

int bgx_abi_version(void) { return BGX_ABI_VERSION; }

int bgx_reload_switches(void) {
  bgx::reload_switches();
  return 0;
}

const char* bgx_last_error(void) { return bgx::g_err; }

const char* bgx_last_kernel(int32_t family) {
  return bgx::noted_kernel(family);
}

int bgx_adafactor_scales(const float* row_dev, int32_t O, const float* col_dev, int32_t I, int32_t dtype,
                         float* row_scale_dev, float* col_scale_dev, void* stream) {
  return bgx::adafactor_scales_impl(row_dev, O, col_dev, I, dtype, row_scale_dev, col_scale_dev, stream);
}

size_t bgx_collect_workspace_bytes(int32_t n_modules, int32_t N, int32_t S, int32_t p) {
  return bgx::collect_workspace_bytes(n_modules, N, S, p);
}

size_t bgx_collect_workspace_bytes_for(const bgx_module_desc* mods_host, int32_t n_modules, int32_t N, int32_t S,
                                       int32_t p, int32_t in_dtype) {
  return bgx::collect_workspace_bytes_for(mods_host, n_modules, N, S, p, in_dtype);
}

int bgx_collect_seq(const bgx_module_desc* mods_host, int32_t n_modules, int32_t N, int32_t S, int32_t p,
                    int32_t in_dtype, const int32_t* lengths_dev, const int64_t* out_rows_dev, void* out_dev,
                    int64_t out_row_stride, int32_t out_dtype, float clamp_lo, float clamp_hi, void* workspace_dev,
                    size_t workspace_bytes, void* stream) {
  return bgx::collect_impl(false, mods_host, n_modules, N, S, p, in_dtype, lengths_dev, out_rows_dev, out_dev,
                           out_row_stride, out_dtype, clamp_lo, clamp_hi, workspace_dev, workspace_bytes, stream);
}

int bgx_collect_tok(const bgx_module_desc* mods_host, int32_t n_modules, int32_t N, int32_t S, int32_t p,
                    int32_t in_dtype, const int32_t* lengths_dev, const int64_t* row_offsets_dev, void* out_dev,
                    int64_t out_row_stride, int32_t out_dtype, float clamp_lo, float clamp_hi, void* workspace_dev,
                    size_t workspace_bytes, void* stream) {
  return bgx::collect_impl(true, mods_host, n_modules, N, S, p, in_dtype, lengths_dev, row_offsets_dev, out_dev,
                           out_row_stride, out_dtype, clamp_lo, clamp_hi, workspace_dev, workspace_bytes, stream);
}

int bgx_collect_seq_static(const bgx_module_desc* mods_host, int32_t n_modules, int32_t N, int32_t S, int32_t p,
                           int32_t in_dtype, const int32_t* lengths_dev, const int64_t* out_rows_dev, void* out_dev,
                           int64_t out_row_stride, int32_t out_dtype, float clamp_lo, float clamp_hi, void* stream) {
  return bgx::collect_seq_static_impl(mods_host, n_modules, N, S, p, in_dtype, lengths_dev, out_rows_dev, out_dev,
                                      out_row_stride, out_dtype, clamp_lo, clamp_hi, stream);
}

size_t bgx_adam_table_bytes(int32_t O, int32_t I, int32_t p, int32_t dtype, int32_t with_bias) {
  return bgx::adam_table_bytes(O, I, p, dtype, with_bias);
}

int bgx_adam_prepare(const void* r_in_dev, const float* weight_avg_sq_dev, const float* bias_col_dev,
                     const float* bias_scale_dev, int32_t O, int32_t I, int32_t p, int32_t dtype, void* table_dev,
                     void* stream) {
  return bgx::adam_prepare_impl(r_in_dev, weight_avg_sq_dev, bias_col_dev, bias_scale_dev, O, I, p, dtype, table_dev,
                                stream);
}

size_t bgx_collect_adam_workspace_bytes(int32_t N, int32_t S, int32_t I, int32_t O, int32_t p, int32_t dtype,
                                        int32_t with_bias, int64_t chunk_tokens) {
  return bgx::collect_adam_workspace_bytes(N, S, I, O, p, dtype, with_bias, chunk_tokens);
}

int bgx_collect_adam(const void* a_dev, const void* g_dev, int64_t a_seq_stride, int64_t a_tok_stride,
                     int64_t g_seq_stride, int64_t g_tok_stride, int32_t N, int32_t S, int32_t I, int32_t O, int32_t p,
                     int32_t dtype, const void* table_dev, const void* r_out_dev, const float* bias_col_dev,
                     const float* bias_scale_dev, int32_t per_token, const int32_t* lengths_dev,
                     const int64_t* rows_dev, void* out_dev, int64_t out_row_stride,
                     int64_t out_col, int32_t out_dtype, float clamp_lo, float clamp_hi, void* workspace_dev,
                     size_t workspace_bytes, int64_t chunk_tokens, void* stream) {
  return bgx::collect_adam_impl(a_dev, g_dev, a_seq_stride, a_tok_stride, g_seq_stride, g_tok_stride, N, S, I, O, p,
                                dtype, table_dev, r_out_dev, bias_col_dev, bias_scale_dev, per_token, lengths_dev,
                                rows_dev, out_dev, out_row_stride,
                                out_col, out_dtype, clamp_lo, clamp_hi, workspace_dev, workspace_bytes, chunk_tokens,
                                stream);
}

int bgx_token_sum(const void* g_dev, int64_t g_seq_stride, int64_t g_tok_stride, int32_t N, int32_t S, int32_t O,
                  int32_t dtype, float* sum_dev, void* stream) {
  return bgx::token_sum_impl(g_dev, g_seq_stride, g_tok_stride, N, S, O, dtype, sum_dev, stream);
}

int bgx_fullgrad_seq(const void* P_dev, int32_t N, int32_t O, int32_t I, int32_t dtype, const float* row_scale_dev,
                     const float* col_scale_dev, const float* adam_v_dev, const float* bias_sum_dev,
                     const float* bias_scale_dev, const int64_t* out_rows_dev, void* out_dev, int64_t out_row_stride,
                     int64_t out_col, int32_t out_dtype, float clamp_lo, float clamp_hi, void* stream) {
  return bgx::fullgrad_seq_impl(P_dev, N, O, I, dtype, row_scale_dev, col_scale_dev, adam_v_dev, bias_sum_dev,
                                bias_scale_dev, out_rows_dev, out_dev, out_row_stride, out_col, out_dtype, clamp_lo,
                                clamp_hi, stream);
}

int bgx_fullgrad_tok(const void* a_dev, const void* g_dev, int64_t a_seq_stride, int64_t a_tok_stride,
                     int64_t g_seq_stride, int64_t g_tok_stride, int32_t N, int32_t S, int32_t I, int32_t O,
                     int32_t dtype, const float* row_scale_dev, const float* col_scale_dev, const float* adam_v_dev,
                     int32_t collect_bias, const float* bias_scale_dev, const int32_t* lengths_dev,
                     const int64_t* row_offsets_dev, void* out_dev, int64_t out_row_stride, int64_t out_col,
                     int32_t out_dtype, float clamp_lo, float clamp_hi, void* stream) {
  return bgx::fullgrad_tok_impl(a_dev, g_dev, a_seq_stride, a_tok_stride, g_seq_stride, g_tok_stride, N, S, I, O, dtype,
                                row_scale_dev, col_scale_dev, adam_v_dev, collect_bias, bias_scale_dev, lengths_dev,
                                row_offsets_dev, out_dev, out_row_stride, out_col, out_dtype, clamp_lo, clamp_hi,
                                stream);
}

int bgx_fullgrad_seq_gemm(const void* a_dev, const void* g_dev, int64_t a_seq_stride, int64_t a_tok_stride,
                          int64_t g_seq_stride, int64_t g_tok_stride, int32_t N, int32_t S, int32_t I, int32_t O,
                          int32_t dtype, const float* row_scale_dev, const float* col_scale_dev,
                          const float* adam_v_dev, int32_t collect_bias, const float* bias_scale_dev,
                          const int32_t* lengths_dev, const int64_t* out_rows_dev, void* out_dev,
                          int64_t out_row_stride, int64_t out_col, int32_t out_dtype, float clamp_lo, float clamp_hi,
                          void* stream) {
  return bgx::fullgrad_seq_gemm_impl(a_dev, g_dev, a_seq_stride, a_tok_stride, g_seq_stride, g_tok_stride, N, S, I, O,
                                     dtype, row_scale_dev, col_scale_dev, adam_v_dev, collect_bias, bias_scale_dev,
                                     lengths_dev, out_rows_dev, out_dev, out_row_stride, out_col, out_dtype, clamp_lo,
                                     clamp_hi, stream);
}

size_t bgx_collect_seq_weight_workspace_bytes(int32_t N, int32_t I, int32_t O, int32_t p) {
  return bgx::collect_seq_weight_workspace_bytes(N, I, O, p);
}

int bgx_collect_seq_weight(const void* a_dev, const void* g_dev, int64_t a_seq_stride, int64_t a_tok_stride,
                           int64_t g_seq_stride, int64_t g_tok_stride, int32_t N, int32_t S, int32_t I, int32_t O,
                           int32_t p, int32_t dtype, const float* row_scale_dev, const float* col_scale_dev,
                           const float* adam_v_dev, const void* left_dev, const void* right_dev, int64_t right_stride,
                           const float* bias_col_dev, const float* bias_scale_dev, const int32_t* lengths_dev,
                           const int64_t* out_rows_dev, void* out_dev, int64_t out_row_stride, int64_t out_col,
                           int32_t out_dtype, float clamp_lo, float clamp_hi, void* workspace_dev,
                           size_t workspace_bytes, void* stream) {
  return bgx::collect_seq_weight_impl(a_dev, g_dev, a_seq_stride, a_tok_stride, g_seq_stride, g_tok_stride, N, S, I, O,
                                      p, dtype, row_scale_dev, col_scale_dev, adam_v_dev, left_dev, right_dev,
                                      right_stride, bias_col_dev, bias_scale_dev, lengths_dev, out_rows_dev, out_dev,
                                      out_row_stride, out_col, out_dtype, clamp_lo, clamp_hi, workspace_dev,
                                      workspace_bytes, stream);
}

size_t bgx_project_rows_workspace_bytes(int64_t n_rows, int64_t width, int32_t P, int32_t dtype) {
  return bgx::project_rows_workspace_bytes(n_rows, width, P, dtype);
}

int bgx_project_rows(const void* rows_dev, int64_t n_rows, int64_t width, int64_t row_stride, int32_t dtype,
                     const void* proj_dev, int32_t P, float* acc_dev, int64_t acc_stride, void* workspace_dev,
                     size_t workspace_bytes, void* stream) {
  return bgx::project_rows_impl(rows_dev, n_rows, width, row_stride, dtype, proj_dev, P, acc_dev, acc_stride,
                                workspace_dev, workspace_bytes, stream);
}

int bgx_collect_timing_enable(int32_t max_launches) { return bgx::collect_timing_enable(max_launches); }

int bgx_collect_timing_read(float* ms_out, int32_t capacity, int32_t* count_out) {
  return bgx::collect_timing_read(ms_out, capacity, count_out);
}

int bgx_unit_normalize_rows(void* rows_dev, int64_t n_rows, int64_t D, int64_t row_stride, int32_t dtype,
                            void* stream) {
  return bgx::unit_normalize_impl(rows_dev, n_rows, D, row_stride, dtype, stream);
}

size_t bgx_scan_workspace_bytes_for(int32_t Q, int32_t k, int64_t chunk_rows, int64_t D, int32_t dtype) {
  return bgx::scan_workspace_bytes_for(Q, k, chunk_rows, D, dtype);
}

size_t bgx_scan_workspace_bytes(int32_t Q, int32_t k, int64_t chunk_rows) {
  return bgx::scan_workspace_bytes(Q, k, chunk_rows);
}

int bgx_scan(const void* store_dev, int64_t n_rows, int64_t D, int64_t store_row_stride, int32_t dtype,
             const void* queries_dev, int32_t Q, float query_scale, int32_t unit_norm, int32_t k, int64_t row_base,
             float* topk_val_dev, int64_t* topk_idx_dev, float* row_max_dev, float* row_mean_dev, float* scores_dev,
             float* sumsq_dev, void* workspace_dev, size_t workspace_bytes, int64_t chunk_rows, void* stream) {
  return bgx::scan_impl(store_dev, n_rows, D, store_row_stride, dtype, queries_dev, Q, query_scale, unit_norm, k,
                        row_base, topk_val_dev, topk_idx_dev, row_max_dev, row_mean_dev, scores_dev, sumsq_dev, nullptr,
                        workspace_dev, workspace_bytes, chunk_rows, stream);
}

int bgx_row_sumsq(const void* store_dev, int64_t n_rows, int64_t D, int64_t store_row_stride, int32_t dtype,
                  float* row_sumsq_dev, void* stream) {
  return bgx::row_sumsq_impl(store_dev, n_rows, D, store_row_stride, dtype, row_sumsq_dev, stream);
}

int bgx_scan_known_norms(const void* store_dev, int64_t n_rows, int64_t D, int64_t store_row_stride, int32_t dtype,
                         const void* queries_dev, int32_t Q, float query_scale, int32_t unit_norm, int32_t k,
                         int64_t row_base, const float* row_sumsq_dev, float* topk_val_dev, int64_t* topk_idx_dev,
                         float* row_max_dev, float* row_mean_dev, float* scores_dev, void* workspace_dev,
                         size_t workspace_bytes, int64_t chunk_rows, void* stream) {
  if (row_sumsq_dev == nullptr) {
    bgx::set_error("scan_known_norms: null row_sumsq");
    return BGX_E_ARG;
  }
  return bgx::scan_impl(store_dev, n_rows, D, store_row_stride, dtype, queries_dev, Q, query_scale, unit_norm, k,
                        row_base, topk_val_dev, topk_idx_dev, row_max_dev, row_mean_dev, scores_dev, nullptr,
                        row_sumsq_dev, workspace_dev, workspace_bytes, chunk_rows, stream);
}

}  // extern "C"
