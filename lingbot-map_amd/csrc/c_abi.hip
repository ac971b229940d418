// extern "C" entry points: argument checks, then the launch helpers of the kernel files.
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include "lbm_internal.h"
#include "tables_logic.h"

namespace {
thread_local char g_last_error[512] = "";
}

int lbm_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int lbm_check_launch(const char* kernel_name) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return LBM_OK;
  return lbm_fail(LBM_ERR_HIP, "%s: %s", kernel_name, hipGetErrorString(e));
}

extern "C" {

int lbm_abi_version(void) { return LBM_ABI_VERSION; }

const char* lbm_last_error(void) { return g_last_error; }

int64_t lbm_tables_words(const lbm_cache_geom* geom) {
  if (!geom || !lbm_geom_valid(*geom)) return 0;
  return lbm_tables_layout(*geom).words;
}

int lbm_tables_step(int32_t* tables, const lbm_cache_geom* geom, int32_t n_streams,
                    const lbm_step_op* ops, int32_t* append_rows, int32_t* kv_rows,
                    int32_t* kv_page_ids, int32_t* kv_page_lens, void* stream) {
  if (!tables || !geom || !ops) return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: null tables, geom or ops");
  if (!lbm_geom_valid(*geom)) return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: invalid cache geometry");
  if (n_streams < 1 || n_streams > LBM_MAX_STREAMS)
    return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: n_streams %d outside [1, %d]", n_streams, LBM_MAX_STREAMS);
  for (int i = 0; i < n_streams; ++i) {
    const lbm_step_op& o = ops[i];
    if (o.ops & ~(LBM_OP_RESET | LBM_OP_ROLLBACK | LBM_OP_APPEND | LBM_OP_EVICT | LBM_OP_PLAN | LBM_OP_PLAN_NEWEST_SELF))
      return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: stream %d has unknown op bits 0x%x", i, o.ops);
    if ((o.ops & LBM_OP_PLAN_NEWEST_SELF) &&
        ((o.ops & (LBM_OP_APPEND | LBM_OP_PLAN)) != (LBM_OP_APPEND | LBM_OP_PLAN) || geom->layout != LBM_LAYOUT_FRAME_PAGES))
      return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: stream %d: LBM_OP_PLAN_NEWEST_SELF goes with LBM_OP_APPEND | "
                      "LBM_OP_PLAN in the frame_pages layout", i);
    if ((o.ops & LBM_OP_PLAN) && !kv_rows && !(kv_page_ids && kv_page_lens))
      return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: PLAN needs kv_rows or the page table outputs");
    if ((o.ops & LBM_OP_PLAN) && (o.expect_kv_tokens == INT32_MIN || o.kv_row_begin < 0 || o.page_out_begin < 0))
      return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: stream %d has a negative plan offset or count", i);
    if ((o.ops & LBM_OP_EVICT) && o.sliding_window < 0)
      return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: stream %d has a negative sliding_window", i);
    if (o.q_begin < 0) return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: stream %d has a negative q_begin", i);
  }
  // Every stream's workgroup writes its tokens_per_frame entries of append_rows (the rows of the
  // new frame, or -1 for a stream that does not append, idle streams included): two streams
  // with overlapping ranges would race inside one launch.
  if (append_rows)
    for (int i = 0; i < n_streams; ++i)
      for (int j = 0; j < i; ++j) {
        const long long d = (long long)ops[i].q_begin - ops[j].q_begin;
        if ((d < 0 ? -d : d) < geom->tokens_per_frame)
          return lbm_fail(LBM_ERR_INVALID, "lbm_tables_step: streams %d and %d overlap in append_rows (q_begin %d and %d, %d tokens per frame)",
                          j, i, ops[j].q_begin, ops[i].q_begin, geom->tokens_per_frame);
      }
  return lbm_launch_tables(tables, *geom, n_streams, ops, append_rows, kv_rows, kv_page_ids,
                           kv_page_lens, (hipStream_t)stream);
}

int lbm_rows_from_pages(const int32_t* kv_page_ids, const int32_t* kv_page_lens,
                        const int32_t* kv_indptr, const int32_t* kv_tokens,
                        const int32_t* kv_row_begin, int32_t n_streams, int32_t page_size,
                        int32_t* kv_rows, void* stream) {
  if (!kv_page_ids || !kv_page_lens || !kv_indptr || !kv_tokens || !kv_row_begin || !kv_rows)
    return lbm_fail(LBM_ERR_INVALID, "lbm_rows_from_pages: null argument");
  if (n_streams < 1 || n_streams > LBM_MAX_STREAMS || page_size <= 0)
    return lbm_fail(LBM_ERR_INVALID, "lbm_rows_from_pages: bad n_streams %d or page_size %d", n_streams, page_size);
  for (int i = 0; i < n_streams; ++i)
    if (kv_indptr[i + 1] < kv_indptr[i] || kv_tokens[i] < 0 || kv_row_begin[i] < 0)
      return lbm_fail(LBM_ERR_INVALID, "lbm_rows_from_pages: stream %d has a decreasing indptr or a negative count", i);
  return lbm_launch_rows_from_pages(kv_page_ids, kv_page_lens, kv_indptr, kv_tokens, kv_row_begin,
                                    n_streams, page_size, kv_rows, (hipStream_t)stream);
}

int lbm_kv_append(const void* k, const void* v, int32_t src_dtype, void* pool, int32_t pool_dtype,
                  const int32_t* append_rows, int32_t n_tokens, int32_t num_heads,
                  int32_t head_dim, int32_t page_size, void* stream) {
  if (n_tokens == 0) return LBM_OK;
  if (!k || !v || !pool || !append_rows) return lbm_fail(LBM_ERR_INVALID, "lbm_kv_append: null argument");
  if (n_tokens < 0 || num_heads <= 0 || head_dim <= 0 || page_size <= 0)
    return lbm_fail(LBM_ERR_INVALID, "lbm_kv_append: non-positive size");
  if ((src_dtype != LBM_DTYPE_BF16 && src_dtype != LBM_DTYPE_F32) ||
      (pool_dtype != LBM_DTYPE_BF16 && pool_dtype != LBM_DTYPE_F32))
    return lbm_fail(LBM_ERR_INVALID, "lbm_kv_append: unknown dtype");
  if ((num_heads * head_dim) % 8 != 0)
    return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_kv_append: num_heads * head_dim must be a multiple of 8");
  return lbm_launch_append(k, v, src_dtype, pool, pool_dtype, append_rows, n_tokens, num_heads,
                           head_dim, page_size, (hipStream_t)stream);
}

int lbm_qkv_prepare(const void* qkv, int32_t src_dtype, const float* q_norm_w, const float* q_norm_b,
                    const float* k_norm_w, const float* k_norm_b, float norm_eps, float q_scale, const float* rope_cs,
                    int32_t rope_layout, void* q_out, void* k_out, void* v_out, int32_t dst_dtype, void* pool,
                    const int32_t* append_rows, int32_t n_tokens, int32_t num_heads, int32_t head_dim,
                    int32_t page_size, void* stream) {
  if (!qkv || !q_out) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: null qkv or q_out");
  if (n_tokens < 0 || num_heads <= 0 || page_size <= 0)
    return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: bad sizes (tokens %d, heads %d, page %d)", n_tokens, num_heads, page_size);
  if (head_dim != 64) return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_qkv_prepare covers head_dim 64 (got %d)", head_dim);
  if ((src_dtype != LBM_DTYPE_BF16 && src_dtype != LBM_DTYPE_F32) || (dst_dtype != LBM_DTYPE_BF16 && dst_dtype != LBM_DTYPE_F32))
    return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: unknown dtype");
  const int n_norm = (q_norm_w != nullptr) + (q_norm_b != nullptr) + (k_norm_w != nullptr) + (k_norm_b != nullptr);
  if (n_norm != 0 && n_norm != 4)
    return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: the four LayerNorm arrays go together");
  if ((k_out == nullptr) != (v_out == nullptr)) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: k_out and v_out go together");
  if (append_rows && !pool) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: append_rows without a pool");
  if (rope_cs && rope_layout != LBM_ROPE_INTERLEAVED && rope_layout != LBM_ROPE_HALF_SPLIT)
    return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: unknown rope_layout %d", rope_layout);
  if (!(q_scale > 0.f)) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_prepare: q_scale must be positive (1 = plain q), got %g", (double)q_scale);
  return lbm_launch_qkv_prepare(qkv, src_dtype, q_norm_w, q_norm_b, k_norm_w, k_norm_b, norm_eps, q_scale, rope_cs, rope_layout, q_out,
                                k_out, v_out, dst_dtype, pool, append_rows, n_tokens, num_heads, page_size,
                                (hipStream_t)stream);
}

int lbm_linear_norm(const void* a, const lbm_row_norm* a_norm, const void* w, const float* bias, const float* gamma,
                    const void* residual, void* out, float* out_stats, int32_t M, int32_t N, int32_t K,
                    int32_t epilogue, void* workspace, size_t workspace_bytes, void* stream) {
  if (!a || !w || !out) return lbm_fail(LBM_ERR_INVALID, "lbm_linear: null a, w or out");
  if (M < 0 || N <= 0 || K <= 0) return lbm_fail(LBM_ERR_INVALID, "lbm_linear: bad shape %d x %d x %d", M, N, K);
  if (epilogue == LBM_LINEAR_BIAS_RESIDUAL && !residual)
    return lbm_fail(LBM_ERR_INVALID, "lbm_linear: the residual epilogue needs a residual");
  if (epilogue != LBM_LINEAR_BIAS_RESIDUAL && (residual || gamma))
    return lbm_fail(LBM_ERR_INVALID, "lbm_linear: residual / gamma given without the residual epilogue");
  return lbm_launch_linear(a, a_norm, w, bias, gamma, residual, out, out_stats, M, N, K, epilogue, workspace,
                           workspace_bytes, (hipStream_t)stream);
}

int lbm_linear_prefetch_hint(const void* next_read, size_t bytes) {
  lbm_set_prefetch_hint(next_read, next_read ? bytes : 0);
  return LBM_OK;
}

size_t lbm_linear_workspace_bytes(int32_t M, int32_t N, int32_t K, int32_t epilogue) {
  if (M <= 0 || N <= 0 || K <= 0 || N % 64 != 0 || K % 128 != 0) return 0;
  return lbm_linear_workspace_for(M, N, K, epilogue);
}

int lbm_linear(const void* a, const void* w, const float* bias, const float* gamma, const void* residual,
               void* out, int32_t M, int32_t N, int32_t K, int32_t epilogue, void* stream) {
  return lbm_linear_norm(a, nullptr, w, bias, gamma, residual, out, nullptr, M, N, K, epilogue, nullptr, 0, stream);
}

int32_t lbm_linear_stats_tiles(int32_t M, int32_t N) {
  if (M < 0 || N <= 0 || N % 64 != 0) return 0;
  return lbm_linear_stats_tiles_for(M, N);
}

int lbm_qkv_linear_prepare(const void* a, const void* w, const float* bias, int32_t M, int32_t K,
                           const float* q_norm_w, const float* q_norm_b, const float* k_norm_w,
                           const float* k_norm_b, float norm_eps, float q_scale, const float* rope_cs, int32_t rope_layout,
                           void* q_out, void* k_out, void* v_out, void* pool, const int32_t* append_rows,
                           int32_t num_heads, int32_t head_dim, int32_t page_size, void* stream) {
  return lbm_qkv_linear_prepare_norm(a, nullptr, w, bias, M, K, q_norm_w, q_norm_b, k_norm_w, k_norm_b, norm_eps, q_scale, rope_cs,
                                     rope_layout, q_out, k_out, v_out, pool, append_rows, num_heads, head_dim, page_size,
                                     stream);
}

int lbm_qkv_linear_prepare_norm(const void* a, const lbm_row_norm* a_norm, const void* w, const float* bias, int32_t M,
                                int32_t K, const float* q_norm_w, const float* q_norm_b, const float* k_norm_w,
                                const float* k_norm_b, float norm_eps, float q_scale, const float* rope_cs, int32_t rope_layout,
                                void* q_out, void* k_out, void* v_out, void* pool, const int32_t* append_rows,
                                int32_t num_heads, int32_t head_dim, int32_t page_size, void* stream) {
  if (!(q_scale > 0.f)) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_linear_prepare: q_scale must be positive (1 = plain q), got %g", (double)q_scale);
  if (!a || !w || !q_out) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_linear_prepare: null a, w or q_out");
  if (M < 0 || K <= 0 || num_heads <= 0) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_linear_prepare: bad shape");
  if (head_dim != 64) return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_qkv_linear_prepare: head_dim must be 64 (got %d)", head_dim);
  const int n_norm = (q_norm_w != nullptr) + (q_norm_b != nullptr) + (k_norm_w != nullptr) + (k_norm_b != nullptr);
  if (n_norm != 0 && n_norm != 4) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_linear_prepare: give all four LayerNorm parameters or none");
  if (rope_cs && rope_layout != LBM_ROPE_INTERLEAVED && rope_layout != LBM_ROPE_HALF_SPLIT)
    return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_linear_prepare: unknown rope_layout %d", rope_layout);
  if (append_rows && !pool) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_linear_prepare: append_rows without a pool");
  if (append_rows && page_size <= 0) return lbm_fail(LBM_ERR_INVALID, "lbm_qkv_linear_prepare: bad page_size");
  return lbm_launch_qkv_linear_prepare(a, a_norm, w, bias, M, K, q_norm_w, q_norm_b, k_norm_w, k_norm_b, norm_eps, q_scale, rope_cs,
                                       rope_layout, q_out, k_out, v_out, pool, append_rows, num_heads, page_size,
                                       (hipStream_t)stream);
}

int lbm_residual_norm(const void* x, const void* y, int32_t dtype, const float* gamma, const float* norm_w,
                      const float* norm_b, float norm_eps, void* x_out, void* n_out, int32_t rows, int32_t cols,
                      void* stream) {
  if (!x || !y || !x_out) return lbm_fail(LBM_ERR_INVALID, "lbm_residual_norm: null x, y or x_out");
  if (rows < 0 || cols <= 0) return lbm_fail(LBM_ERR_INVALID, "lbm_residual_norm: bad shape %d x %d", rows, cols);
  if (dtype != LBM_DTYPE_BF16 && dtype != LBM_DTYPE_F32) return lbm_fail(LBM_ERR_INVALID, "lbm_residual_norm: unknown dtype");
  if ((norm_w == nullptr) != (norm_b == nullptr)) return lbm_fail(LBM_ERR_INVALID, "lbm_residual_norm: norm_w and norm_b go together");
  if (norm_w && !n_out) return lbm_fail(LBM_ERR_INVALID, "lbm_residual_norm: LayerNorm asked for without n_out");
  return lbm_launch_residual_norm(x, y, dtype, gamma, norm_w, norm_b, norm_eps, x_out, n_out, rows, cols, (hipStream_t)stream);
}

static int lbm_check_attn_streams(const lbm_attn_stream* s, int n, const char* who) {
  if (!s) return lbm_fail(LBM_ERR_INVALID, "%s: null streams", who);
  if (n < 1 || n > LBM_MAX_STREAMS) return lbm_fail(LBM_ERR_INVALID, "%s: n_streams %d outside [1, %d]", who, n, LBM_MAX_STREAMS);
  for (int i = 0; i < n; ++i)
    if (s[i].q_begin < 0 || s[i].q_rows < 0 || s[i].kv_row_begin < 0 || s[i].kv_tokens < 0)
      return lbm_fail(LBM_ERR_INVALID, "%s: stream %d has a negative field", who, i);
  return LBM_OK;
}

size_t lbm_attn_workspace_bytes(const lbm_attn_stream* streams, int32_t n_streams,
                                int32_t num_heads, int32_t head_dim) {
  if (lbm_check_attn_streams(streams, n_streams, "lbm_attn_workspace_bytes") != LBM_OK) return 0;
  if (num_heads <= 0 || head_dim <= 0) return 0;
  LbmAttnSchedule sch;
  lbm_attn_schedule(streams, n_streams, num_heads, &sch);
  return lbm_attn_schedule_bytes(sch, num_heads, head_dim);
}

static int lbm_attn_run_impl(const char* who, const void* q, const void* pool, void* out, const void* self_k,
                             const void* self_v, const int32_t* kv_rows, const int32_t* live_kv_tokens,
                             const lbm_attn_stream* streams, int32_t n_streams, int32_t num_heads,
                             int32_t head_dim, int32_t page_size, int32_t dtype, float sm_scale,
                             void* workspace, size_t workspace_bytes, void* stream,
                             const int32_t* append_rows = nullptr, int32_t append_tokens = 0) {
  int rc = lbm_check_attn_streams(streams, n_streams, who);
  if (rc != LBM_OK) return rc;
  if (!q || !pool || !out || !kv_rows) return lbm_fail(LBM_ERR_INVALID, "%s: null q, pool, out or kv_rows", who);
  if (num_heads <= 0 || head_dim <= 0 || page_size <= 0) return lbm_fail(LBM_ERR_INVALID, "%s: non-positive size", who);
  if (!(sm_scale >= 0.f)) return lbm_fail(LBM_ERR_INVALID, "%s: sm_scale must be positive, or 0 for a q that already carries it (got %g)", who, (double)sm_scale);
  if ((self_k == nullptr) != (self_v == nullptr)) return lbm_fail(LBM_ERR_INVALID, "%s: self_k and self_v go together", who);
  if (live_kv_tokens)
    for (int i = 0; i < n_streams; ++i)
      if (streams[i].live_at < 0) return lbm_fail(LBM_ERR_INVALID, "%s: stream %d has a negative live_at", who, i);
  LbmAttnSchedule sch;
  lbm_attn_schedule(streams, n_streams, num_heads, &sch);
  const size_t need = lbm_attn_schedule_bytes(sch, num_heads, head_dim);
  if (need > 0 && (!workspace || workspace_bytes < need))
    return lbm_fail(LBM_ERR_WORKSPACE, "%s: workspace of %zu bytes, %zu needed", who, workspace_bytes, need);
  return lbm_launch_attention(q, pool, out, self_k, self_v, kv_rows, live_kv_tokens, sch, num_heads, head_dim,
                              page_size, dtype, sm_scale, workspace, (hipStream_t)stream, append_rows, append_tokens);
}

int lbm_attn_run(const void* q, const void* pool, void* out, const void* self_k,
                 const void* self_v, const int32_t* kv_rows, const lbm_attn_stream* streams,
                 int32_t n_streams, int32_t num_heads, int32_t head_dim, int32_t page_size,
                 int32_t dtype, float sm_scale, void* workspace, size_t workspace_bytes,
                 void* stream) {
  return lbm_attn_run_impl("lbm_attn_run", q, pool, out, self_k, self_v, kv_rows, nullptr, streams, n_streams,
                           num_heads, head_dim, page_size, dtype, sm_scale, workspace, workspace_bytes, stream);
}

int lbm_attn_run_append(const void* q, void* pool, void* out, const void* new_k, const void* new_v,
                        const int32_t* kv_rows, const int32_t* append_rows, int32_t append_tokens,
                        const lbm_attn_stream* streams, int32_t n_streams, int32_t num_heads,
                        int32_t head_dim, int32_t page_size, int32_t dtype, float sm_scale,
                        void* workspace, size_t workspace_bytes, void* stream) {
  if (!new_k || !new_v || !append_rows)
    return lbm_fail(LBM_ERR_INVALID, "lbm_attn_run_append: null new_k, new_v or append_rows");
  if (append_tokens < 0) return lbm_fail(LBM_ERR_INVALID, "lbm_attn_run_append: negative append_tokens");
  return lbm_attn_run_impl("lbm_attn_run_append", q, pool, out, new_k, new_v, kv_rows, nullptr, streams, n_streams,
                           num_heads, head_dim, page_size, dtype, sm_scale, workspace, workspace_bytes, stream,
                           append_rows, append_tokens);
}

int lbm_attn_run_live(const void* q, const void* pool, void* out, const void* self_k,
                      const void* self_v, const int32_t* kv_rows, const int32_t* live_kv_tokens,
                      const lbm_attn_stream* streams, int32_t n_streams, int32_t num_heads,
                      int32_t head_dim, int32_t page_size, int32_t dtype, float sm_scale,
                      void* workspace, size_t workspace_bytes, void* stream) {
  if (!live_kv_tokens) return lbm_fail(LBM_ERR_INVALID, "lbm_attn_run_live: null live_kv_tokens");
  return lbm_attn_run_impl("lbm_attn_run_live", q, pool, out, self_k, self_v, kv_rows, live_kv_tokens, streams,
                           n_streams, num_heads, head_dim, page_size, dtype, sm_scale, workspace, workspace_bytes,
                           stream);
}

int lbm_attn_run_static(const void* q, const void* pool, void* out, const void* self_k,
                        const void* self_v, const int32_t* kv_rows, const lbm_attn_stream* streams,
                        int32_t n_streams, int32_t num_heads, int32_t head_dim, int32_t page_size,
                        int32_t dtype, float sm_scale, void* stream) {
  int rc = lbm_check_attn_streams(streams, n_streams, "lbm_attn_run_static");
  if (rc != LBM_OK) return rc;
  if (num_heads <= 0 || head_dim <= 0) return lbm_fail(LBM_ERR_INVALID, "lbm_attn_run_static: non-positive size");
  LbmAttnSchedule sch;
  lbm_attn_schedule(streams, n_streams, num_heads, &sch);
  const size_t need = lbm_attn_schedule_bytes(sch, num_heads, head_dim);
  void* ws = nullptr;
  size_t ws_bytes = 0;
  rc = lbm_static_scratch(&ws, &ws_bytes);
  if (rc != LBM_OK) return rc;
  if (need > ws_bytes)
    return lbm_fail(LBM_ERR_WORKSPACE, "lbm_attn_run_static: this batch needs %zu bytes of scratch, the static array holds %zu "
                    "(LBM_STATIC_SCRATCH_MIB = %d); use lbm_attn_run with a workspace of your own",
                    need, ws_bytes, LBM_STATIC_SCRATCH_MIB);
  return lbm_attn_run_impl("lbm_attn_run_static", q, pool, out, self_k, self_v, kv_rows, nullptr, streams, n_streams,
                           num_heads, head_dim, page_size, dtype, sm_scale, ws, ws_bytes, stream);
}

}  // extern "C"
