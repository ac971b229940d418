// Declarations shared by the translation units of the library (not part of the C ABI).
#ifndef LBM_INTERNAL_H
#define LBM_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>
#include "../../include/lbm_paged_attn.h"

// Records `msg` as the calling thread's last error and returns `code`.
int lbm_fail(int code, const char* fmt, ...);
// hipGetLastError() after a launch; LBM_OK or LBM_ERR_HIP with the kernel's name recorded.
int lbm_check_launch(const char* kernel_name);

int lbm_launch_tables(int32_t* tables, const lbm_cache_geom& g, int n_streams,
                      const lbm_step_op* ops, int32_t* append_rows, int32_t* kv_rows,
                      int32_t* page_ids, int32_t* page_lens, hipStream_t stream);
int lbm_launch_rows_from_pages(const int32_t* page_ids, const int32_t* page_lens,
                               const int32_t* indptr, const int32_t* kv_tokens,
                               const int32_t* row_begin, int n_streams, int page_size,
                               int32_t* kv_rows, hipStream_t stream);
int lbm_launch_append(const void* k, const void* v, int src_dtype, void* pool, int pool_dtype,
                      const int32_t* append_rows, int n_tokens, int num_heads, int head_dim,
                      int page_size, hipStream_t stream);

int lbm_launch_qkv_prepare(const void* qkv, int src_dtype, const float* q_norm_w, const float* q_norm_b,
                           const float* k_norm_w, const float* k_norm_b, float norm_eps, float q_scale,
                           const float* rope_cs, int rope_layout, void* q_out, void* k_out, void* v_out,
                           int dst_dtype, void* pool, const int32_t* append_rows, int n_tokens,
                           int num_heads, int page_size, hipStream_t stream);

int lbm_launch_residual_norm(const void* x, const void* y, int dtype, const float* gamma, const float* norm_w,
                             const float* norm_b, float eps, void* x_out, void* n_out, int rows, int cols,
                             hipStream_t stream);

int lbm_launch_linear(const void* a, const lbm_row_norm* a_norm, const void* w, const float* bias, const float* gamma,
                      const void* residual, void* out, float* out_stats, int M, int N, int K, int epilogue,
                      void* workspace, size_t workspace_bytes, hipStream_t stream);
int lbm_linear_stats_tiles_for(int M, int N);
void lbm_set_prefetch_hint(const void* ptr, size_t bytes);
size_t lbm_linear_workspace_for(int M, int N, int K, int epilogue);

int lbm_launch_qkv_linear_prepare(const void* a, const lbm_row_norm* a_norm, const void* w, const float* bias, int M, int K,
                                  const float* q_norm_w, const float* q_norm_b, const float* k_norm_w,
                                  const float* k_norm_b, float norm_eps, float q_scale, const float* rope_cs, int rope_layout,
                                  void* q_out, void* k_out, void* v_out, void* pool, const int32_t* append_rows,
                                  int num_heads, int page_size, hipStream_t stream);

// Split-KV schedule of one attention call, computed on the host from token counts only.
struct LbmAttnStreamPlan {
  int32_t q_begin, q_rows, kv_row_begin, kv_tokens, live_at;
  int32_t n_qtiles, n_splits, tiles_per_split;
  int32_t wg_begin;    // first workgroup of this stream
  int32_t part_begin;  // first partial-result row (unit: q row of one split) in the workspace
};
struct LbmAttnSchedule {
  int32_t n_streams;
  int32_t total_wgs;
  int32_t small;       // every stream's KV is short: the in-workgroup split kernel, no partial results
  int64_t part_rows;   // rows of partial results over all streams (0 when nothing is split)
  LbmAttnStreamPlan s[LBM_MAX_STREAMS];
};
void lbm_attn_schedule(const lbm_attn_stream* streams, int n_streams, int num_heads,
                       LbmAttnSchedule* out);
size_t lbm_attn_schedule_bytes(const LbmAttnSchedule& sch, int num_heads, int head_dim);

int lbm_launch_attention(const void* q, const void* pool, void* out, const void* self_k,
                         const void* self_v, const int32_t* kv_rows, const int32_t* live_kv_tokens,
                         const LbmAttnSchedule& sch,
                         int num_heads, int head_dim, int page_size, int dtype, float sm_scale,
                         void* workspace, hipStream_t stream,
                         const int32_t* append_rows = nullptr, int append_tokens = 0);

// Address and size of the library's static device scratch array on the current device (looked
// up once per device; no allocation).
int lbm_static_scratch(void** ptr, size_t* bytes);

#endif  // LBM_INTERNAL_H
