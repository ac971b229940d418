// Index-only kernels: page-table maintenance (one workgroup per stream) and expansion of a
// FlashInfer-style page table into the row table the attention kernel gathers through.
// These kernels move a few KB of int32 per frame step; they are latency-bound, so each
// stream gets one 1024-thread workgroup and all requested operations run in one launch.
#include <hip/hip_runtime.h>
#include "tables_logic.h"
#include "lbm_internal.h"

struct LbmStepOps { lbm_step_op s[LBM_MAX_STREAMS]; };

__global__ __launch_bounds__(1024) void lbm_tables_kernel(
    int32_t* __restrict__ tables, lbm_cache_geom g, LbmStepOps ops, int32_t* append_rows,
    int32_t* kv_rows, int32_t* page_ids, int32_t* page_lens) {
  const int b = blockIdx.x;
  const lbm_step_op op = ops.s[b];
  const int tid = threadIdx.x, nthr = blockDim.x;
  if (op.ops == 0) {
    if (append_rows)
      for (int t = tid; t < g.tokens_per_frame; t += nthr) append_rows[op.q_begin + t] = -1;
    return;
  }
  const LbmTablesLayout L = lbm_tables_layout(g);
  int32_t* st = tables + (long long)b * L.words;
  LbmHdr h = lbm_hdr_load(st);
  if (op.ops & LBM_OP_RESET) {
    lbm_phase_reset(st, g, L, b * g.pages_per_stream, tid, nthr, h);
    __syncthreads();
  }
  if (op.ops & LBM_OP_ROLLBACK) {
    lbm_phase_rollback(st, g, L, tid, nthr, h);
    __syncthreads();
  }
  if (op.ops & LBM_OP_APPEND) {
    lbm_phase_append(st, g, L, append_rows ? append_rows + op.q_begin : nullptr, tid, nthr, h);
    __syncthreads();
  } else if (append_rows) {
    for (int t = tid; t < g.tokens_per_frame; t += nthr) append_rows[op.q_begin + t] = -1;
  }
  if (op.ops & LBM_OP_EVICT) {
    lbm_phase_evict(st, g, L, op.sliding_window, op.keep_tokens, tid, nthr, h);
    __syncthreads();
  }
  if (op.ops & LBM_OP_PLAN) lbm_phase_plan(st, g, L, op, kv_rows, page_ids, page_lens, tid, nthr, h);
  if (tid == 0) lbm_hdr_store(st, h);
}

struct LbmPageSegs {
  int32_t page_begin[LBM_MAX_STREAMS + 1];
  int32_t kv_tokens[LBM_MAX_STREAMS];
  int32_t row_begin[LBM_MAX_STREAMS];
};

// One workgroup per stream: running exclusive scan of the page lengths in chunks of
// blockDim.x pages, then every thread writes the rows of its page.
__global__ __launch_bounds__(1024) void lbm_rows_from_pages_kernel(
    const int32_t* __restrict__ page_ids, const int32_t* __restrict__ page_lens,
    LbmPageSegs segs, int page_size, int32_t* __restrict__ kv_rows) {
  __shared__ int scan[1024];
  __shared__ int carry;
  const int b = blockIdx.x, tid = threadIdx.x, nthr = blockDim.x;
  const int p0 = segs.page_begin[b], p1 = segs.page_begin[b + 1];
  const int limit = segs.kv_tokens[b];
  int32_t* out = kv_rows + segs.row_begin[b];
  if (tid == 0) carry = 0;
  __syncthreads();
  for (int base = p0; base < p1; base += nthr) {
    const int p = base + tid;
    int len = 0, id = 0;
    if (p < p1) {
      len = page_lens[p];
      id = page_ids[p];
      len = len < 0 ? 0 : (len > page_size ? page_size : len);
    }
    scan[tid] = len;
    __syncthreads();
    for (int off = 1; off < nthr; off <<= 1) {
      const int v = tid >= off ? scan[tid - off] : 0;
      __syncthreads();
      scan[tid] += v;
      __syncthreads();
    }
    const int start = carry + scan[tid] - len;
    for (int s = 0; s < len; ++s)
      if (start + s < limit) out[start + s] = id * 2 * page_size + s;
    __syncthreads();
    if (tid == nthr - 1) carry += scan[tid];
    __syncthreads();
  }
  // A caller whose token count exceeds the table's total still gets defined rows.
  for (int i = carry + tid; i < limit; i += nthr) out[i] = 0;
}

int lbm_launch_tables(int32_t* tables, const lbm_cache_geom& g, int n_streams,
                      const lbm_step_op* ops, int32_t* append_rows, int32_t* kv_rows,
                      int32_t* page_ids, int32_t* page_lens, hipStream_t stream) {
  LbmStepOps o;
  for (int i = 0; i < LBM_MAX_STREAMS; ++i) o.s[i] = lbm_step_op{};
  for (int i = 0; i < n_streams; ++i) o.s[i] = ops[i];
  hipLaunchKernelGGL(lbm_tables_kernel, dim3(n_streams), dim3(1024), 0, stream, tables, g, o,
                     append_rows, kv_rows, page_ids, page_lens);
  return lbm_check_launch("lbm_tables_kernel");
}

int lbm_launch_rows_from_pages(const int32_t* page_ids, const int32_t* page_lens,
                               const int32_t* indptr, const int32_t* kv_tokens,
                               const int32_t* row_begin, int n_streams, int page_size,
                               int32_t* kv_rows, hipStream_t stream) {
  LbmPageSegs s;
  for (int i = 0; i <= LBM_MAX_STREAMS; ++i) s.page_begin[i] = 0;
  for (int i = 0; i < LBM_MAX_STREAMS; ++i) { s.kv_tokens[i] = 0; s.row_begin[i] = 0; }
  for (int i = 0; i < n_streams; ++i) {
    s.page_begin[i] = indptr[i];
    s.kv_tokens[i] = kv_tokens[i];
    s.row_begin[i] = row_begin[i];
  }
  s.page_begin[n_streams] = indptr[n_streams];
  hipLaunchKernelGGL(lbm_rows_from_pages_kernel, dim3(n_streams), dim3(1024), 0, stream,
                     page_ids, page_lens, s, page_size, kv_rows);
  return lbm_check_launch("lbm_rows_from_pages_kernel");
}
