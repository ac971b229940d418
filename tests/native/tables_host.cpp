// CPU build of the page-table state machine for the table tests: the same phase functions
// the HIP kernel runs (csrc/tables_logic.h), executed by one host thread per stream.
// Test infrastructure only; the product library does not contain this entry point.
#include "../../lingbot-map_amd/csrc/tables_logic.h"

extern "C" int lbm_tables_step_host(int32_t* tables, const lbm_cache_geom* geom, int32_t n_streams,
                                    const lbm_step_op* ops, int32_t* append_rows, int32_t* kv_rows,
                                    int32_t* page_ids, int32_t* page_lens) {
  if (!lbm_geom_valid(*geom)) return LBM_ERR_INVALID;
  const lbm_cache_geom g = *geom;
  const LbmTablesLayout L = lbm_tables_layout(g);
  for (int b = 0; b < n_streams; ++b) {
    const lbm_step_op op = ops[b];
    if (op.ops == 0) {
      if (append_rows) for (int t = 0; t < g.tokens_per_frame; ++t) append_rows[op.q_begin + t] = -1;
      continue;
    }
    int32_t* st = tables + (long long)b * L.words;
    LbmHdr h = lbm_hdr_load(st);
    if (op.ops & LBM_OP_RESET) lbm_phase_reset(st, g, L, b * g.pages_per_stream, 0, 1, h);
    if (op.ops & LBM_OP_ROLLBACK) lbm_phase_rollback(st, g, L, 0, 1, h);
    if (op.ops & LBM_OP_APPEND) lbm_phase_append(st, g, L, append_rows ? append_rows + op.q_begin : nullptr, 0, 1, h);
    else if (append_rows) for (int t = 0; t < g.tokens_per_frame; ++t) append_rows[op.q_begin + t] = -1;
    if (op.ops & LBM_OP_EVICT) lbm_phase_evict(st, g, L, op.sliding_window, op.keep_tokens, 0, 1, h);
    if (op.ops & LBM_OP_PLAN) lbm_phase_plan(st, g, L, op, kv_rows, page_ids, page_lens, 0, 1, h);
    lbm_hdr_store(st, h);
  }
  return LBM_OK;
}

extern "C" long long lbm_tables_words_host(const lbm_cache_geom* geom) {
  return lbm_geom_valid(*geom) ? lbm_tables_layout(*geom).words : 0;
}
