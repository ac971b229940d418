// Page-table state machine of one stream, written so that the same code runs as one HIP
// workgroup (tid = threadIdx.x, nthr = blockDim.x, a barrier between phases) or as one host
// thread (tid = 0, nthr = 1) in the CPU build the table tests use.
//
// The policy is the reference's (lingbot_map/layers/flashinfer_cache.py): LIFO free list
// (:496, :538), anchor-then-window routing (:507-510), oldest-first eviction that returns
// pages to the tail of the free list (:252-254), packed special stream (:529-553),
// rollback to the free-list tail (:280-301).  No phase reads a word that the same phase
// writes, so the order of threads inside a phase does not matter.
#ifndef LBM_TABLES_LOGIC_H
#define LBM_TABLES_LOGIC_H

#include "../../include/lbm_paged_attn.h"

#if defined(__HIPCC__)
#define LBM_HD __host__ __device__ __forceinline__
#else
#define LBM_HD inline
#endif

struct LbmTablesLayout {
  int ppf;          // pages a frame takes
  int tpf;          // tokens of a frame stored in those pages
  int kpm;          // most pages a compacted frame keeps
  int ring_frames;  // capacity of the window ring, in frames
  int off_free_patch, off_free_special, off_anchor, off_window, off_special;
  int off_mem_pages, off_mem_tcum, off_mem_pcum;
  long long words;
};

LBM_HD int lbm_ceil_div(int a, int b) { return (a + b - 1) / b; }

LBM_HD bool lbm_geom_valid(const lbm_cache_geom& g) {
  if (g.layout != LBM_LAYOUT_TWO_STREAM && g.layout != LBM_LAYOUT_FRAME_PAGES) return false;
  if (g.page_size <= 0 || g.num_special_tokens < 0 || g.scale_frames < 0) return false;
  if (g.tokens_per_frame <= g.num_special_tokens) return false;  // flashinfer_cache.py:113
  if (g.patch_pages <= 0 || g.special_pages < 0 || g.memory_frames < 0) return false;
  if (g.pages_per_stream < g.patch_pages + g.special_pages) return false;
  return true;
}

LBM_HD LbmTablesLayout lbm_tables_layout(const lbm_cache_geom& g) {
  LbmTablesLayout L;
  const bool two = g.layout == LBM_LAYOUT_TWO_STREAM;
  L.tpf = two ? g.tokens_per_frame - g.num_special_tokens : g.tokens_per_frame;
  L.ppf = lbm_ceil_div(L.tpf, g.page_size);
  L.kpm = two ? 0 : lbm_ceil_div(g.num_special_tokens, g.page_size);
  L.ring_frames = g.patch_pages / L.ppf;
  int off = LBM_HDR_WORDS;
  L.off_free_patch = off;   off += g.patch_pages;
  L.off_free_special = off; off += g.special_pages;
  L.off_anchor = off;       off += g.scale_frames * L.ppf;
  L.off_window = off;       off += L.ring_frames * L.ppf;
  L.off_special = off;      off += g.special_pages;
  L.off_mem_pages = off;    off += g.memory_frames * L.kpm;
  L.off_mem_tcum = off;     off += g.memory_frames + 1;
  L.off_mem_pcum = off;     off += g.memory_frames + 1;
  L.words = off;
  return L;
}

// Header snapshot taken by every thread at the start of a phase.
struct LbmHdr {
  int fc, na, wh, wc, nf, nfs, nsp, stc, nm, nmp, err;
};

LBM_HD LbmHdr lbm_hdr_load(const int32_t* st) {
  LbmHdr h;
  h.fc = st[LBM_HDR_FRAME_COUNT];      h.na = st[LBM_HDR_N_ANCHOR];
  h.wh = st[LBM_HDR_WIN_HEAD];         h.wc = st[LBM_HDR_WIN_COUNT];
  h.nf = st[LBM_HDR_N_FREE_PATCH];     h.nfs = st[LBM_HDR_N_FREE_SPECIAL];
  h.nsp = st[LBM_HDR_N_SPECIAL_PAGES]; h.stc = st[LBM_HDR_SPECIAL_TOKENS];
  h.nm = st[LBM_HDR_N_MEMORY];         h.nmp = st[LBM_HDR_N_MEMORY_PAGES];
  h.err = st[LBM_HDR_ERROR];
  return h;
}

LBM_HD void lbm_hdr_store(int32_t* st, const LbmHdr& h) {
  st[LBM_HDR_FRAME_COUNT] = h.fc;      st[LBM_HDR_N_ANCHOR] = h.na;
  st[LBM_HDR_WIN_HEAD] = h.wh;         st[LBM_HDR_WIN_COUNT] = h.wc;
  st[LBM_HDR_N_FREE_PATCH] = h.nf;     st[LBM_HDR_N_FREE_SPECIAL] = h.nfs;
  st[LBM_HDR_N_SPECIAL_PAGES] = h.nsp; st[LBM_HDR_SPECIAL_TOKENS] = h.stc;
  st[LBM_HDR_N_MEMORY] = h.nm;         st[LBM_HDR_N_MEMORY_PAGES] = h.nmp;
  st[LBM_HDR_ERROR] = h.err;
}

// ---------------------------------------------------------------------------- reset
// flashinfer_cache.py:423-432.  `h` is the header to commit after the phase.
LBM_HD void lbm_phase_reset(int32_t* st, const lbm_cache_geom& g, const LbmTablesLayout& L,
                            int page_base, int tid, int nthr, LbmHdr& h) {
  for (int i = tid; i < g.patch_pages; i += nthr) st[L.off_free_patch + i] = page_base + i;
  for (int i = tid; i < g.special_pages; i += nthr)
    st[L.off_free_special + i] = page_base + g.patch_pages + i;
  if (tid == 0) { st[L.off_mem_tcum] = 0; st[L.off_mem_pcum] = 0; }
  h = LbmHdr{};
  h.nf = g.patch_pages;
  h.nfs = g.special_pages;
}

// ---------------------------------------------------------------------------- rollback
// flashinfer_cache.py:268-301.
LBM_HD void lbm_phase_rollback(int32_t* st, const lbm_cache_geom& g, const LbmTablesLayout& L,
                               int tid, int nthr, LbmHdr& h) {
  const bool two = g.layout == LBM_LAYOUT_TWO_STREAM;
  const bool from_window = h.fc > g.scale_frames;
  int new_count = h.stc, n_pop = 0;
  if (two) {
    new_count = h.stc - g.num_special_tokens;
    n_pop = h.nsp - (new_count > 0 ? lbm_ceil_div(new_count, g.page_size) : 0);
  }
  if (h.fc <= 0 || (from_window ? h.wc <= 0 : h.na <= 0) || new_count < 0) {
    h.err |= LBM_TERR_ROLLBACK;
    return;
  }
  const int32_t* src = from_window
      ? st + L.off_window + ((h.wh + h.wc - 1) % L.ring_frames) * L.ppf
      : st + L.off_anchor + (h.na - 1) * L.ppf;
  for (int j = tid; j < L.ppf; j += nthr) st[L.off_free_patch + h.nf + j] = src[L.ppf - 1 - j];
  for (int k = tid; k < n_pop; k += nthr)
    st[L.off_free_special + h.nfs + k] = st[L.off_special + h.nsp - 1 - k];
  if (from_window) h.wc -= 1; else h.na -= 1;
  h.nf += L.ppf;
  h.nfs += n_pop;
  h.nsp -= n_pop;
  h.stc = new_count;
  h.fc -= 1;
}

// ---------------------------------------------------------------------------- append
// Allocation half of append_frame: flashinfer_cache.py:474-553.  Writes the K row of every
// token of the new frame to rows_out[0 .. tokens_per_frame).
LBM_HD void lbm_phase_append(int32_t* st, const lbm_cache_geom& g, const LbmTablesLayout& L,
                             int32_t* rows_out, int tid, int nthr, LbmHdr& h) {
  const bool two = g.layout == LBM_LAYOUT_TWO_STREAM;
  const int S = g.page_size, n_sp = g.num_special_tokens, T = g.tokens_per_frame;
  const bool to_anchor = h.na < g.scale_frames;
  const int new_sp = two ? lbm_ceil_div(h.stc + n_sp, S) - h.nsp : 0;
  int err = 0;
  if (h.nf < L.ppf) err |= LBM_TERR_PATCH_POOL;
  if (!to_anchor && h.wc >= L.ring_frames) err |= LBM_TERR_WINDOW_RING;
  if (new_sp > h.nfs) err |= LBM_TERR_SPECIAL_POOL;
  if (err) {
    h.err |= err;
    if (rows_out) for (int t = tid; t < T; t += nthr) rows_out[t] = -1;
    return;
  }
  const int32_t* fp = st + L.off_free_patch;
  int32_t* dst = to_anchor ? st + L.off_anchor + h.na * L.ppf
                           : st + L.off_window + ((h.wh + h.wc) % L.ring_frames) * L.ppf;
  for (int j = tid; j < L.ppf; j += nthr) dst[j] = fp[h.nf - 1 - j];
  if (rows_out) {
    for (int t = tid; t < T; t += nthr) {
      int page, slot;
      if (!two) {
        page = fp[h.nf - 1 - t / S]; slot = t % S;
      } else if (t >= n_sp) {
        const int i = t - n_sp;
        page = fp[h.nf - 1 - i / S]; slot = i % S;
      } else {
        const int c = h.stc + t, pi = c / S;
        slot = c % S;
        page = pi < h.nsp ? st[L.off_special + pi] : st[L.off_free_special + h.nfs - 1 - (pi - h.nsp)];
      }
      rows_out[t] = page * 2 * S + slot;
    }
  }
  for (int k = tid; k < new_sp; k += nthr)
    st[L.off_special + h.nsp + k] = st[L.off_free_special + h.nfs - 1 - k];
  if (to_anchor) h.na += 1; else h.wc += 1;
  h.nf -= L.ppf;
  h.nfs -= new_sp;
  h.nsp += new_sp;
  if (two) h.stc += n_sp;
  h.fc += 1;
}

// ---------------------------------------------------------------------------- evict
// flashinfer_cache.py:252-254; in the frame_pages layout the leading pages of an evicted
// frame stay as trajectory memory with `keep` valid tokens
// (lingbot_map/layers/attention.py:690-705), nothing is copied.
LBM_HD void lbm_phase_evict(int32_t* st, const lbm_cache_geom& g, const LbmTablesLayout& L,
                            int window, int keep, int tid, int nthr, LbmHdr& h) {
  const int n_ev = h.wc - window;
  if (n_ev <= 0) return;
  const bool two = g.layout == LBM_LAYOUT_TWO_STREAM;
  if (two || keep < 0) keep = 0;
  if (keep > g.num_special_tokens) keep = g.num_special_tokens;
  const int kp = keep ? lbm_ceil_div(keep, g.page_size) : 0;
  if (keep && h.nm + n_ev > g.memory_frames) { h.err |= LBM_TERR_MEMORY_FULL; return; }
  const int per = L.ppf - kp;
  const int32_t* win = st + L.off_window;
  for (int i = tid; i < n_ev * per; i += nthr) {
    const int e = i / per, j = kp + i % per;
    st[L.off_free_patch + h.nf + i] = win[((h.wh + e) % L.ring_frames) * L.ppf + j];
  }
  for (int i = tid; i < n_ev * kp; i += nthr) {
    const int e = i / kp, j = i % kp;
    st[L.off_mem_pages + h.nmp + i] = win[((h.wh + e) % L.ring_frames) * L.ppf + j];
  }
  if (keep) {
    for (int e = tid; e < n_ev; e += nthr) {
      st[L.off_mem_tcum + h.nm + e + 1] = h.stc + (e + 1) * keep;
      st[L.off_mem_pcum + h.nm + e + 1] = h.nmp + (e + 1) * kp;
    }
    h.nm += n_ev;
    h.nmp += n_ev * kp;
    h.stc += n_ev * keep;
  }
  h.wh = (h.wh + n_ev) % L.ring_frames;
  h.wc -= n_ev;
  h.nf += n_ev * per;
}

// ---------------------------------------------------------------------------- plan
// build_visible_page_table + compute_last_page_len (flashinfer_cache.py:438-470) with a
// valid length per page, plus the dense row table the attention kernel gathers through.
// Never writes more row entries than the host says the table holds (op.expect_kv_tokens, or the
// capacity it gives instead) and publishes a count within that bound, so a host/device
// disagreement cannot make the attention kernel read outside the table (it sets
// LBM_TERR_KV_COUNT instead).
LBM_HD void lbm_phase_plan(int32_t* st, const lbm_cache_geom& g, const LbmTablesLayout& L,
                           const lbm_step_op& op, int32_t* kv_rows, int32_t* page_ids,
                           int32_t* page_lens, int tid, int nthr, LbmHdr& h) {
  const bool two = g.layout == LBM_LAYOUT_TWO_STREAM;
  const int S = g.page_size;
  const int nfr = h.na + h.wc;
  const int frame_tokens = nfr * L.tpf;
  const int self_n = op.self_tokens > 0 ? op.self_tokens : 0;
  // LBM_OP_PLAN_NEWEST_SELF: the newest cached frame (the one this step appended: the last of the
  // frame list) is named by the caller's own rows, in the place its pool rows would take
  const bool newest_self = (op.ops & LBM_OP_PLAN_NEWEST_SELF) != 0 && !two && nfr > 0;
  int total = frame_tokens + h.stc + self_n;
  // expect_kv_tokens >= 0: the host's own count, which must agree; < 0: the host does not track
  // the count and gives the capacity of this stream's part of kv_rows instead
  const bool counted = op.expect_kv_tokens >= 0;
  const int limit = counted ? op.expect_kv_tokens : -op.expect_kv_tokens;
  if (counted ? total != limit : total > limit) h.err |= LBM_TERR_KV_COUNT;
  const int32_t* anchor = st + L.off_anchor;
  const int32_t* win = st + L.off_window;
  if (kv_rows) {
    int32_t* out = kv_rows + op.kv_row_begin;
    // token t of a page list sits in page t / S, slot t % S; page sizes are powers of two in
    // every configuration but one (page = patches per frame), so the common case is a shift
    const int shift = (S & (S - 1)) == 0 ? __builtin_ctz((unsigned)S) : -1;
    // a thread owns token slots t, t + nthr, ... of every frame (consecutive lanes write
    // consecutive rows); eight frames at a time so that their page-id loads are in flight
    // together (no division per token, no load waiting on the previous frame's store)
    for (int t = tid; t < L.tpf; t += nthr) {
      const int pg = shift >= 0 ? t >> shift : t / S;
      const int slot = t - pg * S;
      for (int f0 = 0; f0 < nfr; f0 += 8) {
        int32_t page[8];
#ifdef __HIP_DEVICE_COMPILE__
#pragma unroll
#endif
        for (int k = 0; k < 8; ++k) {
          const int f = f0 + k < nfr ? f0 + k : nfr - 1;
          int r = h.wh + f - h.na;                     // ring slot of window frame f - na
          if (r >= L.ring_frames) r -= L.ring_frames;  // wh < ring_frames and at most ring_frames window frames
          const int32_t* pages = f < h.na ? anchor + f * L.ppf : win + r * L.ppf;
          page[k] = pages[pg];
        }
#ifdef __HIP_DEVICE_COMPILE__
#pragma unroll
#endif
        for (int k = 0; k < 8; ++k) {
          const int i = (f0 + k) * L.tpf + t;
          if (f0 + k < nfr && i < limit)
            out[i] = (newest_self && f0 + k == nfr - 1) ? -1 - (op.q_begin + t) : page[k] * 2 * S + slot;
        }
      }
    }
    if (two) {
      for (int c = tid; c < h.stc; c += nthr) {
        const int pg = shift >= 0 ? c >> shift : c / S;
        if (frame_tokens + c < limit) out[frame_tokens + c] = st[L.off_special + pg] * 2 * S + (c - pg * S);
      }
    } else {
      for (int e = tid; e < h.nm; e += nthr) {
        const int t0 = st[L.off_mem_tcum + e], t1 = st[L.off_mem_tcum + e + 1];
        const int p0 = st[L.off_mem_pcum + e];
        for (int t = 0; t < t1 - t0; ++t) {
          const int pg = shift >= 0 ? t >> shift : t / S;
          if (frame_tokens + t0 + t < limit)
            out[frame_tokens + t0 + t] = st[L.off_mem_pages + p0 + pg] * 2 * S + (t - pg * S);
        }
      }
    }
    for (int t = tid; t < self_n; t += nthr)
      if (frame_tokens + h.stc + t < limit) out[frame_tokens + h.stc + t] = -1 - (op.q_begin + t);
    if (counted)
      for (int i = total + tid; i < limit; i += nthr) out[i] = 0;
  }
  if (total > limit) total = limit;  // what the attention may read
  int n_pages = nfr * L.ppf + (two ? h.nsp : h.nmp);
  if (page_ids && page_lens) {
    int32_t* ids = page_ids + op.page_out_begin;
    int32_t* lens = page_lens + op.page_out_begin;
    for (int i = tid; i < nfr * L.ppf; i += nthr) {
      const int f = i / L.ppf, j = i % L.ppf;
      const int32_t* pages = f < h.na ? anchor + f * L.ppf
                                      : win + ((h.wh + f - h.na) % L.ring_frames) * L.ppf;
      ids[i] = pages[j];
      lens[i] = j < L.ppf - 1 ? S : L.tpf - (L.ppf - 1) * S;
    }
    int32_t* ids2 = ids + nfr * L.ppf;
    int32_t* lens2 = lens + nfr * L.ppf;
    if (two) {
      const int tail = h.stc % S;
      for (int k = tid; k < h.nsp; k += nthr) {
        ids2[k] = st[L.off_special + k];
        lens2[k] = (k < h.nsp - 1 || tail == 0) ? S : tail;
      }
    } else {
      for (int e = tid; e < h.nm; e += nthr) {
        const int keep = st[L.off_mem_tcum + e + 1] - st[L.off_mem_tcum + e];
        const int p0 = st[L.off_mem_pcum + e], p1 = st[L.off_mem_pcum + e + 1];
        for (int j = 0; j < p1 - p0; ++j) {
          ids2[p0 + j] = st[L.off_mem_pages + p0 + j];
          lens2[p0 + j] = j < p1 - p0 - 1 ? S : keep - (p1 - p0 - 1) * S;
        }
      }
    }
  }
  if (tid == 0) {
    st[LBM_HDR_PLAN_KV_TOKENS] = total;
    st[LBM_HDR_PLAN_N_PAGES] = n_pages;
  }
}

#endif  // LBM_TABLES_LOGIC_H
