/*
 * lbm_paged_attn.h - C ABI of the MI355X (gfx950) streaming paged-KV attention library.
 *
 * The reference (Robbyant/lingbot-map) has no FFI on this path: its boundary is the Python
 * KV-cache manager lingbot_map/layers/flashinfer_cache.py:55 and the third-party FlashInfer
 * wrapper it drives.  Each entry point below names the reference interface it stands in for.
 * All pointers are raw device pointers unless marked "host"; all sizes are plain integers;
 * `stream` is a hipStream_t passed as void* (NULL = the null stream).  Every function returns
 * LBM_OK or an LBM_ERR_* code and never throws; lbm_last_error() gives the text of the last
 * failure on the calling thread.  No function synchronises the device.
 *
 * Data layout (flashinfer_cache.py:141-148): one pool per transformer block,
 *   pool[page][2][page_size][num_heads][head_dim]      dim 1: 0 = K, 1 = V
 * A "row" is one token's [num_heads][head_dim] vector; the K row index of (page, slot) is
 * page * 2 * page_size + slot and the matching V row is page_size rows later.
 */
#ifndef LBM_PAGED_ATTN_H
#define LBM_PAGED_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LBM_ABI_VERSION 9

#define LBM_OK 0
#define LBM_ERR_INVALID 1     /* bad argument (null pointer, negative size, bad enum)      */
#define LBM_ERR_UNSUPPORTED 2 /* shape the kernels do not cover (head_dim != 64, ...)       */
#define LBM_ERR_WORKSPACE 3   /* workspace too small; see lbm_attn_workspace_bytes          */
#define LBM_ERR_HIP 4         /* a HIP runtime call failed                                  */

#define LBM_DTYPE_BF16 0
#define LBM_DTYPE_F32 1

#define LBM_LAYOUT_TWO_STREAM 0  /* reference: patch pages + packed special stream         */
#define LBM_LAYOUT_FRAME_PAGES 1 /* whole frame in pages; eviction compacts index-only     */

/* epilogue of lbm_linear */
#define LBM_LINEAR_BIAS 0
#define LBM_LINEAR_BIAS_GELU 1
#define LBM_LINEAR_BIAS_RESIDUAL 2

/* pairing of the rotary embedding in lbm_qkv_prepare */
#define LBM_ROPE_INTERLEAVED 0
#define LBM_ROPE_HALF_SPLIT 1

#define LBM_MAX_STREAMS 16

/* MiB of device memory the library keeps as a static scratch array on every GPU it runs on
 * (lbm_attn_run_static). */
#define LBM_STATIC_SCRATCH_MIB 64

/* Table operations, executed in this fixed order when several bits are set. */
#define LBM_OP_RESET 1
#define LBM_OP_ROLLBACK 2
#define LBM_OP_APPEND 4
#define LBM_OP_EVICT 8
#define LBM_OP_PLAN 16
/* with LBM_OP_PLAN, frame_pages layout (ABI 9): the rows of the newest cached frame - the one
 * this step's LBM_OP_APPEND stored - name the caller's own K/V rows (q_begin + t, as self_tokens
 * rows do) instead of its pool rows, in the same place of the row table.  For a step whose append
 * is carried out by the attention call itself (lbm_attn_run_append), after the pool was read. */
#define LBM_OP_PLAN_NEWEST_SELF 32

/* Sticky bits of the device-side error word (header word LBM_HDR_ERROR). */
#define LBM_TERR_PATCH_POOL 1   /* flashinfer_cache.py:489-494 */
#define LBM_TERR_SPECIAL_POOL 2 /* flashinfer_cache.py:533-537 */
#define LBM_TERR_WINDOW_RING 4
#define LBM_TERR_MEMORY_FULL 8
#define LBM_TERR_ROLLBACK 16    /* flashinfer_cache.py:276-278,290-293 */
#define LBM_TERR_KV_COUNT 32    /* host and device disagree on the visible token count */

/* Header words at the start of each stream's table block. */
#define LBM_HDR_FRAME_COUNT 0
#define LBM_HDR_N_ANCHOR 1
#define LBM_HDR_WIN_HEAD 2
#define LBM_HDR_WIN_COUNT 3
#define LBM_HDR_N_FREE_PATCH 4
#define LBM_HDR_N_FREE_SPECIAL 5
#define LBM_HDR_N_SPECIAL_PAGES 6
#define LBM_HDR_SPECIAL_TOKENS 7
#define LBM_HDR_N_MEMORY 8
#define LBM_HDR_N_MEMORY_PAGES 9
#define LBM_HDR_ERROR 10
#define LBM_HDR_PLAN_KV_TOKENS 11
#define LBM_HDR_PLAN_N_PAGES 12
#define LBM_HDR_WORDS 16

/* Geometry of one stream's cache; the same for every stream of a batch.
 * Mirrors the constructor arguments of FlashInferKVCacheManager
 * (flashinfer_cache.py:75-138) with the page size made a free parameter. */
typedef struct lbm_cache_geom {
  int32_t layout;             /* LBM_LAYOUT_*                                             */
  int32_t tokens_per_frame;   /* specials first, then patches (flashinfer_cache.py:206)   */
  int32_t num_special_tokens;
  int32_t page_size;          /* tokens per page                                          */
  int32_t scale_frames;       /* anchor frames, never evicted                             */
  int32_t patch_pages;        /* recyclable page ids [0, patch_pages) of each stream      */
  int32_t special_pages;      /* append-only ids after them (two_stream), else 0          */
  int32_t memory_frames;      /* capacity of the compacted-frame list (frame_pages)       */
  int32_t pages_per_stream;   /* id distance between streams (>= patch + special pages)   */
} lbm_cache_geom;

/* One stream's share of a lbm_tables_step call. */
typedef struct lbm_step_op {
  int32_t ops;              /* LBM_OP_* bits; 0 = leave this stream alone                  */
  int32_t sliding_window;   /* EVICT: frames the window may keep                           */
  int32_t keep_tokens;      /* EVICT, frame_pages: leading tokens kept per evicted frame   */
  int32_t self_tokens;      /* PLAN: >0 appends the current frame's own K/V (read from the
                               caller's tensors, never stored) after the cached tokens     */
  int32_t q_begin;          /* first row of this stream in the batched q/k/v tensors       */
  int32_t kv_row_begin;     /* PLAN: first entry of this stream in kv_rows                 */
  int32_t expect_kv_tokens; /* PLAN: >= 0: the host's count of visible tokens (a mismatch sets
                               LBM_TERR_KV_COUNT); < 0: the host does not track the count and
                               -expect_kv_tokens is the capacity of this stream's part of
                               kv_rows (more visible tokens than that set the error bit and
                               the count is clamped)                                        */
  int32_t page_out_begin;   /* PLAN: first entry of this stream in kv_page_ids/_lens       */
} lbm_step_op;

/* One stream's share of an attention call (host memory). */
typedef struct lbm_attn_stream {
  int32_t q_begin;      /* first query row                                                 */
  int32_t q_rows;       /* number of query rows                                            */
  int32_t kv_row_begin; /* first entry in kv_rows                                          */
  int32_t kv_tokens;    /* number of entries                                               */
  int32_t live_at;      /* lbm_attn_run_live only: index of this stream's token count in
                           live_kv_tokens                                                  */
} lbm_attn_stream;

int lbm_abi_version(void);
const char* lbm_last_error(void);

/* int32 words of device memory one stream's tables need; 0 if the geometry is invalid. */
int64_t lbm_tables_words(const lbm_cache_geom* geom);

/* Index-only table maintenance, one launch for all streams of a batch.  Replaces the host
 * deque/list bookkeeping of FlashInferKVCacheManager: reset (flashinfer_cache.py:423-432),
 * rollback_last_frame (:268-301), the allocation half of append_frame (:474-553),
 * evict_frames / execute_deferred_eviction (:229-266), and build_visible_page_table +
 * compute_last_page_len + the three table uploads before plan() (:385-400, :438-470).
 *   tables        [n_streams * lbm_tables_words]           in/out
 *   ops           host, n_streams entries
 *   append_rows   APPEND: K row of every token of the new frame, -1 if the stream does not
 *                 append (indexed q_begin + t); may be NULL without APPEND.  When it is given,
 *                 every stream of the call - idle ones (ops == 0) included - gets its
 *                 tokens_per_frame entries written, so the streams' q_begin ranges must not
 *                 overlap (LBM_ERR_INVALID otherwise)
 *   kv_rows       PLAN: K row of every visible token; entries < 0 name row (-1 - e) of the
 *                 caller's own k/v tensors; may be NULL without PLAN
 *   kv_page_ids, kv_page_lens   PLAN: FlashInfer-style page table with a valid length per
 *                 page (optional, NULL to skip) */
int lbm_tables_step(int32_t* tables, const lbm_cache_geom* geom, int32_t n_streams,
                    const lbm_step_op* ops, int32_t* append_rows, int32_t* kv_rows,
                    int32_t* kv_page_ids, int32_t* kv_page_lens, void* stream);

/* Expand a FlashInfer-style page table (any page order, any valid length per page) into
 * the row table the attention kernel reads.  Stands in for the index half of
 * BatchPrefillWithPagedKVCacheWrapper.plan (flashinfer_cache.py:402-414).
 *   kv_indptr  host, n_streams + 1 offsets into kv_page_ids / kv_page_lens
 *   kv_tokens  host, n_streams visible token counts (sum of the stream's page lens)
 *   kv_row_begin host, n_streams offsets into kv_rows */
int lbm_rows_from_pages(const int32_t* kv_page_ids, const int32_t* kv_page_lens,
                        const int32_t* kv_indptr, const int32_t* kv_tokens,
                        const int32_t* kv_row_begin, int32_t n_streams, int32_t page_size,
                        int32_t* kv_rows, void* stream);

/* Keyframe-gated paged append: scatter one batch of new K/V rows into the pool.  Replaces
 * the slice assignments and dtype casts of append_frame (flashinfer_cache.py:215-218,
 * :504-505, :548-549).  Rows whose append_rows entry is negative are not written. */
int lbm_kv_append(const void* k, const void* v, int32_t src_dtype, void* pool,
                  int32_t pool_dtype, const int32_t* append_rows, int32_t n_tokens,
                  int32_t num_heads, int32_t head_dim, int32_t page_size, void* stream);

/* Residual update of a block fused with the LayerNorm that follows it, one pass over the rows:
 *     x_out = x + y * gamma        (x + ls(y): block.py:283, layer_scale.py:21-22)
 *     n_out = LayerNorm(x_out)     (norm2 in front of the MLP: block.py:194-195)
 *   x, y, x_out, n_out  [rows][cols], dtype (bf16 or fp32); x_out may alias x
 *   gamma               [cols] float32 LayerScale, NULL = plain x + y
 *   norm_w, norm_b      [cols] float32, both NULL = no LayerNorm (n_out unused)
 * cols: a multiple of 8, at most 8192.  Roundings follow torch's sequence for the dtype. */
int lbm_residual_norm(const void* x, const void* y, int32_t dtype, const float* gamma,
                      const float* norm_w, const float* norm_b, float norm_eps, void* x_out,
                      void* n_out, int32_t rows, int32_t cols, void* stream);

/* A bf16 linear layer of a transformer block with the elementwise work that follows it fused
 * into the store: out = epilogue(a @ w^T + bias).
 *   LBM_LINEAR_BIAS           the qkv projection (attention.py:413)
 *   LBM_LINEAR_BIAS_GELU      fc1 followed by the exact (erf) GELU (mlp.py:35-36)
 *   LBM_LINEAR_BIAS_RESIDUAL  proj or fc2 followed by LayerScale and the residual add:
 *                             residual + gamma * (a @ w^T + bias) (attention.py:554, mlp.py:38,
 *                             block.py:283, layer_scale.py:21-22)
 *   a         [M][K] bf16          w      [N][K] bf16 (nn.Linear's weight)
 *   bias      [N] float32 or NULL  gamma  [N] float32 or NULL (RESIDUAL only)
 *   residual  [M][N] bf16 (RESIDUAL only; may alias out)       out  [M][N] bf16
 * K: a multiple of 128, N: a multiple of 64, M * K and N * K below 2^31 elements (LBM_ERR_UNSUPPORTED
 * otherwise).  Roundings follow the sequence of separate bf16 torch ops (the
 * linear's output rounded to bf16, then each elementwise op). */
int lbm_linear(const void* a, const void* w, const float* bias, const float* gamma,
               const void* residual, void* out, int32_t M, int32_t N, int32_t K, int32_t epilogue,
               void* stream);

/* The qkv projection with the fused pre-attention producer as its epilogue: lbm_linear
 * (LBM_LINEAR_BIAS) followed by lbm_qkv_prepare on its bf16 output, as one launch - the
 * projection's output never goes to memory.  Replaces self.qkv(x) (attention.py:413) together
 * with everything lbm_qkv_prepare replaces.  Results are bit-identical to the two calls.
 *   a     [M][K] bf16, w [3 * num_heads * 64][K] bf16, bias [3 * num_heads * 64] float32 or NULL
 *   every other argument as in lbm_qkv_prepare, with bf16 activations and a bf16 cache;
 *   head_dim is 64, K a multiple of 128. */
int lbm_qkv_linear_prepare(const void* a, const void* w, const float* bias, int32_t M, int32_t K,
                           const float* q_norm_w, const float* q_norm_b, const float* k_norm_w,
                           const float* k_norm_b, float norm_eps, float q_scale, const float* rope_cs,
                           int32_t rope_layout, void* q_out, void* k_out, void* v_out, void* pool,
                           const int32_t* append_rows, int32_t num_heads, int32_t head_dim,
                           int32_t page_size, void* stream);

/* A LayerNorm folded into the launch that consumes its output.  lbm_linear with the residual
 * epilogue can leave behind, for every row of its output, one (mean, M2 = sum of squared
 * deviations from that mean) pair per column tile of the launch: out_stats [M][tiles][2] float32
 * with tiles = lbm_linear_stats_tiles(M, N).  A following launch that takes that output as its
 * activations standardises each row, (x - mean) * rstd with rstd = 1 / sqrt(M2 / K + eps) merged
 * from the pairs (Chan et al., equal-sized parts), without rewriting it: the product runs on the
 * raw rows and the store applies  rstd * (a @ w^T - mean * w_colsum) + bias.  With the
 * LayerNorm's weight g and bias c folded into the linear layer by the caller,
 *     w[n][k] = W[n][k] * g[k] (rounded to bf16),  w_colsum[n] = sum_k w[n][k] (of the rounded
 *     values),  bias[n] = B[n] + sum_k W[n][k] * c[k],
 * that is LayerNorm(a) @ W^T + B with no launch and no memory traffic for the LayerNorm:
 * norm2(x) in front of the MLP (block.py:194-195) and norm1(x) of the block that follows
 * (block.py:217).  Unlike the separate ops the normalised rows are never rounded to bf16 (the
 * weights' fold is instead): results agree with them to the last bf16 step or two.
 *   stats  [M][stats_tiles][2] float32, stats_tiles divides K        w_colsum  [N] float32 */
typedef struct lbm_row_norm {
  const float* stats;
  const float* w_colsum;
  int32_t stats_tiles;
  float eps;
} lbm_row_norm;

/* Column tiles per row of the statistics lbm_linear_norm writes for an M x N output. */
int32_t lbm_linear_stats_tiles(int32_t M, int32_t N);

/* lbm_linear with a_norm (NULL = none; not with the residual epilogue) applied to the
 * activations and / or out_stats (NULL = none; residual epilogue only) written.
 * workspace (NULL = none): device memory of at least lbm_linear_workspace_bytes(M, N, K, epilogue)
 * bytes that lets a launch with few tiles and a long K (fc2 of one frame: 128 tiles, K = 4096)
 * put several workgroups on each tile, each over a slice of K; the one that finishes a tile last
 * sums the slices in a fixed order, so results do not depend on timing.  The first 256-byte
 * aligned part of the workspace holds one counter per tile: the caller zero-fills the workspace
 * once, every launch leaves the counters at zero.  Launches that overlap in time on one GPU need
 * workspaces of their own, and with a workspace the residual may not alias out. */
int lbm_linear_norm(const void* a, const lbm_row_norm* a_norm, const void* w, const float* bias,
                    const float* gamma, const void* residual, void* out, float* out_stats,
                    int32_t M, int32_t N, int32_t K, int32_t epilogue, void* workspace,
                    size_t workspace_bytes, void* stream);

/* Bytes of workspace with which lbm_linear_norm would split K for this shape and epilogue; 0 when
 * it would not. */
size_t lbm_linear_workspace_bytes(int32_t M, int32_t N, int32_t K, int32_t epilogue);

/* No counterpart in the reference (ABI 8).  A model's weights do not stay in any cache from one
 * frame to the next, and a GEMM of one frame's rows that finds its weights in HBM takes 0.6 to 5 us
 * longer than one that finds them in a cache.  A caller that knows which memory the launch AFTER
 * the next one will read - the weights of the layer that follows - names it here: the next
 * lbm_linear, lbm_linear_norm, lbm_qkv_linear_prepare or lbm_qkv_linear_prepare_norm call of the
 * calling host thread then also reads one dword of every 128-byte line of [next_read, next_read +
 * bytes) while it computes (a ninth wavefront per workgroup that does nothing else), which leaves
 * the lines in the memory-side cache.  The hint is consumed by that one call (launches on
 * 256-row tiles ignore it); results are the same with and without it.  The memory must be
 * readable device memory for as long as that launch can run, replays of a captured graph
 * included.  bytes below 128 or next_read = NULL withdraws a pending hint. */
int lbm_linear_prefetch_hint(const void* next_read, size_t bytes);

/* lbm_qkv_linear_prepare with a_norm (NULL = none) applied to the activations: norm1 of the
 * block (folded as described at lbm_row_norm), its qkv projection and the pre-attention producer
 * as one launch. */
int lbm_qkv_linear_prepare_norm(const void* a, const lbm_row_norm* a_norm, const void* w,
                                const float* bias, int32_t M, int32_t K, const float* q_norm_w,
                                const float* q_norm_b, const float* k_norm_w, const float* k_norm_b,
                                float norm_eps, float q_scale, const float* rope_cs, int32_t rope_layout,
                                void* q_out, void* k_out, void* v_out, void* pool,
                                const int32_t* append_rows, int32_t num_heads, int32_t head_dim,
                                int32_t page_size, void* stream);

/* lbm_attn_run with the token counts read on the device: stream i attends to
 * live_kv_tokens[streams[i].live_at] entries of its row table instead of streams[i].kv_tokens,
 * which then only sizes the launch (number of KV splits, workspace) and should be the host's
 * best knowledge of the count.  Every argument of the call is then the same from frame to frame
 * while the cache grows, so the call can sit in a captured HIP graph; lbm_tables_step with a
 * negative expect_kv_tokens maintains the count (header word LBM_HDR_PLAN_KV_TOKENS).  No
 * counterpart in the reference, whose plan lives on the host (flashinfer_cache.py:385-414). */
int lbm_attn_run_live(const void* q, const void* pool, void* out, const void* self_k,
                      const void* self_v, const int32_t* kv_rows, const int32_t* live_kv_tokens,
                      const lbm_attn_stream* streams, int32_t n_streams, int32_t num_heads,
                      int32_t head_dim, int32_t page_size, int32_t dtype, float sm_scale,
                      void* workspace, size_t workspace_bytes, void* stream);

/* lbm_attn_run followed by the append of the current frames' K/V, as one call (ABI 9): new_k /
 * new_v are the self_k / self_v of lbm_attn_run (rows the table names by negative entries are read
 * from them) and, once the attention has read the pool, row t of them is also stored in pool row
 * append_rows[t] (a negative entry stores nothing), t < append_tokens - by the launch that merges
 * the split-KV partial results where there is one, so that the append costs no launch of its own,
 * by a launch of its own otherwise.  Replaces append_frame (flashinfer_cache.py:474-553, its
 * writes) and prefill_wrapper.run (:418-421) of one streamed frame as lbm_kv_append + lbm_attn_run
 * do, with the same results, for a step whose row table names the newest frame by the caller's
 * rows (LBM_OP_PLAN_NEWEST_SELF); pool and new_k / new_v share the dtype. */
int lbm_attn_run_append(const void* q, void* pool, void* out, const void* new_k, const void* new_v,
                        const int32_t* kv_rows, const int32_t* append_rows, int32_t append_tokens,
                        const lbm_attn_stream* streams, int32_t n_streams, int32_t num_heads,
                        int32_t head_dim, int32_t page_size, int32_t dtype, float sm_scale,
                        void* workspace, size_t workspace_bytes, void* stream);

/* Fused pre-attention producer: per-head LayerNorm of q and k, rotary embedding of q and k
 * (interleaved pairs), [token][head][dim] layout and the keyframe-gated paged append of k and
 * v, in one pass over the output of the qkv projection.  Replaces q_norm / k_norm,
 * apply_rotary_emb and the three permute + contiguous copies of
 * FlashInferAttention.prepare_qkv (attention.py:402-426, rope.py:438-461) together with the
 * writes of append_frame (flashinfer_cache.py:215-218, :504-505, :548-549).  Roundings follow
 * the reference's bf16 sequence when src_dtype is bf16 (LayerNorm output, cos, sin, each
 * product and each sum rounded to bf16) and plain fp32 arithmetic when it is fp32.
 *   qkv          [n_tokens][3][num_heads][head_dim], dtype src_dtype
 *   q_norm_w/_b, k_norm_w/_b   [head_dim] float32 LayerNorm affine; all four NULL = no qk-norm
 *   q_scale      > 0; every q row is multiplied by it in float32 BEFORE the rounding that ends the
 *                row's last operation (rotary sum, else LayerNorm, else the copy).  1 gives the
 *                reference's q.  sm_scale * log2(e) gives a q that lbm_attn_run takes with
 *                sm_scale = 0: the scale then costs q no second rounding to bf16 (the reference
 *                applies it inside its attention kernel, flashinfer_cache.py:418-421).  k and v
 *                are never scaled.
 *   rope_cs      NULL = no rotary embedding; otherwise float32 (cos, sin) pairs:
 *                LBM_ROPE_INTERLEAVED  [n_tokens][head_dim / 2][2], element pairs (2i, 2i+1),
 *                  i.e. torch.view_as_real of the complex freqs of apply_rotary_emb (rope.py:438-461)
 *                LBM_ROPE_HALF_SPLIT   [n_tokens][head_dim][2], one (cos, sin) per element; in each
 *                  half of head_dim element j pairs with j + head_dim/4: x*cos + rotate(x)*sin of
 *                  RotaryPositionEmbedding2D (rope.py:123-198)
 *   q_out        [n_tokens][num_heads][head_dim], dtype dst_dtype (the cache dtype)
 *   k_out, v_out same shape; may be NULL when only the pool copy is wanted (keyframes)
 *   pool, append_rows, page_size   as lbm_kv_append; append_rows NULL = no pool write
 * head_dim must be 64. */
int lbm_qkv_prepare(const void* qkv, int32_t src_dtype, const float* q_norm_w,
                    const float* q_norm_b, const float* k_norm_w, const float* k_norm_b,
                    float norm_eps, float q_scale, const float* rope_cs, int32_t rope_layout, void* q_out,
                    void* k_out, void* v_out, int32_t dst_dtype, void* pool,
                    const int32_t* append_rows, int32_t n_tokens, int32_t num_heads,
                    int32_t head_dim, int32_t page_size, void* stream);

/* Bytes of workspace lbm_attn_run needs for this batch: the split-KV partial results of the
 * bf16 kernel or, when every stream has at most 8 query rows, the per-chunk partials of the
 * fp32 few-query kernels, whichever is larger (the query does not take the dtype). */
size_t lbm_attn_workspace_bytes(const lbm_attn_stream* streams, int32_t n_streams,
                                int32_t num_heads, int32_t head_dim);

/* Ragged gather + softmax(q k^T * sm_scale) v over the rows kv_rows names, non-causal, MHA.
 * Replaces BatchPrefillWithPagedKVCacheWrapper.run (flashinfer_cache.py:418-421) and the
 * gather + F.scaled_dot_product_attention bridge (:324-347, :372-383).
 *   q, out         [rows][num_heads][head_dim], dtype = pool dtype
 *   self_k, self_v the caller's K/V of the current frames, same indexing as q (only read
 *                  for negative kv_rows entries; may be NULL otherwise)
 *   kv_rows        device array; stream i reads entries kv_row_begin .. kv_row_begin + kv_tokens - 1,
 *                  each a K row of the pool (page * 2 * page_size + slot) or -1 - r for row r of
 *                  self_k / self_v.  The entries are trusted: the library cannot see the sizes of
 *                  the pool or of this array, so a table that is too short or names rows outside
 *                  the pool makes the kernel read out of bounds.  Tables written by
 *                  lbm_tables_step / lbm_rows_from_pages satisfy this by construction.
 *   sm_scale       > 0: the softmax scale (the reference's 1 / sqrt(head_dim)).  The bf16 kernels
 *                  fold sm_scale * log2(e) into q, which rounds q to bf16 a second time.
 *                  0: q already carries sm_scale * log2(e) (a producer run with that q_scale)
 *                  and is used as it is.
 *   A stream with kv_tokens == 0 gets zeros; a stream with q_rows == 0 launches nothing. */
int lbm_attn_run(const void* q, const void* pool, void* out, const void* self_k,
                 const void* self_v, const int32_t* kv_rows, const lbm_attn_stream* streams,
                 int32_t n_streams, int32_t num_heads, int32_t head_dim, int32_t page_size,
                 int32_t dtype, float sm_scale, void* workspace, size_t workspace_bytes,
                 void* stream);

/* lbm_attn_run without a workspace argument and without any allocation: the split-KV partials
 * go into a static device array of LBM_STATIC_SCRATCH_MIB MiB that lives in the library (one
 * copy per GPU, held until the process ends).  No counterpart in the reference; it is for
 * callers that cannot allocate device memory - code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  Same arguments, results (bit for bit) and error
 * codes as lbm_attn_run; a batch whose partials do not fit returns LBM_ERR_WORKSPACE and
 * launches nothing.  The first call on a device looks the array's address up (no allocation,
 * but make that call outside a stream capture).  All calls on one GPU share the array: calls
 * that overlap in time on one GPU (two streams, two threads) race on it and must be
 * serialised by the caller; nothing in the array has to be cleared between calls. */
int lbm_attn_run_static(const void* q, const void* pool, void* out, const void* self_k,
                        const void* self_v, const int32_t* kv_rows, const lbm_attn_stream* streams,
                        int32_t n_streams, int32_t num_heads, int32_t head_dim, int32_t page_size,
                        int32_t dtype, float sm_scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LBM_PAGED_ATTN_H */
