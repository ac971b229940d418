// Fused pre-attention producer: one pass over the output of the qkv projection that applies
// the per-head LayerNorm of q and k, the rotary embedding of q and k, writes q (and, when
// asked, k and v) as [token][head][dim] and scatters k and v into the page pool.  It replaces
// q_norm / k_norm, apply_rotary_emb, three permute + contiguous copies
// (lingbot_map/layers/attention.py:402-426, lingbot_map/layers/rope.py:438-461) and the
// append pass (lingbot_map/layers/flashinfer_cache.py:215-218, 504-505, 548-549).
//
// HBM-bound: qkv is read once, q and the pool rows are written once.  Eight lanes own one
// (token, head) row of 64 elements, 8 elements (16 bytes of bf16) each; the LayerNorm
// statistics are reduced over those eight lanes with DPP shuffles; the interleaved rotary
// pairs (2i, 2i+1) of the global blocks stay inside a lane, the half-split pairs (j, j+16) of
// the frame blocks' 2-D embedding (lingbot_map/layers/rope.py:123-198) sit two lanes apart.
//
// Arithmetic follows the reference's order of roundings.  For bf16 activations torch computes
// the LayerNorm in fp32 and rounds its output to bf16; apply_rotary_emb then rounds cos and
// sin to bf16 and rounds after each multiply and after the add.  The kernel rounds at the
// same places, so its q and k match the reference's elementwise sequence (up to the order of
// the fp32 sums inside the LayerNorm).  For fp32 activations everything stays in fp32 with
// separately rounded multiplies and adds, as torch computes them.
#include <hip/hip_runtime.h>
#include "lbm_internal.h"

// Every product and sum below is rounded on its own, as the reference's separate torch ops are.
// The math header's __fmul_rn / __fadd_rn are plain operators compiled with contraction allowed
// (the compiler fuses them into FMAs), so the kernel uses its own, defined under this pragma.
#pragma clang fp contract(off)

#include "qkv_math.h"

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

namespace {

template <int DT>  // 0 = bf16, 1 = f32
__device__ __forceinline__ void load8(const void* base, long long elem, float (&x)[8]) {
  if (DT == 0) {
    const u32x4 a = *(const u32x4*)((const unsigned short*)base + elem);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = __builtin_bit_cast(float, a[i] << 16);
      x[2 * i + 1] = __builtin_bit_cast(float, a[i] & 0xffff0000u);
    }
  } else {
    const f32x4* p = (const f32x4*)((const float*)base + elem);
    const f32x4 a = p[0], b = p[1];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = a[i];
      x[4 + i] = b[i];
    }
  }
}
template <int DT>
__device__ __forceinline__ void store8(void* base, long long elem, const float (&x)[8]) {
  if (DT == 0) {
    bf16x8 a;
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = (__bf16)x[i];
    *(bf16x8*)((unsigned short*)base + elem) = a;
  } else {
    f32x4* p = (f32x4*)((float*)base + elem);
    p[0] = f32x4{x[0], x[1], x[2], x[3]};
    p[1] = f32x4{x[4], x[5], x[6], x[7]};
  }
}

struct PrepareArgs {
  const void* qkv;
  const float* q_norm_w;   // all four NULL: no qk-norm
  const float* q_norm_b;
  const float* k_norm_w;
  const float* k_norm_b;
  const float* rope_cs;
  int rope_layout;
  void* q_out;
  void* k_out;             // k_out / v_out may be NULL (keyframes: only the pool copy is wanted)
  void* v_out;
  void* pool;
  const int32_t* append_rows;
  float eps;
  float q_scale;           // q is multiplied by this in fp32 before its last rounding (1 = plain q)
  int n_tokens, num_heads, page_size;
};

// head_dim 64.  SRC = activation dtype, DST = cache dtype.
//
// The kernel is a chain of short memory latencies, not of bandwidth: 12 MB per frame move in
// about a microsecond, a dependent load costs as much again, and launching a wave costs more
// than the 16 bytes per lane it would move.  So a group of 8 lanes carries three rows, and every
// load it needs - 3 x 16 bytes of qkv, the LayerNorm parameters, the rotary table entries, the
// append row - sits in one straight line of code ahead of the arithmetic.
// ROPE: 0 none, 1 interleaved pairs, 2 half-split pairs; NORM: qk-LayerNorm; APPEND: pool writes.
// Compile-time so that the loads below sit in one straight line of code: the compiler waits
// for every outstanding load at the end of a conditional block.
template <int SRC, int DST, int ROPE, bool NORM, bool APPEND>
__global__ __launch_bounds__(256) void lbm_qkv_prepare_d64_kernel(PrepareArgs a) {
  const int H = a.num_heads;
  // 16 or 32 (token, head) groups per workgroup, 8 lanes each; a group carries the q, k and v
  // row of its head, so the rotary entries and the append row are loaded once for the three and
  // a third as many waves are launched as with a group per row.  The host checks that the group
  // count fits 32 bits.
  const unsigned g = blockIdx.x * (blockDim.x >> 3) + (threadIdx.x >> 3);
  const unsigned groups = (unsigned)a.n_tokens * (unsigned)H;
  // whole 8-lane groups leave together, so the shuffles below see all their lanes
  if (g >= groups) return;
  const int c = (int)(threadIdx.x & 7);
  const int t = (int)(g / (unsigned)H);
  const int h = (int)(g - (unsigned)t * (unsigned)H);
  constexpr bool has_norm = NORM, has_rope = ROPE != 0, interleaved = ROPE == 1;

  // ---- every load of this group, back to back
  const long long in0 = ((long long)t * 3 * H + h) * 64 + c * 8;   // q row; k and v follow H rows apart
  u32x4 raw16[3] = {};
  f32x4 raw32[3][2] = {};
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    if (SRC == 0) {
      raw16[w] = *(const u32x4*)((const unsigned short*)a.qkv + in0 + (long long)w * H * 64);
    } else {
      const f32x4* xp = (const f32x4*)((const float*)a.qkv + in0 + (long long)w * H * 64);
      raw32[w][0] = xp[0];
      raw32[w][1] = xp[1];
    }
  }
  f32x4 w4[2][2] = {}, b4[2][2] = {};
  if (has_norm) {
    const f32x4* qw = (const f32x4*)(a.q_norm_w + c * 8);
    const f32x4* qb = (const f32x4*)(a.q_norm_b + c * 8);
    const f32x4* kw = (const f32x4*)(a.k_norm_w + c * 8);
    const f32x4* kb = (const f32x4*)(a.k_norm_b + c * 8);
    w4[0][0] = qw[0]; w4[0][1] = qw[1]; b4[0][0] = qb[0]; b4[0][1] = qb[1];
    w4[1][0] = kw[0]; w4[1][1] = kw[1]; b4[1][0] = kb[0]; b4[1][1] = kb[1];
  }
  f32x4 cs4[4] = {};
  if (interleaved) {   // (cos, sin) of this lane's four pairs
    const f32x4* cs = (const f32x4*)(a.rope_cs + ((long long)t * 32 + c * 4) * 2);
    cs4[0] = cs[0]; cs4[1] = cs[1];
  } else if (has_rope) {   // (cos, sin) of this lane's eight elements
    const f32x4* cs = (const f32x4*)(a.rope_cs + ((long long)t * 64 + c * 8) * 2);
    cs4[0] = cs[0]; cs4[1] = cs[1]; cs4[2] = cs[2]; cs4[3] = cs[3];
  }
  int pool_row = -1;
  if (APPEND) pool_row = a.append_rows[t];

  float x[3][8];
#pragma unroll
  for (int w = 0; w < 3; ++w) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (SRC == 0) {
        const unsigned pair = raw16[w][i >> 1];
        x[w][i] = __builtin_bit_cast(float, (i & 1) ? (pair & 0xffff0000u) : (pair << 16));
      } else {
        x[w][i] = raw32[w][i >> 2][i & 3];
      }
    }
  }

  // q and k rows: LayerNorm and rotary embedding
#pragma unroll
  for (int w = 0; w < 2; ++w) lbm_qkv::norm_rope<SRC, ROPE, NORM>(x[w], w4[w], b4[w], cs4, c, a.eps, w == 0 ? a.q_scale : 1.0f);

  const long long nhd = ((long long)t * H + h) * 64 + c * 8;
  store8<DST>(a.q_out, nhd, x[0]);
  if (a.k_out) store8<DST>(a.k_out, nhd, x[1]);
  if (a.v_out) store8<DST>(a.v_out, nhd, x[2]);
  if (pool_row >= 0) {
    const long long row_elems = (long long)H * 64;
    const long long d = (long long)pool_row * row_elems + h * 64 + c * 8;
    store8<DST>(a.pool, d, x[1]);
    store8<DST>(a.pool, d + (long long)a.page_size * row_elems, x[2]);
  }
}

}  // namespace

int lbm_launch_qkv_prepare(const void* qkv, int src_dtype, const float* q_norm_w, const float* q_norm_b,
                           const float* k_norm_w, const float* k_norm_b, float norm_eps, float q_scale,
                           const float* rope_cs, int rope_layout, void* q_out, void* k_out, void* v_out,
                           int dst_dtype, void* pool, const int32_t* append_rows, int n_tokens,
                           int num_heads, int page_size, hipStream_t stream) {
  PrepareArgs a;
  a.qkv = qkv;
  a.q_norm_w = q_norm_w; a.q_norm_b = q_norm_b;
  a.k_norm_w = k_norm_w; a.k_norm_b = k_norm_b;
  a.rope_cs = rope_cs;
  a.rope_layout = rope_layout;
  a.q_out = q_out; a.k_out = k_out; a.v_out = v_out;
  a.pool = pool;
  a.append_rows = append_rows;
  a.eps = norm_eps;
  a.q_scale = q_scale;
  a.n_tokens = n_tokens; a.num_heads = num_heads; a.page_size = page_size;
  const long long rows = (long long)n_tokens * 3 * num_heads;
  if (rows == 0) return LBM_OK;
  if (rows > 0x7fffffffLL) return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_qkv_prepare: %lld rows exceed 2^31", rows);
  // one frame (16,064 groups) spreads better over 256 CUs in workgroups of 16 groups; several
  // streams' worth of rows run a little faster in workgroups of 32
  const int bs = rows / 3 <= 32768 ? 128 : 256;
  const dim3 grid((unsigned)((rows / 3 + bs / 8 - 1) / (bs / 8))), block(bs);
  const int rope = !rope_cs ? 0 : (rope_layout == LBM_ROPE_INTERLEAVED ? 1 : 2);
  const bool norm = q_norm_w != nullptr, append = append_rows != nullptr;
#define LBM_PREPARE_LAUNCH(S, D, R, N, A) \
  hipLaunchKernelGGL((lbm_qkv_prepare_d64_kernel<S, D, R, N, A>), grid, block, 0, stream, a)
#define LBM_PREPARE_NA(S, D, R)                            \
  {                                                        \
    if (norm && append) LBM_PREPARE_LAUNCH(S, D, R, true, true);         \
    else if (norm) LBM_PREPARE_LAUNCH(S, D, R, true, false);             \
    else if (append) LBM_PREPARE_LAUNCH(S, D, R, false, true);           \
    else LBM_PREPARE_LAUNCH(S, D, R, false, false);                      \
  }
#define LBM_PREPARE_CASE(S, D)                \
  {                                           \
    if (rope == 0) LBM_PREPARE_NA(S, D, 0)    \
    else if (rope == 1) LBM_PREPARE_NA(S, D, 1) \
    else LBM_PREPARE_NA(S, D, 2)              \
  }
  if (src_dtype == LBM_DTYPE_BF16 && dst_dtype == LBM_DTYPE_BF16) LBM_PREPARE_CASE(0, 0)
  else if (src_dtype == LBM_DTYPE_F32 && dst_dtype == LBM_DTYPE_F32) LBM_PREPARE_CASE(1, 1)
  else if (src_dtype == LBM_DTYPE_F32 && dst_dtype == LBM_DTYPE_BF16) LBM_PREPARE_CASE(1, 0)
  else LBM_PREPARE_CASE(0, 1)
#undef LBM_PREPARE_CASE
#undef LBM_PREPARE_NA
#undef LBM_PREPARE_LAUNCH
  return lbm_check_launch("lbm_qkv_prepare_d64_kernel");
}
