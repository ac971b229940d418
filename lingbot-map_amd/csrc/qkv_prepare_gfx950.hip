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

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

namespace {

// round-to-nearest-even to bf16 and back (torch's .to(bfloat16)); the hardware conversion
// v_cvt_pk_bf16_f32 rounds the same way
__device__ __forceinline__ float round_bf16(float f) { return (float)(__bf16)f; }

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
  const float* norm_w[2];  // q, k
  const float* norm_b[2];
  const float* rope_cs;
  int rope_layout;
  void* out[3];            // q_out, k_out, v_out
  void* pool;
  const int32_t* append_rows;
  float eps;
  int n_tokens, num_heads, page_size;
};

// head_dim 64.  SRC = activation dtype, DST = cache dtype.
template <int SRC, int DST>
__global__ __launch_bounds__(256) void lbm_qkv_prepare_d64_kernel(PrepareArgs a) {
  const int H = a.num_heads;
  // 32 rows of (token, q|k|v, head) per workgroup; the host checks that the row count fits 32 bits
  const unsigned rw = blockIdx.x * 32u + (threadIdx.x >> 3);
  const unsigned rows = (unsigned)a.n_tokens * 3u * (unsigned)H;
  // whole 8-lane groups leave together, so the shuffles below see all their lanes
  if (rw >= rows) return;
  const int c = (int)(threadIdx.x & 7);
  const unsigned th = rw / (unsigned)H;       // token * 3 + which
  const int h = (int)(rw - th * (unsigned)H);
  const int t = (int)(th / 3u);
  const int which = (int)(th - (unsigned)t * 3u);

  float x[8];
  load8<SRC>(a.qkv, (long long)rw * 64 + c * 8, x);

  if (which < 2) {
    if (a.norm_w[which]) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) s += x[i];
      s += __shfl_xor(s, 1);
      s += __shfl_xor(s, 2);
      s += __shfl_xor(s, 4);
      const float mean = s * (1.0f / 64.0f);
      float v = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) v += (x[i] - mean) * (x[i] - mean);
      v += __shfl_xor(v, 1);
      v += __shfl_xor(v, 2);
      v += __shfl_xor(v, 4);
      const float rstd = __builtin_amdgcn_rsqf(v * (1.0f / 64.0f) + a.eps);  // torch's LayerNorm uses rsqrt too
      const float* w = a.norm_w[which] + c * 8;
      const float* b = a.norm_b[which] + c * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float y = __fadd_rn(__fmul_rn(__fmul_rn(x[i] - mean, rstd), w[i]), b[i]);
        x[i] = SRC == 0 ? round_bf16(y) : y;
      }
    }
    if (a.rope_cs && a.rope_layout == LBM_ROPE_INTERLEAVED) {
      const f32x4* cs = (const f32x4*)(a.rope_cs + ((long long)t * 32 + c * 4) * 2);
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const f32x4 q4 = cs[p];  // (cos, sin) of two pairs
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int i = 4 * p + 2 * j;
          float co = q4[2 * j], si = q4[2 * j + 1];
          const float x1 = x[i], x2 = x[i + 1];
          if (SRC == 0) {
            co = round_bf16(co);
            si = round_bf16(si);
            x[i] = round_bf16(__fsub_rn(round_bf16(__fmul_rn(x1, co)), round_bf16(__fmul_rn(x2, si))));
            x[i + 1] = round_bf16(__fadd_rn(round_bf16(__fmul_rn(x1, si)), round_bf16(__fmul_rn(x2, co))));
          } else {
            x[i] = __fsub_rn(__fmul_rn(x1, co), __fmul_rn(x2, si));
            x[i + 1] = __fadd_rn(__fmul_rn(x1, si), __fmul_rn(x2, co));
          }
        }
      }
    } else if (a.rope_cs) {
      // half-split pairs: in each 32-element half, element j < 16 rotates with element j + 16
      // (x * cos + rotate(x) * sin with rotate = (-second, first), rope.py:123-152); the partner
      // sits two lanes away in the 8-lane group
      const f32x4* cs = (const f32x4*)(a.rope_cs + ((long long)t * 64 + c * 8) * 2);
      const bool first = (c & 2) == 0;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const f32x4 q4 = cs[p];  // (cos, sin) of two elements
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int i = 2 * p + j;
          float co = q4[2 * j], si = q4[2 * j + 1];
          const float own = x[i];
          const float other = __shfl_xor(own, 2);
          if (SRC == 0) {
            co = round_bf16(co);
            si = round_bf16(si);
            const float a0 = round_bf16(__fmul_rn(own, co)), b0 = round_bf16(__fmul_rn(other, si));
            x[i] = round_bf16(first ? __fsub_rn(a0, b0) : __fadd_rn(a0, b0));
          } else {
            const float a0 = __fmul_rn(own, co), b0 = __fmul_rn(other, si);
            x[i] = first ? __fsub_rn(a0, b0) : __fadd_rn(a0, b0);
          }
        }
      }
    }
  }

  const long long nhd = ((long long)t * H + h) * 64 + c * 8;
  if (a.out[which]) store8<DST>(a.out[which], nhd, x);
  if (which > 0 && a.append_rows) {
    const int row = a.append_rows[t];
    if (row >= 0) {
      const long long row_elems = (long long)H * 64;
      const long long d = (long long)row * row_elems + (which == 2 ? (long long)a.page_size * row_elems : 0) +
                          h * 64 + c * 8;
      store8<DST>(a.pool, d, x);
    }
  }
}

}  // namespace

int lbm_launch_qkv_prepare(const void* qkv, int src_dtype, const float* q_norm_w, const float* q_norm_b,
                           const float* k_norm_w, const float* k_norm_b, float norm_eps,
                           const float* rope_cs, int rope_layout, void* q_out, void* k_out, void* v_out,
                           int dst_dtype, void* pool, const int32_t* append_rows, int n_tokens,
                           int num_heads, int page_size, hipStream_t stream) {
  PrepareArgs a;
  a.qkv = qkv;
  a.norm_w[0] = q_norm_w; a.norm_b[0] = q_norm_b;
  a.norm_w[1] = k_norm_w; a.norm_b[1] = k_norm_b;
  a.rope_cs = rope_cs;
  a.rope_layout = rope_layout;
  a.out[0] = q_out; a.out[1] = k_out; a.out[2] = v_out;
  a.pool = pool;
  a.append_rows = append_rows;
  a.eps = norm_eps;
  a.n_tokens = n_tokens; a.num_heads = num_heads; a.page_size = page_size;
  const long long rows = (long long)n_tokens * 3 * num_heads;
  if (rows == 0) return LBM_OK;
  if (rows > 0x7fffffffLL) return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_qkv_prepare: %lld rows exceed 2^31", rows);
  const dim3 grid((unsigned)((rows + 31) / 32)), block(256);
#define LBM_PREPARE_CASE(S, D) hipLaunchKernelGGL((lbm_qkv_prepare_d64_kernel<S, D>), grid, block, 0, stream, a)
  if (src_dtype == LBM_DTYPE_BF16 && dst_dtype == LBM_DTYPE_BF16) LBM_PREPARE_CASE(0, 0);
  else if (src_dtype == LBM_DTYPE_F32 && dst_dtype == LBM_DTYPE_F32) LBM_PREPARE_CASE(1, 1);
  else if (src_dtype == LBM_DTYPE_F32 && dst_dtype == LBM_DTYPE_BF16) LBM_PREPARE_CASE(1, 0);
  else LBM_PREPARE_CASE(0, 1);
#undef LBM_PREPARE_CASE
  return lbm_check_launch("lbm_qkv_prepare_d64_kernel");
}
