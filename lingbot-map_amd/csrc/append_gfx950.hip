// Paged K/V append: scatters the rows of one batch of new frames into the page pool.
// HBM-bound copy (read k,v once, write them once); each thread moves one 16-byte piece of
// a K row and the matching piece of the V row, so a wavefront writes 1 KiB contiguous per
// row half and every store is a full 128-bit transaction.  A negative destination row
// gates the write off (non-keyframes, streams that do not append in this step).
#include <hip/hip_runtime.h>
#include "lbm_internal.h"

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// round-to-nearest-even, NaN kept quiet: the rounding torch's .to(bfloat16) applies
// (the reference casts with .to(self.dtype), flashinfer_cache.py:215-218)
__device__ __forceinline__ unsigned int lbm_f32_to_bf16_bits(float f) {
  unsigned int u = __builtin_bit_cast(unsigned int, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ unsigned int lbm_pack_bf16(float lo, float hi) {
  return lbm_f32_to_bf16_bits(lo) | (lbm_f32_to_bf16_bits(hi) << 16);
}

// SRC/DST: 0 = bf16, 1 = f32.  `row_elems` = num_heads * head_dim, a multiple of 8.
template <int SRC, int DST>
__global__ __launch_bounds__(256) void lbm_kv_append_kernel(
    const void* __restrict__ k, const void* __restrict__ v, void* __restrict__ pool,
    const int32_t* __restrict__ append_rows, int n_tokens, int row_elems, int page_size) {
  const int pieces = row_elems / 8;  // 8 elements per thread
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)n_tokens * pieces) return;
  const int t = (int)(idx / pieces), piece = (int)(idx % pieces);
  const int row = append_rows[t];
  if (row < 0) return;
  const long long src = (long long)t * row_elems + piece * 8;
  const long long dk = (long long)row * row_elems + piece * 8;
  const long long dv = dk + (long long)page_size * row_elems;
  if (SRC == 0 && DST == 0) {
    const u32x4 a = *(const u32x4*)((const unsigned short*)k + src);
    const u32x4 b = *(const u32x4*)((const unsigned short*)v + src);
    *(u32x4*)((unsigned short*)pool + dk) = a;
    *(u32x4*)((unsigned short*)pool + dv) = b;
  } else if (SRC == 1 && DST == 1) {
    const f32x4* ks = (const f32x4*)((const float*)k + src);
    const f32x4* vs = (const f32x4*)((const float*)v + src);
    f32x4* kd = (f32x4*)((float*)pool + dk);
    f32x4* vd = (f32x4*)((float*)pool + dv);
    const f32x4 a0 = ks[0], a1 = ks[1], b0 = vs[0], b1 = vs[1];
    kd[0] = a0; kd[1] = a1; vd[0] = b0; vd[1] = b1;
  } else if (SRC == 1 && DST == 0) {
    const f32x4* ks = (const f32x4*)((const float*)k + src);
    const f32x4* vs = (const f32x4*)((const float*)v + src);
    const f32x4 a0 = ks[0], a1 = ks[1], b0 = vs[0], b1 = vs[1];
    u32x4 a, b;
    a[0] = lbm_pack_bf16(a0[0], a0[1]); a[1] = lbm_pack_bf16(a0[2], a0[3]);
    a[2] = lbm_pack_bf16(a1[0], a1[1]); a[3] = lbm_pack_bf16(a1[2], a1[3]);
    b[0] = lbm_pack_bf16(b0[0], b0[1]); b[1] = lbm_pack_bf16(b0[2], b0[3]);
    b[2] = lbm_pack_bf16(b1[0], b1[1]); b[3] = lbm_pack_bf16(b1[2], b1[3]);
    *(u32x4*)((unsigned short*)pool + dk) = a;
    *(u32x4*)((unsigned short*)pool + dv) = b;
  } else {  // bf16 -> f32
    const u32x4 a = *(const u32x4*)((const unsigned short*)k + src);
    const u32x4 b = *(const u32x4*)((const unsigned short*)v + src);
    f32x4* kd = (f32x4*)((float*)pool + dk);
    f32x4* vd = (f32x4*)((float*)pool + dv);
    f32x4 a0, a1, b0, b1;
    for (int i = 0; i < 2; ++i) {
      a0[2 * i] = __builtin_bit_cast(float, a[i] << 16);     a0[2 * i + 1] = __builtin_bit_cast(float, a[i] & 0xffff0000u);
      a1[2 * i] = __builtin_bit_cast(float, a[2 + i] << 16); a1[2 * i + 1] = __builtin_bit_cast(float, a[2 + i] & 0xffff0000u);
      b0[2 * i] = __builtin_bit_cast(float, b[i] << 16);     b0[2 * i + 1] = __builtin_bit_cast(float, b[i] & 0xffff0000u);
      b1[2 * i] = __builtin_bit_cast(float, b[2 + i] << 16); b1[2 * i + 1] = __builtin_bit_cast(float, b[2 + i] & 0xffff0000u);
    }
    kd[0] = a0; kd[1] = a1; vd[0] = b0; vd[1] = b1;
  }
}

int lbm_launch_append(const void* k, const void* v, int src_dtype, void* pool, int pool_dtype,
                      const int32_t* append_rows, int n_tokens, int num_heads, int head_dim,
                      int page_size, hipStream_t stream) {
  const int row_elems = num_heads * head_dim;
  const long long work = (long long)n_tokens * (row_elems / 8);
  if (work == 0) return LBM_OK;
  const dim3 grid((unsigned)((work + 255) / 256)), block(256);
#define LBM_APPEND_CASE(S, D)                                                                  \
  hipLaunchKernelGGL((lbm_kv_append_kernel<S, D>), grid, block, 0, stream, k, v, pool,         \
                     append_rows, n_tokens, row_elems, page_size)
  if (src_dtype == LBM_DTYPE_BF16 && pool_dtype == LBM_DTYPE_BF16) LBM_APPEND_CASE(0, 0);
  else if (src_dtype == LBM_DTYPE_F32 && pool_dtype == LBM_DTYPE_F32) LBM_APPEND_CASE(1, 1);
  else if (src_dtype == LBM_DTYPE_F32 && pool_dtype == LBM_DTYPE_BF16) LBM_APPEND_CASE(1, 0);
  else LBM_APPEND_CASE(0, 1);
#undef LBM_APPEND_CASE
  return lbm_check_launch("lbm_kv_append_kernel");
}
