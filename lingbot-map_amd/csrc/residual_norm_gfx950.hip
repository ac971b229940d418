// Residual update of a transformer block fused with the LayerNorm that follows it:
//     x_out = x + y * gamma            (x + ls(y), lingbot_map/layers/block.py:283,
//                                       lingbot_map/layers/layer_scale.py:21-22)
//     n_out = LayerNorm(x_out)         (the block's norm2 in front of the MLP, block.py:194-195)
// One pass over the rows instead of three elementwise / normalisation kernels.  HBM-bound:
// reads x and y once, writes x_out and n_out once.
//
// Rows of up to 2048 elements take one wavefront each (butterfly sums, no LDS); longer rows one
// 128-thread workgroup: a thread owns 8 consecutive elements per 1024-element chunk of the row
// (up to 8 chunks).  Either way the row stays in registers between the statistics and the output.
// Rounding follows torch for bf16 activations: y * gamma rounded to bf16, the sum rounded to
// bf16, the LayerNorm computed in fp32 on those bf16 values (two-pass mean / variance) and
// rounded once.  For fp32 activations every step is a separately rounded fp32 operation.
#include <hip/hip_runtime.h>
#include "lbm_internal.h"
#include "qkv_math.h"

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

namespace {

constexpr int kThreads = 128;
constexpr int kMaxChunks = 8;  // rows of up to 8192 elements

__device__ __forceinline__ float round_bf16(float f) { return (float)(__bf16)f; }

template <int DT>
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

// sum over the 128 threads of the workgroup (two wavefronts)
__device__ __forceinline__ float block_sum(float v, float* lds2) {
  v = lbm_qkv::sum_of_wave(v);
  const int wave = threadIdx.x >> 6;
  __syncthreads();  // lds2 may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) lds2[wave] = v;
  __syncthreads();
  return lds2[0] + lds2[1];
}

struct ResidualNormArgs {
  const void* x;
  const void* y;
  const float* gamma;   // LayerScale, or NULL for x + y
  const float* norm_w;  // NULL: no LayerNorm output
  const float* norm_b;
  void* x_out;
  void* n_out;
  float eps;
  int rows, cols;
};

// NCH = 1024-element chunks a row may have (1, 2, 4 or 8): sizes the register array
template <int DT, int NCH>
__global__ __launch_bounds__(kThreads) void lbm_residual_norm_kernel(ResidualNormArgs a) {
  __shared__ float lds2[2];
  const int row = blockIdx.x;
  const long long base = (long long)row * a.cols;
  const int n_chunks = (a.cols + 1023) >> 10;
  float v[NCH][8];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int col = c * 1024 + threadIdx.x * 8;
    if (c < n_chunks && col < a.cols) {
      float x[8], y[8];
      load8<DT>(a.x, base + col, x);
      load8<DT>(a.y, base + col, y);
      f32x4 ga[2] = {{1.f, 1.f, 1.f, 1.f}, {1.f, 1.f, 1.f, 1.f}};
      if (a.gamma) {   // a launch parameter: uniform
        ga[0] = *(const f32x4*)(a.gamma + col);
        ga[1] = *(const f32x4*)(a.gamma + col + 4);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = y[i];
        if (a.gamma) t = DT == 0 ? round_bf16(__fmul_rn(t, ga[i >> 2][i & 3])) : __fmul_rn(t, ga[i >> 2][i & 3]);
        const float s = __fadd_rn(x[i], t);
        v[c][i] = DT == 0 ? round_bf16(s) : s;
        sum += v[c][i];
      }
      store8<DT>(a.x_out, base + col, v[c]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[c][i] = 0.f;
    }
  }
  if (!a.norm_w) return;  // uniform: a launch parameter
  const float mean = block_sum(sum, lds2) / (float)a.cols;
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int col = c * 1024 + threadIdx.x * 8;
    if (c < n_chunks && col < a.cols) {
#pragma unroll
      for (int i = 0; i < 8; ++i) sq += (v[c][i] - mean) * (v[c][i] - mean);
    }
  }
  const float rstd = __builtin_amdgcn_rsqf(block_sum(sq, lds2) / (float)a.cols + a.eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int col = c * 1024 + threadIdx.x * 8;
    if (c < n_chunks && col < a.cols) {
      const f32x4 w0 = *(const f32x4*)(a.norm_w + col), w1 = *(const f32x4*)(a.norm_w + col + 4);
      const f32x4 b0 = *(const f32x4*)(a.norm_b + col), b1 = *(const f32x4*)(a.norm_b + col + 4);
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        o[i] = __fadd_rn(__fmul_rn(__fmul_rn(v[c][i] - mean, rstd), i < 4 ? w0[i & 3] : w1[i & 3]), i < 4 ? b0[i & 3] : b1[i & 3]);
      store8<DT>(a.n_out, base + col, o);
    }
  }
}

// Rows of up to 2048 elements: one wavefront per row, four rows per workgroup.  A lane owns 8
// consecutive elements per 512-element chunk (NV chunks), the two statistics are butterfly
// sums over the 64 lanes - no LDS, no barrier.
template <int DT, int NV>
__global__ __launch_bounds__(256) void lbm_residual_norm_wave_kernel(ResidualNormArgs a) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) return;   // whole wavefronts leave; nothing below synchronises across them
  const long long base = (long long)row * a.cols;
  const bool has_gamma = a.gamma != nullptr, has_norm = a.norm_w != nullptr;   // launch parameters: uniform
  // Every load of the row is issued before the first use of any of them - x, y, LayerScale and
  // the LayerNorm parameters: the kernel is a chain of memory latencies, not of bandwidth.
  float x[NV][8], y[NV][8];
  f32x4 ga[NV][2], nw[NV][2], nb[NV][2];
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int col = (c * 64 + lane) * 8;
    ga[c][0] = ga[c][1] = f32x4{1.f, 1.f, 1.f, 1.f};
    nw[c][0] = nw[c][1] = nb[c][0] = nb[c][1] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (col < a.cols) {
      load8<DT>(a.x, base + col, x[c]);
      load8<DT>(a.y, base + col, y[c]);
      if (has_gamma) {
        ga[c][0] = *(const f32x4*)(a.gamma + col);
        ga[c][1] = *(const f32x4*)(a.gamma + col + 4);
      }
      if (has_norm) {
        nw[c][0] = *(const f32x4*)(a.norm_w + col);
        nw[c][1] = *(const f32x4*)(a.norm_w + col + 4);
        nb[c][0] = *(const f32x4*)(a.norm_b + col);
        nb[c][1] = *(const f32x4*)(a.norm_b + col + 4);
      }
    }
  }
  float v[NV][8];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int col = (c * 64 + lane) * 8;
    if (col < a.cols) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = y[c][i];
        // without LayerScale the factor is 1 and the product is y itself
        if (has_gamma) t = DT == 0 ? round_bf16(__fmul_rn(t, ga[c][i >> 2][i & 3])) : __fmul_rn(t, ga[c][i >> 2][i & 3]);
        const float s = __fadd_rn(x[c][i], t);
        v[c][i] = DT == 0 ? round_bf16(s) : s;
        sum += v[c][i];
      }
      store8<DT>(a.x_out, base + col, v[c]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[c][i] = 0.f;
    }
  }
  if (!has_norm) return;
  sum = lbm_qkv::sum_of_wave(sum);
  const float mean = sum / (float)a.cols;
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < NV; ++c)
    if ((c * 64 + lane) * 8 < a.cols) {
#pragma unroll
      for (int i = 0; i < 8; ++i) sq += (v[c][i] - mean) * (v[c][i] - mean);
    }
  sq = lbm_qkv::sum_of_wave(sq);
  const float rstd = __builtin_amdgcn_rsqf(sq / (float)a.cols + a.eps);
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int col = (c * 64 + lane) * 8;
    if (col < a.cols) {
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        o[i] = __fadd_rn(__fmul_rn(__fmul_rn(v[c][i] - mean, rstd), nw[c][i >> 2][i & 3]), nb[c][i >> 2][i & 3]);
      store8<DT>(a.n_out, base + col, o);
    }
  }
}

}  // namespace

int lbm_launch_residual_norm(const void* x, const void* y, int dtype, const float* gamma, const float* norm_w,
                             const float* norm_b, float eps, void* x_out, void* n_out, int rows, int cols,
                             hipStream_t stream) {
  if (rows == 0) return LBM_OK;
  if (cols % 8 != 0 || cols > 1024 * kMaxChunks)
    return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_residual_norm: cols must be a multiple of 8 and at most %d (got %d)",
                    1024 * kMaxChunks, cols);
  ResidualNormArgs a{x, y, gamma, norm_w, norm_b, x_out, n_out, eps, rows, cols};
  if (cols <= 2048) {
    const int nv = (cols + 511) >> 9;
    const dim3 grid((rows + 3) / 4);
#define LBM_RN_WAVE(DT, NV) hipLaunchKernelGGL((lbm_residual_norm_wave_kernel<DT, NV>), grid, dim3(256), 0, stream, a)
    if (dtype == LBM_DTYPE_BF16) {
      if (nv <= 1) LBM_RN_WAVE(0, 1);
      else if (nv <= 2) LBM_RN_WAVE(0, 2);
      else LBM_RN_WAVE(0, 4);
    } else {
      if (nv <= 1) LBM_RN_WAVE(1, 1);
      else if (nv <= 2) LBM_RN_WAVE(1, 2);
      else LBM_RN_WAVE(1, 4);
    }
#undef LBM_RN_WAVE
    return lbm_check_launch("lbm_residual_norm_wave_kernel");
  }
  const int n_chunks = (cols + 1023) >> 10;
#define LBM_RN_LAUNCH(DT, NCH) hipLaunchKernelGGL((lbm_residual_norm_kernel<DT, NCH>), dim3(rows), dim3(kThreads), 0, stream, a)
  if (dtype == LBM_DTYPE_BF16) {
    if (n_chunks <= 1) LBM_RN_LAUNCH(0, 1);
    else if (n_chunks <= 2) LBM_RN_LAUNCH(0, 2);
    else if (n_chunks <= 4) LBM_RN_LAUNCH(0, 4);
    else LBM_RN_LAUNCH(0, 8);
  } else {
    if (n_chunks <= 1) LBM_RN_LAUNCH(1, 1);
    else if (n_chunks <= 2) LBM_RN_LAUNCH(1, 2);
    else if (n_chunks <= 4) LBM_RN_LAUNCH(1, 4);
    else LBM_RN_LAUNCH(1, 8);
  }
#undef LBM_RN_LAUNCH
  return lbm_check_launch("lbm_residual_norm_kernel");
}
