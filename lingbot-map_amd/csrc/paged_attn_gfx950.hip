// Ragged paged attention forward for gfx950: out = softmax(q k^T * scale) v over the K/V
// rows a row table names (pool pages in any order, partially filled pages already squeezed
// out by the table, optional read-only tail from the caller's own K/V).
//
// bf16 kernel, head_dim 64.  One workgroup = 4 wavefronts x 64 query rows of one head over
// one contiguous run of 64-token KV tiles (split-KV; partial results are merged by
// lbm_attn_combine_kernel).  Per tile a wavefront computes
//     S^T = K Q^T      v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q in registers
//     P   = exp2(S*c - m)   one query row per lane column, so row max/sum stay in-lane
//                           except one half-swap (v_permlane32_swap)
//     O^T += V^T P^T   A = V^T read with ds_read_b64_tr_b16 from the row-major V tile,
//                      B = P^T straight from the accumulator registers of S^T
// The running maximum is only raised when a tile exceeds it by more than kTau (in log2
// units): the rescale of the 64 output registers is skipped on almost every tile and the
// result is mathematically unchanged because the same stale maximum divides out.
#include <hip/hip_runtime.h>
#include "lbm_internal.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

namespace {

constexpr int kKvTile = 64;             // KV tokens per tile
constexpr int kQPerWave = 64;           // query rows per wavefront (two 32-row MFMA blocks)
constexpr int kWaves = 4;
constexpr int kQTile = kQPerWave * kWaves;
constexpr int kKStride = 72;            // bf16 per LDS row of K: 144 B, b128 reads hit 64 distinct banks
constexpr int kVStride = 96;            // bf16 per LDS row of V: 192 B, 4-row transpose reads conflict-free
constexpr float kTau = 8.0f;            // lazy-rescale threshold, log2 units

struct AttnArgs {
  const unsigned short* q;
  const unsigned short* pool;
  unsigned short* out;
  const unsigned short* self_k;
  const unsigned short* self_v;
  const int32_t* kv_rows;
  float* part_o;
  float* part_lse;
  int num_heads;
  int page_size;
  float scale_log2;
  LbmAttnSchedule sch;
};

// Exchange between lane l and lane l^32.  v_permlane32_swap swaps the upper half of its first
// register with the lower half of its second; fed two copies of x it leaves {x_lo, x_lo} in
// the first and {x_hi, x_hi} in the second.  Written as inline asm because the compiler
// folds the builtin's two results into one; the s_nop covers the VALU-write to permlane-read
// wait states the compiler can no longer see.
__device__ __forceinline__ void swap_halves(float x, float& lo, float& hi) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  lo = a;
  hi = b;
}
__device__ __forceinline__ float swap_max(float x) {
  float lo, hi;
  swap_halves(x, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float swap_sum(float x) {
  float lo, hi;
  swap_halves(x, lo, hi);
  return lo + hi;
}

}  // namespace

__global__ __launch_bounds__(256, 2) void lbm_attn_bf16_d64_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) unsigned short lds_k[2][kKvTile * kKStride];
  __shared__ __attribute__((aligned(16))) unsigned short lds_v[2][kKvTile * kVStride];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n32 = lane & 31, g = lane >> 5;

  // ---- which piece of work is this workgroup
  int b = 0;
  for (int i = 1; i < a.sch.n_streams; ++i)
    if ((int)blockIdx.x >= a.sch.s[i].wg_begin) b = i;
  const LbmAttnStreamPlan sp = a.sch.s[b];
  const int H = a.num_heads;
  const int local = (int)blockIdx.x - sp.wg_begin;
  const int n_hs = H * sp.n_splits;
  int qt, hs;
  if ((n_hs & 7) == 0) {
    // Workgroups are dealt to the 8 XCDs round-robin: keep the query tiles that share one
    // (head, split) - hence the same K/V rows - on one XCD so its L2 serves the re-reads.
    const int x = local & 7, i = local >> 3;
    qt = i % sp.n_qtiles;
    hs = (i / sp.n_qtiles) * 8 + x;
  } else {
    qt = local % sp.n_qtiles;
    hs = local / sp.n_qtiles;
  }
  if (local >= sp.n_qtiles * n_hs) return;  // padding between streams
  const int head = hs % H, split = hs / H;
  const int n_tiles = (sp.kv_tokens + kKvTile - 1) / kKvTile;
  const int t0 = split * sp.tiles_per_split;
  const int t1 = min(t0 + sp.tiles_per_split, n_tiles);
  const size_t row_elems = (size_t)H * 64;
  const size_t v_off = (size_t)a.page_size * row_elems;

  // ---- Q fragments (B operand of S^T = K Q^T): lane holds q row n32, d = ks*16 + g*8 .. +8
  bf16x8 qf[2][4];
  const int q_row0 = qt * kQTile + wave * kQPerWave;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int r = q_row0 + qb * 32 + n32;
    const unsigned short* qp = a.q + ((size_t)(sp.q_begin + r) * H + head) * 64 + g * 8;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (r < sp.q_rows) v = *(const u32x4*)(qp + ks * 16);
      qf[qb][ks] = __builtin_bit_cast(bf16x8, v);
    }
  }

  f32x16 o[2][2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
  float m_run[2] = {-INFINITY, -INFINITY};
  float l_run[2] = {0.f, 0.f};

  // ---- tile staging: each thread moves two 16-byte pieces of K and of V per tile
  const int ld_r = tid >> 3, ld_c = (tid & 7) * 8;
  u32x4 kreg[2], vreg[2];
  auto fetch = [&](int t) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int kvi = t * kKvTile + ld_r + 32 * i;
      u32x4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
      if (kvi < sp.kv_tokens) {
        const int e = a.kv_rows[sp.kv_row_begin + kvi];
        const unsigned short *kp, *vp;
        if (e >= 0) {
          kp = a.pool + ((size_t)e * H + head) * 64 + ld_c;
          vp = kp + v_off;
        } else {
          const size_t off = ((size_t)(-1 - e) * H + head) * 64 + ld_c;
          kp = a.self_k + off;
          vp = a.self_v + off;
        }
        kk = *(const u32x4*)kp;
        vv = *(const u32x4*)vp;
      }
      kreg[i] = kk;
      vreg[i] = vv;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = ld_r + 32 * i;
      *(u32x4*)&lds_k[buf][r * kKStride + ld_c] = kreg[i];
      *(u32x4*)&lds_v[buf][r * kVStride + ld_c] = vreg[i];
    }
  };

  fetch(t0);
  stage(0);
  __syncthreads();

  for (int t = t0; t < t1; ++t) {
    const int buf = (t - t0) & 1;
    if (t + 1 < t1) fetch(t + 1);

    // ---- S^T = K Q^T : s[kvb][qb][i] is kv = kvb*32 + 8*(i/4) + 4*g + i%4, q = qb*32 + n32
    f32x16 s[2][2];
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kvb][qb][i] = 0.f;
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 ka = __builtin_bit_cast(
            bf16x8, *(const u32x4*)&lds_k[buf][(kvb * 32 + n32) * kKStride + ks * 16 + g * 8]);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          s[kvb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[qb][ks], s[kvb][qb], 0, 0, 0);
      }
    }

    const int n_valid = sp.kv_tokens - t * kKvTile;
    if (n_valid < kKvTile) {
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int kv = kvb * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          if (kv >= n_valid) {
            s[kvb][0][i] = -INFINITY;
            s[kvb][1][i] = -INFINITY;
          }
        }
    }

    // ---- softmax numerators, packed to bf16 as the B operand of O^T += V^T P^T
    bf16x8 pb[2][4];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float mx = s[0][qb][0];
#pragma unroll
      for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s[0][qb][i]);
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[1][qb][i]);
      mx = swap_max(mx);
      const float ms = mx * a.scale_log2;
      const bool raise = ms > m_run[qb] + kTau;
      if (__builtin_amdgcn_ballot_w64(raise)) {
        const float m_new = raise ? ms : m_run[qb];
        const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_new);
        m_run[qb] = m_new;
        l_run[qb] *= alpha;
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha;
      }
      const float mr = m_run[qb];
      float lsum = 0.f;
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          f32x8 p;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kvb][qb][hh * 8 + j], a.scale_log2, -mr));
            lsum += p[j];
          }
          pb[qb][kvb * 2 + hh] = __builtin_convertvector(p, bf16x8);
        }
      }
      l_run[qb] += lsum;
    }

    // ---- O^T += V^T P^T : o[qb][db][i] is d = db*32 + 8*(i/4) + 4*g + i%4, q = qb*32 + n32
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int db = 0; db < 2; ++db) {
        const int row = ks * 16 + 4 * g + ((lane & 15) >> 2);
        const int col = db * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3)))*)&lds_v[buf][row * kVStride + col]);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3)))*)&lds_v[buf][(row + 8) * kVStride + col]);
        s16x8 both;
        both[0] = lo[0]; both[1] = lo[1]; both[2] = lo[2]; both[3] = lo[3];
        both[4] = hi[0]; both[5] = hi[1]; both[6] = hi[2]; both[7] = hi[3];
        const bf16x8 va = __builtin_bit_cast(bf16x8, both);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[qb][ks], o[qb][db], 0, 0, 0);
      }
    }

    if (t + 1 < t1) stage(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int r = q_row0 + qb * 32 + n32;
    const float l_tot = swap_sum(l_run[qb]);
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    if (r >= sp.q_rows) continue;
    if (sp.n_splits == 1) {
      unsigned short* op = a.out + ((size_t)(sp.q_begin + r) * H + head) * 64;
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          f32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = o[qb][db][c4 * 4 + e] * inv;
          *(bf16x4*)(op + db * 32 + c4 * 8 + g * 4) = __builtin_convertvector(w, bf16x4);
        }
    } else {
      const size_t prow = ((size_t)sp.part_begin + (size_t)split * sp.q_rows + r) * H + head;
      float* po = a.part_o + prow * 64;
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
          f32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = o[qb][db][c4 * 4 + e] * inv;
          *(f32x4*)(po + db * 32 + c4 * 8 + g * 4) = w;
        }
      if (g == 0) a.part_lse[prow] = m_run[qb] + __builtin_amdgcn_logf(l_tot);
    }
  }
}

// Merge split-KV partial results: out = sum_s w_s * o_s with w_s = 2^(lse_s - max) / sum.
// One thread per (query row, head, 4 consecutive d).
__global__ __launch_bounds__(256) void lbm_attn_combine_bf16_kernel(AttnArgs a) {
  const LbmAttnStreamPlan sp = a.sch.s[blockIdx.y];
  if (sp.n_splits <= 1) return;
  const int H = a.num_heads;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)sp.q_rows * H * 16) return;
  const int d4 = (int)(idx & 15);
  const long long rh = idx >> 4;  // r * H + h
  const long long split_stride = (long long)sp.q_rows * H;
  const float* lse = a.part_lse + (long long)sp.part_begin * H + rh;
  float mx = -INFINITY;
  for (int s = 0; s < sp.n_splits; ++s) mx = fmaxf(mx, lse[s * split_stride]);
  float wsum = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const float* po = a.part_o + ((long long)sp.part_begin * H + rh) * 64 + d4 * 4;
  for (int s = 0; s < sp.n_splits; ++s) {
    const float w = __builtin_amdgcn_exp2f(lse[s * split_stride] - mx);
    const f32x4 v = *(const f32x4*)(po + s * split_stride * 64);
    wsum += w;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] += w * v[e];
  }
  const float inv = 1.0f / wsum;
  const long long r = rh / H, h = rh % H;
  unsigned short* op = a.out + ((size_t)(sp.q_begin + r) * H + h) * 64 + d4 * 4;
#pragma unroll
  for (int e = 0; e < 4; ++e) acc[e] *= inv;
  *(bf16x4*)op = __builtin_convertvector(acc, bf16x4);
}

// ---------------------------------------------------------------------------- schedule
void lbm_attn_schedule(const lbm_attn_stream* streams, int n_streams, int num_heads,
                       LbmAttnSchedule* out) {
  // Aim at two workgroups on each of the 256 CUs, all with about the same number of tiles.
  const long long target_wgs = 512;
  LbmAttnSchedule& sch = *out;
  sch = LbmAttnSchedule{};
  sch.n_streams = n_streams;
  long long work = 0;
  for (int i = 0; i < n_streams; ++i) {
    const long long qt = (streams[i].q_rows + kQTile - 1) / kQTile;
    const long long nt = (streams[i].kv_tokens + kKvTile - 1) / kKvTile;
    work += qt * num_heads * nt;
  }
  long long tps_target = (work + target_wgs - 1) / target_wgs;
  if (tps_target < 4) tps_target = 4;
  int wg = 0;
  long long part = 0;
  for (int i = 0; i < n_streams; ++i) {
    LbmAttnStreamPlan& p = sch.s[i];
    p.q_begin = streams[i].q_begin;
    p.q_rows = streams[i].q_rows;
    p.kv_row_begin = streams[i].kv_row_begin;
    p.kv_tokens = streams[i].kv_tokens;
    p.n_qtiles = (p.q_rows + kQTile - 1) / kQTile;
    const int nt = (p.kv_tokens + kKvTile - 1) / kKvTile;
    int ns = (int)((nt + tps_target - 1) / tps_target);
    if (ns < 1) ns = 1;
    if (ns > 64) ns = 64;
    p.tiles_per_split = nt > 0 ? (nt + ns - 1) / ns : 1;
    p.n_splits = nt > 0 ? (nt + p.tiles_per_split - 1) / p.tiles_per_split : 1;
    // keep each stream's first workgroup on XCD 0 so the in-kernel XCD mapping lines up
    wg = (wg + 7) & ~7;
    p.wg_begin = wg;
    p.part_begin = (int32_t)part;
    wg += p.n_qtiles * num_heads * p.n_splits;
    if (p.n_splits > 1) part += (long long)p.n_splits * p.q_rows;
  }
  sch.total_wgs = wg;
  sch.part_rows = part;
}

size_t lbm_attn_schedule_bytes(const LbmAttnSchedule& sch, int num_heads, int head_dim) {
  return (size_t)sch.part_rows * num_heads * (head_dim + 1) * sizeof(float);
}

int lbm_launch_attention(const void* q, const void* pool, void* out, const void* self_k,
                         const void* self_v, const int32_t* kv_rows, const LbmAttnSchedule& sch,
                         int num_heads, int head_dim, int page_size, int dtype, float sm_scale,
                         void* workspace, hipStream_t stream) {
  if (dtype != LBM_DTYPE_BF16 || head_dim != 64)
    return lbm_fail(LBM_ERR_UNSUPPORTED, "attention kernel covers bf16 with head_dim 64 (got dtype %d, head_dim %d)", dtype, head_dim);
  AttnArgs a;
  a.q = (const unsigned short*)q;
  a.pool = (const unsigned short*)pool;
  a.out = (unsigned short*)out;
  a.self_k = (const unsigned short*)self_k;
  a.self_v = (const unsigned short*)self_v;
  a.kv_rows = kv_rows;
  a.part_o = (float*)workspace;
  a.part_lse = a.part_o + (size_t)sch.part_rows * num_heads * head_dim;
  a.num_heads = num_heads;
  a.page_size = page_size;
  a.scale_log2 = sm_scale * 1.4426950408889634f;
  a.sch = sch;
  if (sch.total_wgs == 0) return LBM_OK;
  hipLaunchKernelGGL(lbm_attn_bf16_d64_kernel, dim3(sch.total_wgs), dim3(256), 0, stream, a);
  int rc = lbm_check_launch("lbm_attn_bf16_d64_kernel");
  if (rc != LBM_OK) return rc;
  if (sch.part_rows > 0) {
    int max_rows = 0;
    for (int i = 0; i < sch.n_streams; ++i)
      if (sch.s[i].n_splits > 1 && sch.s[i].q_rows > max_rows) max_rows = sch.s[i].q_rows;
    const long long threads = (long long)max_rows * num_heads * 16;
    hipLaunchKernelGGL(lbm_attn_combine_bf16_kernel, dim3((unsigned)((threads + 255) / 256), sch.n_streams),
                       dim3(256), 0, stream, a);
    rc = lbm_check_launch("lbm_attn_combine_bf16_kernel");
  }
  return rc;
}
