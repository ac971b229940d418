// Ragged paged attention forward for gfx950: out = softmax(q k^T * scale) v over the K/V
// rows a row table names (pool pages in any order, partially filled pages already squeezed
// out by the table, optional read-only tail from the caller's own K/V).
//
// bf16 kernel, head_dim 64.  One workgroup = 8 wavefronts x 64 query rows of one head over
// one contiguous run of 64-token KV tiles (split-KV; partial results are merged by
// lbm_attn_combine_bf16_kernel).  Per tile a wavefront computes
//     S^T = K Q^T      v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q in registers
//     P   = exp2(S*c - m)   one query row per lane column, so row max/sum stay in-lane
//                           except one half-swap (v_permlane32_swap)
//     O^T += V^T P^T   A = V^T read with ds_read_b64_tr_b16 from the row-major V tile,
//                      B = P^T straight from the accumulator registers of S^T
// The running maximum is only raised when a tile exceeds it by more than kTau (in log2
// units): the rescale of the 64 output registers is skipped on almost every tile and the
// result is mathematically unchanged because the same stale maximum divides out.
//
// Schedule.  A SIMD cannot overlap the matrix pipe with the vector ALU when its two waves
// run the same phase at the same time (measured: MFMA-busy + VALU-busy = kernel time).  The
// eight waves therefore form two groups of four (one wave of each group per SIMD) that are
// kept one phase apart by the workgroup barrier: while one group issues the 32 MFMAs of a
// tile (PV of the previous tile, QK of the next), the other runs the softmax VALU work of
// its tile.  K/V tiles are shared by all eight waves through a three-stage LDS ring.
#include <hip/hip_runtime.h>
#include <climits>
#include "lbm_internal.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

#ifndef LBM_PRIO_MODE
#define LBM_PRIO_MODE 1
#endif
#if LBM_PRIO_MODE == 1   // matrix phase runs at raised priority
#define LBM_PRIO_MATRIX_BEGIN __builtin_amdgcn_s_setprio(1)
#define LBM_PRIO_MATRIX_END __builtin_amdgcn_s_setprio(0)
#elif LBM_PRIO_MODE == 2  // vector phase runs at raised priority
#define LBM_PRIO_MATRIX_BEGIN __builtin_amdgcn_s_setprio(0)
#define LBM_PRIO_MATRIX_END __builtin_amdgcn_s_setprio(1)
#else                    // equal priority; sched_barrier keeps the phase boundaries
#define LBM_PRIO_MATRIX_BEGIN __builtin_amdgcn_sched_barrier(0)
#define LBM_PRIO_MATRIX_END __builtin_amdgcn_sched_barrier(0)
#endif

#ifdef LBM_TRACE
__device__ long long g_lbm_trace[2 * 64 * 8];
#define LBM_TRACE_POINT(slot) do { if (blockIdx.x == 0 && (wave == 0 || wave == 4) && lane == 0 && trace_i < 64) \
    g_lbm_trace[((wave >> 2) * 64 + trace_i) * 8 + (slot)] = __builtin_readcyclecounter(); } while (0)
extern "C" int lbm_debug_trace_read(long long* dst) {
  return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(g_lbm_trace), sizeof(g_lbm_trace));
}
#else
#define LBM_TRACE_POINT(slot) do { } while (0)
#endif

namespace {

constexpr int kKvTile = 64;             // KV tokens per tile
constexpr int kQPerWave = 64;           // query rows per wavefront (two 32-row MFMA blocks)
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kQTile = kQPerWave * kWaves;
constexpr int kStages = 3;              // LDS ring depth
constexpr int kKStride = 72;            // bf16 per LDS row of K: 144 B, b128 reads hit 64 distinct banks
constexpr int kVStride = 96;            // bf16 per LDS row of V: 192 B, 4-row transpose reads conflict-free
constexpr float kTau = 8.0f;            // lazy-rescale threshold, log2 units
constexpr int kTargetWgs = 256;         // one 8-wave workgroup per CU

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
// Forces a value to exist in registers at this point of the program: the compiler otherwise
// sinks the softmax arithmetic below the workgroup barrier into the next phase, where it
// would run on the vector ALU at the same time as the other group's softmax.
__device__ __forceinline__ void pin(bf16x8& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(f32x16& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }

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

__global__ __launch_bounds__(kThreads, 1) void lbm_attn_bf16_d64_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) unsigned short lds_k[kStages][kKvTile * kKStride];
  __shared__ __attribute__((aligned(16))) unsigned short lds_v[kStages][kKvTile * kVStride];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n32 = lane & 31, g = lane >> 5;
  const int group = wave >> 2;  // waves w and w+4 share a SIMD and run opposite phases

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
  const int n = t1 - t0;
  const size_t row_elems = (size_t)H * 64;

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

  // ---- tile staging: each thread moves one 16-byte piece of a K row and of a V row per tile
  const int ld_r = tid >> 3, ld_c = (tid & 7) * 8;
  const unsigned short* pool_k = a.pool + (size_t)head * 64 + ld_c;
  const unsigned short* pool_v = pool_k + (size_t)a.page_size * row_elems;
  const unsigned short* own_k = a.self_k + (size_t)head * 64 + ld_c;
  const unsigned short* own_v = a.self_v + (size_t)head * 64 + ld_c;
  const int32_t* rows = a.kv_rows + sp.kv_row_begin;
  // Row-table entry of this thread's row in tile t; INT_MIN marks "no token" (zero fill).
  auto row_entry = [&](int t) -> int {
    const int kvi = t * kKvTile + ld_r;
    return (t < t1 && kvi < sp.kv_tokens) ? rows[kvi] : INT_MIN;
  };
  auto fetch = [&](int e, const unsigned short* pool_base, const unsigned short* own_base) -> u32x4 {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (e != INT_MIN) {
      const bool own = e < 0;
      const unsigned short* base = own ? own_base : pool_base;
      const size_t r = own ? (size_t)(-1 - e) : (size_t)e;
      v = *(const u32x4*)(base + r * row_elems);
    }
    return v;
  };
  auto put_k = [&](int stage, u32x4 v) { *(u32x4*)&lds_k[stage][ld_r * kKStride + ld_c] = v; };
  auto put_v = [&](int stage, u32x4 v) { *(u32x4*)&lds_v[stage][ld_r * kVStride + ld_c] = v; };

  f32x16 s[2][2];   // s[kvb][qb][i]: kv = kvb*32 + 8*(i/4) + 4*g + i%4, q = qb*32 + n32
  bf16x8 pb[2][4];  // softmax numerators as the B operand of O^T += V^T P^T

  // S^T = K Q^T for the tile in K stage `st`
  auto qk = [&](int st) {
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 ka = __builtin_bit_cast(
            bf16x8, *(const u32x4*)&lds_k[st][(kvb * 32 + n32) * kKStride + ks * 16 + g * 8]);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          if (ks == 0) {
            f32x16 z;
#pragma unroll
            for (int i = 0; i < 16; ++i) z[i] = 0.f;
            s[kvb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[qb][ks], z, 0, 0, 0);
          } else {
            s[kvb][qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[qb][ks], s[kvb][qb], 0, 0, 0);
          }
        }
      }
    }
  };
  // O^T += V^T P^T : o[qb][db][i] is d = db*32 + 8*(i/4) + 4*g + i%4, q = qb*32 + n32
  auto pv = [&](int st) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int db = 0; db < 2; ++db) {
        const int row = ks * 16 + 4 * g + ((lane & 15) >> 2);
        const int col = db * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3)))*)&lds_v[st][row * kVStride + col]);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3)))*)&lds_v[st][(row + 8) * kVStride + col]);
        s16x8 both;
        both[0] = lo[0]; both[1] = lo[1]; both[2] = lo[2]; both[3] = lo[3];
        both[4] = hi[0]; both[5] = hi[1]; both[6] = hi[2]; both[7] = hi[3];
        const bf16x8 va = __builtin_bit_cast(bf16x8, both);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[qb][ks], o[qb][db], 0, 0, 0);
      }
    }
  };
  // softmax numerators of tile t from s into pb; maintains m_run, l_run, rescales o lazily
  auto softmax = [&](int t) {
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
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
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
      float lsum = l_run[qb];
#pragma unroll
      for (int kvb = 0; kvb < 2; ++kvb) {
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          f32x8 p;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kvb][qb][hh * 8 + j], a.scale_log2, -mr));
          const bf16x8 pk = __builtin_convertvector(p, bf16x8);
          pb[qb][kvb * 2 + hh] = pk;
          // the denominator sums the bf16-rounded numerators the PV product actually uses
#pragma unroll
          for (int j = 0; j < 8; j += 2) {
            const bf16x2 pr = {pk[j], pk[j + 1]};
            lsum = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, lsum, false);
          }
        }
      }
      l_run[qb] = lsum;
    }
  };

  // ---- prologue: K(0), K(1), V(0) into the ring
  put_k(0, fetch(row_entry(t0), pool_k, own_k));
  put_k(1, fetch(row_entry(t0 + 1), pool_k, own_k));
  put_v(0, fetch(row_entry(t0), pool_v, own_v));
  int ek = row_entry(t0 + 2), ev = row_entry(t0 + 1);   // entries of the next pieces to fetch
  __syncthreads();
  if (group == 1) __syncthreads();  // puts the second group one phase behind the first

  // matrix phase 0
  u32x4 kreg = fetch(ek, pool_k, own_k), vreg = fetch(ev, pool_v, own_v);
  LBM_PRIO_MATRIX_BEGIN;
  qk(0);
  LBM_PRIO_MATRIX_END;
#pragma unroll
  for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) pin(s[kvb][qb]);
  __syncthreads();

  int st_k = 0, st_v = 0;  // stage of K(i) and of V(i)
  for (int i = 0; i < n; ++i) {
    const int t = t0 + i;
    const int trace_i = i; (void)trace_i;
    LBM_TRACE_POINT(0);
    // ---- vector phase i: softmax of tile i; land K(i+2), V(i+1) in the ring
    ek = row_entry(t + 3);
    ev = row_entry(t + 2);
#ifndef LBM_SKIP_VECTOR
    softmax(t);
#endif
    int st_k2 = st_k + 2; if (st_k2 >= kStages) st_k2 -= kStages;
    int st_v1 = st_v + 1; if (st_v1 >= kStages) st_v1 -= kStages;
    if (i + 2 < n) put_k(st_k2, kreg);
    if (i + 1 < n) put_v(st_v1, vreg);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) pin(pb[qb][ks]);
      pin(l_run[qb]);
    }
    LBM_TRACE_POINT(1);
    __syncthreads();
    LBM_TRACE_POINT(2);
    // ---- matrix phase i+1: PV of tile i, QK of tile i+1; start fetching K(i+3), V(i+2)
    kreg = fetch(ek, pool_k, own_k);
    vreg = fetch(ev, pool_v, own_v);
    int st_k1 = st_k + 1; if (st_k1 >= kStages) st_k1 -= kStages;
    LBM_PRIO_MATRIX_BEGIN;
#ifndef LBM_SKIP_MATRIX
    pv(st_v);
    qk(st_k1);  // on the last tile this reads a stale stage and its result is never used
    // LDS fragment reads run three steps (of two MFMAs) ahead of the MFMAs that use them:
    // 8 PV steps with two transpose reads each, then 8 QK steps with one 128-bit read each.
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
    for (int step = 0; step < 16; ++step) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      const int ahead = step + 3;
      if (ahead < 8) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      else if (ahead < 16) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#endif
    LBM_PRIO_MATRIX_END;
#pragma unroll
    for (int kvb = 0; kvb < 2; ++kvb)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) pin(s[kvb][qb]);
    LBM_TRACE_POINT(3);
    __syncthreads();
    LBM_TRACE_POINT(4);
    st_k = st_k1;
    st_v = st_v1;
  }
  if (group == 0) __syncthreads();  // both groups pass the same number of barriers

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
  // Aim at one 8-wave workgroup on each of the 256 CUs, all with about the same number of tiles.
  const long long target_wgs = kTargetWgs;
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
  hipLaunchKernelGGL(lbm_attn_bf16_d64_kernel, dim3(sch.total_wgs), dim3(kThreads), 0, stream, a);
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
