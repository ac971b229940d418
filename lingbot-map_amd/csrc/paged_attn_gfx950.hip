// Ragged paged attention forward for gfx950: out = softmax(q k^T * scale) v over the K/V
// rows a row table names (pool pages in any order, partially filled pages already squeezed
// out by the table, optional read-only tail from the caller's own K/V).
//
// bf16 kernel, head_dim 64.  One workgroup = 8 wavefronts x 64 query rows of one head over
// one contiguous run of 64-token KV tiles (split-KV; partial results are merged by
// lbm_attn_combine_bf16_kernel).  Per tile a wavefront computes
//     S^T = K Q^T      v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = Q in registers; the
//                      softmax scale (in log2 units) is folded into Q, so S arrives ready
//                      for exp2
//     P   = exp2(S)    one query row per lane column; v_exp_f32 + v_cvt_pk_bf16_f32
//     O^T += V^T P^T   A = V^T read with ds_read_b64_tr_b16 from the row-major V tile,
//                      B = P^T straight from the registers the packing wrote
//     l   += 1^T P^T   row sums on the matrix pipe too (16x16x32 with a 0/1 selector)
// Common path: no softmax reference at all.  2^score is exact softmax arithmetic as long as
// nothing leaves the range of fp32 / bf16; a range check on O and l after the last tile
// decides, per workgroup, whether that held.  If not - scores beyond about +-100 in log2
// units - the workgroup repeats its split in an out-of-line function (lbm_attn_split_safe)
// with a reference m carried into the QK^T contraction as one more k-step: m is kHeadroom
// above the row maximum seen when it was last set and is only raised when a numerator
// reaches 2 (a bf16 numerator is >= 2 or infinite exactly when the top bit of its exponent
// field is set: a few OR instructions per half tile), with O, l and the scores in flight
// rescaled on that rare path.  The same extra k-step masks the rows past the last token on
// the ragged last tiles of either path.
//
// Why it is built this way.  Measured on MI355X with two wavefronts per SIMD: v_exp_f32 issues
// every ~4.6 ns per SIMD, v_cvt_pk_bf16_f32 (like v_max3_f32, v_dot2c_f32_bf16) every ~2.7 ns, plain
// fp32 adds and multiplies every ~1.4 ns, and a 32x32x16 MFMA occupies the matrix pipe for
// 13.8 ns.  With head_dim 64 every score needs one exp2 and half a packing instruction, so the
// vector ALU is as busy as the matrix pipe; everything that can run as an MFMA (scale, row
// sums, masking of the ragged tail, the reference subtraction of the repeat pass) does, and
// the vector ALU is left with exp2 and packing.
//
// Schedule.  Each wavefront runs a software pipeline over 32-token half tiles: while the
// vector ALU turns the scores of one half into numerators, the MFMAs of the next half's QK^T
// and of the previous half's PV and row sums are issued in between.  A half-step is one basic
// block written as 20 slices (22 with the extra k-step; one MFMA plus its share of the vector
// work and LDS reads each) fenced with sched_barrier, and the two wavefronts of a SIMD fill
// each other's issue gaps.  K/V tiles are shared by all eight waves through a three-stage
// LDS ring with one workgroup barrier per tile; the rows go from global memory straight into
// the ring (global_load_lds_dwordx4), no staging registers and no LDS store instructions.
#include <hip/hip_runtime.h>
#include <climits>
#include <mutex>
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

namespace {

constexpr int kKvTile = 64;             // KV tokens per tile
constexpr int kQPerWave = 64;           // query rows per wavefront (two 32-row MFMA blocks)
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kQTile = kQPerWave * kWaves;
constexpr int kStages = 3;              // LDS ring depth
constexpr int kRingRow = 64;            // bf16 per row of a K/V tile in the LDS ring: 128 B, unpadded, 16-byte chunks swizzled
constexpr int kKStride = 72;            // bf16 per row of a padded patch (Q, short-KV K, output transpose): 144 B, b128 reads hit 64 distinct banks
constexpr int kVStride = 96;            // bf16 per row of the short-KV kernel's V patch: 192 B, 4-row transpose reads conflict-free
constexpr float kHeadroom = 11.0f;      // the softmax reference is set this far above the row maxima (log2 units)

struct AttnCore {
  const unsigned short* q;
  const unsigned short* pool;
  unsigned short* out;
  const unsigned short* self_k;
  const unsigned short* self_v;
  const int32_t* kv_rows;
  const int32_t* live_kv_tokens;  // device-side token counts (NULL: the host's counts in the plan)
  unsigned short* part_o;  // split-KV partial outputs, normalised, bf16
  float* part_lse;
  int num_heads;
  int page_size;
  float scale_log2;
  // the append carried by the merging launch: row t of self_k / self_v to pool row append_rows[t]
  const int32_t* append_rows;
  int append_tokens;
  int combine_blocks;      // blocks (per stream) of that launch that merge; those beyond them append
};
struct AttnArgs : AttnCore {
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
// The same for neighbouring rows of 16 lanes: v_permlane16_swap swaps the odd rows of its first
// register with the even rows of its second; fed two copies of x it leaves rows {0, 0, 2, 2}
// in the first and rows {1, 1, 3, 3} in the second.
__device__ __forceinline__ void swap_rows(float x, float& even, float& odd) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  even = a;
  odd = b;
}
// Built with -fno-honor-nans, fmaxf chains become v_max3_f32 without NaN-quieting moves.
__device__ __forceinline__ float max3(float a, float b, float c) { return fmaxf(fmaxf(a, b), c); }
__device__ __forceinline__ float max2(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ float swap_max(float x) {
  float lo, hi;
  swap_halves(x, lo, hi);
  return max2(lo, hi);
}

// LDS of the split-KV kernel, at namespace scope because the kernel and the out-of-line second
// pass below both work in it.
__shared__ __attribute__((aligned(1024))) unsigned short lds_k[kStages][kKvTile * kRingRow];
__shared__ __attribute__((aligned(1024))) unsigned short lds_v[kStages][kKvTile * kRingRow];
__shared__ __attribute__((aligned(16))) unsigned short lds_q[kWaves][kQPerWave * kKStride];   // per-wave patch: Q on the way in, O on the way out

// The repeat pass is a function of its own, not inlined: it is entered once in a blue moon,
// and compiled into the kernel body its registers would push the common path into scratch
// memory (spill stores and reloads on every launch, tens of MB of HBM traffic).
// (it takes the 130 bytes it needs, not the whole argument block with its sixteen stream plans:
// what is passed by value sizes the kernel's scratch frame)
__device__ __noinline__ void lbm_attn_split_safe(AttnCore a, LbmAttnStreamPlan sp);

// One workgroup's share of the split-KV attention: 512 query rows of one head over one run of
// KV tiles, start to finish.  SAFE = false is the common path (no softmax reference, range
// check at the end); when the check fails it writes nothing, hands the workgroup to the
// repeat pass and ends the program there, so that nothing of the common path is live across
// the call.  SAFE = true is the repeat with a reference that follows the row maxima.
template <bool SAFE>
__device__ __forceinline__ void lbm_attn_split(const AttnCore& a, const LbmAttnStreamPlan& sp) {
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n32 = lane & 31, g = lane >> 5;

  // ---- which piece of this stream's work is this workgroup
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
  // With device-side token counts the split count stays the host's choice (it fixes the grid
  // and the workspace layout) and the tiles are dealt to the splits from the live count.
  const int kv_tokens = a.live_kv_tokens ? a.live_kv_tokens[sp.live_at] : sp.kv_tokens;
  if (kv_tokens <= 0 && sp.n_splits == 1) {
    // nothing visible: the reference returns zeros (lingbot_map/layers/flashinfer_cache.py:368-370)
    for (int k = 0; k < kQPerWave / 8; ++k) {
      const int r = qt * kQTile + wave * kQPerWave + k * 8 + (lane >> 3);
      if (r < sp.q_rows)
        *(u32x4*)(a.out + ((size_t)(sp.q_begin + r) * H + head) * 64 + (lane & 7) * 8) = u32x4{0u, 0u, 0u, 0u};
    }
    return;
  }
  const int n_tiles = (max(kv_tokens, 0) + kKvTile - 1) / kKvTile;
  const int tiles_per_split = a.live_kv_tokens ? max((n_tiles + sp.n_splits - 1) / sp.n_splits, 1) : sp.tiles_per_split;
  const int t0 = split * tiles_per_split;
  const int t1 = min(t0 + tiles_per_split, n_tiles);  // an empty split (t1 <= t0) contributes weight 0
  const int n = t1 - t0;
  const unsigned row_bytes = (unsigned)H * 128u;

  // ---- tile staging: each thread moves one 16-byte piece of a K row and of a V row per tile,
  // global -> LDS without a stop in registers (global_load_lds_dwordx4: the wavefront's 64
  // pieces land on 1 KiB of consecutive LDS starting at M0, i.e. on eight 128-byte rows).  A
  // tile in the ring is therefore 64 unpadded rows, and what keeps the fragment reads off each
  // other's banks is the order of the eight 16-byte chunks within a row, which each lane
  // chooses by the global address it reads: chunk c of K row r sits at position
  // c ^ ((r >> 1) & 7) (the b128 fragment reads of 16 rows x one chunk hit all 64 banks), chunk
  // c of V row r at c ^ 4 ((r >> 1) & 1) (the 8-byte transposed reads touch four rows x 64
  // bytes; rows r+2 and r+3 move to the other half).  The compiler does not count these loads
  // (its own waits only get stricter by that); LBM_DMA_LANDED waits for them before the
  // barrier that publishes a tile.  M0 is declared clobbered, so the compiler keeps nothing of
  // its own in it across a load.
  // Rows past the last token re-read the last token (finite data; the softmax masks them).
  const int ld_r = tid >> 3;
  const int ld_ck = ((lane & 7) ^ ((ld_r >> 1) & 7)) * 8, ld_cv = ((lane & 7) ^ (((ld_r >> 1) & 1) * 4)) * 8;
  const char* pool_k = (const char*)(a.pool + (size_t)head * 64 + ld_ck);
  const char* pool_v = (const char*)(a.pool + (size_t)head * 64 + ld_cv) + (size_t)a.page_size * row_bytes;
  const char* own_k = (const char*)(a.self_k + (size_t)head * 64 + ld_ck);
  const char* own_v = (const char*)(a.self_v + (size_t)head * 64 + ld_cv);
  const int32_t* rows = a.kv_rows + sp.kv_row_begin;
  const int last_token = max(kv_tokens - 1, 0);
  // Tiles past the end of this split re-read its last tile: the data lands in ring stages
  // nobody reads any more, and the code stays free of branches.
  auto row_entry = [&](int t) -> int { return rows[min(max(min(t, t1 - 1), 0) * kKvTile + ld_r, last_token)]; };
  auto dma = [&](int e, const char* pool_base, const char* own_base, const unsigned short* lds_tile) {
    // negative entries name rows of the caller's own K/V (read-only tail of a non-keyframe)
    const char* base = e < 0 ? own_base : pool_base;
    const unsigned r = (unsigned)(e ^ (e >> 31));
    const char* src = base + (unsigned long long)r * row_bytes;
    const unsigned m0v = (unsigned)(size_t)(__attribute__((address_space(3))) const void*)(lds_tile + wave * (8 * kRingRow));
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(src), "s"(__builtin_amdgcn_readfirstlane(m0v))
                 : "memory", "m0");
  };
#define LBM_DMA_LANDED() __builtin_amdgcn_s_waitcnt(0x0F70)   /* vmcnt(0); expcnt and lgkmcnt untouched */

  // The first tiles' rows are asked for before anything else: the row table entry, then the K/V
  // row it names, is the longest chain of memory latencies in front of the first MFMA, and the
  // Q rows below travel at the same time.
  const int e_t0 = row_entry(t0), e_t1 = row_entry(t0 + 1);
  int ek = row_entry(t0 + 2), ev = e_t1;   // entries of the loads of the first iteration
  dma(e_t0, pool_k, own_k, lds_k[0]);
  dma(e_t1, pool_k, own_k, lds_k[1]);
  dma(e_t0, pool_v, own_v, lds_v[0]);

  // ---- Q fragments (B operand of S^T = K Q^T): lane holds q row n32, d = ks*16 + g*8 .. +8.
  // Each wavefront reads its 64 query rows as whole 128-byte rows (eight lanes per row), parks
  // them in its own LDS patch and picks the fragments up from there; read directly in the
  // fragment layout every load instruction would touch 64 different rows with 16 bytes each.
  // The softmax scale and log2(e) are folded into Q here (one extra bf16 rounding of q; none
  // when the producer already multiplied q by them before its own rounding and the caller
  // passed sm_scale = 0), so the MFMA result is already the exponent of 2.
  bf16x8 qf[2][4];
  const int q_row0 = qt * kQTile + wave * kQPerWave;
  {
    unsigned short* patch = lds_q[wave];
    u32x4 raw[kQPerWave / 8];
#pragma unroll
    for (int k = 0; k < kQPerWave / 8; ++k) {
      // rows past the stream's last query row re-read that row: their results are never stored,
      // and eight unconditional loads go out back to back (a load inside a conditional block
      // ends up with a wait for everything in flight behind it)
      const int r = max(min(q_row0 + k * 8 + (lane >> 3), sp.q_rows - 1), 0);
      raw[k] = *(const u32x4*)(a.q + ((size_t)(sp.q_begin + r) * H + head) * 64 + (lane & 7) * 8);
    }
#pragma unroll
    for (int k = 0; k < kQPerWave / 8; ++k)
      *(u32x4*)&patch[(k * 8 + (lane >> 3)) * kKStride + (lane & 7) * 8] = raw[k];
    __syncthreads();   // (a wavefront only reads its own patch; the barrier orders its lanes' writes and reads)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 rawf = __builtin_bit_cast(bf16x8, *(const u32x4*)&patch[(qb * 32 + n32) * kKStride + ks * 16 + g * 8]);
        f32x8 f = __builtin_convertvector(rawf, f32x8);
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] *= a.scale_log2;
        // (a q that already carries the scale - scale_log2 == 1 - comes back bit for bit: x * 1 is exact)
        qf[qb][ks] = __builtin_convertvector(f, bf16x8);
      }
  }
  // One more 16-wide step of the QK contraction carries the softmax reference: K side is the
  // constant row (-1, -1, 0, ...), Q side is (m_hi, m_lo, 0, ...) with m_hi + m_lo = m_run
  // exactly, so S arrives as score*scale - m_run at no vector-ALU cost.
  // A third element masks the rows past the last token: K side -1 on such rows (0 elsewhere),
  // Q side 2^100, so their scores arrive as about -2^100 and their numerators are exactly 0.
  u32x4 kaug_bits = {0u, 0u, 0u, 0u};
  if (g == 0) kaug_bits[0] = 0xBF80BF80u;
  u32x4 qaug_bits[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
  if (g == 0) qaug_bits[0][1] = qaug_bits[1][1] = 0x7180u;  // bf16 2^100

  // Accumulators and softmax reference; (re)initialised at the start of each pass below.
  f32x16 o[2][2];
  float m_run[2];
  // Row sums (softmax denominators) are accumulated by the matrix pipe as well: a 16x16x32 MFMA
  // with a 0/1 selector as A and the numerators, exactly as they sit in the registers for PV,
  // as B.  Read as a 32x16 B operand the numerator registers hold, for column n, query n in
  // k rows 0-7 and 16-23 and query n+16 in k rows 8-15 and 24-31; selector row 0 picks the
  // former and row 1 the latter, so lane n < 16 ends up with the sums of query n (element 0)
  // and of query n+16 (element 1) of the block, and every other element stays 0.
  f32x4 lacc[2];
  const unsigned sel_word = (lane == 0 || lane == 32 || lane == 17 || lane == 49) ? 0x3F803F80u : 0u;
  const bf16x8 lsel = __builtin_bit_cast(bf16x8, u32x4{sel_word, sel_word, sel_word, sel_word});

  // Register state of the software pipeline.  A 64-token tile is processed as two 32-token
  // halves; while the vector ALU turns the scores of one half into softmax numerators, the
  // matrix pipe computes the scores of the next half and folds the numerators of the
  // previous half into O.  The two halves alternate between the A and B register sets.
  f32x16 sA[2], sB[2];        // s[qb][i]: kv = 32*half + 8*(i/4) + 4*g + i%4, q = qb*32 + n32
  bf16x8 pA[2][2], pB[2][2];  // numerators [qb][k-step] as the B operand of O^T += V^T P^T
  bf16x8 vnext[2];            // V^T fragments of the next PV's first k-step, read early

  // V^T fragment (A operand): lane holds d = db*32 + n32 and the kv rows
  // ks*16 + {4g..4g+3, 8+4g..8+4g+3} of the V tile in stage st
  auto v_frag = [&](int st, int ks, int db) -> bf16x8 {
    const int row = ks * 16 + 4 * g + ((lane & 15) >> 2);
    const int col = (db * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4) ^ (((lane >> 3) & 1) * 32);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (s16x4 __attribute__((address_space(3)))*)&lds_v[st][row * kRingRow + col]);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (s16x4 __attribute__((address_space(3)))*)&lds_v[st][(row + 8) * kRingRow + col]);
    s16x8 both;
    both[0] = lo[0]; both[1] = lo[1]; both[2] = lo[2]; both[3] = lo[3];
    both[4] = hi[0]; both[5] = hi[1]; both[6] = hi[2]; both[7] = hi[3];
    return __builtin_bit_cast(bf16x8, both);
  };
  // One k-step (16 kv rows) of O^T += V^T P^T; o[qb][db][i] is d = db*32 + 8*(i/4) + 4*g + i%4
  auto pv_step = [&](const bf16x8 (&va)[2], const bf16x8 (&p)[2][2], int kk) {
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
        o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[db], p[qb][kk], o[qb][db], 0, 0, 0);
  };
  // S^T = K Q^T - m_run for the 32 kv rows of half h of the K tile in stage st
  auto qk_half = [&](int st, int h, int n_valid, f32x16 (&sd)[2]) {
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    u32x4 kb = kaug_bits;
    kb[1] = (g == 0 && h * 32 + n32 >= n_valid) ? 0xBF80u : 0u;
    const bf16x8 kaug = __builtin_bit_cast(bf16x8, kb);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
      sd[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kaug, __builtin_bit_cast(bf16x8, qaug_bits[qb]), z, 0, 0, 0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const bf16x8 ka = __builtin_bit_cast(
          bf16x8, *(const u32x4*)&lds_k[st][(h * 32 + n32) * kRingRow + ((ks * 2 + g) ^ ((n32 >> 1) & 7)) * 8]);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
        sd[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[qb][ks], sd[qb], 0, 0, 0);
    }
  };
  // Row maxima of one half, per query block (the lane's own 16 scores, then the other
  // half-wave's through one swap).
  auto row_max = [&](const f32x16 (&sc)[2], float (&mx)[2]) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float m0 = max3(sc[qb][0], sc[qb][1], sc[qb][2]), m1 = max3(sc[qb][3], sc[qb][4], sc[qb][5]);
      m0 = max3(m0, sc[qb][6], sc[qb][7]);
      m1 = max3(m1, sc[qb][8], sc[qb][9]);
      m0 = max3(m0, sc[qb][10], sc[qb][11]);
      m1 = max3(m1, sc[qb][12], sc[qb][13]);
      m0 = max3(m0, sc[qb][14], sc[qb][15]);
      mx[qb] = swap_max(max2(m0, m1));
    }
  };
  // Numerators 2^s packed to bf16.
  auto numerators = [&](const f32x16 (&sc)[2], bf16x8 (&pd)[2][2]) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        f32x8 e;
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(sc[qb][kk * 8 + j]);
        pd[qb][kk] = __builtin_convertvector(e, bf16x8);
      }
  };
  // Move the reference of query block qb to m_run + rise (rounded so that two bf16 values
  // carry it exactly) and return how far it moved.
  auto move_reference = [&](int qb, float rise) -> float {
    const float want = m_run[qb] + rise;
    const float hi = (float)(__bf16)want;
    const float lo = (float)(__bf16)(want - hi);
    const float d = (hi + lo) - m_run[qb];
    m_run[qb] = hi + lo;
    const bf16x2 pair = {(__bf16)hi, (__bf16)lo};
    qaug_bits[qb][0] = g == 0 ? __builtin_bit_cast(unsigned, pair) : 0u;
    return d;
  };
  // Rare path of a half-step: a numerator of `cur` came out as 2 or more, i.e. a score
  // exceeded the reference by at least 1 (in log2 units; an overflow to infinity included).
  // Nothing has consumed these numerators yet.  Raise the reference to kHeadroom above the row
  // maxima, rescale what is already expressed in the old one (O, the row sums, and the scores
  // of `cur` and of `next`, which the MFMAs of this half-step produced with the old reference)
  // and recompute the numerators, which are then at most 2^-kHeadroom.
  auto raise_reference = [&](f32x16 (&cur)[2], bf16x8 (&pd)[2][2], f32x16 (&next)[2]) {
    float mx[2];
    row_max(cur, mx);
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float d = move_reference(qb, max2(mx[qb] + kHeadroom, 0.f));
      const float alpha = __builtin_amdgcn_exp2f(-d);
      // row sums: lane n < 16 holds query n in element 0 and query n + 16 in element 1
      const float alpha_hi = __builtin_bit_cast(
          float, __builtin_amdgcn_ds_bpermute(4 * ((lane & 15) + 16), __builtin_bit_cast(int, alpha)));
      lacc[qb][0] *= alpha;
      lacc[qb][1] *= alpha_hi;
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        cur[qb][i] -= d;
        next[qb][i] -= d;
      }
    }
    numerators(cur, pd);
  };
// One half-step is one basic block of 22 MFMAs, written as 22 slices fenced by
// sched_barrier so that the interleaving is the one spelled out here.  Slice j issues MFMA j
//    0-3   O += V^T P^T, k-step 0 of `prev`        4-7   the same, k-step 1
//    8-11  row sums of `prev` (16x16x32)           12-13 reference step of the next scores
//   14-21  their four K steps
// then its share of the vector work on `cur` (two exp2 each in slices 0-15, the bf16 packing
// one slice later, then the OR of the packed words whose exponent bits tell whether any
// numerator reached 2) and the LDS reads of operands a few slices ahead of their MFMA.
//   cur/pd    scores of this half and where its numerators go
//   prev      numerators of the previous half; their V rows: k-step 0 already in vnext,
//             k-step 1 = k-step ks_pv of the V tile in stage st_pv
//   next      scores of the next half: K tile in stage st_qk, half h_qk, nv_qk valid tokens left
//   st_vn, ks_vn   V tile / k-step whose V^T goes to vnext for the following half-step
#define LBM_SLICE(j, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)           \
  {                                                                                              \
    /* ---- the MFMA of this slice */                                                            \
    if ((j) < 4)                                                                                 \
      o[(j) & 1][(j) >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                            \
          vnext[(j) >> 1], prev[(j) & 1][0], o[(j) & 1][(j) >> 1], 0, 0, 0);                     \
    else if ((j) < 8)                                                                            \
      o[(j) & 1][((j) - 4) >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                      \
          va[((j) - 4) >> 1], prev[(j) & 1][1], o[(j) & 1][((j) - 4) >> 1], 0, 0, 0);            \
    else if ((j) < 12)                                                                           \
      lacc[(j) & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(                                   \
          lsel, prev[(j) & 1][((j) - 8) >> 1], lacc[(j) & 1], 0, 0, 0);                          \
    else if ((j) < 14)                                                                           \
      next[(j) & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                                   \
          kaug, __builtin_bit_cast(bf16x8, qaug_bits[(j) & 1]), zero16, 0, 0, 0);                \
    else                                                                                         \
      next[(j) & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                                   \
          ka[((j) - 14) >> 1], qf[(j) & 1][((j) - 14) >> 1], next[(j) & 1], 0, 0, 0);            \
    /* ---- numerators of cur: exp2 of scores 2j, 2j+1; packing of the pair of slice j-1 */      \
    if ((j) < 16) {                                                                              \
      e[2 * (j)] = __builtin_amdgcn_exp2f(cur[(j) >> 3][(2 * (j)) & 15]);                        \
      e[2 * (j) + 1] = __builtin_amdgcn_exp2f(cur[(j) >> 3][(2 * (j) + 1) & 15]);                \
    }                                                                                            \
    if ((j) >= 1 && (j) <= 16) {                                                                 \
      constexpr int c = (j) - 1, ci = (2 * c) & 15;                                              \
      pd[c >> 3][ci >> 3][ci & 7] = (__bf16)e[2 * c];                                            \
      pd[c >> 3][ci >> 3][(ci & 7) + 1] = (__bf16)e[2 * c + 1];                                  \
    }                                                                                            \
    /* ---- OR of the packed numerators, one 4-word group per two slices once it is complete */  \
    if ((j) >= 5 && (j) <= 18 && (((j) - 5) & 3) < 2) {                                          \
      constexpr int grp = ((j) - 5) >> 2, w = (((j) - 5) & 3) * 2;                               \
      const u32x4 words = __builtin_bit_cast(u32x4, pd[grp >> 1][grp & 1]);                      \
      chk = ((j) == 5 ? 0u : chk) | words[w] | words[w + 1];                                     \
    }                                                                                            \
    /* ---- LDS reads */                                                                         \
    if ((j) == 0) va[0] = v_frag(st_pv, ks_pv, 0);                                               \
    if ((j) == 1) va[1] = v_frag(st_pv, ks_pv, 1);                                               \
    if ((j) == 10 || (j) == 12 || (j) == 14 || (j) == 16)                                        \
      ka[((j) - 10) >> 1] = __builtin_bit_cast(                                                  \
          bf16x8, *(const u32x4*)&lds_k[st_qk][((h_qk) * 32 + n32) * kRingRow + (((((j) - 10) >> 1) * 2 + g) ^ ((n32 >> 1) & 7)) * 8]); \
    if ((j) == 17) vnext[0] = v_frag(st_vn, ks_vn, 0);                                           \
    if ((j) == 18) vnext[1] = v_frag(st_vn, ks_vn, 1);                                           \
    hook(j)                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                           \
  }
#define LBM_S4(j, ...) LBM_SLICE(j, __VA_ARGS__) LBM_SLICE(j + 1, __VA_ARGS__) LBM_SLICE(j + 2, __VA_ARGS__) LBM_SLICE(j + 3, __VA_ARGS__)
// `hot` tells whether a numerator of `cur` reached 2 (bf16 exponent field >= 128)
#define LBM_HALF_STEP(cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, nv_qk, st_vn, ks_vn, hot, hook) \
  {                                                                                              \
    u32x4 kb = kaug_bits;                                                                        \
    kb[1] = (g == 0 && (h_qk) * 32 + n32 >= (nv_qk)) ? 0xBF80u : 0u;                             \
    const bf16x8 kaug = __builtin_bit_cast(bf16x8, kb);                                          \
    bf16x8 va[2], ka[4];                                                                         \
    float e[32];                                                                                 \
    unsigned chk;                                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                           \
    LBM_S4(0, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                       \
    LBM_S4(4, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                       \
    LBM_S4(8, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                       \
    LBM_S4(12, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                      \
    LBM_S4(16, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                      \
    LBM_SLICE(20, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                   \
    LBM_SLICE(21, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                   \
    /* the numerators exist before the test that follows, not only on its common branch */       \
    asm volatile("" : "+v"(pd[0][0]), "+v"(pd[0][1]), "+v"(pd[1][0]), "+v"(pd[1][1]));             \
    hot = (chk & 0x40004000u) != 0u;                                                             \
  }
// The same half-step without a softmax reference (scores go to exp2 as they come out of the
// QK^T product) and without the test: 20 slices, QK^T in slices 12-19 with its first k-step
// starting from zero.  Only for half-steps whose 32 KV rows are all valid tokens.
#define LBM_FSLICE(j, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)          \
  {                                                                                              \
    if ((j) < 4)                                                                                 \
      o[(j) & 1][(j) >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                            \
          vnext[(j) >> 1], prev[(j) & 1][0], o[(j) & 1][(j) >> 1], 0, 0, 0);                     \
    else if ((j) < 8)                                                                            \
      o[(j) & 1][((j) - 4) >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                      \
          va[((j) - 4) >> 1], prev[(j) & 1][1], o[(j) & 1][((j) - 4) >> 1], 0, 0, 0);            \
    else if ((j) < 12)                                                                           \
      lacc[(j) & 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(                                   \
          lsel, prev[(j) & 1][((j) - 8) >> 1], lacc[(j) & 1], 0, 0, 0);                          \
    else if ((j) < 14)                                                                           \
      next[(j) & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[0], qf[(j) & 1][0], zero16, 0, 0, 0); \
    else                                                                                         \
      next[(j) & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(                                   \
          ka[((j) - 12) >> 1], qf[(j) & 1][((j) - 12) >> 1], next[(j) & 1], 0, 0, 0);            \
    if ((j) < 16) {                                                                              \
      e[2 * (j)] = __builtin_amdgcn_exp2f(cur[(j) >> 3][(2 * (j)) & 15]);                        \
      e[2 * (j) + 1] = __builtin_amdgcn_exp2f(cur[(j) >> 3][(2 * (j) + 1) & 15]);                \
    }                                                                                            \
    if ((j) >= 1 && (j) <= 16) {                                                                 \
      constexpr int c = (j) - 1, ci = (2 * c) & 15;                                              \
      pd[c >> 3][ci >> 3][ci & 7] = (__bf16)e[2 * c];                                            \
      pd[c >> 3][ci >> 3][(ci & 7) + 1] = (__bf16)e[2 * c + 1];                                  \
    }                                                                                            \
    if ((j) == 0) va[0] = v_frag(st_pv, ks_pv, 0);                                               \
    if ((j) == 1) va[1] = v_frag(st_pv, ks_pv, 1);                                               \
    if ((j) == 8 || (j) == 10 || (j) == 12 || (j) == 14)                                         \
      ka[((j) - 8) >> 1] = __builtin_bit_cast(                                                   \
          bf16x8, *(const u32x4*)&lds_k[st_qk][((h_qk) * 32 + n32) * kRingRow + (((((j) - 8) >> 1) * 2 + g) ^ ((n32 >> 1) & 7)) * 8]); \
    if ((j) == 16) vnext[0] = v_frag(st_vn, ks_vn, 0);                                           \
    if ((j) == 17) vnext[1] = v_frag(st_vn, ks_vn, 1);                                           \
    hook(j)                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                           \
  }
#define LBM_F4(j, ...) LBM_FSLICE(j, __VA_ARGS__) LBM_FSLICE(j + 1, __VA_ARGS__) LBM_FSLICE(j + 2, __VA_ARGS__) LBM_FSLICE(j + 3, __VA_ARGS__)
#define LBM_FAST_HALF_STEP(cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)     \
  {                                                                                              \
    bf16x8 va[2], ka[4];                                                                         \
    float e[32];                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                           \
    LBM_F4(0, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                       \
    LBM_F4(4, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                       \
    LBM_F4(8, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                       \
    LBM_F4(12, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                      \
    LBM_F4(16, cur, pd, prev, next, st_pv, ks_pv, st_qk, h_qk, st_vn, ks_vn, hook)                      \
  }
  f32x16 zero16;
#pragma unroll
  for (int i = 0; i < 16; ++i) zero16[i] = 0.f;

  // Iterations [0, n_fast) of this split see only complete 32-token halves (their own second
  // half and the first half of the tile after them) and take the half-step without reference;
  // the iterations around the ragged end of the KV list take the one with the masking k-step.
  const int n_fast = min(max((kv_tokens - 96) / kKvTile - t0 + (kv_tokens >= 96 ? 1 : 0), 0), n);

  // Two passes at most.  The first one uses no softmax reference at all: the numerators are
  // 2^score, which is exact softmax arithmetic as long as nothing leaves the range of fp32 /
  // bf16 (both carry 8 exponent bits and the relative precision does not depend on the
  // magnitude).  Scores in log2 units beyond about +-100 - unheard of behind a q/k LayerNorm -
  // make a row sum or an output overflow or vanish; the check after the pass sees that and the
  // whole workgroup repeats its split with a reference that follows the row maxima (pass 1).
  {
    constexpr bool safe = SAFE;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
      lacc[qb] = f32x4{0.f, 0.f, 0.f, 0.f};
      m_run[qb] = 0.f;
      qaug_bits[qb][0] = 0u;
    }

    // ---- prologue: K(0), K(1), V(0) are on their way into the ring; the V stage the first PV
    // reads is zeroed
    *(u32x4*)&lds_v[2][tid * 8] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) pB[qb][kk] = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
    LBM_DMA_LANDED();
    __syncthreads();
    qk_half(0, 0, kv_tokens - t0 * kKvTile, sA);
    if (safe) {
      // the reference starts kHeadroom above the maxima of the first half
      float mx[2];
      row_max(sA, mx);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const float d = move_reference(qb, mx[qb] + kHeadroom);
#pragma unroll
        for (int i = 0; i < 16; ++i) sA[qb][i] -= d;
      }
    }
    vnext[0] = v_frag(2, 2, 0);
    vnext[1] = v_frag(2, 2, 1);

    int st_k = 0, st_v = 0, st_vm1 = 2;  // stages of K(i), V(i), V(i-1)
    // Common frame of one tile iteration.  The loads of K(i+2) and V(i+1) into their ring
    // stages (free since the barrier that ended iteration i-1) and the fetch of the next row
    // entry are issued from inside the first half-step's slices (LBM_STAGING_HOOK), not in front
    // of it: after the barrier every wavefront goes straight to matrix instructions whose
    // operands it already holds, and the address arithmetic of the staging shares slices with
    // them instead of leaving the matrix pipe idle on all four SIMDs at once.  The loads have
    // the rest of the iteration to land; the wait for them sits right before the barrier that
    // ends it.  Past the last tile the data lands in stages nobody reads any more.  The row
    // entry fetched for K now serves V in the next iteration.
#define LBM_NO_HOOK(j)
#define LBM_STAGING_HOOK(j)                                                          \
    if ((j) == 1) dma(ek, pool_k, own_k, lds_k[st_k2]);                              \
    if ((j) == 2) dma(ev, pool_v, own_v, lds_v[st_v1]);                              \
    if ((j) == 3) {                                                                  \
      ev = ek;                                                                       \
      ek = row_entry(t + 3);                                                         \
    }
#define LBM_TILE_ITERATION(PRE, HALF0, HALF1)                                        \
    {                                                                                \
      const int t = t0 + i;                                                          \
      int st_k1 = st_k + 1; if (st_k1 >= kStages) st_k1 -= kStages;                  \
      int st_k2 = st_k1 + 1; if (st_k2 >= kStages) st_k2 -= kStages;                 \
      int st_v1 = st_v + 1; if (st_v1 >= kStages) st_v1 -= kStages;                  \
      PRE                                                                            \
      HALF0                                                                          \
      HALF1                                                                          \
      LBM_DMA_LANDED();                                                              \
      __syncthreads();                                                               \
      st_k = st_k1;                                                                  \
      st_vm1 = st_v;                                                                 \
      st_v = st_v1;                                                                  \
    }
    // The same frame with the ring stages as compile-time constants (the ring has three stages,
    // so three iterations bring it back to where it started): every LDS address of the
    // iteration is then one per-lane register plus an immediate offset, and the thirty-odd vector
    // and scalar instructions per tile that add a run-time stage base to it are gone.
#define LBM_TILE_ITERATION_AT(U, SK, HALF0, HALF1)                                   \
    {                                                                                \
      const int t = t0 + i + (U);                                                    \
      constexpr int st_k = (SK), st_v = (SK), st_vm1 = ((SK) + 2) % kStages;          \
      constexpr int st_k1 = ((SK) + 1) % kStages, st_k2 = ((SK) + 2) % kStages;       \
      constexpr int st_v1 = ((SK) + 1) % kStages;                                    \
      HALF0                                                                          \
      HALF1                                                                          \
      LBM_DMA_LANDED();                                                              \
      __syncthreads();                                                               \
    }
    int i = 0;
    // half 0 of tile i: softmax(sA) -> pA | PV(tile i-1, half 1) with pB | QK(tile i, half 1) -> sB
    // half 1 of tile i: softmax(sB) -> pB | PV(tile i, half 0) with pA | QK(tile i+1, half 0) -> sA
    const int n_f = safe ? 0 : n_fast;
#define LBM_FAST_ITERATION_AT(U, SK)                                                              \
      LBM_TILE_ITERATION_AT(U, SK,                                                                 \
        LBM_FAST_HALF_STEP(sA, pA, pB, sB, st_vm1, 3, st_k, 1, st_v, 0, LBM_STAGING_HOOK);,        \
        LBM_FAST_HALF_STEP(sB, pB, pA, sA, st_v, 1, st_k1, 0, st_v, 2, LBM_NO_HOOK);)
    for (; i + kStages <= n_f; i += kStages) {   // (entered with st_k = st_v = 0, st_vm1 = 2, and left so)
      LBM_FAST_ITERATION_AT(0, 0)
      LBM_FAST_ITERATION_AT(1, 1)
      LBM_FAST_ITERATION_AT(2, 2)
    }
#undef LBM_FAST_ITERATION_AT
#undef LBM_TILE_ITERATION_AT
    for (; i < n_f; ++i)
      LBM_TILE_ITERATION(
        ,
        LBM_FAST_HALF_STEP(sA, pA, pB, sB, st_vm1, 3, st_k, 1, st_v, 0, LBM_STAGING_HOOK);,
        LBM_FAST_HALF_STEP(sB, pB, pA, sA, st_v, 1, st_k1, 0, st_v, 2, LBM_NO_HOOK);
      )
    for (; i < n; ++i)
      LBM_TILE_ITERATION(
        const int n_valid = kv_tokens - t * kKvTile;
        bool hot;,
        LBM_HALF_STEP(sA, pA, pB, sB, st_vm1, 3, st_k, 1, n_valid, st_v, 0, hot, LBM_STAGING_HOOK);
        if (safe && __builtin_amdgcn_ballot_w64(hot)) raise_reference(sA, pA, sB);,
        /* after the last tile this QK reads a stale stage; its result is unused */
        LBM_HALF_STEP(sB, pB, pA, sA, st_v, 1, st_k1, 0, n_valid - kKvTile, st_v, 2, hot, LBM_NO_HOOK);
        if (safe && __builtin_amdgcn_ballot_w64(hot)) raise_reference(sB, pB, sA);
      )
#undef LBM_TILE_ITERATION
#undef LBM_STAGING_HOOK
#undef LBM_NO_HOOK
    // PV and row sums of the last half: pB with half 1 of V(n-1), first k-step already in vnext
    {
      pv_step(vnext, pB, 0);
      bf16x8 va[2] = {v_frag(st_vm1, 3, 0), v_frag(st_vm1, 3, 1)};
      pv_step(va, pB, 1);
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
          lacc[qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lsel, pB[qb][kk], lacc[qb], 0, 0, 0);
    }
    // Did the pass without reference stay in range?  Compared as integers (non-negative floats
    // order like their bit patterns; NaN, infinity and negative values land above every bound).
    bool bad = false;
    if (!safe && n > 0) {
      unsigned top = 0u;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) top = max(top, __builtin_bit_cast(unsigned, o[qb][db][i]) & 0x7FFFFFFFu);
      bad = top >= 0x7F800000u;
      if (lane < 16) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int h2 = 0; h2 < 2; ++h2) {
            const unsigned lb = __builtin_bit_cast(unsigned, lacc[qb][h2]);
            bad = bad || lb < 0x12800000u /* 2^-90 */ || lb > 0x71800000u /* 2^100 */;
          }
      }
    }
    if (!safe && __builtin_amdgcn_readfirstlane(__syncthreads_or(bad))) {
      lbm_attn_split_safe(a, sp);
      __builtin_amdgcn_endpgm();
    }
  }
#undef LBM_FAST_HALF_STEP
#undef LBM_F4
#undef LBM_FSLICE
#undef LBM_HALF_STEP
#undef LBM_S4
#undef LBM_SLICE

  // ---- epilogue.  The accumulators hold O^T (a lane owns 4-element runs of 32 different
  // rows); written straight out that is 32 scattered 8-byte stores per instruction.  Each
  // wavefront instead transposes its rows through its Q patch (idle since the prologue) and
  // stores whole 128-byte rows, eight lanes per row.
  unsigned short* stage = lds_q[wave];
  const bool direct = sp.n_splits == 1;
  unsigned short* dst = direct ? a.out : a.part_o;
  const size_t dst_row0 = direct ? (size_t)sp.q_begin : (size_t)sp.part_begin + (size_t)split * sp.q_rows;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    // the row sum of query n32 of this block sits in lane n32 % 16, element n32 / 16
    // (the two elements go through an opaque asm: fed two elements of one vector, the compiler
    // folds the select below into the permute's data operand, which picks by the wrong lane)
    float sum_lo = lacc[qb][0], sum_hi = lacc[qb][1];
    asm volatile("" : "+v"(sum_lo), "+v"(sum_hi));
    const float l_lo = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(4 * (lane & 15), __builtin_bit_cast(int, sum_lo)));
    const float l_hi = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(4 * (lane & 15), __builtin_bit_cast(int, sum_hi)));
    const float l_tot = (n32 & 16) ? l_hi : l_lo;
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        f32x4 w;
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = o[qb][db][c4 * 4 + e] * inv;
        *(bf16x4*)&stage[n32 * kKStride + db * 32 + c4 * 8 + g * 4] = __builtin_convertvector(w, bf16x4);
      }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int row = k * 8 + (lane >> 3);
      const u32x4 v = *(const u32x4*)&stage[row * kKStride + (lane & 7) * 8];
      const int r = q_row0 + qb * 32 + row;
      if (r < sp.q_rows) *(u32x4*)(dst + ((dst_row0 + r) * H + head) * 64 + (lane & 7) * 8) = v;
    }
    const int r = q_row0 + qb * 32 + n32;
    if (!direct && g == 0 && r < sp.q_rows)
      a.part_lse[(dst_row0 + r) * H + head] = m_run[qb] + __builtin_amdgcn_logf(l_tot);
  }
}

__device__ __noinline__ void lbm_attn_split_safe(AttnCore a, LbmAttnStreamPlan sp) { lbm_attn_split<true>(a, sp); }

}  // namespace

__global__ __launch_bounds__(kThreads, 1) void lbm_attn_bf16_d64_kernel(AttnArgs a) {
  int b = 0;   // which stream's work is this workgroup
  for (int i = 1; i < a.sch.n_streams; ++i)
    if ((int)blockIdx.x >= a.sch.s[i].wg_begin) b = i;
  const LbmAttnStreamPlan sp = a.sch.s[b];
  lbm_attn_split<false>(a, sp);
}

// ---------------------------------------------------------------------------- bf16, short KV
// Streams with at most kSmMaxKv KV tokens - the frame blocks' attention of a frame over itself
// (lingbot_map/layers/block.py:27-101: 1004 x 1004 tokens), the first frames of a stream - have
// too few KV tiles to amortise the split-KV machinery above (a workgroup per (512 rows, head,
// split) with a prologue of several tile-times, partial results through HBM and a second
// kernel).  Here one 8-wave workgroup owns 64 query rows of one head and the KV axis is split
// INSIDE it: wavefront w walks its own eighth of the KV axis in 32-token pieces with its own
// K/V patch in LDS (rows loaded as whole 128-byte lines, eight lanes per row, one piece ahead in
// registers), two wavefronts per SIMD covering each other's waits, and the eight partial
// results are summed through LDS at the end.  No workspace, no second kernel.  Same arithmetic
// as the main kernel's first pass: scores straight into exp2 without a reference, a range
// check at the end, and - only if that fails - a second pass with the textbook running-maximum
// recurrence.
namespace {
constexpr int kSmWaves = 8;
constexpr int kSmThreads = kSmWaves * 64;
constexpr int kSmMaxKv = 4096;
constexpr int kSmPiece = 32;     // KV tokens per step of a wavefront
constexpr int kSmOStride = 68;   // floats per row of a partial output parked in LDS (4-bank shift per row)
constexpr int kSmPatchBytes = kSmPiece * (kKStride + kVStride) * 2;             // one wave's K and V piece
constexpr int kSmMergeBytes = kSmWaves * (kQPerWave * kSmOStride + 2 * kQPerWave) * 4;
constexpr int kSmQBytes = kQPerWave * kKStride * 2;                              // Q on its way to the fragments
constexpr int kSmLdsBytes = kSmMergeBytes > kSmWaves * kSmPatchBytes ? kSmMergeBytes : kSmWaves * kSmPatchBytes;
static_assert(kSmLdsBytes >= kSmQBytes && kSmLdsBytes <= 160 * 1024, "LDS budget of the short-KV kernel");
}  // namespace

__global__ __launch_bounds__(kSmThreads, 1) void lbm_attn_bf16_d64_small_kernel(AttnArgs a) {
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kSmLdsBytes];
  // (the wavefront index is uniform by construction; said so, or the loop over this wavefront's
  // pieces is compiled as divergent control flow)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n32 = lane & 31, g = lane >> 5;
  unsigned short* patch_k = (unsigned short*)(lds_raw + wave * kSmPatchBytes);
  unsigned short* patch_v = patch_k + kSmPiece * kKStride;

  // ---- which (stream, 64 query rows, head)
  int b = 0;
  for (int i = 1; i < a.sch.n_streams; ++i)
    if ((int)blockIdx.x >= a.sch.s[i].wg_begin) b = i;
  const LbmAttnStreamPlan sp = a.sch.s[b];
  const int H = a.num_heads;
  const int local = (int)blockIdx.x - sp.wg_begin;
  int qb64, head;
  if ((H & 7) == 0) {   // the query blocks of one head on one XCD (blockIdx mod 8): its L2 serves their K/V
    const int x = local & 7, i = local >> 3;
    head = (i % (H >> 3)) * 8 + x;
    qb64 = i / (H >> 3);
  } else {
    head = local % H;
    qb64 = local / H;
  }
  if (qb64 >= sp.n_qtiles) return;   // padding between streams (whole workgroups)
  const int kv_tokens = max(a.live_kv_tokens ? a.live_kv_tokens[sp.live_at] : sp.kv_tokens, 0);
  const int n_pieces = (kv_tokens + kSmPiece - 1) / kSmPiece;
  const int pps = (n_pieces + kSmWaves - 1) / kSmWaves;
  const int p0 = wave * pps, p1 = min(p0 + pps, n_pieces);   // this wavefront's pieces (possibly none)
  const unsigned row_bytes = (unsigned)H * 128u;
  const int q_row0 = qb64 * kQPerWave;
  if (n_pieces == 0) {
    // nothing visible: the reference returns zeros (lingbot_map/layers/flashinfer_cache.py:368-370).
    // Decided before the first load, so that every load below is unconditional.
    const int r = q_row0 + (tid >> 3);
    if (r < sp.q_rows)
      *(u32x4*)(a.out + ((size_t)(sp.q_begin + r) * H + head) * 64 + (tid & 7) * 8) = u32x4{0u, 0u, 0u, 0u};
    return;
  }

  // ---- K/V rows of a piece: lane l takes the 16-byte part (l & 7) of rows (l >> 3) + 8 j
  const char* pool_k = (const char*)(a.pool + (size_t)head * 64 + (lane & 7) * 8);
  const char* pool_v = pool_k + (size_t)a.page_size * row_bytes;
  const char* own_k = (const char*)(a.self_k + (size_t)head * 64 + (lane & 7) * 8);
  const char* own_v = (const char*)(a.self_v + (size_t)head * 64 + (lane & 7) * 8);
  const int32_t* rows = a.kv_rows + sp.kv_row_begin;
  const int last_token = max(kv_tokens - 1, 0);
  auto fetch = [&](int e, const char* pool_base, const char* own_base) -> u32x4 {
    const char* base = e < 0 ? own_base : pool_base;
    const unsigned r = (unsigned)(e ^ (e >> 31));
    return *(const u32x4*)(base + (unsigned long long)r * row_bytes);
  };
  constexpr int kRowsPerPass = 8, kPasses = kSmPiece / kRowsPerPass;
  // rows past the last token re-read the last token: finite data, masked below
  auto load_piece = [&](int pc, u32x4 (&kk)[kPasses], u32x4 (&vv)[kPasses]) {
    const int mine = rows[min(pc * kSmPiece + n32, last_token)];   // lanes l and l + 32: the entry of the piece's row l
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
      const int e = __builtin_amdgcn_ds_bpermute(4 * (j * kRowsPerPass + (lane >> 3)), mine);
      kk[j] = fetch(e, pool_k, own_k);
      vv[j] = fetch(e, pool_v, own_v);
    }
  };
  // Loads in the order their data is needed and their chains are long: this thread's piece of a
  // Q row first (the load counter retires in order, so the wait for it must not sit behind the
  // K/V rows), then the first piece's row entries and, once those are back, its K/V rows.
  const int q_r = max(min(q_row0 + (tid >> 3), sp.q_rows - 1), 0);   // rows past the last one re-read it (never stored)
  const u32x4 q_raw = *(const u32x4*)(a.q + ((size_t)(sp.q_begin + q_r) * H + head) * 64 + (tid & 7) * 8);
  // (a wavefront without pieces loads the last piece and drops it: a load inside a conditional
  // block would make the wait for the Q row a wait for everything in flight)
  u32x4 kk[kPasses], vv[kPasses];
  load_piece(min(p0, n_pieces - 1), kk, vv);

  // ---- Q: the workgroup reads the 64 rows once as whole rows, every wavefront picks its
  // fragments up from LDS; scale * log2(e) folded in (as in the main kernel)
  bf16x8 qf[2][4];
  {
    unsigned short* patch_q = (unsigned short*)lds_raw;
    *(u32x4*)&patch_q[(tid >> 3) * kKStride + (tid & 7) * 8] = q_raw;
    __syncthreads();
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 rawf = __builtin_bit_cast(bf16x8, *(const u32x4*)&patch_q[(qb * 32 + n32) * kKStride + ks * 16 + g * 8]);
        f32x8 f = __builtin_convertvector(rawf, f32x8);
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] *= a.scale_log2;
        qf[qb][ks] = __builtin_convertvector(f, bf16x8);
      }
    __syncthreads();   // the patches below overlay the Q rows
  }

  auto store_piece = [&](const u32x4 (&kk)[kPasses], const u32x4 (&vv)[kPasses]) {
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
      *(u32x4*)&patch_k[(j * kRowsPerPass + (lane >> 3)) * kKStride + (lane & 7) * 8] = kk[j];
      *(u32x4*)&patch_v[(j * kRowsPerPass + (lane >> 3)) * kVStride + (lane & 7) * 8] = vv[j];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };
  auto v_frag = [&](int ks, int db) -> bf16x8 {   // as in the main kernel, on this wave's patch
    const int row = ks * 16 + 4 * g + ((lane & 15) >> 2);
    const int col = db * 32 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (s16x4 __attribute__((address_space(3)))*)&patch_v[row * kVStride + col]);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (s16x4 __attribute__((address_space(3)))*)&patch_v[(row + 8) * kVStride + col]);
    s16x8 both;
    both[0] = lo[0]; both[1] = lo[1]; both[2] = lo[2]; both[3] = lo[3];
    both[4] = hi[0]; both[5] = hi[1]; both[6] = hi[2]; both[7] = hi[3];
    return __builtin_bit_cast(bf16x8, both);
  };

  f32x16 o[2][2];
  f32x4 lacc[2];                 // first pass: row sums on the matrix pipe (layout as in the main kernel)
  float m_run[2], l_lane[2];     // second pass: running maximum of the row, this lane's share of its sum
  const unsigned sel_word = (lane == 0 || lane == 32 || lane == 17 || lane == 49) ? 0x3F803F80u : 0u;
  const bf16x8 lsel = __builtin_bit_cast(bf16x8, u32x4{sel_word, sel_word, sel_word, sel_word});
  f32x16 zero16;
#pragma unroll
  for (int i = 0; i < 16; ++i) zero16[i] = 0.f;

  bool safe = false;
  for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
      for (int db = 0; db < 2; ++db) o[qb][db] = zero16;
      lacc[qb] = f32x4{0.f, 0.f, 0.f, 0.f};
      m_run[qb] = safe ? -INFINITY : 0.f;
      l_lane[qb] = 0.f;
    }
    if (pass > 0 && p0 < p1) load_piece(p0, kk, vv);   // (the first pass's first piece is already on its way)
    for (int pc = p0; pc < p1; ++pc) {
      store_piece(kk, vv);
      if (pc + 1 < p1) load_piece(pc + 1, kk, vv);   // in flight while this piece is computed
      const int n_valid = kv_tokens - pc * kSmPiece;
      // S^T = K Q^T for the piece's 32 kv rows: sc[qb][i] is kv = 8 (i / 4) + 4 g + i % 4, q = 32 qb + n32
      f32x16 sc[2] = {zero16, zero16};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 ka = __builtin_bit_cast(bf16x8, *(const u32x4*)&patch_k[n32 * kKStride + ks * 16 + g * 8]);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) sc[qb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[qb][ks], sc[qb], 0, 0, 0);
      }
      const bf16x8 va0[2] = {v_frag(0, 0), v_frag(0, 1)};   // requested early: they arrive under the exp2 work
      const bf16x8 va1[2] = {v_frag(1, 0), v_frag(1, 1)};
      if (n_valid < kSmPiece) {   // the ragged last piece of the stream
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (8 * (i >> 2) + 4 * g + (i & 3) >= n_valid) sc[qb][i] = -INFINITY;
      }
      bf16x8 p[2][2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        if (safe) {
          float mx = max3(sc[qb][0], sc[qb][1], sc[qb][2]);
#pragma unroll
          for (int i = 3; i < 15; i += 2) mx = max3(mx, sc[qb][i], sc[qb][i + 1]);
          mx = swap_max(max2(mx, sc[qb][15]));
          const float m_new = max2(m_run[qb], mx);     // finite: the first row of a piece is a token
          const float alpha = __builtin_amdgcn_exp2f(m_run[qb] - m_new);   // 0 on the first piece
          m_run[qb] = m_new;
          l_lane[qb] *= alpha;
#pragma unroll
          for (int db = 0; db < 2; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha;
#pragma unroll
          for (int i = 0; i < 16; ++i) sc[qb][i] -= m_new;
        }
#pragma unroll
        for (int kk2 = 0; kk2 < 2; ++kk2) {
          f32x8 e;
#pragma unroll
          for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(sc[qb][kk2 * 8 + j]);
          p[qb][kk2] = __builtin_convertvector(e, bf16x8);
          if (safe) {
#pragma unroll
            for (int j = 0; j < 8; ++j) l_lane[qb] += e[j];
          } else {
            lacc[qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lsel, p[qb][kk2], lacc[qb], 0, 0, 0);
          }
        }
      }
      // O^T += V^T P^T over the piece's two 16-row k-steps
#pragma unroll
      for (int db = 0; db < 2; ++db)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va0[db], p[qb][0], o[qb][db], 0, 0, 0);
          o[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va1[db], p[qb][1], o[qb][db], 0, 0, 0);
        }
    }
    if (safe) break;
    // range check of the pass without reference (integer compares, see the main kernel)
    bool bad = false;
    if (p0 < p1) {
      unsigned top = 0u;
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
          for (int i = 0; i < 16; ++i) top = max(top, __builtin_bit_cast(unsigned, o[qb][db][i]) & 0x7FFFFFFFu);
      bad = top >= 0x7F800000u;
      if (lane < 16) {
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int h2 = 0; h2 < 2; ++h2) {
            const unsigned lb = __builtin_bit_cast(unsigned, lacc[qb][h2]);
            bad = bad || lb < 0x12800000u /* 2^-90 */ || lb > 0x71800000u /* 2^100 */;
          }
      }
    }
    if (!__syncthreads_or(bad)) break;
    safe = true;
  }

  // ---- merge the wavefronts' partial results through LDS (the patches are dead)
  __syncthreads();
  float* so = (float*)lds_raw + wave * (kQPerWave * kSmOStride);
  float* sl = (float*)lds_raw + kSmWaves * (kQPerWave * kSmOStride);   // [wave][64] row sums, then [wave][64] references
  float* sm = sl + kSmWaves * kQPerWave;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
    for (int db = 0; db < 2; ++db)
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4)
        *(f32x4*)&so[(qb * 32 + n32) * kSmOStride + db * 32 + c4 * 8 + g * 4] =
            f32x4{o[qb][db][c4 * 4], o[qb][db][c4 * 4 + 1], o[qb][db][c4 * 4 + 2], o[qb][db][c4 * 4 + 3]};
    if (safe) {
      float lo, hi;
      swap_halves(l_lane[qb], lo, hi);
      if (g == 0) sl[wave * kQPerWave + qb * 32 + n32] = lo + hi;
    } else if (lane < 16) {
      sl[wave * kQPerWave + qb * 32 + lane] = lacc[qb][0];
      sl[wave * kQPerWave + qb * 32 + 16 + lane] = lacc[qb][1];
    }
    if (g == 0) sm[wave * kQPerWave + qb * 32 + n32] = (p0 < p1) ? m_run[qb] : -INFINITY;
  }
  __syncthreads();
  {
    // wavefront w finishes rows 8 w .. 8 w + 7: eight lanes per row, 8 head dims (16 bytes) each
    const int row = wave * (kQPerWave / kSmWaves) + (lane >> 3), d0 = (lane & 7) * 8;
    float mw[kSmWaves], mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < kSmWaves; ++w) {
      mw[w] = sm[w * kQPerWave + row];
      mx = max2(mx, mw[w]);
    }
    f32x8 acc;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    float l_tot = 0.f;
#pragma unroll
    for (int w = 0; w < kSmWaves; ++w) {
      // a wavefront without pieces (reference -inf) weighs nothing; with a common reference the weights are 1
      const float wgt = mw[w] > -INFINITY ? __builtin_amdgcn_exp2f(mw[w] - mx) : 0.f;
      l_tot += wgt * sl[w * kQPerWave + row];
      const float* src = (const float*)lds_raw + w * (kQPerWave * kSmOStride) + row * kSmOStride + d0;
      const f32x4 x0 = *(const f32x4*)src, x1 = *(const f32x4*)(src + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[e] += wgt * x0[e];
        acc[4 + e] += wgt * x1[e];
      }
    }
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;   // nothing visible: zeros (flashinfer_cache.py:368-370)
    const int r = q_row0 + row;
    if (r < sp.q_rows) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] *= inv;
      *(bf16x8*)(a.out + ((size_t)(sp.q_begin + r) * H + head) * 64 + d0) = __builtin_convertvector(acc, bf16x8);
    }
  }
}

// Merge split-KV partial results: out = sum_s w_s * o_s with w_s = 2^(lse_s - max) / sum.
// One thread per (query row, head, 8 consecutive d).
//
// Up to NJ splits (n <= NJ): all 2 NJ loads - the log-sum-exps and the partial rows - are issued
// before the first use of any of them, one round trip of memory latency instead of three.  NJ is
// the next of 2, 4, 8 above the split count, so that a launch with two splits (several streams'
// frame blocks) does not load its last split seven times over.
template <int NJ>
__device__ __forceinline__ void lbm_combine_upto(const float* lse, const unsigned short* po, long long split_stride, int n,
                                                 float& wsum, f32x8& acc) {
  float t[NJ];
  bf16x8 v[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const long long s = min(j, n - 1);
    t[j] = lse[s * split_stride];
    v[j] = *(const bf16x8*)(po + s * split_stride * 64);
  }
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < NJ; ++j) mx = fmaxf(mx, t[j]);
  if (mx == -INFINITY) mx = 0.f;  // every split empty (no visible token): weights 0, output 0
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const float w = j < n ? __builtin_amdgcn_exp2f(t[j] - mx) : 0.f;
    const f32x8 vf = __builtin_convertvector(v[j], f32x8);
    wsum += w;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += w * vf[e];
  }
}

__global__ __launch_bounds__(256) void lbm_attn_combine_bf16_kernel(AttnArgs a) {
  if ((int)blockIdx.x >= a.combine_blocks) {
    // The append's share of the launch (lbm_attn_run_append): the main kernel has read the pool,
    // the new frames' rows - attended to from the caller's tensors - now go into their pages.  One
    // 16-byte piece of a K row and of the matching V row per thread, as lbm_kv_append_kernel.
    if (blockIdx.y != 0) return;
    const int pieces = a.num_heads * 8;
    const long long idx = (long long)((int)blockIdx.x - a.combine_blocks) * 256 + threadIdx.x;
    if (idx >= (long long)a.append_tokens * pieces) return;
    const int t = (int)(idx / pieces), piece = (int)(idx % pieces);
    const int row = a.append_rows[t];
    if (row < 0) return;
    const long long row_elems = (long long)a.num_heads * 64;
    const long long src = t * row_elems + piece * 8, dk = row * row_elems + piece * 8;
    unsigned short* pool = const_cast<unsigned short*>(a.pool);
    const u32x4 kk = *(const u32x4*)(a.self_k + src), vv = *(const u32x4*)(a.self_v + src);
    *(u32x4*)(pool + dk) = kk;
    *(u32x4*)(pool + dk + (long long)a.page_size * row_elems) = vv;
    return;
  }
  const LbmAttnStreamPlan sp = a.sch.s[blockIdx.y];
  if (sp.n_splits <= 1) return;
  const int H = a.num_heads;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)sp.q_rows * H * 8) return;
  const int d8 = (int)(idx & 7);
  const long long rh = idx >> 3;  // r * H + h
  const long long split_stride = (long long)sp.q_rows * H;
  const float* lse = a.part_lse + (long long)sp.part_begin * H + rh;
  const int n = sp.n_splits;
  const unsigned short* po = a.part_o + ((long long)sp.part_begin * H + rh) * 64 + d8 * 8;
  float wsum = 0.f;
  f32x8 acc;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (n <= 2) {
    lbm_combine_upto<2>(lse, po, split_stride, n, wsum, acc);
  } else if (n <= 4) {
    lbm_combine_upto<4>(lse, po, split_stride, n, wsum, acc);
  } else if (n <= 8) {
    lbm_combine_upto<8>(lse, po, split_stride, n, wsum, acc);
  } else {
    // loads are issued in batches (the split count is a run-time value, a plain loop would
    // wait for each load in turn)
    float mx = -INFINITY;
    for (int s0 = 0; s0 < n; s0 += 8) {
      float t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) t[j] = lse[min(s0 + j, n - 1) * split_stride];
#pragma unroll
      for (int j = 0; j < 8; ++j) mx = fmaxf(mx, t[j]);
    }
    if (mx == -INFINITY) mx = 0.f;
    for (int s0 = 0; s0 < n; s0 += 4) {
      float t[4];
      bf16x8 v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const long long s = min(s0 + j, n - 1);
        t[j] = lse[s * split_stride];
        v[j] = *(const bf16x8*)(po + s * split_stride * 64);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float w = s0 + j < n ? __builtin_amdgcn_exp2f(t[j] - mx) : 0.f;
        const f32x8 vf = __builtin_convertvector(v[j], f32x8);
        wsum += w;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += w * vf[e];
      }
    }
  }
  const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
  const long long r = rh / H, h = rh % H;
  unsigned short* op = a.out + ((size_t)(sp.q_begin + r) * H + h) * 64 + d8 * 8;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] *= inv;
  *(bf16x8*)op = __builtin_convertvector(acc, bf16x8);
}

// ---------------------------------------------------------------------------- fp32 path
// Same contract as the bf16 kernel for pools kept in fp32 (the reference's force_fp32 mode,
// lingbot_map/layers/flashinfer_cache.py:118-127,372-383), head_dim 64, and 128 for the camera
// head's one-token-per-frame cache (lingbot_map/heads/camera_head.py:284-377: 16 heads of 128).
// Full fp32 products and sums on the matrix pipe (v_mfma_f32_16x16x4_f32), exact running
// maximum, no split-KV across workgroups.  One workgroup per (64 query rows, head), four waves
// (head_dim 64) or two (128) per 16 query rows.
//
// A lane is (n = lane % 16, g = lane / 16).  Scores are kept transposed, S^T = K Q^T: the
// 16x16x4 product takes K[kv = n][dim k_g] from every lane as A and Q[q = n][dim k_g] as B and
// leaves S^T[kv = 4g + i][q = n] in element i of lane (n, g), so a lane's four elements
// belong to ONE query row and the softmax statistics are per lane plus two cross-lane steps
// over g.  Which head dimension lane group g contributes in step t is free as long as A and B
// agree; dim = (D/4) g + t makes the K operand four consecutive floats per four steps (one
// ds_read_b128) and the Q operand a contiguous quarter row held in registers.  For O^T = V^T P^T
// the same freedom is used on the KV index: step (c, i) contracts kv = 16c + 4g + i over g,
// which is exactly where element i of the score block c already sits - P goes from the
// accumulator into the B operand without a shuffle.  Output block e takes head dimension
// (D/16) n + e from lane n as its A operand (one ds_read_b128 of V per lane and KV row covers
// four blocks), which leaves O^T[dim = (D/16)(4g + i) + e][q = n] in element i of block e:
// consecutive dims across the blocks, 16-byte stores.
namespace {
constexpr int kF32Rows = 64;
struct AttnArgsF32 {
  const float* q;
  const float* pool;
  float* out;
  const float* self_k;
  const float* self_v;
  const int32_t* kv_rows;
  const int32_t* live_kv_tokens;
  int num_heads;
  int page_size;
  float scale_log2;
  int n_streams;
  lbm_attn_stream s[LBM_MAX_STREAMS];
  int wg_begin[LBM_MAX_STREAMS + 1];
};
}  // namespace

// Maximum over the four lanes n, n + 16, n + 32, n + 48 that share a query row, on the vector
// ALU (no LDS round trip): rows of 16 lanes pairwise, then the two halves of the wavefront.
__device__ __forceinline__ float max_over_lane_groups(float x) {
  float a, b;
  swap_rows(x, a, b);
  x = fmaxf(a, b);
  swap_halves(x, a, b);
  return fmaxf(a, b);
}

template <int D>
__global__ __launch_bounds__(D == 64 ? 1024 : 512) void lbm_attn_f32_kernel(AttnArgsF32 a) {
  // NG groups of four waves: wave w of every group owns the same 16 query rows, group j takes
  // KV tiles j, j + NG, ... (NG waves per SIMD, so one wave's softmax, LDS waits and barriers
  // overlap the others' matrix work); the partial results are merged through LDS at the end.
  constexpr int NG = D == 64 ? 4 : 2;          // wave groups = tiles staged per iteration
  constexpr int kThreadsF32 = 256 * NG;
  constexpr int kTile = 16;                    // KV tokens per tile = one 16-token score block
  constexpr int kStage = kTile * D / 256;      // floats of K (and of V) a thread stages per iteration
  constexpr int kRowThreads = D / kStage;      // threads that stage one row
  constexpr int LD = D + 4;                    // LDS row stride: rows stay 16-byte aligned and shift by 4 banks
  constexpr int NE = D / 16;                   // 16-dim output blocks
  constexpr int DG = D / 4;                    // head dims one lane group contributes to q.k
  static_assert(kThreadsF32 / kRowThreads == NG * kTile && kStage % 4 == 0, "the threads stage NG tiles");
  constexpr int kTileFloats = NG * kTile * LD;  // NG tiles of K (and as many again of V)
  constexpr int kMergeFloats = (NE * 4 + 2) * 256 * (NG / 2);
  constexpr int kLdsFloats = 2 * kTileFloats > kMergeFloats ? 2 * kTileFloats : kMergeFloats;
  __shared__ __attribute__((aligned(16))) float lds_raw[kLdsFloats];
  float (*lds_k)[LD] = (float (*)[LD])lds_raw;
  float (*lds_v)[LD] = (float (*)[LD])(lds_raw + kTileFloats);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = (tid >> 6) & 3, grp = tid >> 8;
  const int n16 = lane & 15, g = lane >> 4;
  int b = 0;
  for (int i = 1; i < a.n_streams; ++i)
    if ((int)blockIdx.x >= a.wg_begin[i]) b = i;
  lbm_attn_stream sp = a.s[b];
  if (a.live_kv_tokens) sp.kv_tokens = max(a.live_kv_tokens[sp.live_at], 0);
  const int H = a.num_heads;
  const int local = (int)blockIdx.x - a.wg_begin[b];
  const int head = local % H, qt = local / H;
  const int r = qt * kF32Rows + wave * 16 + n16;   // this lane's query row
  const size_t row_elems = (size_t)H * D;
  const bool row_ok = r < sp.q_rows;

  // Q[r][DG g .. DG g + DG - 1], pre-multiplied by scale * log2(e)
  float q[DG];
  {
    const float* qp = a.q + ((size_t)(sp.q_begin + (row_ok ? r : 0)) * H + head) * D + DG * g;
#pragma unroll
    for (int d4 = 0; d4 < DG / 4; ++d4) {
      const f32x4 x = row_ok ? ((const f32x4*)qp)[d4] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) q[4 * d4 + j] = x[j] * a.scale_log2;
    }
  }
  f32x4 o[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;   // running maximum of the row; this lane's share of the row sum

  const int ld_r = tid / kRowThreads, ld_c = (tid % kRowThreads) * kStage;
  const int n_tiles = (sp.kv_tokens + kTile - 1) / kTile;
  const int n_iters = (n_tiles + NG - 1) / NG;
  // Two-deep prefetch: the row-table entry of iteration it + 2 is requested while iteration it
  // is computed, so the K/V loads of iteration it + 1 can be issued without waiting for it.
  f32x4 kk[kStage / 4], vv[kStage / 4];
  constexpr int kNoRow = INT32_MIN;   // not a row: past the end of the stream's KV
  auto entry = [&](int it) -> int {
    const int kvi = it * NG * kTile + ld_r;
    return kvi < sp.kv_tokens ? a.kv_rows[sp.kv_row_begin + kvi] : kNoRow;
  };
  auto fetch = [&](int e) {
#pragma unroll
    for (int i = 0; i < kStage / 4; ++i) kk[i] = vv[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (e != kNoRow) {
      const float *kp, *vp;
      if (e >= 0) {
        kp = a.pool + ((size_t)e * H + head) * D + ld_c;
        vp = kp + (size_t)a.page_size * row_elems;
      } else {
        const size_t off = ((size_t)(-1 - e) * H + head) * D + ld_c;
        kp = a.self_k + off;
        vp = a.self_v + off;
      }
#pragma unroll
      for (int i = 0; i < kStage / 4; ++i) {
        kk[i] = ((const f32x4*)kp)[i];
        vv[i] = ((const f32x4*)vp)[i];
      }
    }
  };
  int e_next = kNoRow;
  if (n_iters > 0) {
    fetch(entry(0));
    if (n_iters > 1) e_next = entry(1);
  }
  for (int it = 0; it < n_iters; ++it) {
    __syncthreads();  // the previous tiles are no longer being read
#pragma unroll
    for (int i = 0; i < kStage / 4; ++i) {
      *(f32x4*)&lds_k[ld_r][ld_c + 4 * i] = kk[i];
      *(f32x4*)&lds_v[ld_r][ld_c + 4 * i] = vv[i];
    }
    __syncthreads();
    if (it + 1 < n_iters) {                // in flight while these tiles are computed
      fetch(e_next);
      e_next = it + 2 < n_iters ? entry(it + 2) : kNoRow;
    }
    const int t = NG * it + grp;           // this wave's tile
    if (t >= n_tiles) continue;            // the last iteration may not have a tile for every group
    const int row0 = grp * kTile;

    // S^T block: sc[i] = score of kv token 4g + i of the tile for query row n16
    // every LDS operand of the tile is requested up front: the V reads complete under the
    // score MFMAs instead of stalling each output MFMA
    f32x4 kf[DG / 4];
#pragma unroll
    for (int d4 = 0; d4 < DG / 4; ++d4) kf[d4] = *(const f32x4*)&lds_k[row0 + n16][DG * g + 4 * d4];
    f32x4 vf[4][NE / 4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int h = 0; h < NE / 4; ++h) vf[i][h] = *(const f32x4*)&lds_v[row0 + 4 * g + i][NE * n16 + 4 * h];
    f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int d4 = 0; d4 < DG / 4; ++d4)
#pragma unroll
      for (int j = 0; j < 4; ++j) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[d4][j], q[4 * d4 + j], sc, 0, 0, 0);
    const int n_valid = sp.kv_tokens - t * kTile;
    if (n_valid < kTile) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (4 * g + i >= n_valid) sc[i] = -INFINITY;
    }
    float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
    mx = max_over_lane_groups(mx);
    mx = fmaxf(mx, m);                                    // finite: token 0 of every tile is valid
    const float alpha = __builtin_amdgcn_exp2f(m - mx);   // m = -inf on the first tile gives 0
    m = mx;
    l *= alpha;
#pragma unroll
    for (int e = 0; e < NE; ++e) o[e] *= alpha;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[i] = __builtin_amdgcn_exp2f(sc[i] - m);
      l += sc[i];
    }
    // O^T += V^T P^T, contraction step i over kv = 4g + i; block e holds dims NE * m + e
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < NE; ++e)
        o[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[i][e / 4][e % 4], sc[i], o[e], 0, 0, 0);
  }
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);

  // merge the groups pairwise: the upper half of the remaining groups writes (o, m, l) per
  // lane, the lower half rescales and adds; the last round normalises and stores
  float* merge = lds_raw;
  const int slot = tid & 255;
#pragma unroll
  for (int stride = NG / 2; stride >= 1; stride /= 2) {
    __syncthreads();
    if (grp >= stride && grp < 2 * stride) {
      float* mb = merge + (size_t)(grp - stride) * (NE * 4 + 2) * 256;
#pragma unroll
      for (int e = 0; e < NE; ++e)
#pragma unroll
        for (int i = 0; i < 4; ++i) mb[(4 * e + i) * 256 + slot] = o[e][i];
      mb[(4 * NE) * 256 + slot] = m;
      mb[(4 * NE + 1) * 256 + slot] = l;
    }
    __syncthreads();
    if (grp < stride) {
      const float* mb = merge + (size_t)grp * (NE * 4 + 2) * 256;
      const float m1 = mb[(4 * NE) * 256 + slot], l1 = mb[(4 * NE + 1) * 256 + slot];
      const float mt = fmaxf(m, m1);
      // a group that saw no tile has m = -inf and contributes nothing
      const float w0 = m > -INFINITY ? exp2f(m - mt) : 0.f;
      const float w1 = m1 > -INFINITY ? exp2f(m1 - mt) : 0.f;
      l = l * w0 + l1 * w1;
      m = mt;
#pragma unroll
      for (int e = 0; e < NE; ++e)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[e][i] = o[e][i] * w0 + mb[(4 * e + i) * 256 + slot] * w1;
    }
  }
  if (grp == 0 && row_ok) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;   // no KV at all leaves zeros
    float* op = a.out + ((size_t)(sp.q_begin + r) * H + head) * D + NE * 4 * g;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int h = 0; h < NE / 4; ++h)
        *(f32x4*)(op + NE * i + 4 * h) =
            f32x4{o[4 * h][i], o[4 * h + 1][i], o[4 * h + 2][i], o[4 * h + 3][i]} * inv;
  }
}

// ---------------------------------------------------------------------------- fp32, few queries
// Streams with at most kDecQ query rows (the camera head: one token per frame attending to
// every frame so far, lingbot_map/heads/camera_head.py:296-346) are bound by reading K and V
// once, not by arithmetic, and have far too few rows for the matrix kernel's (64 rows, head)
// workgroups to fill the chip.  Here the KV range of a (stream, head) is cut into n_chunks
// pieces, one workgroup per piece and query row; a workgroup walks its piece in blocks of 256
// tokens: scores by fp32 dot products (D/4 lanes per K row, 16 bytes each, summed with DPP
// steps), block maximum and exp2 through LDS, then the V rows of the block weighted into the
// output accumulator, with the usual running-maximum rescale between blocks.  Each workgroup
// leaves one partial (maximum, sum, unnormalised output); a second small kernel merges them.
namespace {
constexpr int kDecQ = 8;         // query rows per stream this path takes
constexpr int kDecBlock = 256;   // tokens a workgroup handles between two softmax updates
constexpr int kDecMaxChunks = 64;

struct DecodeArgs {
  AttnArgsF32 f;
  float* part;                           // [sum n_chunks][q_rows][H][D + 2]
  int n_chunks[LBM_MAX_STREAMS];
  int part_begin[LBM_MAX_STREAMS];       // in (chunk, query row) units
  int max_q;                             // most query rows of any stream
};

__device__ __forceinline__ float block_reduce_256(float v, bool is_max, float* red) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    const float w = __shfl_xor(v, o);
    v = is_max ? fmaxf(v, w) : v + w;
  }
  __syncthreads();   // red may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return is_max ? fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) : (red[0] + red[1]) + (red[2] + red[3]);
}
}  // namespace

// sum over the LPR = D/4 lanes that share a K row, on the vector ALU: four DPP steps inside a
// row of 16 lanes, and for 32-lane groups one exchange between neighbouring rows
template <int LPR>
__device__ __forceinline__ float row_group_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));  // row_mirror
  if (LPR == 32) {
    float even, odd;
    swap_rows(v, even, odd);
    v = even + odd;
  }
  return v;
}

// grid: x = chunk of the KV axis, y = head, z = stream * max_q + query row
template <int D>
__global__ __launch_bounds__(256) void lbm_attn_f32_decode_kernel(DecodeArgs a) {
  constexpr int LPR = D / 4;         // lanes per K/V row, 16 bytes each
  constexpr int RPP = 256 / LPR;     // rows per pass of the workgroup
  constexpr int NPASS = kDecBlock / RPP;
  constexpr int kBatch = 8;          // rows per lane in flight
  __shared__ float sc[kDecBlock];               // scores, then numerators, of the block
  __shared__ __attribute__((aligned(16))) float acc_red[RPP][D];   // per row-group partial outputs
  __shared__ float red[4];
  const int tid = threadIdx.x;
  const int b = blockIdx.z / a.max_q, qi = blockIdx.z % a.max_q, head = blockIdx.y, chunk = blockIdx.x;
  lbm_attn_stream sp = a.f.s[b];
  if (chunk >= a.n_chunks[b] || qi >= sp.q_rows) return;
  if (a.f.live_kv_tokens) sp.kv_tokens = max(a.f.live_kv_tokens[sp.live_at], 0);
  const int H = a.f.num_heads;
  const size_t row_elems = (size_t)H * D;
  // this workgroup's piece of the KV axis, a whole number of blocks
  const int per = ((sp.kv_tokens + a.n_chunks[b] - 1) / a.n_chunks[b] + kDecBlock - 1) / kDecBlock * kDecBlock;
  const int t_begin = chunk * per, t_end = min(t_begin + per, sp.kv_tokens);
  const int grp = tid / LPR, ln = tid % LPR;   // row group of a pass, lane within the row

  const f32x4 q4 = *(const f32x4*)(a.f.q + ((size_t)(sp.q_begin + qi) * H + head) * D + 4 * ln) * a.f.scale_log2;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  auto row_ptr = [&](int token, bool want_v) -> const float* {
    const int e = a.f.kv_rows[sp.kv_row_begin + token];
    if (e >= 0) return a.f.pool + ((size_t)e * H + head) * D + 4 * ln + (want_v ? (size_t)a.f.page_size * row_elems : 0);
    return (want_v ? a.f.self_v : a.f.self_k) + ((size_t)(-1 - e) * H + head) * D + 4 * ln;
  };

  for (int t0 = t_begin; t0 < t_end; t0 += kDecBlock) {
    // ---- scores of the block, kBatch rows per lane in flight
    __syncthreads();   // sc of the previous block is no longer read
#pragma unroll 1
    for (int pb = 0; pb < NPASS; pb += kBatch) {
      f32x4 kx[kBatch];
#pragma unroll
      for (int p = 0; p < kBatch; ++p) {
        const int token = t0 + (pb + p) * RPP + grp;
        kx[p] = token < t_end ? *(const f32x4*)row_ptr(token, false) : f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int p = 0; p < kBatch; ++p) {
        const int local = (pb + p) * RPP + grp;
        const float d = row_group_sum<LPR>(kx[p][0] * q4[0] + kx[p][1] * q4[1] + kx[p][2] * q4[2] + kx[p][3] * q4[3]);
        if (ln == 0) sc[local] = t0 + local < t_end ? d : -INFINITY;
      }
    }
    __syncthreads();
    // ---- running maximum, numerators, running sum (thread tid owns token tid of the block)
    const float s = sc[tid];
    const float m_new = fmaxf(m_run, block_reduce_256(s, true, red));   // finite: token t0 is valid
    const float pr = exp2f(s - m_new);
    sc[tid] = pr;
    const float alpha = exp2f(m_run - m_new);   // 0 on the first block
    l_run = l_run * alpha + block_reduce_256(pr, false, red);
    m_run = m_new;
    __syncthreads();
    // ---- weighted V rows
    acc *= alpha;
#pragma unroll 1
    for (int pb = 0; pb < NPASS; pb += kBatch) {
      f32x4 vx[kBatch];
#pragma unroll
      for (int p = 0; p < kBatch; ++p) {
        const int token = t0 + (pb + p) * RPP + grp;
        vx[p] = token < t_end ? *(const f32x4*)row_ptr(token, true) : f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int p = 0; p < kBatch; ++p) acc += vx[p] * sc[(pb + p) * RPP + grp];
    }
  }
  // ---- sum the row groups' accumulators, write the partial
  *(f32x4*)&acc_red[grp][4 * ln] = acc;
  __syncthreads();
  if (tid < D) {
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < RPP; ++r) o += acc_red[r][tid];
    float* pp = a.part + (((size_t)a.part_begin[b] + (size_t)chunk * sp.q_rows + qi) * H + head) * (D + 2);
    pp[tid] = o;
    if (tid == 0) {
      pp[D] = m_run;       // identical in every thread
      pp[D + 1] = l_run;
    }
  }
}

// one 128-thread workgroup per (stream, query row, head): merge the chunks' partials.  Thread
// c reads chunk c's maximum and sum (all chunks at once), the weights go through LDS, then
// thread d sums the weighted outputs with several loads in flight.
template <int D>
__global__ __launch_bounds__(128) void lbm_attn_f32_decode_merge_kernel(DecodeArgs a) {
  static_assert(kDecMaxChunks <= 128 && D <= 128, "one thread per chunk, one per head dimension");
  __shared__ float w[kDecMaxChunks];
  __shared__ float red[2][2];
  const int b = blockIdx.z, head = blockIdx.y, qi = blockIdx.x, tid = threadIdx.x;
  const lbm_attn_stream sp = a.f.s[b];
  if (qi >= sp.q_rows) return;
  const int H = a.f.num_heads, nc = a.n_chunks[b];
  const size_t stride = (size_t)sp.q_rows * H * (D + 2);      // from one chunk's partial to the next
  const float* base = a.part + (((size_t)a.part_begin[b] + qi) * H + head) * (D + 2);
  float m_c = -INFINITY, l_c = 0.f;
  if (tid < nc) {
    m_c = base[tid * stride + D];
    l_c = base[tid * stride + D + 1];
  }
  float m = m_c;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  if ((tid & 63) == 0) red[0][tid >> 6] = m;
  __syncthreads();
  m = fmaxf(red[0][0], red[0][1]);
  const float w_c = m_c > -INFINITY ? exp2f(m_c - m) : 0.f;   // a chunk without tokens weighs nothing
  if (tid < nc) w[tid] = w_c;
  float l = l_c * w_c;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) l += __shfl_xor(l, o);
  if ((tid & 63) == 0) red[1][tid >> 6] = l;
  __syncthreads();
  l = red[1][0] + red[1][1];
  if (tid >= D) return;
  float o = 0.f;
  int c = 0;
  for (; c + 8 <= nc; c += 8) {
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = base[(c + j) * stride + tid];
#pragma unroll
    for (int j = 0; j < 8; ++j) o += x[j] * w[c + j];
  }
  for (; c < nc; ++c) o += base[c * stride + tid] * w[c];
  a.f.out[((size_t)(sp.q_begin + qi) * H + head) * D + tid] = l > 0.f ? o / l : 0.f;
}

// Chunks per stream for the few-query path, and the floats of partials they need.  Depends on
// row and token counts only (never on the dtype), so the workspace query can include it.
static int lbm_decode_chunks(int kv_tokens) {
  int n = (kv_tokens + kDecBlock - 1) / kDecBlock;
  return n < 1 ? 1 : (n > kDecMaxChunks ? kDecMaxChunks : n);
}
static bool lbm_decode_applies(const LbmAttnSchedule& sch) {
  for (int i = 0; i < sch.n_streams; ++i)
    if (sch.s[i].q_rows > kDecQ) return false;
  return sch.n_streams > 0;
}
static size_t lbm_decode_bytes(const LbmAttnSchedule& sch, int num_heads, int head_dim) {
  if (!lbm_decode_applies(sch)) return 0;
  size_t rows = 0;
  for (int i = 0; i < sch.n_streams; ++i) rows += (size_t)lbm_decode_chunks(sch.s[i].kv_tokens) * sch.s[i].q_rows;
  return rows * num_heads * (head_dim + 2) * sizeof(float);
}

// ---------------------------------------------------------------------------- schedule
// How many KV splits each stream gets.  All workgroups of one launch compete for the 256 CUs
// (one 8-wave workgroup per CU at a time, handed out in blockIdx order), so the choice is a
// small scheduling problem: few long workgroups leave CUs idle at the end, many short ones
// pay the per-workgroup prologue/epilogue and more split-KV partials.  A handful of candidate
// tile counts per workgroup is priced with the measured costs below by simulating the
// hand-out (streams with the longest workgroups first), and the cheapest wins.  The result
// depends on row and tile counts only and is remembered for the next call with the same ones
// (every block of a frame asks for the same schedule).
namespace {
constexpr double kTileUs = 1.95;      // one 64-token tile iteration of a workgroup
constexpr double kWgTiles = 3.0;      // prologue + epilogue of a workgroup, in tile iterations
constexpr double kCombineUs = 2.5;    // launch + latency of the combine kernel
constexpr double kCombineBytesPerUs = 5.0e6;
// the short-KV kernel (one workgroup per 64 query rows and head, no partial results)
constexpr double kSmLaunchUs = 1.8;   // launch to first instruction
constexpr double kSmWgUs = 4.0;       // a workgroup's fixed part: Q rows, range check, merge through LDS, store
constexpr double kSmTileUs = 0.3625;  // per 64-token tile: 1.45 us per step of eight 32-token pieces

struct ScheduleKey {
  int n_streams = -1, num_heads = 0;
  bool small = false;
  int q_rows[LBM_MAX_STREAMS], n_tiles[LBM_MAX_STREAMS];
  int order[LBM_MAX_STREAMS], n_splits[LBM_MAX_STREAMS];
};
thread_local ScheduleKey g_last_schedule;

double price_candidate(const int* qt, const int* nt, int n_streams, int num_heads, int tps, const int* q_rows,
                       int* n_splits_out) {
  // streams sorted by tiles per workgroup, longest first
  int tiles[LBM_MAX_STREAMS], order[LBM_MAX_STREAMS];
  double part_bytes = 0;
  for (int i = 0; i < n_streams; ++i) {
    int ns = nt[i] > 0 ? (nt[i] + tps - 1) / tps : 1;
    if (ns > 64) ns = 64;
    if (ns < 1) ns = 1;
    tiles[i] = nt[i] > 0 ? (nt[i] + ns - 1) / ns : 0;
    n_splits_out[i] = nt[i] > 0 ? (nt[i] + tiles[i] - 1) / tiles[i] : 1;
    if (n_splits_out[i] > 1) part_bytes += (double)n_splits_out[i] * q_rows[i] * num_heads * (64 * 2 + 4);
    order[i] = i;
  }
  for (int i = 1; i < n_streams; ++i)
    for (int j = i; j > 0 && tiles[order[j]] > tiles[order[j - 1]]; --j) { int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
  // hand the workgroups out to the CUs in order; each goes to the CU that frees up first.  A
  // binary heap over 256 finish times.
  double heap[256];
  for (int i = 0; i < 256; ++i) heap[i] = 0.0;
  double makespan = 0.0;
  for (int oi = 0; oi < n_streams; ++oi) {
    const int i = order[oi];
    const long long wgs = (long long)qt[i] * num_heads * n_splits_out[i];
    const double dur = kWgTiles + tiles[i];
    for (long long w = 0; w < wgs; ++w) {
      const double t = heap[0] + dur;
      if (t > makespan) makespan = t;
      // replace the root and sift down
      int k = 0;
      for (;;) {
        int c = 2 * k + 1;
        if (c >= 256) break;
        if (c + 1 < 256 && heap[c + 1] < heap[c]) ++c;
        if (heap[c] >= t) break;
        heap[k] = heap[c];
        k = c;
      }
      heap[k] = t;
    }
  }
  return makespan * kTileUs + (part_bytes > 0 ? kCombineUs + 2.0 * part_bytes / kCombineBytesPerUs : 0.0);
}
}  // namespace

void lbm_attn_schedule(const lbm_attn_stream* streams, int n_streams, int num_heads,
                       LbmAttnSchedule* out) {
  LbmAttnSchedule& sch = *out;
  sch = LbmAttnSchedule{};
  sch.n_streams = n_streams;
  int qt[LBM_MAX_STREAMS], nt[LBM_MAX_STREAMS], q_rows[LBM_MAX_STREAMS];
  long long work = 0;
  int max_nt = 0;
  for (int i = 0; i < n_streams; ++i) {
    q_rows[i] = streams[i].q_rows;
    qt[i] = (streams[i].q_rows + kQTile - 1) / kQTile;
    nt[i] = (streams[i].kv_tokens + kKvTile - 1) / kKvTile;
    work += (long long)qt[i] * num_heads * nt[i];
    if (nt[i] > max_nt) max_nt = nt[i];
  }
  // Short KV everywhere: the in-workgroup split kernel (one workgroup per 64 query rows and head,
  // no partial results) is a candidate, priced against the split-KV plan: it wins on one frame's
  // 1,004 x 1,004 (256 workgroups of 16 tiles: 12 us against 19), the split-KV pair wins once
  // several streams would take the CUs four rounds of such workgroups (31 against 43 us).
  bool small_ok = n_streams > 0;
  for (int i = 0; i < n_streams; ++i) small_ok = small_ok && streams[i].kv_tokens <= kSmMaxKv;
  ScheduleKey& memo = g_last_schedule;
  bool hit = memo.n_streams == n_streams && memo.num_heads == num_heads;
  for (int i = 0; hit && i < n_streams; ++i) hit = memo.q_rows[i] == q_rows[i] && memo.n_tiles[i] == nt[i];
  if (!hit) {
    int best_splits[LBM_MAX_STREAMS], cand_splits[LBM_MAX_STREAMS];
    double best = -1.0;
    auto consider = [&](long long tps) {
      if (tps < 2) tps = 2;
      if (tps > max_nt) tps = max_nt > 0 ? max_nt : 1;
      const double c = price_candidate(qt, nt, n_streams, num_heads, (int)tps, q_rows, cand_splits);
      if (best < 0 || c < best) {
        best = c;
        for (int i = 0; i < n_streams; ++i) best_splits[i] = cand_splits[i];
      }
    };
    // the longest stream cut into 1..12 pieces, and the total work spread over 1..3 rounds of 256
    for (int k = 1; k <= 12; ++k) consider((max_nt + k - 1) / k);
    for (int k = 1; k <= 3; ++k) consider((work + 256LL * k - 1) / (256LL * k));
    memo.small = false;
    if (small_ok) {
      double longest = 0.0, total = 0.0;
      for (int i = 0; i < n_streams; ++i) {
        const double dur = kSmWgUs + kSmTileUs * (nt[i] > 0 ? nt[i] : 1);
        const double wgs = (double)((q_rows[i] + kQPerWave - 1) / kQPerWave) * num_heads;
        if (wgs > 0 && dur > longest) longest = dur;
        total += wgs * dur;
      }
      const double small_price = kSmLaunchUs + (total / 256.0 > longest ? total / 256.0 : longest);
      // (the short-KV kernel unless the pair is clearly ahead: it merges its partial results in
      // fp32 inside the workgroup, the pair rounds them to bf16 on their way through memory)
      memo.small = best < 0 || 0.85 * small_price <= best;
    }
    memo.n_streams = n_streams;
    memo.num_heads = num_heads;
    int tiles[LBM_MAX_STREAMS];
    for (int i = 0; i < n_streams; ++i) {
      memo.q_rows[i] = q_rows[i];
      memo.n_tiles[i] = nt[i];
      memo.n_splits[i] = best_splits[i];
      memo.order[i] = i;
      tiles[i] = nt[i] > 0 ? (nt[i] + best_splits[i] - 1) / best_splits[i] : 0;
    }
    for (int i = 1; i < n_streams; ++i)
      for (int j = i; j > 0 && tiles[memo.order[j]] > tiles[memo.order[j - 1]]; --j) {
        int t = memo.order[j]; memo.order[j] = memo.order[j - 1]; memo.order[j - 1] = t;
      }
  }
  if (memo.small) {
    sch.small = 1;
    int wg = 0;
    for (int i = 0; i < n_streams; ++i) {
      LbmAttnStreamPlan& p = sch.s[i];
      p.q_begin = streams[i].q_begin;
      p.q_rows = streams[i].q_rows;
      p.kv_row_begin = streams[i].kv_row_begin;
      p.kv_tokens = streams[i].kv_tokens;
      p.live_at = streams[i].live_at;
      p.n_qtiles = (streams[i].q_rows + kQPerWave - 1) / kQPerWave;
      p.n_splits = 1;
      p.tiles_per_split = nt[i] > 0 ? nt[i] : 1;
      wg = (wg + 7) & ~7;   // each stream starts on XCD 0 so the in-kernel head -> XCD map lines up
      p.wg_begin = wg;
      p.part_begin = 0;
      // whole groups of 8 workgroups when the heads are dealt over the XCDs
      const int per_q = num_heads;
      wg += p.n_qtiles * per_q;
    }
    sch.total_wgs = wg;
    sch.part_rows = 0;
    return;
  }
  int wg = 0;
  long long part = 0;
  for (int oi = 0; oi < n_streams; ++oi) {
    const int i = memo.order[oi];
    LbmAttnStreamPlan& p = sch.s[oi];   // plans in launch order: blockIdx ranges ascend with the index
    p.q_begin = streams[i].q_begin;
    p.q_rows = streams[i].q_rows;
    p.kv_row_begin = streams[i].kv_row_begin;
    p.kv_tokens = streams[i].kv_tokens;
    p.live_at = streams[i].live_at;
    p.n_qtiles = qt[i];
    const int ns = memo.n_splits[i];
    p.tiles_per_split = nt[i] > 0 ? (nt[i] + ns - 1) / ns : 1;
    p.n_splits = nt[i] > 0 ? (nt[i] + p.tiles_per_split - 1) / p.tiles_per_split : 1;
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
  // bf16 partial outputs followed by one float log-sum-exp per (row, head); or, when every
  // stream has only a few query rows, the fp32 partials of the few-query path (the query does
  // not know the dtype, so it covers both)
  const size_t split_kv = (size_t)sch.part_rows * num_heads * (head_dim * 2 + 4);
  const size_t few_q = lbm_decode_bytes(sch, num_heads, head_dim);
  return split_kv > few_q ? split_kv : few_q;
}

namespace {
int lbm_launch_attention_only(const void* q, const void* pool, void* out, const void* self_k,
                              const void* self_v, const int32_t* kv_rows, const int32_t* live_kv_tokens,
                              const LbmAttnSchedule& sch, int num_heads, int head_dim, int page_size, int dtype,
                              float sm_scale, void* workspace, hipStream_t stream, const int32_t* append_rows,
                              int append_tokens, bool* appended);
}  // namespace

// append_rows (lbm_attn_run_append): rows of self_k / self_v that are stored in the pool after the
// attention has read it - inside the launch that merges the split-KV partials when the schedule has
// one, by lbm_kv_append_kernel behind the attention otherwise.
int lbm_launch_attention(const void* q, const void* pool, void* out, const void* self_k,
                         const void* self_v, const int32_t* kv_rows, const int32_t* live_kv_tokens,
                         const LbmAttnSchedule& sch,
                         int num_heads, int head_dim, int page_size, int dtype, float sm_scale,
                         void* workspace, hipStream_t stream, const int32_t* append_rows, int append_tokens) {
  bool appended = false;
  int rc = lbm_launch_attention_only(q, pool, out, self_k, self_v, kv_rows, live_kv_tokens, sch, num_heads, head_dim,
                                     page_size, dtype, sm_scale, workspace, stream, append_rows, append_tokens, &appended);
  if (rc != LBM_OK || !append_rows || append_tokens <= 0 || appended) return rc;
  return lbm_launch_append(self_k, self_v, dtype, const_cast<void*>(pool), dtype, append_rows, append_tokens, num_heads,
                           head_dim, page_size, stream);
}

namespace {
int lbm_launch_attention_only(const void* q, const void* pool, void* out, const void* self_k,
                              const void* self_v, const int32_t* kv_rows, const int32_t* live_kv_tokens,
                              const LbmAttnSchedule& sch, int num_heads, int head_dim, int page_size, int dtype,
                              float sm_scale, void* workspace, hipStream_t stream, const int32_t* append_rows,
                              int append_tokens, bool* appended) {
  if (head_dim != 64 && !(head_dim == 128 && dtype == LBM_DTYPE_F32))
    return lbm_fail(LBM_ERR_UNSUPPORTED, "attention kernels cover head_dim 64 (bf16, fp32) and 128 (fp32), got %d", head_dim);
  if (dtype == LBM_DTYPE_F32) {
    AttnArgsF32 f;
    f.q = (const float*)q;
    f.pool = (const float*)pool;
    f.out = (float*)out;
    f.self_k = (const float*)self_k;
    f.self_v = (const float*)self_v;
    f.kv_rows = kv_rows;
    f.live_kv_tokens = live_kv_tokens;
    f.num_heads = num_heads;
    f.page_size = page_size;
    f.scale_log2 = sm_scale == 0.f ? 1.0f : sm_scale * 1.4426950408889634f;   // 0: q already carries scale * log2(e)
    f.n_streams = sch.n_streams;
    int wg = 0;
    for (int i = 0; i < LBM_MAX_STREAMS; ++i) {
      f.s[i] = lbm_attn_stream{0, 0, 0, 0, 0};
      f.wg_begin[i] = wg;
      if (i < sch.n_streams) {
        f.s[i] = lbm_attn_stream{sch.s[i].q_begin, sch.s[i].q_rows, sch.s[i].kv_row_begin, sch.s[i].kv_tokens, sch.s[i].live_at};
        wg += ((sch.s[i].q_rows + kF32Rows - 1) / kF32Rows) * num_heads;
      }
    }
    f.wg_begin[LBM_MAX_STREAMS] = wg;
    if (wg == 0) return LBM_OK;
    if (lbm_decode_applies(sch)) {
      DecodeArgs d;
      d.f = f;
      d.part = (float*)workspace;
      int max_chunks = 0, max_q = 0, part = 0;
      for (int i = 0; i < LBM_MAX_STREAMS; ++i) {
        d.n_chunks[i] = 0;
        d.part_begin[i] = part;
        if (i < sch.n_streams) {
          d.n_chunks[i] = lbm_decode_chunks(sch.s[i].kv_tokens);
          part += d.n_chunks[i] * sch.s[i].q_rows;
          if (d.n_chunks[i] > max_chunks) max_chunks = d.n_chunks[i];
          if (sch.s[i].q_rows > max_q) max_q = sch.s[i].q_rows;
        }
      }
      if (max_q == 0) return LBM_OK;
      d.max_q = max_q;
      const dim3 grid(max_chunks, num_heads, sch.n_streams * max_q), mgrid(max_q, num_heads, sch.n_streams);
      if (head_dim == 64) {
        hipLaunchKernelGGL(lbm_attn_f32_decode_kernel<64>, grid, dim3(256), 0, stream, d);
        hipLaunchKernelGGL(lbm_attn_f32_decode_merge_kernel<64>, mgrid, dim3(128), 0, stream, d);
      } else {
        hipLaunchKernelGGL(lbm_attn_f32_decode_kernel<128>, grid, dim3(256), 0, stream, d);
        hipLaunchKernelGGL(lbm_attn_f32_decode_merge_kernel<128>, mgrid, dim3(128), 0, stream, d);
      }
      return lbm_check_launch("lbm_attn_f32_decode_kernel");
    }
    if (head_dim == 64) hipLaunchKernelGGL(lbm_attn_f32_kernel<64>, dim3(wg), dim3(1024), 0, stream, f);
    else hipLaunchKernelGGL(lbm_attn_f32_kernel<128>, dim3(wg), dim3(512), 0, stream, f);
    return lbm_check_launch("lbm_attn_f32_kernel");
  }
  if (dtype != LBM_DTYPE_BF16) return lbm_fail(LBM_ERR_INVALID, "unknown dtype %d", dtype);
  AttnArgs a;
  a.q = (const unsigned short*)q;
  a.pool = (const unsigned short*)pool;
  a.out = (unsigned short*)out;
  a.self_k = (const unsigned short*)self_k;
  a.self_v = (const unsigned short*)self_v;
  a.kv_rows = kv_rows;
  a.live_kv_tokens = live_kv_tokens;
  a.part_o = (unsigned short*)workspace;
  a.part_lse = (float*)(a.part_o + (size_t)sch.part_rows * num_heads * head_dim);
  a.num_heads = num_heads;
  a.page_size = page_size;
  a.scale_log2 = sm_scale == 0.f ? 1.0f : sm_scale * 1.4426950408889634f;   // 0: q already carries scale * log2(e)
  a.append_rows = nullptr;
  a.append_tokens = 0;
  a.combine_blocks = 0x7fffffff;
  a.sch = sch;
  if (sch.total_wgs == 0) return LBM_OK;
  if (sch.small) {
    hipLaunchKernelGGL(lbm_attn_bf16_d64_small_kernel, dim3(sch.total_wgs), dim3(kSmThreads), 0, stream, a);
    return lbm_check_launch("lbm_attn_bf16_d64_small_kernel");
  }
  hipLaunchKernelGGL(lbm_attn_bf16_d64_kernel, dim3(sch.total_wgs), dim3(kThreads), 0, stream, a);
  int rc = lbm_check_launch("lbm_attn_bf16_d64_kernel");
  if (rc != LBM_OK) return rc;
  if (sch.part_rows > 0) {
    int max_rows = 0;
    for (int i = 0; i < sch.n_streams; ++i)
      if (sch.s[i].n_splits > 1 && sch.s[i].q_rows > max_rows) max_rows = sch.s[i].q_rows;
    const long long threads = (long long)max_rows * num_heads * 8;
    unsigned blocks = (unsigned)((threads + 255) / 256);
    a.combine_blocks = (int)blocks;
    if (append_rows && append_tokens > 0) {
      a.append_rows = append_rows;
      a.append_tokens = append_tokens;
      blocks += (unsigned)(((long long)append_tokens * num_heads * 8 + 255) / 256);
      *appended = true;
    }
    hipLaunchKernelGGL(lbm_attn_combine_bf16_kernel, dim3(blocks, sch.n_streams), dim3(256), 0, stream, a);
    rc = lbm_check_launch("lbm_attn_combine_bf16_kernel");
  }
  return rc;
}
}  // namespace

// ---------------------------------------------------------------------------- static scratch
// Workspace for callers that cannot allocate (lbm_attn_run_static): split-KV partials and the
// few-query partials go into this file-scope device array instead of a caller's buffer.  Every
// GPU the library runs on holds its own copy at its own address until the process ends; the
// array's name is only a host-side handle, so the address is looked up once per device with
// that device current and the kernels get the looked-up pointer like any other workspace.
// Nothing in it has to start at zero: every partial a launch reads was written by that launch.
namespace {
constexpr size_t kStaticScratchBytes = (size_t)LBM_STATIC_SCRATCH_MIB << 20;
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

int lbm_static_scratch(void** ptr, size_t* bytes) {
  int dev = -1;
  const hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return lbm_fail(LBM_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return lbm_fail(LBM_ERR_UNSUPPORTED, "device ordinal %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    const hipError_t es = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (es != hipSuccess || !p)
      return lbm_fail(LBM_ERR_HIP, "hipGetSymbolAddress(static scratch) on device %d: %s", dev, hipGetErrorString(es));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  *bytes = kStaticScratchBytes;
  return LBM_OK;
}
