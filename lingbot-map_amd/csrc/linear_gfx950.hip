// bf16 linear layers of a transformer block for gfx950, with the elementwise work that follows
// them fused into the store:
//     out = epilogue(a @ w^T + bias)      a [M, K], w [N, K] (nn.Linear's weight), bf16 in and out
//   LBM_LINEAR_BIAS            the qkv projection                (lingbot_map/layers/attention.py:413)
//   LBM_LINEAR_BIAS_GELU       fc1 + exact (erf) GELU            (lingbot_map/layers/mlp.py:35-36)
//   LBM_LINEAR_BIAS_RESIDUAL   proj / fc2 + LayerScale + residual: x + gamma * (a @ w^T + bias)
//                              (attention.py:554, mlp.py:38, lingbot_map/layers/block.py:283,
//                              lingbot_map/layers/layer_scale.py:21-22)
// Roundings follow the sequence of separate bf16 torch ops: the linear's output is rounded to
// bf16, then each elementwise op rounds again.
//
// Around that, so that a transformer block needs no LayerNorm, residual or producer launch:
//   * the residual epilogue can leave the row statistics (mean, M2 per column tile) of what it
//     stores (block.py:283-285 feeding the next LayerNorm);
//   * a launch can take activations whose LayerNorm is still to be applied: the product runs on
//     the raw rows and the store applies rstd * (acc - mean * colsum(w)) + bias, the LayerNorm's
//     affine part folded into w and bias by the caller (block.py:194-195, 217; the normalised rows
//     are then never rounded to bf16, the folded weights are);
//   * the qkv projection can carry the pre-attention producer as its epilogue (kEpiQkvPrepare);
//   * a launch with few tiles and a long K can put several workgroups on a tile (SPLITK).
//
// Shapes this is written for: M about 1,000 rows per stream (one frame), K, N in 1024 .. 4096.
// At that size a launch has only a few hundred tiles and 16-64 k-steps, so what counts is a
// tile count that matches the 256 CUs and a short prologue, not asymptotic throughput.
//
// One workgroup = 8 wavefronts on a 128 x 128 tile of the output (TN = 64: 128 x 64).  The product
// is computed transposed, C^T = W A^T with v_mfma_f32_32x32x16_bf16 (A operand = 32 rows of W, B
// operand = 32 rows of the activations), so an accumulator register holds four consecutive output
// columns of one row.  The eight wavefronts are two groups of four: each group covers the whole
// tile (a wavefront owns 64 x TN / 2 of it) over its own half of every K slice, which gives each
// SIMD two wavefronts to cover each other's LDS and barrier waits without giving up the fragment
// reuse of the large per-wave tile; the two groups' sums meet through LDS once, at the end.
// Both operands are K-contiguous and travel global -> LDS directly (global_load_lds_dwordx4, no
// registers and no LDS store instructions in between) in 64-wide slices of K, four LDS stages,
// three slices ahead of the multiply; rows are unpadded and their 16-byte chunks XOR-swizzled by
// the choice of source address, so the b128 fragment reads are free of bank conflicts.  One
// workgroup barrier per slice.  The tile leaves through LDS as whole rows: 16-byte stores, and
// the residual is read the same way.
#include <type_traits>
#include <hip/hip_runtime.h>
#include "lbm_internal.h"
#include "qkv_math.h"

#pragma clang fp contract(off)

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

constexpr int kGK = 128;         // K granularity the launches accept
constexpr int kGM = 128;         // activation rows per tile
constexpr int kGThreads = 512;
constexpr int kGTouchThreads = 64;   // lbm_linear_bf16_kernel: one more wavefront that only asks for weight lines ahead of the loop
constexpr int kKS = 64;          // K elements per LDS stage
constexpr int kStagesG = 4;      // LDS stages: three being loaded while one is multiplied (six stages for the 64-column tile,
                                 // which has the room: slower, 8.4 -> 8.8 us for proj - the longer prologue costs more than the depth gains)

struct LinearArgs {
  const unsigned short* a;       // [M, K]
  const unsigned short* w;       // [N, K]
  const float* bias;             // [N] or null
  const float* gamma;            // [N] LayerScale (RESIDUAL only) or null
  const unsigned short* res;     // [M, N] residual (RESIDUAL only)
  unsigned short* out;           // [M, N]
  int M, N, K;
  int m_tiles, n_tiles;
  // LBM_LINEAR_QKV_PREPARE: the fused pre-attention producer as the epilogue of the qkv projection
  const float* q_norm_w;         // all four null: no qk-norm
  const float* q_norm_b;
  const float* k_norm_w;
  const float* k_norm_b;
  const float* rope_cs;
  unsigned short* k_out;         // out is q_out; k_out / v_out may be null
  unsigned short* v_out;
  unsigned short* pool;
  const int32_t* append_rows;    // null: nothing is appended
  float eps;
  float q_scale;                 // q rows are multiplied by this in fp32 before their last rounding (1 = plain q)
  int num_heads, page_size;
  // LNA kernels: the rows of the activations are standardised, (x - mean) * rstd, without ever
  // being rewritten: the product runs on the raw rows and the store applies
  // rstd * (a @ w^T - mean * colsum(w)) + bias.  The statistics come from the launch that
  // produced the activations (one (mean, M2) pair per row and column tile of that launch).
  const float* ln_colsum;        // [N]: sum over k of w[n][k]
  const float* ln_stats;         // [M][ln_tiles][2]
  int ln_tiles;
  float ln_eps;
  // LBM_LINEAR_BIAS_RESIDUAL: (mean, M2) of every output row over this tile's columns,
  // [M][n_tiles][2], or null
  float* stats_out;
  // SPLITK kernels: k_splits workgroups share a tile, each over its own slice of K.  Every one
  // parks its fp32 partial tile in `split_part` and takes a ticket from the tile's counter; the
  // one that draws the last ticket sums the partials in slice order (the same sum whoever is
  // last) and runs the epilogue.  Counters start at zero and are left at zero.
  // memory the launch after this one will read (lbm_linear_prefetch_hint): the ninth wavefronts of
  // lbm_linear_bf16_kernel ask for it
  const char* touch;
  unsigned touch_lines;          // 128-byte lines
  int k_splits;
  unsigned* split_counters;      // [m_tiles * n_tiles]
  float* split_part;             // [m_tiles * n_tiles][k_splits][8 waves][NT * 16][64 lanes]
};
constexpr int kEpiQkvPrepare = 3;   // internal: reached through lbm_qkv_linear_prepare only

__device__ __forceinline__ float round_bf16(float f) { return (float)(__bf16)f; }
__device__ __forceinline__ float bf16_bits_to_f32(unsigned v) { return __builtin_bit_cast(float, v << 16); }
// The GELU of the fused fc1 epilogue (torch's exact-erf nn.GELU, lingbot_map/layers/mlp.py:24) acts
// on a value already rounded to bf16 and is rounded to bf16 again: a function from 16 bits to
// 16 bits.  Evaluated per element it costs about 32 vector instructions, 4 us of a 20 us launch;
// instead it is tabulated for |v| in [2^-12, 2^3) - 15 binades x 128 mantissas x 2 signs, 7.5 KB,
// exact values rounded once (gen_gelu_table.py) - and each workgroup pulls the table into LDS with
// one 16-byte LDS-direct load per thread, ahead of its first operand tiles, and looks the
// elements up, without a branch, so that the lookups of a lane's 32 elements overlap.
// Outside the table the function has closed forms that agree with torch's fp32 evaluation
// after the rounding to bf16: below 2^-12, 1 + erf differs from 1 by less than 2^-12 and
// v / 2 is the nearest bf16 value (zeros and denormals included); from 8 up erff is exactly
// +-1, so the result is v on the positive side (+inf and NaN included) and v * 0 on the
// negative side (-0, and NaN for -inf and NaN, like 0.5 * v * (1 - 1)).  Between -8 and -3,
// where torch's 1 + erff cancels and its result carries the last bits of its erff, the table
// holds the exact value, within one bf16 step of torch's.
constexpr int kGeluE0 = 127 - 12;              // biased exponent of the first tabulated binade
constexpr int kGeluHalf = 15 * 128;            // entries per sign
constexpr int kGeluEntries = 2 * kGeluHalf;
static __device__ __attribute__((aligned(16))) const unsigned short g_gelu_table[kGeluEntries] = {
#include "gelu_table.inc"
};
// GELU of a value that is already a bf16 (v), rounded to bf16, from the table copy in LDS
__device__ __forceinline__ float gelu_of_bf16(float v, const unsigned short* tab) {
  const unsigned b16 = __builtin_bit_cast(unsigned, v) >> 16;
  const unsigned mag = b16 & 0x7fffu, neg = b16 >> 15;
  const unsigned rel = mag - (unsigned)(kGeluE0 << 7);
  const unsigned looked_up = tab[min(rel, (unsigned)(kGeluHalf - 1)) + neg * kGeluHalf];
  // outside the table: v / 2 below it, v or v * 0 above it (see kGeluE0)
  const float outside = mag < (unsigned)(kGeluE0 << 7) ? 0.5f * v : (neg ? v * 0.0f : v);
  return rel < (unsigned)kGeluHalf ? bf16_bits_to_f32(looked_up) : outside;
}

// Workgroup b's tile.  Workgroups are dealt to the 8 XCDs round-robin (b % 8), 32 of a round of 256
// to each; an XCD's 32 take consecutive tiles of an order that walks panels of 8 column tiles row
// by row, i.e. 4 row tiles x 8 column tiles (8 x 4 in a last panel of 4): 12 operand tiles per
// k-step for the XCD's L2 to hold instead of 17 to 33, which is what sets the latency of the
// operand loads.
__device__ __forceinline__ void lbm_tile_of_workgroup(int b, int m_tiles, int n_tiles, int& mt, int& nt) {
  const int x = b & 7, i = b >> 3;
  const int base = (i >> 5) * 256;
  const int in_round = min(m_tiles * n_tiles - base, 256);
  const int t = base + x * (in_round >> 3) + min(x, in_round & 7) + (i & 31);
  const int panel_tiles = m_tiles * 8;
  const int panel = t / panel_tiles, rem = t - panel * panel_tiles;
  const int width = min(8, n_tiles - panel * 8);
  mt = rem / width;
  nt = panel * 8 + rem - mt * width;
}

// TN: output columns per tile (128 or 64); a wavefront owns 64 x (TN / 2) of the tile.
// ROPE / NORM: rotary layout (0 none, 1 interleaved, 2 half-split) and qk-LayerNorm of the
// kEpiQkvPrepare epilogue; 0 / false otherwise.
// LNA: the activations' rows are standardised by the store (see LinearArgs).
// SPLITK: several workgroups per tile, each over a slice of K (see LinearArgs).
template <int EPI, int TN, int ROPE = 0, bool NORM = false, bool LNA = false, bool SPLITK = false>
__global__ __launch_bounds__(kGThreads + kGTouchThreads, 1) void lbm_linear_bf16_kernel(LinearArgs p) {
  constexpr int NT = TN / 64;   // 32-column blocks of W per wavefront
  // [buffer][k half][row][64 + pad]
  // [stage][row][64]: 64-wide slices of K, kStagesG of them in flight or in use
  __shared__ __attribute__((aligned(16))) unsigned short lds_a[kStagesG][kGM * kKS];
  __shared__ __attribute__((aligned(16))) unsigned short lds_w[kStagesG][TN * kKS];
  __shared__ __attribute__((aligned(16))) unsigned short gelu_tab[EPI == LBM_LINEAR_BIAS_GELU ? kGeluEntries : 8];
  __shared__ __attribute__((aligned(8))) float ln_rows[LNA ? kGM * 2 : 2];   // per row of the tile: rstd, -mean * rstd
  __shared__ __attribute__((aligned(16))) float colvec[3][TN];               // bias, column sums of w (LNA), LayerScale

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n32 = lane & 31, g = lane >> 5;
  const int kh = wave >> 2, ws = wave & 3;    // k half of this wave's group, its sub-tile
  // Workgroups are dealt to the 8 XCDs round-robin: an XCD keeps its own column tiles of W (read
  // from HBM once, by it alone) and walks all row tiles of the activations with them.
  // (the workgroups that share a tile under SPLITK land on the same XCD as well)
  int mt, nt, split = 0;
  {
    const int n_tiles_all = p.m_tiles * p.n_tiles;
    if (!SPLITK) {
      lbm_tile_of_workgroup((int)blockIdx.x, p.m_tiles, p.n_tiles, mt, nt);
    } else if ((p.n_tiles & 7) == 0) {
      const int x = blockIdx.x & 7;
      int i = blockIdx.x >> 3;
      split = i / (n_tiles_all >> 3);
      i -= split * (n_tiles_all >> 3);
      mt = i % p.m_tiles;
      nt = (i / p.m_tiles) * 8 + x;
    } else {
      int i = (int)blockIdx.x;
      if (SPLITK) {
        split = i / n_tiles_all;
        i -= split * n_tiles_all;
      }
      mt = i % p.m_tiles;
      nt = i / p.m_tiles;
    }
  }
  const int m0 = mt * kGM, n0 = nt * TN;
  const int wm = (ws & 1) * 64, wn = (ws >> 1) * (TN / 2);

  // ---- staging.  Operands travel global -> LDS without passing through registers
  // (global_load_lds_dwordx4: a wavefront's 64 lanes x 16 bytes land as one contiguous KB, i.e.
  // eight whole 128-byte rows of a 64-wide K slice; wavefront w covers rows 8 w .. 8 w + 7 of every
  // block of 64 rows).  Rows are not padded; instead the 16-byte chunk c of row r sits at chunk
  // position c ^ ((r >> 1) & 7), which the lane arranges by asking for the chunk that belongs at
  // ITS position - then the b128 fragment reads of 16 rows at one logical chunk hit all 64 banks.
  constexpr int kPassA = kGM / 64, kPassW = TN / 64;
  const int ld_r = wave * 8 + (lane >> 3);                                   // row within a block of 64
  const unsigned sw_c = (unsigned)(((lane & 7) ^ ((ld_r >> 1) & 7)) * 8);    // logical element offset this lane fetches
  unsigned a_off[kPassA];
#pragma unroll
  for (int j = 0; j < kPassA; ++j) a_off[j] = ((unsigned)min(m0 + ld_r + 64 * j, p.M - 1) * (unsigned)p.K + sw_c) * 2u;   // rows past M re-read the last row
  const unsigned w_off = ((unsigned)ld_r * (unsigned)p.K + sw_c) * 2u;
  const int nk = (SPLITK ? p.K / p.k_splits : p.K) / kKS;   // 64-wide steps of this workgroup
  const size_t k_first = SPLITK ? (size_t)split * nk * kKS : 0;
  const char* a_base = (const char*)(p.a + k_first);
  const char* w_base = (const char*)(p.w + (size_t)n0 * p.K + k_first);
  if (wave >= kGThreads / 64) {   // (a scalar condition: the whole wavefront branches)
    // The ninth wavefront holds no operand and joins no barrier (a wavefront that has ended is not
    // waited for).  In a model every launch finds its weights in HBM - a frame walks through far
    // more weight bytes than the caches hold - and the loop's three steps of look-ahead do not
    // cover that latency: the same launch takes 0.6 to 5 us longer on weights that no cache holds.
    // A caller that knows which memory the launch AFTER this one will read says so
    // (lbm_linear_prefetch_hint), and these wavefronts, all workgroups' together, read one dword of
    // every 128-byte line of it: the lines are then in the memory-side cache (or an L2) when that
    // launch starts, having travelled while this one computed.
    // (plain loads whose results the compiler sees - a load whose result it does not know of could
    // land in a register it has reused: eight in flight per lane, their values folded into a word
    // that is stored only under a condition that never holds)
    unsigned folded = 0;
    const unsigned stride = gridDim.x * 64u;
    for (unsigned first = blockIdx.x * 64u + (unsigned)lane; first < p.touch_lines; first += 8u * stride) {
      unsigned got[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const unsigned line = first + (unsigned)j * stride;
        got[j] = line < p.touch_lines ? *(const unsigned*)(p.touch + (size_t)line * 128) : 0u;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) folded ^= got[j];
    }
    if (folded == 0x5bd1e995u && p.M < 0) p.out[lane] = (unsigned short)folded;   // (M is never negative)
    return;
  }
  // The loads are written as inline assembly: the compiler would otherwise wait for every
  // LDS-direct load in flight before any LDS read that might alias it (it cannot tell the two
  // buffers apart), which serialises load and multiply.  M0 carries the LDS address of the
  // wavefront's KB (declared as clobbered, so the compiler keeps nothing of its own in M0 across
  // the load).  The waits for these loads are placed
  // by hand (dma_wait) - the compiler's own counts only see fewer loads in flight than there
  // are, which makes its waits stricter, never laxer.
  auto dma_row = [&](const char* base, unsigned voff, const unsigned short* lds_dst) {
    const unsigned m0v = (unsigned)(size_t)(__attribute__((address_space(3))) const void*)lds_dst;
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(base), "s"(__builtin_amdgcn_readfirstlane(m0v))
                 : "memory", "m0");
  };
  auto dma_step = [&](int ks, int stage) {
#pragma unroll
    for (int j = 0; j < kPassA; ++j)
      dma_row(a_base + ks * (kKS * 2), a_off[j], &lds_a[stage][(64 * j + 8 * wave) * kKS]);
#pragma unroll
    for (int j = 0; j < kPassW; ++j)
      dma_row(w_base + ((size_t)(64 * j) * p.K + (size_t)ks * kKS) * 2, w_off, &lds_w[stage][(64 * j + 8 * wave) * kKS]);
  };
  // the same loads one by one, for the loop: M0 values and row offsets as integers, so that
  // nothing but two scalar adds and the load itself sits between the MFMAs
  const unsigned m0_a = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) unsigned short*)&lds_a[0][0] + (unsigned)wave * 1024u);
  const unsigned m0_w = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) unsigned short*)&lds_w[0][0] + (unsigned)wave * 1024u);
  unsigned w_offs[kPassW];
#pragma unroll
  for (int j = 0; j < kPassW; ++j) w_offs[j] = w_off + (unsigned)(64 * j) * (unsigned)p.K * 2u;
  auto dma_one = [&](int ks, int stage, int j) {
    const char* base = (j < kPassA ? a_base : w_base) + (size_t)ks * (kKS * 2);
    const unsigned voff = j < kPassA ? a_off[j < kPassA ? j : 0] : w_offs[j < kPassA ? 0 : j - kPassA];
    const unsigned m0v = j < kPassA ? m0_a + (unsigned)(stage * kGM * kKS * 2 + 64 * j * kKS * 2)
                                    : m0_w + (unsigned)(stage * TN * kKS * 2 + 64 * (j - kPassA) * kKS * 2);
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base), "s"(m0v) : "memory", "m0");
  };
  // loads of this wavefront still allowed in flight: N (vmcnt(N); expcnt and lgkmcnt untouched)
  constexpr int kDmaPerStep = kPassA + kPassW;
#define LBM_DMA_WAIT(N) __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14))

  f32x16 acc[NT][2];   // [column block of W][row block of A]; element i: column 8 (i / 4) + 4 g + i % 4, row n32
#pragma unroll
  for (int a = 0; a < NT; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  // One 64-wide step: each wave group multiplies its 32-wide half.  The fragments of a step are
  // read during the step before it, one read in between two MFMAs (a burst of reads fills the LDS
  // queue and holds the MFMAs behind it back), into the other half of the fragment registers.
  const int sw_r = (n32 >> 1) & 7;
  bf16x8 wf[2][2][NT], af[2][2][2];   // [step parity][16-wide slice][block]
  auto read_one = [&](int stage, int buf, int i) {   // read i of a step's 2 (NT + 2), in the order the MFMAs use them
    const unsigned short* la = &lds_a[stage][0];
    const unsigned short* lw = &lds_w[stage][0];
    const int k16 = i / (NT + 2), j = i % (NT + 2);
    const int pos = ((kh * 4 + k16 * 2 + g) ^ sw_r) * 8;
    if (j == 0) wf[buf][k16][0] = __builtin_bit_cast(bf16x8, *(const u32x4*)&lw[(wn + n32) * kKS + pos]);
    else if (j <= 2) af[buf][k16][j - 1] = __builtin_bit_cast(bf16x8, *(const u32x4*)&la[(wm + ((j - 1) ^ kh) * 32 + n32) * kKS + pos]);
    else wf[buf][k16][j - 2] = __builtin_bit_cast(bf16x8, *(const u32x4*)&lw[(wn + (j - 2) * 32 + n32) * kKS + pos]);
  };
  auto read_slice = [&](int stage, int buf, int k16) {
#pragma unroll
    for (int i = 0; i < NT + 2; ++i) read_one(stage, buf, k16 * (NT + 2) + i);
  };
  auto read_step = [&](int stage, int buf) {
    read_slice(stage, buf, 0);
    read_slice(stage, buf, 1);
  };
  auto mfma_slice = [&](int buf, int k16) {
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[buf][k16][a], af[buf][k16][b], acc[a][b], 0, 0, 0);
  };

  // LNA, row statistics: row r of the tile is handled by threads 4 r .. 4 r + 3, each taking every
  // fourth (mean, M2) partial; equal-sized partials merge as mean = avg(mean_i),
  // M2 = sum(M2_i) + n_i * sum((mean_i - mean)^2) (Chan et al.), variance = M2 / K.  The partials
  // are asked for before the operand tiles (loads return in order) and merged while those travel.
  constexpr int kLnHeld = 4;     // partials a thread keeps in registers (up to 16 column tiles)
  f32x2 ln_part[kLnHeld] = {};
  const float* ln_st = nullptr;
  if (LNA) {
    ln_st = p.ln_stats + (size_t)min(m0 + (tid >> 2), p.M - 1) * p.ln_tiles * 2;
#pragma unroll
    for (int i = 0; i < kLnHeld; ++i)
      if ((tid & 3) + 4 * i < p.ln_tiles) ln_part[i] = *(const f32x2*)(ln_st + 2 * ((tid & 3) + 4 * i));
  }
  // The per-column vectors of the epilogue (bias, column sums of w, LayerScale) are asked for now
  // and parked in LDS behind the first operand loads; the loop's barriers publish them.
  float cv_bias = 0.f, cv_sum = 0.f, cv_gamma = 1.f;
  if (tid < TN) {
    if (p.bias) cv_bias = p.bias[n0 + tid];
    if (LNA) cv_sum = p.ln_colsum[n0 + tid];
    if (EPI == LBM_LINEAR_BIAS_RESIDUAL && p.gamma) cv_gamma = p.gamma[n0 + tid];
  }
  // The GELU table travels first (480 threads x 16 bytes; the loads return in order, so the wait
  // for the first operand tile covers it and the barrier behind that wait publishes it) ...
  if (EPI == LBM_LINEAR_BIAS_GELU && tid < kGeluEntries / 8)
    dma_row((const char*)g_gelu_table, (unsigned)tid * 16u, &gelu_tab[wave * 512]);
  // ... then three steps ahead: steps 0, 1, 2 on their way before anything else happens
#pragma unroll
  for (int i = 0; i < kStagesG - 1; ++i)
    if (i < nk) dma_step(i, i);
  if (tid < TN) {
    colvec[0][tid] = cv_bias;
    colvec[1][tid] = cv_sum;
    colvec[2][tid] = cv_gamma;
  }
  if (LNA) {
    const int r = tid >> 2, part = tid & 3;
    float sm = 0.f;
#pragma unroll
    for (int i = 0; i < kLnHeld; ++i)
      if (part + 4 * i < p.ln_tiles) sm += ln_part[i][0];
    for (int i = part + 4 * kLnHeld; i < p.ln_tiles; i += 4) sm += ln_st[2 * i];
    sm += lbm_qkv::lane_xor1(sm);
    sm += lbm_qkv::lane_xor2(sm);
    const float mean = sm / (float)p.ln_tiles;
    const float n_i = (float)p.K / (float)p.ln_tiles;
    float m2 = 0.f;
#pragma unroll
    for (int i = 0; i < kLnHeld; ++i)
      if (part + 4 * i < p.ln_tiles) {
        const float d = ln_part[i][0] - mean;
        m2 += ln_part[i][1] + n_i * d * d;
      }
    for (int i = part + 4 * kLnHeld; i < p.ln_tiles; i += 4) {
      const float d = ln_st[2 * i] - mean;
      m2 += ln_st[2 * i + 1] + n_i * d * d;
    }
    m2 += lbm_qkv::lane_xor1(m2);
    m2 += lbm_qkv::lane_xor2(m2);
    const float rstd = __builtin_amdgcn_rsqf(m2 / (float)p.K + p.ln_eps);
    if (part == 0) {
      ln_rows[2 * r] = rstd;
      ln_rows[2 * r + 1] = -mean * rstd;
    }
    // (read in the epilogue, many barriers from here)
  }
  // Step 0's fragments: its rows have landed (steps 1 and 2 may still be in flight), barrier, read.
  if (2 < nk) LBM_DMA_WAIT(2 * kDmaPerStep);
  else LBM_DMA_WAIT(kDmaPerStep);
  __syncthreads();
  read_step(0, 0);
  if (kStagesG - 1 < nk) dma_step(kStagesG - 1, kStagesG - 1);
  // Step s: wait until the rows of step s + 1 have landed (the loads of steps s + 2 and s + 3 may
  // still be in flight), barrier (everyone's rows of step s + 1 are there, and everyone holds the
  // fragments of step s in registers, so its stage is free), then the MFMAs of step s with the
  // fragment reads of step s + 1 in between, then the loads of step s + 4 into the freed stage.
  static_assert(kStagesG == 4, "the loop is written for a ring of four stages");
#define LBM_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
  for (int s0 = 0; s0 < nk; s0 += kStagesG) {
#pragma unroll
    for (int st = 0; st < kStagesG; ++st) {
      const int sidx = s0 + st;
      if (sidx < nk) {
        if (sidx + 3 < nk) LBM_DMA_WAIT(2 * kDmaPerStep);
        else if (sidx + 2 < nk) LBM_DMA_WAIT(kDmaPerStep);
        else LBM_DMA_WAIT(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        const bool more = sidx + kStagesG < nk;
#pragma unroll
        for (int k16 = 0; k16 < 2; ++k16) {
          read_slice((st + 1) % kStagesG, (st + 1) & 1, k16);   // (past the last step: stale rows, never used)
          mfma_slice(st & 1, k16);
#pragma unroll
          for (int i = 0; i < NT + 2; ++i) { LBM_SGB(0x008, 1); LBM_SGB(0x100, 1); }
          __builtin_amdgcn_sched_barrier(0);
          if (more) {
#pragma unroll
            for (int j = 0; j < kDmaPerStep; ++j)
              if (j * 2 / kDmaPerStep == k16) dma_one(sidx + kStagesG, st, j);
          }
        }
      }
    }
  }
#undef LBM_SGB
  __syncthreads();

  // What the epilogue needs from global memory beyond the per-column vectors is asked for here,
  // all at once, and arrives while the wave groups exchange their sums (asked for where it is
  // used - per pass - every load would wait out a trip to L2 or HBM on its own, and behind the
  // stores of the pass before it; asked for before the multiply, it delays the first operand
  // tiles):
  // the residual rows of the store passes (a workgroup that shares its tile under SPLITK
  // asks only once it knows that it is the one to store).
  constexpr int kPieces = TN / 8;                 // 16-byte pieces per row of the tile
  constexpr int kRowsPerPass = kGThreads / kPieces;
  constexpr int kPasses = kGM / kRowsPerPass;
  u32x4 res_v[kPasses] = {};
  auto load_residual = [&]() {
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
      const int row = min(m0 + j * kRowsPerPass + tid / kPieces, p.M - 1);   // rows past M: read, never stored
      res_v[j] = *(const u32x4*)(p.res + (size_t)row * p.N + n0 + (tid % kPieces) * 8);
    }
  };
  if (EPI == LBM_LINEAR_BIAS_RESIDUAL && !SPLITK) load_residual();
  // The producer's own inputs - q/k norm weights, every pass's rotary table entries and pool rows -
  // are asked for now as well.
  const int H = p.num_heads;
  struct {
    int c, which, h, c8;
    lbm_qkv::f32x4 w4[2], b4[2], cs4[kPasses][4];
    int pool_row[kPasses];
  } pq = {};
  if (EPI == kEpiQkvPrepare) {
    typedef lbm_qkv::f32x4 qf4;
    pq.c = (tid % kPieces) * 8;
    const int col = n0 + pq.c;                    // column of the projection: [q|k|v][head][64]
    pq.which = col / (H * 64);                    // uniform over the workgroup (H * 64 is a multiple of TN)
    pq.h = (col - pq.which * H * 64) >> 6;
    pq.c8 = (col & 63) >> 3;                      // = tid % 8: the lane's place in its row of 64
    if (NORM && pq.which < 2) {
      const qf4* wp = (const qf4*)((pq.which == 0 ? p.q_norm_w : p.k_norm_w) + pq.c8 * 8);
      const qf4* bp = (const qf4*)((pq.which == 0 ? p.q_norm_b : p.k_norm_b) + pq.c8 * 8);
      pq.w4[0] = wp[0]; pq.w4[1] = wp[1];
      pq.b4[0] = bp[0]; pq.b4[1] = bp[1];
    }
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
      const int t = min(m0 + j * kRowsPerPass + tid / kPieces, p.M - 1);
      if (ROPE == 1 && pq.which < 2) {
        const qf4* cs = (const qf4*)(p.rope_cs + ((long long)t * 32 + pq.c8 * 4) * 2);
        pq.cs4[j][0] = cs[0]; pq.cs4[j][1] = cs[1];
      } else if (ROPE == 2 && pq.which < 2) {
        const qf4* cs = (const qf4*)(p.rope_cs + ((long long)t * 64 + pq.c8 * 8) * 2);
        pq.cs4[j][0] = cs[0]; pq.cs4[j][1] = cs[1]; pq.cs4[j][2] = cs[2]; pq.cs4[j][3] = cs[3];
      }
      pq.pool_row[j] = -1;
      if (pq.which > 0 && p.append_rows) pq.pool_row[j] = p.append_rows[t];
    }
  }
  // ---- the two wave groups' sums meet: group 0 finishes row block 0 of every sub-tile, group 1
  // row block 1; each parks the other's half in LDS (the operand buffers are dead)
  float* xch = (float*)&lds_a[0][0];            // [wave][NT][4][64 lanes][4] floats
  static_assert(8 * NT * 16 * 64 * 4 <= (int)sizeof(lds_a), "the exchanged halves fit the activation buffers");
  // (the second wave group reads its activation fragments with the two row blocks swapped, so
  // for both groups acc[.][0] is the block they finish and acc[.][1] the one they hand over)
  f32x16 fin[NT];
  {
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        f32x4 give;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          give[e] = acc[a][1][q * 4 + e];
          fin[a][q * 4 + e] = acc[a][0][q * 4 + e];
        }
        *(f32x4*)&xch[(((wave * NT + a) * 4 + q) * 64 + lane) * 4] = give;
      }
    // (a barrier that waits for the LDS writes only: the loads asked for above stay in flight)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const int peer = wave ^ 4;
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x4 got = *(const f32x4*)&xch[(((peer * NT + a) * 4 + q) * 64 + lane) * 4];
#pragma unroll
        for (int e = 0; e < 4; ++e) fin[a][q * 4 + e] += got[e];
      }
  }
  const int b = kh;     // the row block this wave finishes
  if (SPLITK) {
    // Partials and counters travel as scope-qualified relaxed atomics, which go past the caches
    // that are not coherent between workgroups (the CU's and, between XCDs, the L2) - a
    // device-wide fence would write back and invalidate the whole L2 instead, once per
    // workgroup (measured: 60 us on a 25 us launch).  Order: every thread waits until its own
    // stores are acknowledged (an explicit s_waitcnt vmcnt(0): the stores are write-through, so an
    // acknowledged store is visible device-wide, and a workgroup-scope fence alone does not wait
    // for it), the barrier collects all threads, only then thread 0 draws the ticket.
    __shared__ unsigned ticket_lds;
    const int tile = mt * p.n_tiles + nt;
    constexpr int kPartFloats = 8 * NT * 16 * 64;                 // one workgroup's partial tile
    float* tile_part = p.split_part + (size_t)tile * p.k_splits * kPartFloats;
    float* mine = tile_part + (size_t)split * kPartFloats + (size_t)wave * (NT * 16 * 64);
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        __hip_atomic_store(&mine[(a * 16 + i) * 64 + lane], fin[a][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    LBM_DMA_WAIT(0);
    __syncthreads();
    if (tid == 0) ticket_lds = __hip_atomic_fetch_add(&p.split_counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket_lds != (unsigned)(p.k_splits - 1)) return;          // (uniform over the workgroup)
    if (tid == 0) __hip_atomic_store(&p.split_counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // as the next launch expects it
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (EPI == LBM_LINEAR_BIAS_RESIDUAL) load_residual();
    // two slices: this workgroup's own sum is still in its registers and a + b = b + a; more
    // slices: all of them from memory, in slice order, so the sum does not depend on who is last
    const bool pair = p.k_splits == 2;
    if (!pair) {
#pragma unroll
      for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int i = 0; i < 16; ++i) fin[a][i] = 0.f;
    }
    for (int sidx = pair ? 1 - split : 0; sidx < (pair ? 2 - split : p.k_splits); ++sidx) {
      const float* src = tile_part + (size_t)sidx * kPartFloats + (size_t)wave * (NT * 16 * 64);
#pragma unroll
      for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          fin[a][i] += __hip_atomic_load(&src[(a * 16 + i) * 64 + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }

  // ---- epilogue.  In registers: + bias, round (the linear's output), GELU or LayerScale, round.
  // Then the tile goes through LDS and leaves as whole rows.
  constexpr int kCStride = TN + 4;   // bf16 per staged row: 8-byte writes of 32 rows hit 64 distinct banks
  unsigned short* stage = (unsigned short*)&lds_w[0][0];
  f32x2 row_f = {1.f, 0.f};   // this lane's output row: rstd, -mean * rstd
  if (LNA) row_f = *(const f32x2*)&ln_rows[2 * (wm + b * 32 + n32)];
  static_assert(kGM * kCStride * 2 <= (int)sizeof(lds_w), "the staged tile fits the weight buffers");
#pragma unroll
  for (int a = 0; a < NT; ++a)
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) {
      const int col = wn + a * 32 + c4 * 8 + g * 4;     // four consecutive output columns
      const f32x4 bias4 = *(const f32x4*)&colvec[0][col], colsum4 = *(const f32x4*)&colvec[1][col], gamma4 = *(const f32x4*)&colvec[2][col];
      f32x4 y;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float lin = fin[a][c4 * 4 + e];
        if (LNA) lin = __builtin_fmaf(lin, row_f[0], row_f[1] * colsum4[e]);   // rstd * acc - mean * rstd * colsum
        float v = round_bf16(lin + bias4[e]);
        if (EPI == LBM_LINEAR_BIAS_GELU) v = gelu_of_bf16(v, gelu_tab);
        if (EPI == LBM_LINEAR_BIAS_RESIDUAL && p.gamma) v = v * gamma4[e];
        y[e] = v;
      }
      *(bf16x4*)&stage[(wm + b * 32 + n32) * kCStride + col] = __builtin_convertvector(y, bf16x4);
    }
  __syncthreads();
  if (EPI == kEpiQkvPrepare) {
    // The staged tile holds the projection's output rounded to bf16, 8 consecutive columns per
    // thread: exactly the producer's layout (8 lanes per (token, q|k|v, head) row of 64), so its
    // LayerNorm, rotary embedding and scatter run here instead of in a pass of their own
    // (lingbot_map/layers/attention.py:402-426, rope.py:438-461, flashinfer_cache.py:215-218).
    unsigned short* dst_plain = pq.which == 0 ? p.out : (pq.which == 1 ? p.k_out : p.v_out);
#pragma unroll
    for (int j = 0; j < kPasses; ++j) {
      const int r = j * kRowsPerPass + tid / kPieces;
      const bool valid = m0 + r < p.M;            // rows past M computed on the last token's entries, never stored
      const u32x2 lo = *(const u32x2*)&stage[r * kCStride + pq.c], hi = *(const u32x2*)&stage[r * kCStride + pq.c + 4];
      const u32x4 raw = {lo[0], lo[1], hi[0], hi[1]};
      bf16x8 o8 = __builtin_bit_cast(bf16x8, raw);   // v rows leave as they are
      if (pq.which < 2) {
        // q and k rows: the row's last rounding is the conversion that packs it
        float x[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = __builtin_bit_cast(float, (i & 1) ? (raw[i >> 1] & 0xffff0000u) : (raw[i >> 1] << 16));
        lbm_qkv::norm_rope_unrounded<0, ROPE, NORM>(x, pq.w4, pq.b4, pq.cs4[j], pq.c8, p.eps, pq.which == 0 ? p.q_scale : 1.0f);
#pragma unroll
        for (int i = 0; i < 8; ++i) o8[i] = (__bf16)x[i];
      }
      if (valid) {
        const long long nhd = ((long long)(m0 + r) * H + pq.h) * 64 + pq.c8 * 8;
        if (dst_plain) *(bf16x8*)(dst_plain + nhd) = o8;
        if (pq.which > 0 && pq.pool_row[j] >= 0) {
          const long long row_elems = (long long)H * 64;
          const long long d = (long long)pq.pool_row[j] * row_elems + (pq.which == 2 ? (long long)p.page_size * row_elems : 0) +
                              pq.h * 64 + pq.c8 * 8;
          *(bf16x8*)(p.pool + d) = o8;
        }
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < kPasses; ++j) {
    const int r = j * kRowsPerPass + tid / kPieces, c = (tid % kPieces) * 8;
    const int row = m0 + r;
    // (an 8-byte aligned read of the padded row: two halves)
    const u32x2 lo = *(const u32x2*)&stage[r * kCStride + c], hi = *(const u32x2*)&stage[r * kCStride + c + 4];
    u32x4 v = {lo[0], lo[1], hi[0], hi[1]};
    if (row < p.M) {
      unsigned short* dst = p.out + (size_t)row * p.N + n0 + c;
      if (EPI == LBM_LINEAR_BIAS_RESIDUAL) {
        const u32x4 x = res_v[j];
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float s0 = bf16_bits_to_f32(x[e] & 0xffffu) + bf16_bits_to_f32(v[e] & 0xffffu);
          const float s1 = bf16_bits_to_f32(x[e] >> 16) + bf16_bits_to_f32(v[e] >> 16);
          o[e] = (unsigned)__builtin_bit_cast(unsigned short, (__bf16)s0) | ((unsigned)__builtin_bit_cast(unsigned short, (__bf16)s1) << 16);
        }
        v = o;
      }
      *(u32x4*)dst = v;
    }
    if (EPI == LBM_LINEAR_BIAS_RESIDUAL && p.stats_out) {
      // (mean, M2) of the row's TN stored values: the kPieces lanes that hold the row are
      // neighbours inside one 16-lane group
      float x[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[2 * e] = bf16_bits_to_f32(v[e] & 0xffffu);
        x[2 * e + 1] = bf16_bits_to_f32(v[e] >> 16);
      }
      float sm = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
      sm = lbm_qkv::sum_of_8(sm);
      if (kPieces == 16) sm += lbm_qkv::other_half_of_16(sm);
      const float mean = sm / (float)TN;
      float m2 = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) m2 += (x[e] - mean) * (x[e] - mean);
      m2 = lbm_qkv::sum_of_8(m2);
      if (kPieces == 16) m2 += lbm_qkv::other_half_of_16(m2);
      if (row < p.M && (tid % kPieces) == 0) {
        float* so = p.stats_out + ((size_t)row * p.n_tiles + nt) * 2;
        so[0] = mean;
        so[1] = m2;
      }
    }
  }
}


// ---------------------------------------------------------------------------- several streams' rows
// The same product on 256 x 256 (or 192 x 256) tiles, for launches with enough rows to give most
// of the 256 CUs such a tile (four streams' 4,016 rows x the qkv projection's 3,072 or fc1's
// 4,096 columns): a 256 x 256 tile moves 64 KB of operands per 64 of K for 8.4 MFLOP - 128 FLOP
// per byte on the way from L2 into LDS, which is what bounds the 128 x 128 tiles above at 64.
// Eight wavefronts, each on 64 rows x 128 columns of the tile (96 x 64 of a 192-row tile) over
// the whole K slice, no K split inside the workgroup and so no exchange at the end.  Two LDS
// stages: a 64-wide step is 24-32 MFMAs per wavefront, longer than a trip to memory, so one step
// of prefetch is enough; the loads of a step are issued at the end of the step before the one
// they replace, right behind the barrier that frees its stage.  Same operand path (global -> LDS directly, swizzled 16-byte chunks), same
// epilogue arithmetic and rounding sequence.  Epilogues: bias, bias + GELU, and the
// pre-attention producer; the folded LayerNorm of the activations; not the residual forms (their
// 1,024 columns make too few such tiles).  The per-column vectors wait in LDS instead of
// registers (the accumulators take half the register file).  192-row tiles are for shapes whose
// 256-row tiles would leave a quarter of the CUs idle (4,016 x 3,072: 192 against 252 tiles).
constexpr int kBN = 256;
constexpr int kBCStride = kBN + 4;                          // bf16 per staged output row
constexpr int lbm_big_lds_bytes(int bm) {
  return bm * kBCStride * 2 > 2 * (bm + kBN) * kKS * 2 ? bm * kBCStride * 2 : 2 * (bm + kBN) * kKS * 2;
}
static_assert(lbm_big_lds_bytes(256) + kGeluEntries * 2 + 2 * kBN * 4 + 256 * 8 <= 160 * 1024, "LDS budget of the 256 x 256 tile");

template <int BM, int EPI, int ROPE = 0, bool NORM = false, bool LNA = false>
__global__ __launch_bounds__(kGThreads, 1) void lbm_linear_bf16_big_kernel(LinearArgs p) {
  constexpr int kRowGroups = BM == 256 ? 4 : 2;             // wavefronts along the rows of the tile
  constexpr int kColGroups = 8 / kRowGroups;
  constexpr int RB = BM / 32 / kRowGroups, CB = kBN / 32 / kColGroups;   // 32 x 32 blocks per wavefront: 2 x 4 or 3 x 2
  constexpr int kStageBytes = (BM + kBN) * kKS * 2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[lbm_big_lds_bytes(BM)];   // two operand stages, then the staged output tile
  __shared__ __attribute__((aligned(16))) float colvec[2][kBN];                             // bias, column sums of w (LNA)
  __shared__ __attribute__((aligned(16))) unsigned short gelu_tab[EPI == LBM_LINEAR_BIAS_GELU ? kGeluEntries : 8];
  __shared__ __attribute__((aligned(8))) float ln_rows[LNA ? BM * 2 : 2];                   // per row: rstd, -mean * rstd

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n32 = lane & 31, g = lane >> 5;
  const int rg = wave % kRowGroups, cg = wave / kRowGroups;
  const int wm = rg * (RB * 32), wn = cg * (CB * 32);       // this wavefront's corner of the tile
  int mt, nt;
  lbm_tile_of_workgroup((int)blockIdx.x, p.m_tiles, p.n_tiles, mt, nt);
  const int m0 = mt * BM, n0 = nt * kBN;

  // ---- staging (as in the kernel above: eight 128-byte rows per wavefront and load)
  constexpr int kPassA = BM / 64, kPassW = kBN / 64;
  const int ld_r = wave * 8 + (lane >> 3);
  const unsigned sw_c = (unsigned)(((lane & 7) ^ ((ld_r >> 1) & 7)) * 8);
  unsigned a_off[kPassA];
#pragma unroll
  for (int j = 0; j < kPassA; ++j) a_off[j] = ((unsigned)min(m0 + ld_r + 64 * j, p.M - 1) * (unsigned)p.K + sw_c) * 2u;
  const unsigned w_off = ((unsigned)ld_r * (unsigned)p.K + sw_c) * 2u;
  const int nk = p.K / kKS;
  const char* a_base = (const char*)p.a;
  const char* w_base = (const char*)(p.w + (size_t)n0 * p.K);
  auto dma_row = [&](const char* base, unsigned voff, const unsigned char* lds_dst) {
    const unsigned m0v = (unsigned)(size_t)(__attribute__((address_space(3))) const void*)lds_dst;
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(base), "s"(__builtin_amdgcn_readfirstlane(m0v))
                 : "memory", "m0");
  };
  // load j of step ks: the activations' passes first, then the weights'
  auto dma_one = [&](int ks, int stage, int j) {
    unsigned char* st = lds_raw + stage * kStageBytes;
    if (j < kPassA) dma_row(a_base + ks * (kKS * 2), a_off[j], st + (64 * j + 8 * wave) * (kKS * 2));
    else dma_row(w_base + ((size_t)(64 * (j - kPassA)) * p.K + (size_t)ks * kKS) * 2, w_off,
                 st + BM * kKS * 2 + (64 * (j - kPassA) + 8 * wave) * (kKS * 2));
  };
  constexpr int kDma = kPassA + kPassW;

  // the folded LayerNorm's row statistics: two threads per row, each every second partial
  constexpr int kLnHeld = 8;
  f32x2 ln_part[kLnHeld] = {};
  if (LNA) {
    const float* ln_st = p.ln_stats + (size_t)min(m0 + (tid >> 1), p.M - 1) * p.ln_tiles * 2;
#pragma unroll
    for (int i = 0; i < kLnHeld; ++i)
      if ((tid & 1) + 2 * i < p.ln_tiles) ln_part[i] = *(const f32x2*)(ln_st + 2 * ((tid & 1) + 2 * i));
  }
  // per-column vectors of the tile into LDS (read in the epilogue, many barriers from here)
  float cv_bias = 0.f, cv_sum = 0.f;
  if (tid < kBN) {
    if (p.bias) cv_bias = p.bias[n0 + tid];
    if (LNA) cv_sum = p.ln_colsum[n0 + tid];
  }
  if (EPI == LBM_LINEAR_BIAS_GELU && tid < kGeluEntries / 8)
    dma_row((const char*)g_gelu_table, (unsigned)tid * 16u, (const unsigned char*)&gelu_tab[wave * 512]);
#pragma unroll
  for (int j = 0; j < kDma; ++j) dma_one(0, 0, j);
  if (tid < kBN) {
    colvec[0][tid] = cv_bias;
    colvec[1][tid] = cv_sum;
  }
  if (LNA && (tid >> 1) < BM) {
    const int r = tid >> 1, part = tid & 1;
    const float* ln_st = p.ln_stats + (size_t)min(m0 + r, p.M - 1) * p.ln_tiles * 2;
    float sm = 0.f;
#pragma unroll
    for (int i = 0; i < kLnHeld; ++i)
      if (part + 2 * i < p.ln_tiles) sm += ln_part[i][0];
    for (int i = part + 2 * kLnHeld; i < p.ln_tiles; i += 2) sm += ln_st[2 * i];
    sm += lbm_qkv::lane_xor1(sm);
    const float mean = sm / (float)p.ln_tiles;
    const float n_i = (float)p.K / (float)p.ln_tiles;
    float m2 = 0.f;
#pragma unroll
    for (int i = 0; i < kLnHeld; ++i)
      if (part + 2 * i < p.ln_tiles) {
        const float d = ln_part[i][0] - mean;
        m2 += ln_part[i][1] + n_i * d * d;
      }
    for (int i = part + 2 * kLnHeld; i < p.ln_tiles; i += 2) {
      const float d = ln_st[2 * i] - mean;
      m2 += ln_st[2 * i + 1] + n_i * d * d;
    }
    m2 += lbm_qkv::lane_xor1(m2);
    const float rstd = __builtin_amdgcn_rsqf(m2 / (float)p.K + p.ln_eps);
    if (part == 0) {
      ln_rows[2 * r] = rstd;
      ln_rows[2 * r + 1] = -mean * rstd;
    }
  }

  f32x16 acc[CB][RB];   // [column block of w][row block of a]; element i: column 8 (i / 4) + 4 g + i % 4, row n32
#pragma unroll
  for (int a = 0; a < CB; ++a)
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  const int sw_r = (n32 >> 1) & 7;
  // M0 values as integers (no pointer cast inside the loop): this wavefront's KB of every block of 64 rows
  const unsigned m0_wave = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds_raw + (unsigned)wave * 1024u);
  unsigned w_offs[kPassW];
#pragma unroll
  for (int j = 0; j < kPassW; ++j) w_offs[j] = w_off + (unsigned)(64 * j) * (unsigned)p.K * 2u;
  auto dma_at = [&](const char* base, unsigned voff, unsigned m0v) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base), "s"(m0v) : "memory", "m0");
  };
  auto dma_step = [&](int ks, unsigned stage_bytes) {
    const char* ab = a_base + (size_t)ks * (kKS * 2);
    const char* wb = w_base + (size_t)ks * (kKS * 2);
#pragma unroll
    for (int j = 0; j < kPassA; ++j) dma_at(ab, a_off[j], m0_wave + stage_bytes + (unsigned)(64 * j * kKS * 2));
#pragma unroll
    for (int j = 0; j < kPassW; ++j) dma_at(wb, w_offs[j], m0_wave + stage_bytes + (unsigned)((BM + 64 * j) * kKS * 2));
  };
  bf16x8 wf[2][CB], af[2][RB];
  auto read = [&](unsigned stage_bytes, int kq, bf16x8 (&wfr)[CB], bf16x8 (&afr)[RB]) {
    const unsigned char* la = lds_raw + stage_bytes;
    const unsigned char* lw = la + BM * kKS * 2;
    const int posb = ((kq * 2 + g) ^ sw_r) * 16;
#pragma unroll
    for (int a = 0; a < CB; ++a)
      wfr[a] = __builtin_bit_cast(bf16x8, *(const u32x4*)(lw + (wn + a * 32 + n32) * (kKS * 2) + posb));
#pragma unroll
    for (int b = 0; b < RB; ++b)
      afr[b] = __builtin_bit_cast(bf16x8, *(const u32x4*)(la + (wm + b * 32 + n32) * (kKS * 2) + posb));
  };
  auto mfmas = [&](int kq, int from, int to) {
#pragma unroll
    for (int a = 0; a < CB; ++a)
#pragma unroll
      for (int b = 0; b < RB; ++b)
        if (a * RB + b >= from && a * RB + b < to)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[kq & 1][a], af[kq & 1][b], acc[a][b], 0, 0, 0);
  };
#define LBM_SGB(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
  // One 64-wide step on the stage at byte `here`.  The fragment reads of a quarter step are
  // issued one by one in between the MFMAs of the quarter before it (a burst of them fills the
  // LDS queue and stalls the wavefront's MFMAs behind it).  The barrier that hands the other
  // stage over sits in the middle of the last quarter: behind it come the first fragment reads
  // of the next step, covered by the quarter's remaining MFMAs, and at the end of the step the
  // loads of the step after the next one, which have a whole step to land.
  constexpr int kQ = CB * RB, kR = CB + RB, kH = kQ / 2;
  auto step = [&](int s, auto stage_c) {
    constexpr unsigned here = decltype(stage_c)::value * kStageBytes, there = kStageBytes - here;
#pragma unroll
    for (int kq = 0; kq < 3; ++kq) {
      read(here, kq + 1, wf[(kq + 1) & 1], af[(kq + 1) & 1]);
      mfmas(kq, 0, kQ);
#pragma unroll
      for (int i = 0; i < kR; ++i) { LBM_SGB(0x008, 1); LBM_SGB(0x100, 1); }
      LBM_SGB(0x008, kQ - kR);
      __builtin_amdgcn_sched_barrier(0);
    }
    mfmas(3, 0, kH);
    __builtin_amdgcn_sched_barrier(0);
    LBM_DMA_WAIT(0);
    __syncthreads();   // the other stage has landed everywhere, and everyone has read all of this one
    __builtin_amdgcn_sched_barrier(0);
    read(there, 0, wf[0], af[0]);
    mfmas(3, kH, kQ);
    LBM_SGB(0x100, kR - (kQ - kH) + 1 > 0 ? kR - (kQ - kH) + 1 : 0);
#pragma unroll
    for (int i = 0; i < kQ - kH; ++i) { LBM_SGB(0x008, 1); LBM_SGB(0x100, 1); }
    __builtin_amdgcn_sched_barrier(0);
    if (s + 2 < nk) dma_step(s + 2, here);
  };
  LBM_DMA_WAIT(0);
  __syncthreads();
  dma_step(1, kStageBytes);
  read(0, 0, wf[0], af[0]);
  for (int s = 0; s < nk; s += 2) {
    step(s, std::integral_constant<unsigned, 0>{});
    step(s + 1, std::integral_constant<unsigned, 1>{});
  }
#undef LBM_SGB

  // ---- epilogue.  What the producer's first passes need from global memory is asked for now and
  // arrives while the tile is staged.
  constexpr int kPieces = kBN / 8;                    // 16-byte pieces per row of the tile: 32
  constexpr int kRowsPerPass = kGThreads / kPieces;   // 16
  constexpr int kPasses = BM / kRowsPerPass;          // 16 or 12
  constexpr int kGroup = 4;                           // passes whose rotary entries and pool rows travel together
  const int pr = tid / kPieces, pc = (tid % kPieces) * 8;
  typedef lbm_qkv::f32x4 qf4;
  const int H = p.num_heads;
  const int pq_col = n0 + pc;
  const int which = EPI == kEpiQkvPrepare ? pq_col / (H * 64) : 0;   // uniform over the workgroup (H * 64 is a multiple of 256)
  const int ph = (pq_col - which * H * 64) >> 6, c8 = (pq_col & 63) >> 3;
  qf4 w4[2] = {}, b4[2] = {};
  qf4 cs4[2][kGroup][4] = {};
  int pool_row[2][kGroup];
  auto ask = [&](int grp, qf4 (&cs)[kGroup][4], int (&rows)[kGroup]) {
#pragma unroll
    for (int j = 0; j < kGroup; ++j) {
      const int t = min(m0 + (grp * kGroup + j) * kRowsPerPass + pr, p.M - 1);
      if (ROPE == 1 && which < 2) {
        const qf4* src = (const qf4*)(p.rope_cs + ((long long)t * 32 + c8 * 4) * 2);
        cs[j][0] = src[0]; cs[j][1] = src[1];
      } else if (ROPE == 2 && which < 2) {
        const qf4* src = (const qf4*)(p.rope_cs + ((long long)t * 64 + c8 * 8) * 2);
        cs[j][0] = src[0]; cs[j][1] = src[1]; cs[j][2] = src[2]; cs[j][3] = src[3];
      }
      rows[j] = -1;
      if (which > 0 && p.append_rows) rows[j] = p.append_rows[t];
    }
  };
  if (EPI == kEpiQkvPrepare) {
    if (NORM && which < 2) {
      const qf4* wp = (const qf4*)((which == 0 ? p.q_norm_w : p.k_norm_w) + c8 * 8);
      const qf4* bp = (const qf4*)((which == 0 ? p.q_norm_b : p.k_norm_b) + c8 * 8);
      w4[0] = wp[0]; w4[1] = wp[1];
      b4[0] = bp[0]; b4[1] = bp[1];
    }
    ask(0, cs4[0], pool_row[0]);
  }
  __syncthreads();   // the operand stages are dead: the output tile is staged over them
  // In registers: the folded LayerNorm's scale and correction, + bias, round (the linear's
  // output), GELU, round; then the tile goes through LDS and leaves as whole rows.
  unsigned short* stage = (unsigned short*)lds_raw;
#pragma unroll
  for (int b = 0; b < RB; ++b) {
    const int row = wm + b * 32 + n32;
    f32x2 row_f = {1.f, 0.f};
    if (LNA) row_f = *(const f32x2*)&ln_rows[2 * row];
#pragma unroll
    for (int a = 0; a < CB; ++a)
#pragma unroll
      for (int c4 = 0; c4 < 4; ++c4) {
        const int col = wn + a * 32 + c4 * 8 + g * 4;
        const f32x4 bias4 = *(const f32x4*)&colvec[0][col], colsum4 = *(const f32x4*)&colvec[1][col];
        f32x4 y;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float lin = acc[a][b][c4 * 4 + e];
          if (LNA) lin = __builtin_fmaf(lin, row_f[0], row_f[1] * colsum4[e]);
          float v = round_bf16(lin + bias4[e]);
          if (EPI == LBM_LINEAR_BIAS_GELU) v = gelu_of_bf16(v, gelu_tab);
          y[e] = v;
        }
        *(bf16x4*)&stage[row * kBCStride + col] = __builtin_convertvector(y, bf16x4);
      }
  }
  __syncthreads();
  if (EPI == kEpiQkvPrepare) {
    // the producer on the staged tile, as in the kernel above; the rotary entries and pool rows of
    // four passes are asked for while the four before them are worked on
    unsigned short* dst_plain = which == 0 ? p.out : (which == 1 ? p.k_out : p.v_out);
    const float post = which == 0 ? p.q_scale : 1.0f;
    auto work = [&](int grp, const qf4 (&cs)[kGroup][4], const int (&rows)[kGroup]) {
#pragma unroll
      for (int j = 0; j < kGroup; ++j) {
        const int r = (grp * kGroup + j) * kRowsPerPass + pr;
        const bool valid = m0 + r < p.M;
        const u32x2 lo = *(const u32x2*)&stage[r * kBCStride + pc], hi = *(const u32x2*)&stage[r * kBCStride + pc + 4];
        const u32x4 raw = {lo[0], lo[1], hi[0], hi[1]};
        bf16x8 o8 = __builtin_bit_cast(bf16x8, raw);   // v rows leave as they are
        if (which < 2) {
          // q and k rows: the row's last rounding is the conversion that packs it
          float x[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) x[i] = __builtin_bit_cast(float, (i & 1) ? (raw[i >> 1] & 0xffff0000u) : (raw[i >> 1] << 16));
          lbm_qkv::norm_rope_unrounded<0, ROPE, NORM>(x, w4, b4, cs[j], c8, p.eps, post);
#pragma unroll
          for (int i = 0; i < 8; ++i) o8[i] = (__bf16)x[i];
        }
        if (valid) {
          const long long nhd = ((long long)(m0 + r) * H + ph) * 64 + c8 * 8;
          if (dst_plain) *(bf16x8*)(dst_plain + nhd) = o8;
          if (which > 0 && rows[j] >= 0) {
            const long long row_elems = (long long)H * 64;
            const long long d = (long long)rows[j] * row_elems + (which == 2 ? (long long)p.page_size * row_elems : 0) + ph * 64 + c8 * 8;
            *(bf16x8*)(p.pool + d) = o8;
          }
        }
      }
    };
#pragma unroll
    for (int grp = 0; grp < kPasses / kGroup; ++grp) {
      if (grp + 1 < kPasses / kGroup) ask(grp + 1, cs4[(grp + 1) & 1], pool_row[(grp + 1) & 1]);
      work(grp, cs4[grp & 1], pool_row[grp & 1]);
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < kPasses; ++j) {
    const int r = j * kRowsPerPass + pr, row = m0 + r;
    const u32x2 lo = *(const u32x2*)&stage[r * kBCStride + pc], hi = *(const u32x2*)&stage[r * kBCStride + pc + 4];
    if (row < p.M) *(u32x4*)(p.out + (size_t)row * p.N + n0 + pc) = u32x4{lo[0], lo[1], hi[0], hi[1]};
  }
}

}  // namespace

namespace {
// tile width: 128 columns when that gives the 256 CUs at least most of a round of workgroups (and
// N splits into 128s), 64 otherwise (N = 1024 at one frame: 128 tiles of 128 x 64 instead of 64
// of 128 x 128)
int lbm_linear_tiles(LinearArgs& p) {
  p.m_tiles = (p.M + kGM - 1) / kGM;
  const bool wide = (p.N % 128 == 0) && ((long long)p.m_tiles * (p.N / 128) >= 160);
  const int tn = wide ? 128 : 64;
  p.n_tiles = p.N / tn;
  return tn;
}
}  // namespace

namespace {
// 256- or 192-row tiles of 256 columns when they give at least half of the 256 CUs a workgroup
// (several streams' rows into the 3,072 or 4,096 columns of the qkv projection or fc1): the row
// count of the tile (the one that needs fewer rounds of the CUs times rows), or 0; sets the tile
// counts
int lbm_linear_big_tiles(LinearArgs& p) {
  if (p.N % kBN != 0) return 0;
  const int nt = p.N / kBN;
  int best = 0;
  long long best_cost = 0;
  for (int bm : {256, 192}) {
    const long long tiles = (long long)((p.M + bm - 1) / bm) * nt;
    if (tiles < 128) continue;
    const long long cost = ((tiles + 255) / 256) * bm;      // rounds of the 256 CUs x rows per tile
    if (!best || cost < best_cost) best = bm, best_cost = cost;
  }
  if (!best) return 0;
  p.m_tiles = (p.M + best - 1) / best;
  p.n_tiles = nt;
  return best;
}
}  // namespace

namespace {
// the kernel addresses a row of either operand with a 32-bit byte offset from a 64-bit base
bool lbm_offsets_fit(int M, int N, int K) {
  return (long long)M * K * 2 < (1LL << 32) && (long long)N * K * 2 < (1LL << 32);
}
}  // namespace

namespace {
// the folded LayerNorm of the activations, checked and copied into the kernel arguments
int lbm_set_row_norm(LinearArgs& p, const lbm_row_norm* ln, const char* who) {
  if (!ln) return LBM_OK;
  if (!ln->w_colsum || !ln->stats || ln->stats_tiles <= 0 || p.K % ln->stats_tiles != 0)
    return lbm_fail(LBM_ERR_INVALID, "%s: standardised rows need w_colsum, stats and a tile count that divides K (got %d for K %d)",
                    who, ln->stats_tiles, p.K);
  p.ln_colsum = ln->w_colsum;
  p.ln_stats = ln->stats;
  p.ln_tiles = ln->stats_tiles;
  p.ln_eps = ln->eps;
  return LBM_OK;
}
}  // namespace

namespace {
// K slices per tile: as many as still leave every workgroup eight k-steps and fit one round of
// the 256 CUs (fc2 of one frame: 128 tiles x 2); the residual epilogue only
int lbm_linear_splits(const LinearArgs& p, int epilogue) {
  if (epilogue != LBM_LINEAR_BIAS_RESIDUAL) return 1;
  const int tiles = p.m_tiles * p.n_tiles, nk = p.K / kGK;
  for (int s = 4; s >= 2; s >>= 1)
    if (tiles * s <= 256 && nk % s == 0 && nk / s >= 8) return s;
  return 1;
}
size_t lbm_linear_counter_bytes(const LinearArgs& p) { return ((size_t)p.m_tiles * p.n_tiles * 4 + 255) & ~(size_t)255; }
}  // namespace

size_t lbm_linear_workspace_for(int M, int N, int K, int epilogue) {
  LinearArgs p = {};
  p.M = M; p.N = N; p.K = K;
  const int tn = lbm_linear_tiles(p);
  const int s = lbm_linear_splits(p, epilogue);
  if (s == 1) return 0;
  return lbm_linear_counter_bytes(p) + (size_t)p.m_tiles * p.n_tiles * s * kGM * tn * 4;
}

int lbm_linear_stats_tiles_for(int M, int N) {
  LinearArgs p = {};
  p.M = M; p.N = N;
  lbm_linear_tiles(p);
  return p.n_tiles;
}

namespace {
// what the calling thread's next GEMM launch is to ask for on behalf of the launch after it
thread_local const char* g_prefetch_hint = nullptr;
thread_local size_t g_prefetch_hint_bytes = 0;
void lbm_take_prefetch_hint(LinearArgs& p) {
  p.touch = g_prefetch_hint;
  p.touch_lines = (unsigned)(g_prefetch_hint ? g_prefetch_hint_bytes / 128 : 0);
  g_prefetch_hint = nullptr;
  g_prefetch_hint_bytes = 0;
}
}  // namespace

void lbm_set_prefetch_hint(const void* ptr, size_t bytes) {
  g_prefetch_hint = bytes >= 128 ? (const char*)ptr : nullptr;
  g_prefetch_hint_bytes = g_prefetch_hint ? bytes : 0;
}

int lbm_launch_linear(const void* a, const lbm_row_norm* a_norm, const void* w, const float* bias, const float* gamma,
                      const void* residual, void* out, float* out_stats, int M, int N, int K, int epilogue,
                      void* workspace, size_t workspace_bytes, hipStream_t stream) {
  if (M == 0) {
    lbm_set_prefetch_hint(nullptr, 0);   // a hint is for the next call, whatever that call does
    return LBM_OK;
  }
  if (K % kGK != 0 || N % 64 != 0)
    return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_linear: K must be a multiple of 128 and N of 64 (got K %d, N %d)", K, N);
  if (!lbm_offsets_fit(M, N, K))
    return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_linear: M * K and N * K must stay below 2^31 elements (32-bit byte offsets), got %d x %d x %d", M, N, K);
  if (a_norm && epilogue == LBM_LINEAR_BIAS_RESIDUAL)
    return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_linear: no row standardisation with the residual epilogue");
  if (out_stats && epilogue != LBM_LINEAR_BIAS_RESIDUAL)
    return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_linear: row statistics come with the residual epilogue only");
  LinearArgs p = {};
  p.stats_out = out_stats;
  p.a = (const unsigned short*)a;
  p.w = (const unsigned short*)w;
  p.bias = bias;
  p.gamma = gamma;
  p.res = (const unsigned short*)residual;
  p.out = (unsigned short*)out;
  p.M = M; p.N = N; p.K = K;
  lbm_take_prefetch_hint(p);
  if (int rc = lbm_set_row_norm(p, a_norm, "lbm_linear_norm")) return rc;
  const bool lna = a_norm != nullptr;
  const dim3 block(kGThreads), block_s(kGThreads + kGTouchThreads);
  if (epilogue == LBM_LINEAR_BIAS || epilogue == LBM_LINEAR_BIAS_GELU) {
    if (const int bm = lbm_linear_big_tiles(p)) {
      const dim3 grid_b((unsigned)(p.m_tiles * p.n_tiles));
#define LBM_BIG_LAUNCH(E, L)                                                                                         \
      {                                                                                                              \
        if (bm == 256) hipLaunchKernelGGL((lbm_linear_bf16_big_kernel<256, E, 0, false, L>), grid_b, block, 0, stream, p); \
        else hipLaunchKernelGGL((lbm_linear_bf16_big_kernel<192, E, 0, false, L>), grid_b, block, 0, stream, p);           \
      }
      if (epilogue == LBM_LINEAR_BIAS && lna) LBM_BIG_LAUNCH(LBM_LINEAR_BIAS, true)
      else if (epilogue == LBM_LINEAR_BIAS) LBM_BIG_LAUNCH(LBM_LINEAR_BIAS, false)
      else if (lna) LBM_BIG_LAUNCH(LBM_LINEAR_BIAS_GELU, true)
      else LBM_BIG_LAUNCH(LBM_LINEAR_BIAS_GELU, false)
#undef LBM_BIG_LAUNCH
      return lbm_check_launch("lbm_linear_bf16_big_kernel");
    }
  }
  const bool wide = lbm_linear_tiles(p) == 128;
  if (workspace) {
    const int splits = lbm_linear_splits(p, epilogue);
    if (splits > 1 && workspace_bytes >= lbm_linear_workspace_for(M, N, K, epilogue)) {
      if (residual == out)   // a workgroup that is not the tile's last would see the other's store
        return lbm_fail(LBM_ERR_INVALID, "lbm_linear_norm: with a workspace the residual may not alias out");
      p.k_splits = splits;
      p.split_counters = (unsigned*)workspace;
      p.split_part = (float*)((char*)workspace + lbm_linear_counter_bytes(p));
      const dim3 grid_s((unsigned)(p.m_tiles * p.n_tiles * splits));
      if (wide) hipLaunchKernelGGL((lbm_linear_bf16_kernel<LBM_LINEAR_BIAS_RESIDUAL, 128, 0, false, false, true>), grid_s, block_s, 0, stream, p);
      else hipLaunchKernelGGL((lbm_linear_bf16_kernel<LBM_LINEAR_BIAS_RESIDUAL, 64, 0, false, false, true>), grid_s, block_s, 0, stream, p);
      return lbm_check_launch("lbm_linear_bf16_kernel<split K>");
    }
  }
  const dim3 grid((unsigned)(p.m_tiles * p.n_tiles));
#define LBM_LINEAR_LAUNCH(E, L)                                                                                  \
  {                                                                                                              \
    if (wide) hipLaunchKernelGGL((lbm_linear_bf16_kernel<E, 128, 0, false, L>), grid, block_s, 0, stream, p);    \
    else hipLaunchKernelGGL((lbm_linear_bf16_kernel<E, 64, 0, false, L>), grid, block_s, 0, stream, p);          \
  }
  if (epilogue == LBM_LINEAR_BIAS && lna) LBM_LINEAR_LAUNCH(LBM_LINEAR_BIAS, true)
  else if (epilogue == LBM_LINEAR_BIAS) LBM_LINEAR_LAUNCH(LBM_LINEAR_BIAS, false)
  else if (epilogue == LBM_LINEAR_BIAS_GELU && lna) LBM_LINEAR_LAUNCH(LBM_LINEAR_BIAS_GELU, true)
  else if (epilogue == LBM_LINEAR_BIAS_GELU) LBM_LINEAR_LAUNCH(LBM_LINEAR_BIAS_GELU, false)
  else if (epilogue == LBM_LINEAR_BIAS_RESIDUAL) LBM_LINEAR_LAUNCH(LBM_LINEAR_BIAS_RESIDUAL, false)
  else return lbm_fail(LBM_ERR_INVALID, "lbm_linear: unknown epilogue %d", epilogue);
#undef LBM_LINEAR_LAUNCH
  return lbm_check_launch("lbm_linear_bf16_kernel");
}

int lbm_launch_qkv_linear_prepare(const void* a, const lbm_row_norm* a_norm, const void* w, const float* bias, int M, int K,
                                  const float* q_norm_w, const float* q_norm_b, const float* k_norm_w,
                                  const float* k_norm_b, float norm_eps, float q_scale, const float* rope_cs, int rope_layout,
                                  void* q_out, void* k_out, void* v_out, void* pool, const int32_t* append_rows,
                                  int num_heads, int page_size, hipStream_t stream) {
  if (M == 0) return LBM_OK;
  const int N = 3 * num_heads * 64;
  if (K % kGK != 0) return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_qkv_linear_prepare: K must be a multiple of 128 (got %d)", K);
  if (!lbm_offsets_fit(M, N, K))
    return lbm_fail(LBM_ERR_UNSUPPORTED, "lbm_qkv_linear_prepare: M * K and N * K must stay below 2^31 elements (32-bit byte offsets), got %d x %d x %d", M, N, K);
  LinearArgs p = {};
  p.a = (const unsigned short*)a;
  p.w = (const unsigned short*)w;
  p.bias = bias;
  p.out = (unsigned short*)q_out;
  p.M = M; p.N = N; p.K = K;
  lbm_take_prefetch_hint(p);
  p.q_norm_w = q_norm_w; p.q_norm_b = q_norm_b; p.k_norm_w = k_norm_w; p.k_norm_b = k_norm_b;
  p.rope_cs = rope_cs;
  p.k_out = (unsigned short*)k_out; p.v_out = (unsigned short*)v_out;
  p.pool = (unsigned short*)pool;
  p.append_rows = append_rows;
  p.eps = norm_eps;
  p.q_scale = q_scale;
  p.num_heads = num_heads; p.page_size = page_size;
  if (int rc = lbm_set_row_norm(p, a_norm, "lbm_qkv_linear_prepare_norm")) return rc;
  const bool lna = a_norm != nullptr;
  const int rope = !rope_cs ? 0 : (rope_layout == LBM_ROPE_INTERLEAVED ? 1 : 2);
  const bool norm = q_norm_w != nullptr;
  // 256-wide tiles: four whole heads each, so that a tile does not straddle q | k | v
  if (const int bm = (num_heads & 3) == 0 ? lbm_linear_big_tiles(p) : 0) {
    const dim3 grid_b((unsigned)(p.m_tiles * p.n_tiles)), block_b(kGThreads);
#define LBM_QKV_BIG_M(BM, R, NRM)                                                                                               \
    {                                                                                                                           \
      if (lna) hipLaunchKernelGGL((lbm_linear_bf16_big_kernel<BM, kEpiQkvPrepare, R, NRM, true>), grid_b, block_b, 0, stream, p);  \
      else hipLaunchKernelGGL((lbm_linear_bf16_big_kernel<BM, kEpiQkvPrepare, R, NRM, false>), grid_b, block_b, 0, stream, p);     \
    }
#define LBM_QKV_BIG(R, NRM)                                                  \
    {                                                                        \
      if (bm == 256) LBM_QKV_BIG_M(256, R, NRM) else LBM_QKV_BIG_M(192, R, NRM) \
    }
    if (rope == 0 && !norm) LBM_QKV_BIG(0, false)
    else if (rope == 0) LBM_QKV_BIG(0, true)
    else if (rope == 1 && !norm) LBM_QKV_BIG(1, false)
    else if (rope == 1) LBM_QKV_BIG(1, true)
    else if (!norm) LBM_QKV_BIG(2, false)
    else LBM_QKV_BIG(2, true)
#undef LBM_QKV_BIG
#undef LBM_QKV_BIG_M
    return lbm_check_launch("lbm_linear_bf16_big_kernel<qkv prepare>");
  }
  // a tile must not straddle q | k | v: 128-wide tiles need an even number of heads
  bool wide = lbm_linear_tiles(p) == 128;
  if (wide && (num_heads & 1)) {
    wide = false;
    p.n_tiles = N / 64;
  }
  const dim3 grid((unsigned)(p.m_tiles * p.n_tiles)), block(kGThreads + kGTouchThreads);
#define LBM_QKV_LAUNCH_L(R, NRM, L)                                                                                   \
  {                                                                                                                   \
    if (wide) hipLaunchKernelGGL((lbm_linear_bf16_kernel<kEpiQkvPrepare, 128, R, NRM, L>), grid, block, 0, stream, p); \
    else hipLaunchKernelGGL((lbm_linear_bf16_kernel<kEpiQkvPrepare, 64, R, NRM, L>), grid, block, 0, stream, p);       \
  }
#define LBM_QKV_LAUNCH(R, NRM)                                                                                        \
  {                                                                                                                   \
    if (lna) LBM_QKV_LAUNCH_L(R, NRM, true) else LBM_QKV_LAUNCH_L(R, NRM, false)                                      \
  }
  if (rope == 0 && !norm) LBM_QKV_LAUNCH(0, false)
  else if (rope == 0) LBM_QKV_LAUNCH(0, true)
  else if (rope == 1 && !norm) LBM_QKV_LAUNCH(1, false)
  else if (rope == 1) LBM_QKV_LAUNCH(1, true)
  else if (!norm) LBM_QKV_LAUNCH(2, false)
  else LBM_QKV_LAUNCH(2, true)
#undef LBM_QKV_LAUNCH_L
#undef LBM_QKV_LAUNCH
  return lbm_check_launch("lbm_linear_bf16_kernel<qkv prepare>");
}
