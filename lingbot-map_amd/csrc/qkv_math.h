// Arithmetic shared by the fused pre-attention producer (qkv_prepare_gfx950.hip) and the qkv
// projection that carries the producer as its epilogue (linear_gfx950.hip): per-head LayerNorm
// and rotary embedding of one q or k row of 64 elements held by 8 consecutive lanes, 8 elements
// each (lingbot_map/layers/attention.py:402-426, lingbot_map/layers/rope.py:123-198,438-461).
// Compiled with floating-point contraction off: every product and sum is rounded on its own, as
// the reference's separate torch ops are.
#ifndef LBM_QKV_MATH_H
#define LBM_QKV_MATH_H

#include <hip/hip_runtime.h>

#pragma clang fp contract(off)

namespace lbm_qkv {

typedef __attribute__((ext_vector_type(4))) float f32x4;

// (the math header's __fmul_rn / __fadd_rn are plain operators compiled with contraction allowed)
__device__ __forceinline__ float mul_rn(float a, float b) { return a * b; }
__device__ __forceinline__ float add_rn(float a, float b) { return a + b; }
__device__ __forceinline__ float sub_rn(float a, float b) { return a - b; }
// round-to-nearest-even to bf16 and back (torch's .to(bfloat16)); the hardware conversion
// v_cvt_pk_bf16_f32 rounds the same way
__device__ __forceinline__ float round_bf16(float f) { return (float)(__bf16)f; }

// Lane exchanges inside aligned groups of 4, 8 and 16 lanes as DPP moves (vector ALU, no LDS
// round trip as the permute instructions behind __shfl_xor make): xor 1 and xor 2 are quad
// permutations; once a quad's lanes agree, the mirror of a half row (lane i <-> 7 - i of 8) or of a
// row (i <-> 15 - i of 16) brings in the value of the other quad / other half, which is what xor 4 /
// xor 8 would have fetched.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  const int i = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float lane_xor1(float v) { return dpp_move<0xB1>(v); }          // quad_perm [1, 0, 3, 2]
__device__ __forceinline__ float lane_xor2(float v) { return dpp_move<0x4E>(v); }          // quad_perm [2, 3, 0, 1]
__device__ __forceinline__ float other_quad_of_8(float v) { return dpp_move<0x141>(v); }   // row_half_mirror
__device__ __forceinline__ float other_half_of_16(float v) { return dpp_move<0x140>(v); }  // row_mirror
// sum over an aligned group of 8 lanes, every lane ends up with it (same additions, in the same
// order, as s += xor 1; s += xor 2; s += xor 4)
__device__ __forceinline__ float sum_of_8(float s) {
  s += lane_xor1(s);
  s += lane_xor2(s);
  s += other_quad_of_8(s);
  return s;
}

// sum over the 64 lanes of a wavefront, every lane ends up with it: 16-lane rows by DPP, the four
// row sums through scalar registers
__device__ __forceinline__ float sum_of_wave(float s) {
  s = sum_of_8(s);
  s += other_half_of_16(s);
  const int bits = __builtin_bit_cast(int, s);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
  return (r0 + r1) + (r2 + r3);
}

// two fp32 values rounded to bf16 and back by ONE conversion (v_cvt_pk_bf16_f32 takes a pair) and
// two bit operations, where round_bf16 on each would take a conversion and a shift apiece
__device__ __forceinline__ void round_bf16_pair(float a, float b, float& ra, float& rb) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  const unsigned pk = __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, bf16x2));
  ra = __builtin_bit_cast(float, pk << 16);
  rb = __builtin_bit_cast(float, pk & 0xffff0000u);
}

// x: this lane's elements 8 c .. 8 c + 7 of the row (c = lane % 8; the row's 8 lanes are
// consecutive and aligned, so the shuffles below stay inside it).  SRC 0: bf16 activations
// (roundings after the LayerNorm, of cos and sin, and after every product and sum), 1: fp32.
// ROPE 0 none, 1 interleaved pairs (cs4[0..1] = (cos, sin) of this lane's four pairs), 2
// half-split pairs (cs4[0..3] = (cos, sin) of its eight elements).  w4 / b4: LayerNorm weight
// and bias of the lane's eight elements.
// post: a factor the row is multiplied by in fp32 BEFORE the rounding that ends its last
// operation (the rotary sum, else the LayerNorm, else the plain copy), so that a scaled q row
// is rounded once; 1.0f leaves every result as it was (x * 1.0f is exact).
// norm_rope_unrounded leaves that last rounding of a bf16 row (SRC 0) to the caller, who makes it
// with the conversion that packs the row for its store; every rounding before it is made here.
template <int SRC, int ROPE, bool NORM>
__device__ __forceinline__ void norm_rope_unrounded(float (&x)[8], const f32x4 (&w4)[2], const f32x4 (&b4)[2],
                                                    const f32x4 (&cs4)[4], int c, float eps, float post = 1.0f) {
  const float post_norm = ROPE == 0 ? post : 1.0f;
  if (!NORM && ROPE == 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = mul_rn(x[i], post);
  }
  if (NORM) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += x[i];
    s = sum_of_8(s);
    const float mean = s * (1.0f / 64.0f);
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) v += (x[i] - mean) * (x[i] - mean);
    v = sum_of_8(v);
    const float rstd = __builtin_amdgcn_rsqf(v * (1.0f / 64.0f) + eps);  // torch's LayerNorm uses rsqrt too
#pragma unroll
    for (int i = 0; i < 8; ++i)
      x[i] = mul_rn(add_rn(mul_rn(mul_rn(x[i] - mean, rstd), w4[i >> 2][i & 3]), b4[i >> 2][i & 3]), post_norm);
    if (SRC == 0 && ROPE != 0) {
#pragma unroll
      for (int i = 0; i < 8; i += 2) round_bf16_pair(x[i], x[i + 1], x[i], x[i + 1]);
    }
  }
  if (ROPE == 1) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const f32x4 q4 = cs4[p];  // (cos, sin) of two pairs
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int i = 4 * p + 2 * j;
        float co = q4[2 * j], si = q4[2 * j + 1];
        const float x1 = x[i], x2 = x[i + 1];
        if (SRC == 0) {
          round_bf16_pair(co, si, co, si);
          float cc, ss, sc, cs;
          round_bf16_pair(mul_rn(x1, co), mul_rn(x2, si), cc, ss);
          round_bf16_pair(mul_rn(x1, si), mul_rn(x2, co), sc, cs);
          x[i] = mul_rn(sub_rn(cc, ss), post);
          x[i + 1] = mul_rn(add_rn(sc, cs), post);
        } else {
          x[i] = mul_rn(sub_rn(mul_rn(x1, co), mul_rn(x2, si)), post);
          x[i + 1] = mul_rn(add_rn(mul_rn(x1, si), mul_rn(x2, co)), post);
        }
      }
    }
  } else if (ROPE != 0) {
    // half-split pairs: in each 32-element half, element j < 16 rotates with element j + 16
    // (x * cos + rotate(x) * sin with rotate = (-second, first), rope.py:123-152); the partner
    // sits two lanes away in the 8-lane group.  a - b is a + (-b) bit for bit, so the lanes of
    // the first 16 flip the sign of the second product instead of choosing between two results.
    const unsigned flip = (c & 2) == 0 ? 0x80000000u : 0u;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const f32x4 q4 = cs4[p];  // (cos, sin) of two elements
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int i = 2 * p + j;
        float co = q4[2 * j], si = q4[2 * j + 1];
        const float own = x[i];
        const float other = lane_xor2(own);
        float a0, b0;
        if (SRC == 0) {
          round_bf16_pair(co, si, co, si);
          round_bf16_pair(mul_rn(own, co), mul_rn(other, si), a0, b0);
        } else {
          a0 = mul_rn(own, co), b0 = mul_rn(other, si);
        }
        b0 = __builtin_bit_cast(float, __builtin_bit_cast(unsigned, b0) ^ flip);
        x[i] = mul_rn(add_rn(a0, b0), post);
      }
    }
  }
}

// the same with the last rounding of a bf16 row made here: x holds bf16 values as fp32
template <int SRC, int ROPE, bool NORM>
__device__ __forceinline__ void norm_rope(float (&x)[8], const f32x4 (&w4)[2], const f32x4 (&b4)[2],
                                          const f32x4 (&cs4)[4], int c, float eps, float post = 1.0f) {
  norm_rope_unrounded<SRC, ROPE, NORM>(x, w4, b4, cs4, c, eps, post);
  if (SRC == 0) {
#pragma unroll
    for (int i = 0; i < 8; i += 2) round_bf16_pair(x[i], x[i + 1], x[i], x[i + 1]);
  }
}

}  // namespace lbm_qkv

#endif  // LBM_QKV_MATH_H
