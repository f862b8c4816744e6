// Shared pieces of the zoo (linear attention / GLA / DeltaNet / KDA) INT8 chunk kernels.
//
// Tensor layouts: q, k (B,T,H,K) and v (B,T,H,V) fp16 contiguous; g fp32 (B,T,H) or (B,T,H,K) holding the
// chunk-local cumulative log decay; scales fp32.  The per-chunk INT8 stored state is kept V-major,
// hT[b][chunk][h][v][k] (contraction axis K contiguous), which is what both its consumers want as an MFMA
// operand; it is an internal buffer of the wrappers.
#pragma once

#include "lq_common.h"

// _q8 of the reference (linquant/kernels/zoo/simple_gla.py:15-20): y = x * inv_scale, round half away, clamp.
LQ_DEV int zoo_q8(float x, float inv_scale, int qmax) { return lq_q_rha(x * inv_scale, qmax); }

LQ_DEV uint32_t zoo_pack_codes(int a, int b, int c, int d) {
  const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x04000c0cu);
  return lo | hi;
}

LQ_DEV _Float16 zoo_half_of(uint32_t w, int hi) {
  return __builtin_bit_cast(_Float16, (uint16_t)(hi ? (w >> 16) : (w & 0xffffu)));
}

// 4 int8 codes (one dword) -> 4 exact fp16 values as two packed dwords
LQ_DEV void zoo_i8x4_to_f16x4(uint32_t w, uint32_t& lo, uint32_t& hi) {
  const uint32_t u = w ^ 0x80808080u;
  const uint32_t a = __builtin_amdgcn_perm(0x64646464u, u, 0x05010400u);
  const uint32_t b = __builtin_amdgcn_perm(0x64646464u, u, 0x05030402u);
  const lq_v2h off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
  lo = __builtin_bit_cast(uint32_t, __builtin_bit_cast(lq_v2h, a) + off);
  hi = __builtin_bit_cast(uint32_t, __builtin_bit_cast(lq_v2h, b) + off);
}

LQ_DEV uint32_t zoo_pack_h2(float a, float b) {
  const lq_v2h v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(uint32_t, v);
}

static inline bool zoo_al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

// exp on the hardware exp2 unit (x * log2(e), then v_exp_f32): the arithmetic tl.exp lowers to in the reference's
// Triton kernels.  Large negative arguments give 0, never NaN.
LQ_DEV float zoo_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// ---- activation dtype: q, k, v (and the prepared Hw, W, U, E) are fp16 or bf16; `bf` is uniform per launch.
// Pointers are typed _Float16* for their 2-byte element stride only.
LQ_DEV void zoo_dec2(uint32_t w, bool bf, float& lo, float& hi) {
  if (bf) {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
  } else {
    const lq_v2h h = __builtin_bit_cast(lq_v2h, w);
    lo = (float)h[0];
    hi = (float)h[1];
  }
}
LQ_DEV float zoo_dec1(uint32_t bits16, bool bf) {
  return bf ? __uint_as_float(bits16 << 16) : (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
LQ_DEV void zoo_ld8(const _Float16* p, bool bf, float (&o)[8]) {
  const lq_v4i raw = *(const lq_v4i*)p;
#pragma unroll
  for (int d = 0; d < 4; ++d) zoo_dec2((uint32_t)raw[d], bf, o[2 * d], o[2 * d + 1]);
}
LQ_DEV void zoo_ld4(const _Float16* p, bool bf, float (&o)[4]) {
  const lq_v2i raw = *(const lq_v2i*)p;
#pragma unroll
  for (int d = 0; d < 2; ++d) zoo_dec2((uint32_t)raw[d], bf, o[2 * d], o[2 * d + 1]);
}
// round-to-nearest-even bf16 bits of a finite fp32 value
LQ_DEV uint32_t zoo_bf16_bits(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
LQ_DEV uint32_t zoo_enc2(float a, float b, bool bf) {
  return bf ? (zoo_bf16_bits(a) | (zoo_bf16_bits(b) << 16)) : zoo_pack_h2(a, b);
}
LQ_DEV uint16_t zoo_enc1(float a, bool bf) {
  return bf ? (uint16_t)zoo_bf16_bits(a) : __builtin_bit_cast(uint16_t, (_Float16)a);
}
// x rounded to the activation dtype and back: what a consumer reads when a producer stored x there
LQ_DEV float zoo_round_act(float x, bool bf) { return zoo_dec1((uint32_t)zoo_enc1(x, bf), bf); }

// a * b as an fp32 value of its own: a conversion to half precision that follows is a second rounding (left to the
// compiler, it is folded into the multiply: one rounding of the exact product)
LQ_DEV float zoo_mul_rn(float a, float b) {
  float p = a * b;
  asm volatile("" : "+v"(p));
  return p;
}

// x / d rounded once to fp32 (the IEEE quotient) from r = RN(1 / d): q0 = RN(x r), rem = x - q0 d (exact in the fused
// multiply-add), q = RN(q0 + rem r).  Correct for finite d > 0 and half-precision x (checked over every fp16 and bf16
// value on the CPU); three instructions instead of the division sequence.
LQ_DEV float zoo_div_rn(float x, float d, float r) {
  const float q0 = x * r;
  const float rem = __builtin_fmaf(-q0, d, x);
  float q = __builtin_fmaf(rem, r, q0);
  // the quotient exists as an fp32 value before anything narrows it: without this the compiler folds a following
  // conversion to half precision into the multiply-add (one rounding instead of two)
  asm volatile("" : "+v"(q));
  return q;
}

// ---- fast Walsh-Hadamard transform of a row spread over LPR adjacent lanes (LPR = 8 or 16, rows aligned to LPR lanes),
// eight adjacent channels per lane: butterflies 1, 2, 4 inside the lane, then across lanes l ^ 1, l ^ 2, l ^ 4 (, l ^ 8)
// through DPP lane permutations (no LDS traffic).  fp32 sums in a fixed order: y = sum_i x_i H_ij, unnormalized.
template <int M>
LQ_DEV float zoo_lane_xor(float v) {
  int x = __float_as_int(v);
  // every lane has a source, so nothing depends on the "old" operand
  if constexpr (M == 1) x = __builtin_amdgcn_update_dpp(x, x, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
  if constexpr (M == 2) x = __builtin_amdgcn_update_dpp(x, x, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
  if constexpr (M == 4) {  // l ^ 7 (mirror of each half row) followed by l ^ 3 (mirror of each quad)
    x = __builtin_amdgcn_update_dpp(x, x, 0x141, 0xf, 0xf, true);  // row_half_mirror
    x = __builtin_amdgcn_update_dpp(x, x, 0x1B, 0xf, 0xf, true);   // quad_perm [3,2,1,0]
  }
  if constexpr (M == 8) x = __builtin_amdgcn_update_dpp(x, x, 0x128, 0xf, 0xf, true);  // row_ror:8
  return __int_as_float(x);
}

template <int M>
LQ_DEV void zoo_fwht_stage(float (&v)[8], int sub) {
  // lanes whose bit M is set hold the difference o - v = (-v) + o, the others the sum v + o
  const uint32_t neg = (sub & M) ? 0x80000000u : 0u;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = __uint_as_float(__float_as_uint(v[e]) ^ neg) + zoo_lane_xor<M>(v[e]);
}

template <int LPR>
LQ_DEV void zoo_fwht(float (&v)[8], int sub) {
#pragma unroll
  for (int h2 = 1; h2 < 8; h2 <<= 1)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if ((e & h2) == 0) {
        const float a = v[e], c = v[e + h2];
        v[e] = a + c;
        v[e + h2] = a - c;
      }
  zoo_fwht_stage<1>(v, sub);
  zoo_fwht_stage<2>(v, sub);
  zoo_fwht_stage<4>(v, sub);
  if constexpr (LPR == 16) zoo_fwht_stage<8>(v, sub);
}
