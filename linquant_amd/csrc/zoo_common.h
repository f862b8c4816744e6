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
