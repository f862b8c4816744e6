// Shared device helpers for the gfx950 INT8 chunkwise-recurrence kernels.
//
// Everything that produces an INT8 code goes through the helpers in this file so that the
// arithmetic is a fixed sequence of individually rounded IEEE fp32 operations (the library is
// built with -ffp-contract=off; fused multiply-adds appear only where written as fmaf).  The
// CPU checker restates the same sequences in numpy, which makes code tensors comparable bit
// for bit.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#define LQ_OK 0
#define LQ_ERR_SHAPE (-22)      // bad / unsupported shape, stride or flag
#define LQ_ERR_LAUNCH (-5)      // hipGetLastError() reported a launch failure
#define LQ_ERR_NULL (-14)       // required pointer missing
#define LQ_ERR_STATE (-11)      // set-up needed that cannot run now (stream under graph capture)

typedef int lq_v4i __attribute__((ext_vector_type(4)));
typedef int lq_v2i __attribute__((ext_vector_type(2)));
typedef int lq_v16i __attribute__((ext_vector_type(16)));
typedef float lq_v4f __attribute__((ext_vector_type(4)));
typedef float lq_v16f __attribute__((ext_vector_type(16)));
typedef _Float16 lq_v8h __attribute__((ext_vector_type(8)));
typedef _Float16 lq_v4h __attribute__((ext_vector_type(4)));
typedef _Float16 lq_v2h __attribute__((ext_vector_type(2)));

#define LQ_DEV __device__ __forceinline__

// ---------------------------------------------------------------------------------------------
// Deterministic exp / log (plain fp32 mul/add/sub/div, no FMA, no hardware transcendental).
// ---------------------------------------------------------------------------------------------

// exp(x): Cody-Waite reduction by ln2 (hi part has 16 significant bits so n*hi is exact), degree-7
// Taylor polynomial on |r| <= 0.3466, result scaled by 2^n built from the exponent bits.
// x <= -86 returns 0 (keeps every result a normal number), x > 88 returns +inf, NaN propagates.
LQ_DEV float lq_expf(float x) {
#pragma clang fp contract(off)
  // evaluated without a branch on a clamped argument, the special cases selected at the end: as early returns they
  // became a branch per call, and a load whose value feeds a branch is waited for on the spot
  const float xin = x;
  x = fminf(fmaxf(x, -86.0f), 88.0f);  // NaN -> -86, replaced below
  float t = x * 1.44269502162933349609375f;
  float n = __builtin_rintf(t);
  float r = x - n * 0.693145751953125f;
  r = r - n * 1.42860676533018704504e-06f;
  float p = 1.98412701138295233250e-04f;   // 1/5040
  p = p * r + 1.38888892251998186111e-03f; // 1/720
  p = p * r + 8.33333376795053482056e-03f; // 1/120
  p = p * r + 4.16666679084300994873e-02f; // 1/24
  p = p * r + 1.66666671633720397949e-01f; // 1/6
  p = p * r + 0.5f;
  p = p * r + 1.0f;
  p = p * r + 1.0f;
  int e = ((int)n + 127) << 23;
  float y = p * __int_as_float(e);
  y = xin > 88.0f ? __builtin_inff() : y;
  y = !(xin > -86.0f) ? 0.0f : y;
  return xin != xin ? xin : y;
}

// log(y) for normal y > 0: y = m * 2^e with m in [sqrt(1/2), sqrt(2)), s = (m-1)/(m+1),
// log m = 2*(s + s^3/3 + s^5/5 + s^7/7 + s^9/9 + s^11/11).
LQ_DEV float lq_logf(float y) {
#pragma clang fp contract(off)
  int bits = __float_as_int(y);
  int e = ((bits >> 23) & 0xff) - 127;
  float m = __int_as_float((bits & 0x007fffff) | 0x3f800000);  // [1, 2)
  if (m > 1.41421353816986083984375f) {
    m = m * 0.5f;
    e = e + 1;
  }
  float s = (m - 1.0f) / (m + 1.0f);
  float s2 = s * s;
  float p = 9.09090936183929443359e-02f;    // 1/11
  p = p * s2 + 1.11111111938953399658e-01f; // 1/9
  p = p * s2 + 1.42857149243354797363e-01f; // 1/7
  p = p * s2 + 2.00000002980232238770e-01f; // 1/5
  p = p * s2 + 3.33333343267440795898e-01f; // 1/3
  p = p * s2 + 1.0f;
  float lm = (s + s) * p;
  float fe = (float)e;
  return fe * 0.693145751953125f + (fe * 1.42860676533018704504e-06f + lm);
}

// ---------------------------------------------------------------------------------------------
// Rounding to the INT8 grid.
// ---------------------------------------------------------------------------------------------

// Round half away from zero: floor(y + 0.5) for y >= 0, ceil(y - 0.5) otherwise.  y + copysign(0.5, y)
// is the same fp32 sum in both branches and truncation toward zero equals floor / ceil on its sign.
// The float->int conversion saturates, the caller clamps to the code range.
LQ_DEV int lq_rha_i32(float y) { return (int)(y + __builtin_copysignf(0.5f, y)); }

LQ_DEV int lq_clampi(int v, int lo, int hi) { return min(max(v, lo), hi); }

// clamp(rha(y), -qmax, qmax)
LQ_DEV int lq_q_rha(float y, int qmax) { return lq_clampi(lq_rha_i32(y), -qmax, qmax); }

// clamp(rint(y), lo, hi) with IEEE round-half-even
LQ_DEV int lq_q_rint(float y, int lo, int hi) {
  float r = __builtin_rintf(y);
  r = fminf(fmaxf(r, (float)lo), (float)hi);
  return (int)r;
}

LQ_DEV uint32_t lq_pack4(int a, int b, int c, int d) {
  return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) | ((uint32_t)d << 24);
}

LQ_DEV int lq_sbyte(uint32_t w, int i) { return (int)(int8_t)(w >> (8 * i)); }

// ---------------------------------------------------------------------------------------------
// MFMA wrappers (wave64).  Operand layout used throughout:
//   i8  16x16x64: lane l supplies row/col (l & 15) and the 16 contraction slots of group (l >> 4)
//   f16 16x16x32: lane l supplies row/col (l & 15) and the 8 contraction slots of group (l >> 4)
//   accumulator : lane l holds column (l & 15), rows 4*(l >> 4) + {0,1,2,3}
// A and B use the same slot numbering, so any assignment of real contraction indices to slots is
// valid as long as both operands agree.
// ---------------------------------------------------------------------------------------------
LQ_DEV lq_v4i lq_mfma_i8(lq_v4i a, lq_v4i b, lq_v4i c) {
  return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}
LQ_DEV lq_v4f lq_mfma_f16(lq_v8h a, lq_v8h b, lq_v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

LQ_DEV float lq_h2f(_Float16 h) { return (float)h; }

static inline int lq_check_launch() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LQ_OK : LQ_ERR_LAUNCH;
}
