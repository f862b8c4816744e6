// Rotation + quantize prologue: B/C lanes of the post-conv xBC slab -> signed Kronecker Hadamard -> INT8,
// and the standalone rotation used for the key-side fp16 B.
// Replaces linquant/kernels/mamba2/fused_split_rotate_xBC.py:31-227 (launcher :236-329) and
// linquant/kernels/hadamard.py:38-103 (launcher :141-179).
//
// Reference arithmetic per B or C row b (N = 2*BS channels, halves b0 | b1):
//   [b = fp16(b * dqk)]; v = bf16(b * signs); w_half = v . H_BS (H_BS = +-bf16(1/sqrt(BS)), fp32 accumulate)
//   y0 = (w0 + w1) * (1/sqrt 2), y1 = (w0 - w1) * (1/sqrt 2); y -> fp16;
//   q = clamp(rint(float(y) * inv_scale), -128, 127)
// The Sylvester matrix product is evaluated as a fast Walsh-Hadamard transform in fp32 (exact additions of
// bf16 inputs whenever the row's dynamic range fits 24 bits) followed by one multiply with bf16(1/sqrt(BS)):
// HBM-bound byte work, no matrix core needed.  A row is spread over N/8 lanes, 8 contiguous channels
// (16 bytes) per lane; butterfly stages 1,2,4 run in registers, the rest through wave shuffles, in the
// fixed order 1,2,4,...,BS/2 and then the H2 step across the halves.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

// fp32 -> bf16 -> fp32 with round-to-nearest-even (finite inputs)
LQ_DEV float bf16_round(float x) {
  uint32_t u = __float_as_uint(x);
  u += 0x7fffu + ((u >> 16) & 1u);
  return __uint_as_float(u & 0xffff0000u);
}

LQ_DEV float load_sign(const void* s, int64_t i, int dtype) {
  if (dtype == LQ_DT_F16) return (float)((const _Float16*)s)[i];
  if (dtype == LQ_DT_F32) return ((const float*)s)[i];
  return (float)((const int8_t*)s)[i];
}

// v[8]: this lane's 8 channels of one row; sub = lane index inside the row (0 .. N/8-1); LPH = lanes per half.
// Returns the rotated row in place: w * kron for both halves combined by the H2 step.
template <int LPH>
LQ_DEV void fwht_row(float* v, int sub, float hb, float kron) {
#pragma unroll
  for (int h = 1; h < 8; h <<= 1)
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if ((i & h) == 0) {
        const float a = v[i], b = v[i + h];
        v[i] = a + b;
        v[i + h] = a - b;
      }
#pragma unroll
  for (int m = 1; m < LPH; m <<= 1)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float o = __shfl_xor(v[i], m, 64);
      v[i] = (sub & m) ? (o - v[i]) : (v[i] + o);
    }
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = v[i] * hb;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float o = __shfl_xor(v[i], LPH, 64);
    const float s = (sub & LPH) ? (o - v[i]) : (v[i] + o);
    v[i] = s * kron;
  }
}

// VEC: signs and dqk are 16-byte aligned, so a lane's eight entries are fetched as whole pieces, requested together with
// its row piece before anything is used (element by element, behind a run-time dtype switch, they formed a chain of
// memory round trips several times longer than the transform itself).
// BF: the rows are bf16 in and out (stand-alone rotation only; the fused prologue rounds through fp16 by definition).
template <int N, bool QUANT, bool VEC, bool BF = false>
__global__ __launch_bounds__(256) void rotate_kernel(const _Float16* __restrict__ src, int64_t s_b, int64_t s_t,
                                                     int64_t s_seg, int nseg_per_side, int64_t side_off,
                                                     void* __restrict__ dst0, void* __restrict__ dst1, _Float16* __restrict__ fp0,
                                                     const void* __restrict__ signs, int signs_dtype,
                                                     const float* __restrict__ inv0, const float* __restrict__ inv1,
                                                     const float* __restrict__ dqk0, const float* __restrict__ dqk1,
                                                     int T, float hb, float kron, float* __restrict__ rowmax) {
  constexpr int LPR = N / 8;       // lanes per row
  constexpr int LPH = LPR / 2;     // lanes per half
  constexpr int RPB = 256 / LPR;   // rows per block
  const int sub = threadIdx.x % LPR;
  const int t = blockIdx.x * RPB + threadIdx.x / LPR;
  const int nside = QUANT ? 2 : 1;
  const int b = blockIdx.y / (nside * nseg_per_side);
  const int rem = blockIdx.y % (nside * nseg_per_side);
  const int side = rem / nseg_per_side, seg = rem % nseg_per_side;
  const bool live = t < T;
  const int tt = live ? t : T - 1;  // inactive rows still take part in the shuffles

  const _Float16* sp = src + (int64_t)b * s_b + (int64_t)tt * s_t + side * side_off + (int64_t)seg * s_seg + sub * 8;
  const lq_v4i hraw = *(const lq_v4i*)sp;
  const lq_v8h hv = __builtin_bit_cast(lq_v8h, hraw);
  float xin[8];  // the row piece as fp32
#pragma unroll
  for (int i = 0; i < 8; ++i)
    xin[i] = BF ? __uint_as_float(((uint32_t)hraw[i >> 1] >> (16 * (i & 1))) << 16) : (float)hv[i];
  float v[8];
  const float* dqk = side ? dqk1 : dqk0;
  if constexpr (VEC) {
    // absent operands are read from a valid dummy address (the start of the row) and ignored
    const int64_t e0 = (int64_t)seg * N + sub * 8;
    const float* dq = (QUANT && dqk) ? dqk + e0 : (const float*)(sp - sub * 8);
    const lq_v4f d0 = *(const lq_v4f*)dq, d1 = *(const lq_v4f*)(dq + 4);
    const int es = signs_dtype == LQ_DT_F16 ? 2 : (signs_dtype == LQ_DT_F32 ? 4 : 1);
    const char* sgp = signs ? (const char*)signs + e0 * es : (const char*)(sp - sub * 8);
    const lq_v4i s0 = *(const lq_v4i*)(es == 1 ? sgp - ((uintptr_t)sgp & 8) : sgp);          // int8: the aligned 16 bytes around the 8
    const lq_v4i s1 = *(const lq_v4i*)(es == 4 ? sgp + 16 : sgp - ((uintptr_t)sgp & 15));    // fp32: second half
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = xin[i];
    if (QUANT && dqk) {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (float)(_Float16)(v[i] * (i < 4 ? d0[i & 3] : d1[i & 3]));
    }
    if (signs) {
      const lq_v8h sh = __builtin_bit_cast(lq_v8h, s0);
      const int boff = (int)((uintptr_t)sgp & 8) >> 2;  // int8: dword index of the lane's 8 bytes inside s0
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float f16v = (float)sh[i];
        const float f32v = __int_as_float(i < 4 ? s0[i & 3] : s1[i & 3]);
        const float i8v = (float)lq_sbyte((uint32_t)(boff ? s0[2 + (i >> 2)] : s0[i >> 2]), i & 3);
        const float sg = es == 2 ? f16v : (es == 4 ? f32v : i8v);
        v[i] = bf16_round(v[i] * sg);
      }
      fwht_row<LPH>(v, sub, hb, kron);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = xin[i];
    if (QUANT && dqk) {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (float)(_Float16)(v[i] * dqk[seg * N + sub * 8 + i]);
    }
    if (signs) {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = bf16_round(v[i] * load_sign(signs, (int64_t)seg * N + sub * 8 + i, signs_dtype));
      fwht_row<LPH>(v, sub, hb, kron);
    }
  }
  // max |fp16 value| of the rotated B row, for the key-side chunk state's zero-slab test: the same comparison sequence as
  // its own pre-pass (a NaN wins, so a row holding one is never left out)
  float rmax = 0.0f;
  if (QUANT && rowmax && side == 0) {  // uniform over the block
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float a = __builtin_fabsf((float)(_Float16)v[i]);
      rmax = (a > rmax || a != a) ? a : rmax;
    }
#pragma unroll
    for (int o = 1; o < LPR; o <<= 1) {
      const float t2 = __shfl_xor(rmax, o, 64);
      rmax = (t2 > rmax || t2 != t2) ? t2 : rmax;
    }
  }
  if (!live) return;
  if (QUANT) {
    const float inv = (side ? inv1 : inv0)[seg];
    int code[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) code[i] = lq_q_rint((float)(_Float16)v[i] * inv, -128, 127);
    int8_t* dp = (int8_t*)(side ? dst1 : dst0) + (((int64_t)b * T + t) * nseg_per_side + seg) * N + sub * 8;
    lq_v2i o;
    o[0] = (int)lq_pack4(code[0], code[1], code[2], code[3]);
    o[1] = (int)lq_pack4(code[4], code[5], code[6], code[7]);
    *(lq_v2i*)dp = o;
    if (fp0 && side == 0) {  // the rotated fp16 B itself, for the key-side chunk state
      lq_v8h f;
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = (_Float16)v[i];
      *(lq_v8h*)(fp0 + (((int64_t)b * T + t) * nseg_per_side + seg) * N + sub * 8) = f;
      if (rowmax && sub == 0) rowmax[((int64_t)b * T + t) * nseg_per_side + seg] = rmax;
    }
  } else {
    _Float16* dp = (_Float16*)dst0 + (((int64_t)b * T + t) * nseg_per_side + seg) * N + sub * 8;
    if constexpr (BF) {
      lq_v4i o;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = __float_as_uint(bf16_round(v[2 * i])) >> 16, hi = __float_as_uint(bf16_round(v[2 * i + 1])) & 0xffff0000u;
        o[i] = (int)(lo | hi);
      }
      *(lq_v4i*)dp = o;
    } else {
      lq_v8h o;
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = (_Float16)v[i];
      *(lq_v8h*)dp = o;
    }
  }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

// bf16(1/sqrt(bs)) as float
float hblock_value(int bs) {
  float x = 1.0f / sqrtf((float)bs);
  uint32_t u;
  __builtin_memcpy(&u, &x, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  __builtin_memcpy(&x, &u, 4);
  return x;
}

}  // namespace

extern "C" int lq_split_rotate_quant_xBC(const lq_split_rotate_quant_xBC_args* a, hipStream_t stream) {
  if (!a || !a->xBC || !a->qB || !a->qC || !a->B_inv_scale || !a->C_inv_scale) return LQ_ERR_NULL;
  if ((a->dqk_b == nullptr) != (a->dqk_c == nullptr)) return LQ_ERR_NULL;
  const int N = a->dstate, G = a->ngroups;
  if (a->batch <= 0 || a->seqlen <= 0 || G <= 0 || a->d_ssm < 0) return LQ_ERR_SHAPE;
  if (N != 64 && N != 128) return LQ_ERR_SHAPE;
  if (a->d_ssm % 8 || a->xBC_stride_b % 8 || a->xBC_stride_t % 8 || !al(a->xBC, 16) || !al(a->qB, 8) || !al(a->qC, 8))
    return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * 2 * G > 65535) return LQ_ERR_SHAPE;
  if (a->b_fp && !al(a->b_fp, 16)) return LQ_ERR_SHAPE;
  if (a->b_rowmax && !a->b_fp) return LQ_ERR_NULL;
  const _Float16* src = (const _Float16*)a->xBC + a->d_ssm;
  const float hb = hblock_value(N / 2);
  const float kron = (float)(1.0 / sqrt(2.0));
  const int rpb = 256 / (N / 8);
  dim3 grid((a->seqlen + rpb - 1) / rpb, a->batch * 2 * G);
  const bool vec = (!a->signs || al(a->signs, 16)) && (!a->dqk_b || (al(a->dqk_b, 16) && al(a->dqk_c, 16)));
#define LQ_ROT_LAUNCH(NN, VV)                                                                                          \
  hipLaunchKernelGGL((rotate_kernel<NN, true, VV>), grid, dim3(256), 0, stream, src, a->xBC_stride_b, a->xBC_stride_t, \
                     (int64_t)N, G, (int64_t)G * N, a->qB, a->qC, (_Float16*)a->b_fp, a->signs, a->signs_dtype,         \
                     a->B_inv_scale, a->C_inv_scale, a->dqk_b, a->dqk_c, a->seqlen, hb, kron, a->b_fp ? a->b_rowmax : nullptr)
  if (N == 128) {
    if (vec) LQ_ROT_LAUNCH(128, true); else LQ_ROT_LAUNCH(128, false);
  } else {
    if (vec) LQ_ROT_LAUNCH(64, true); else LQ_ROT_LAUNCH(64, false);
  }
#undef LQ_ROT_LAUNCH
  return lq_check_launch();
}

extern "C" int lq_kron_hadamard(const lq_kron_hadamard_args* a, hipStream_t stream) {
  if (!a || !a->x || !a->y || !a->signs) return LQ_ERR_NULL;
  const int D = a->dim, H = a->nheads;
  if (a->batch <= 0 || a->seqlen <= 0 || H <= 0) return LQ_ERR_SHAPE;
  if (D != 64 && D != 128 && D != 256 && D != 512) return LQ_ERR_SHAPE;  // a row is spread over D / 8 lanes of one wave
  if (a->x_dtype != LQ_DT_F16 && a->x_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  if (a->x_stride_b % 8 || a->x_stride_t % 8 || a->x_stride_h % 8 || !al(a->x, 16) || !al(a->y, 16)) return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * H > 65535) return LQ_ERR_SHAPE;
  const float hb = hblock_value(D / 2);
  const float kron = (float)(1.0 / sqrt(2.0));
  const int rpb = 256 / (D / 8);
  dim3 grid((a->seqlen + rpb - 1) / rpb, a->batch * H);
  const bool vec = al(a->signs, 16), bf = a->x_dtype == LQ_DT_BF16;
#define LQ_KRON_LAUNCH(NN, VV, BB)                                                                                      \
  hipLaunchKernelGGL((rotate_kernel<NN, false, VV, BB>), grid, dim3(256), 0, stream, (const _Float16*)a->x, a->x_stride_b, \
                     a->x_stride_t, a->x_stride_h, H, (int64_t)0, a->y, (void*)nullptr, (_Float16*)nullptr, a->signs,      \
                     a->signs_dtype, (const float*)nullptr, (const float*)nullptr, (const float*)nullptr,                  \
                     (const float*)nullptr, a->seqlen, hb, kron, (float*)nullptr)
#define LQ_KRON_DISPATCH(NN)                     \
  do {                                           \
    if (vec && bf) LQ_KRON_LAUNCH(NN, true, true);       \
    else if (vec) LQ_KRON_LAUNCH(NN, true, false);       \
    else if (bf) LQ_KRON_LAUNCH(NN, false, true);        \
    else LQ_KRON_LAUNCH(NN, false, false);               \
  } while (0)
  switch (D) {
    case 64: LQ_KRON_DISPATCH(64); break;
    case 128: LQ_KRON_DISPATCH(128); break;
    case 256: LQ_KRON_DISPATCH(256); break;
    default: LQ_KRON_DISPATCH(512); break;
  }
#undef LQ_KRON_DISPATCH
#undef LQ_KRON_LAUNCH
  return lq_check_launch();
}
