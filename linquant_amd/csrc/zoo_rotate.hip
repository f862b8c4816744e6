// Zoo prologue: the persistent operand rotations R_QK (on q, k) and R_V (on v) and the diagonal q / k rescaling D_QK,
// one launch for all three tensors.
// Replaces the three bf16 GEMMs q @ R, k @ R, v @ R_V of the reference's timing script (bench/zoo_kernels.py:135-140,
// "not fused yet"), the rotation the oracle applies on entry (linquant/reference.py:42-46: mat(q @ rot_qk),
// mat(k @ rot_qk), mat(v @ rot_v)) and the D_QK input transform (linquant/harness.py:68-88: q' = q D, k' = k / D, the
// quotient rounded once as the division there rounds it).
//
// R = H_n / sqrt(n) . diag(signs) with the Sylvester H_n (linquant/reference.py:232-239), so a row is rotated by a fast
// Walsh-Hadamard transform instead of a GEMM: y_j = signs_j / sqrt(n) * sum_i (x_i d_i) H_ij.  HBM-bound byte work:
// a row of n channels is spread over n / 8 lanes, 16 bytes per lane in and out; butterfly stages 1, 2, 4 run in
// registers, the rest through DPP lane permutations.  fp32 sums of at most 128 half-precision values, one multiply, one
// rounding to the activation dtype.
#include "zoo_common.h"
#include "../../include/linquant_hip.h"

namespace {

struct RotParams {
  const uint16_t* src[3];
  uint16_t* dst[3];
  const float* diag[3];   // (H, D) multiplier, or nullptr
  const float* divd[3];   // (H, D) divisor whose reciprocal diag holds (the row is divided, rounded once), or nullptr
  const float* signs[3];  // (D,) or nullptr: no rotation
  int64_t rows;           // B * T * H
  int nheads;
  float rsqrt_n;
};

LQ_DEV float bf16_to_f(uint16_t u) { return __uint_as_float((uint32_t)u << 16); }
LQ_DEV uint16_t f_to_bf16(float x) {  // round to nearest even (finite inputs)
  uint32_t u = __float_as_uint(x);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// R rows per thread (R * 256 / (D / 8) rows per workgroup): all R requests of a thread are issued before the first row is
// transformed, so a workgroup has R times the bytes in flight of the one-row form (a thread that moves 16 bytes in and
// 16 bytes out and exits spends most of its life on the way in and out of the machine).
template <int D, bool BF16, int R>
__global__ __launch_bounds__(256) void zoo_rotate_kernel(RotParams p) {
  constexpr int LPR = D / 8;      // lanes per row
  constexpr int RPB = 256 / LPR;  // rows per pass of the workgroup
  const int which = blockIdx.y;
  const uint16_t* src = p.src[which];
  if (!src) return;  // block-uniform: this tensor is not part of the call
  const float* diag = p.diag[which];
  const float* divd = p.divd[which];
  const float* signs = p.signs[which];
  const int sub = threadIdx.x % LPR;
  const int64_t row0 = (int64_t)blockIdx.x * (R * RPB) + threadIdx.x / LPR;
  lq_v4i raw[R];
  int hh[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t rr = min(row0 + r * RPB, p.rows - 1);  // surplus rows still take part in the shuffles
    hh[r] = (int)(rr % p.nheads);
    raw[r] = *(const lq_v4i*)(src + rr * D + sub * 8);
  }
  // operands that are absent are read from a valid address and ignored: every request is issued before the first use
  const float* sp = signs ? signs + sub * 8 : (const float*)src;
  const lq_v4f s0 = *(const lq_v4f*)sp, s1 = *(const lq_v4f*)(signs ? sp + 4 : sp);
  lq_v4f d0[R], d1[R], e0[R], e1[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float* dp = diag ? diag + (int64_t)hh[r] * D + sub * 8 : sp;
    d0[r] = *(const lq_v4f*)dp, d1[r] = *(const lq_v4f*)(diag ? dp + 4 : dp);
    const float* ep = divd ? divd + (int64_t)hh[r] * D + sub * 8 : sp;
    e0[r] = *(const lq_v4f*)ep, e1[r] = *(const lq_v4f*)(divd ? ep + 4 : ep);
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + r * RPB;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint16_t u = (uint16_t)((uint32_t)raw[r][i >> 1] >> (16 * (i & 1)));
      v[i] = BF16 ? bf16_to_f(u) : (float)__builtin_bit_cast(_Float16, u);
    }
    if (divd) {  // the quotient rounded once, as a division would give it
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = zoo_div_rn(v[i], i < 4 ? e0[r][i & 3] : e1[r][i & 3], i < 4 ? d0[r][i & 3] : d1[r][i & 3]);
    } else if (diag) {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = zoo_mul_rn(v[i], i < 4 ? d0[r][i & 3] : d1[r][i & 3]);
    }
    if (signs) {
      zoo_fwht<LPR>(v, sub);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (v[i] * p.rsqrt_n) * (i < 4 ? s0[i & 3] : s1[i & 3]);
    }
    if (row < p.rows) {
      lq_v4i out;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint16_t lo, hi;
        if (BF16) {
          lo = f_to_bf16(v[2 * i]), hi = f_to_bf16(v[2 * i + 1]);
        } else {
          lo = __builtin_bit_cast(uint16_t, (_Float16)v[2 * i]), hi = __builtin_bit_cast(uint16_t, (_Float16)v[2 * i + 1]);
        }
        out[i] = (int)((uint32_t)lo | ((uint32_t)hi << 16));
      }
      *(lq_v4i*)(p.dst[which] + row * D + sub * 8) = out;
    }
  }
}

bool al16(const void* q) { return ((uintptr_t)q % 16) == 0; }

// Rows per thread: four for the pure rescaling (a copy with one multiply: 537 MB in 117 -> 104 us at B2 T8192 H32 K128),
// two with the butterflies (their lane exchanges keep the vector ALU busy; one, two and four rows measured 56.6, 55.7
// and 61 us for 268 MB).
template <int D, int R>
int launch_r(const RotParams& p, bool bf16, int64_t rows, hipStream_t stream) {
  constexpr int RPB = R * 256 / (D / 8);
  const int64_t gx = (rows + RPB - 1) / RPB;
  if (gx > 0x7fffffffLL) return LQ_ERR_SHAPE;
  dim3 grid((unsigned)gx, 3);
  if (bf16)
    hipLaunchKernelGGL((zoo_rotate_kernel<D, true, R>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_rotate_kernel<D, false, R>), grid, dim3(256), 0, stream, p);
  return lq_check_launch();
}

template <int D>
int launch(const RotParams& p, bool bf16, int64_t rows, hipStream_t stream) {
  const bool rotates = p.signs[0] || p.signs[1] || p.signs[2];
  return rotates ? launch_r<D, 2>(p, bf16, rows, stream) : launch_r<D, 4>(p, bf16, rows, stream);
}

}  // namespace

extern "C" int lq_zoo_rotate_qkv(const lq_zoo_rotate_qkv_args* a, hipStream_t stream) {
  if (!a) return LQ_ERR_NULL;
  if ((a->q && !a->q_out) || (a->k && !a->k_out) || (a->v && !a->v_out)) return LQ_ERR_NULL;
  if (!a->q && !a->k && !a->v) return LQ_ERR_NULL;
  if (a->k && a->dk && !a->dq) return LQ_ERR_NULL;  // k is divided by dq; dk is its reciprocal
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  const int K = a->kdim, V = a->vdim;
  if ((a->q || a->k) && K != 64 && K != 128) return LQ_ERR_SHAPE;
  if (a->v && V != 64 && V != 128) return LQ_ERR_SHAPE;
  const void* ptrs[] = {a->q, a->k, a->v, a->q_out, a->k_out, a->v_out, a->dq, a->dk, a->signs_qk, a->signs_v};
  for (const void* q : ptrs)
    if (q && !al16(q)) return LQ_ERR_SHAPE;
  const int64_t rows = (int64_t)a->batch * a->seqlen * a->nheads;
  const bool bf16 = a->act_dtype == LQ_DT_BF16;
  // one launch per distinct row width: q and k share K, v joins them when V == K
  for (int pass = 0; pass < 2; ++pass) {
    const bool qk = pass == 0;
    const int D = qk ? K : V;
    RotParams p = {};
    p.rows = rows, p.nheads = a->nheads;
    p.rsqrt_n = (float)(1.0 / sqrt((double)D));
    if (qk) {
      p.src[0] = (const uint16_t*)a->q, p.dst[0] = (uint16_t*)a->q_out, p.diag[0] = a->dq, p.signs[0] = a->signs_qk;
      p.src[1] = (const uint16_t*)a->k, p.dst[1] = (uint16_t*)a->k_out, p.diag[1] = a->dk, p.signs[1] = a->signs_qk;
      p.divd[1] = a->dk ? a->dq : nullptr;
      if (a->v && V == K) p.src[2] = (const uint16_t*)a->v, p.dst[2] = (uint16_t*)a->v_out, p.signs[2] = a->signs_v;
      if (!a->q && !a->k && !(a->v && V == K)) continue;
    } else {
      if (!a->v || V == K) continue;
      p.src[2] = (const uint16_t*)a->v, p.dst[2] = (uint16_t*)a->v_out, p.signs[2] = a->signs_v;
    }
    const int rc = D == 128 ? launch<128>(p, bf16, rows, stream) : launch<64>(p, bf16, rows, stream);
    if (rc != LQ_OK) return rc;
  }
  return LQ_OK;
}
