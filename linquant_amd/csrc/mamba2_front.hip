// Element-wise stages in front of the Mamba-2 SSD prologue (pure HBM streaming, 16 bytes per lane).
//   lq_fp16_to_int8     replaces _fused_fp16_to_int8 (linquant/w4a8_linear.py:36-98):
//                       q = clamp(rint(x * (1/s)) | rint(x / s), clamp_min, 127), s a device scalar
//   lq_causal_conv1d    replaces causal_conv1d_fn(x, weight, bias, activation="silu") as called at
//                       linquant/quantized_mamba2.py:262-268 (channel-last layout):
//                       y[t, c] = silu(bias[c] + sum_j weight[c, j] * x[t - (W-1) + j, c]), fp32, taps in order j = 0..W-1,
//                       silu(a) = a * rcp(1 + exp2(-a * log2 e)) on the hardware exp2 / reciprocal units (1 ulp each; the
//                       fp16 output absorbs them except at rounding boundaries)
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

__global__ __launch_bounds__(256) void fp16_to_int8_kernel(const _Float16* __restrict__ x, int64_t x_stride,
                                                           int8_t* __restrict__ out, const void* __restrict__ scale,
                                                           int scale_dtype, int rows, int cols, float clamp_min,
                                                           int reciprocal) {
  const float s = scale_dtype == LQ_DT_F16 ? (float)*(const _Float16*)scale : *(const float*)scale;
  const float inv = 1.0f / s;  // correctly rounded
  // x / s with a uniform divisor: q0 = RN(x * inv), r = x - q0 * s (exact in one fma), q = RN(q0 + r * inv) is the
  // correctly rounded quotient whenever nothing under- or overflows (Markstein's final-quotient step). fp16 inputs span
  // 2^-24 .. 2^16, so a scale within 2^-60 .. 2^60 keeps x, q0, r and r * inv in the normal range; outside it the plain
  // IEEE divide runs.
  const float as = __builtin_fabsf(s);
  const bool fast_div = as > 0x1p-60f && as < 0x1p60f;
  const uint32_t c8n = (uint32_t)cols >> 3;  // 16-byte pieces per row
  const uint32_t total = (uint32_t)rows * c8n;  // the launcher rejects 2^32 pieces or more
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < total; i += gridDim.x * 256u) {
    const uint32_t r = i / c8n;
    const uint32_t c = (i - r * c8n) * 8u;
    const lq_v8h v = *(const lq_v8h*)(x + (int64_t)r * x_stride + c);
    int code[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float xf = (float)v[e];
      float y = xf * inv;
      if (!reciprocal) {
        if (fast_div) {
          const float rem = __builtin_fmaf(-y, s, xf);
          const float y2 = __builtin_fmaf(rem, inv, y);
          y = y2 == y2 ? y2 : y;  // an infinite x gives rem = NaN: keep the infinite first quotient
        } else {
          y = xf / s;
        }
      }
      code[e] = (int)fminf(fmaxf(__builtin_rintf(y), clamp_min), 127.0f);
    }
    lq_v2i o;
    o[0] = (int)lq_pack4(code[0], code[1], code[2], code[3]);
    o[1] = (int)lq_pack4(code[4], code[5], code[6], code[7]);
    *(lq_v2i*)(out + (int64_t)r * cols + c) = o;
  }
}

constexpr int kTL = 16;  // tokens per thread: the W-1 halo rows are re-read once per 16 outputs

template <int W>
__global__ __launch_bounds__(256) void causal_conv1d_kernel(const _Float16* __restrict__ x, int64_t sx_b, int64_t sx_l,
                                                            const _Float16* __restrict__ weight,
                                                            const _Float16* __restrict__ bias, _Float16* __restrict__ out,
                                                            int L, int D, int silu) {
  const int c8n = D >> 3;
  const int idx = blockIdx.x * 256 + threadIdx.x;  // (token block, channel group), channel groups fastest
  const int cg = idx % c8n, tb = idx / c8n;
  const int b = blockIdx.y;
  const int t0 = tb * kTL;
  if (t0 >= L) return;
  const int c = cg * 8;
  // Every request of the thread is issued before the first use and outside any branch: the taps of its 8 channels are
  // 8 W contiguous halves (W 16-byte pieces; element-wise loads, a branch on `bias` and one on `t >= 0` per halo row
  // made a chain of about eight memory round trips in front of the x rows), the bias piece comes from a valid dummy
  // address when there is none, halo rows before the sequence start re-read row 0 and are zeroed in registers.
  lq_v8h wraw[W];
#pragma unroll
  for (int j = 0; j < W; ++j) wraw[j] = *(const lq_v8h*)(weight + (int64_t)c * W + 8 * j);
  const lq_v8h braw = *(const lq_v8h*)(bias ? bias + c : weight + (int64_t)c * W);
  const _Float16* xp = x + (int64_t)b * sx_b + c;
  lq_v8h halo[W - 1];
#pragma unroll
  for (int j = 0; j < W - 1; ++j) halo[j] = *(const lq_v8h*)(xp + (int64_t)max(t0 - (W - 1) + j, 0) * sx_l);
  _Float16* op = out + ((int64_t)b * L) * D + c;
  // all rows of the block are requested before the first one is used (the clamped row index keeps a ragged last block
  // inside the sequence; its surplus rows are computed and not stored)
  lq_v8h rows[kTL];
#pragma unroll
  for (int i = 0; i < kTL; ++i) {
    const int t = t0 + i < L ? t0 + i : L - 1;
    rows[i] = *(const lq_v8h*)(xp + (int64_t)t * sx_l);
  }
  float w[W][8], bv[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    bv[e] = bias ? (float)braw[e] : 0.0f;
#pragma unroll
    for (int j = 0; j < W; ++j) w[j][e] = (float)wraw[(e * W + j) >> 3][(e * W + j) & 7];  // weight[(c + e) * W + j]
  }
  float win[W][8];  // sliding window: win[j] = x[t - (W-1) + j]
#pragma unroll
  for (int j = 0; j < W - 1; ++j) {
    const bool in = t0 - (W - 1) + j >= 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) win[j + 1][e] = in ? (float)halo[j][e] : 0.0f;
  }
#pragma unroll
  for (int i = 0; i < kTL; ++i) {
    const int t = t0 + i;
#pragma unroll
    for (int j = 0; j < W - 1; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) win[j][e] = win[j + 1][e];
    lq_v8h o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      win[W - 1][e] = (float)rows[i][e];
      float a = bv[e];
#pragma unroll
      for (int j = 0; j < W; ++j) a = a + w[j][e] * win[j][e];
      if (silu) a = a * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(a * -1.44269504088896340736f));
      o[e] = (_Float16)a;
    }
    if (t < L) __builtin_nontemporal_store(o, (lq_v8h*)(op + (int64_t)t * D));
  }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

}  // namespace

extern "C" int lq_fp16_to_int8(const lq_fp16_to_int8_args* a, hipStream_t stream) {
  if (!a || !a->x || !a->out || !a->scale) return LQ_ERR_NULL;
  if (a->rows <= 0 || a->cols <= 0 || a->cols % 8 != 0 || a->x_stride % 8 != 0) return LQ_ERR_SHAPE;
  if (a->scale_dtype != LQ_DT_F16 && a->scale_dtype != LQ_DT_F32) return LQ_ERR_SHAPE;
  if (!al(a->x, 16) || !al(a->out, 8)) return LQ_ERR_SHAPE;
  if (!(a->clamp_min >= -128.0f && a->clamp_min <= 0.0f)) return LQ_ERR_SHAPE;
  const int64_t total = (int64_t)a->rows * (a->cols / 8);
  if (total >= ((int64_t)1 << 32) - 256 * 256 * 32) return LQ_ERR_SHAPE;  // the kernel indexes pieces in 32 bits
  const int64_t blocks = (total + 255) / 256;
  const unsigned grid = (unsigned)(blocks < 256 * 32 ? blocks : 256 * 32);
  hipLaunchKernelGGL(fp16_to_int8_kernel, dim3(grid), dim3(256), 0, stream, (const _Float16*)a->x, a->x_stride, a->out,
                     a->scale, a->scale_dtype, a->rows, a->cols, a->clamp_min, a->reciprocal);
  return lq_check_launch();
}

extern "C" int lq_causal_conv1d(const lq_causal_conv1d_args* a, hipStream_t stream) {
  if (!a || !a->x || !a->weight || !a->out) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->dim <= 0 || a->dim % 8 != 0 || a->batch > 65535) return LQ_ERR_SHAPE;
  if (a->width < 2 || a->width > 4) return LQ_ERR_SHAPE;
  if (a->x_stride_b % 8 != 0 || a->x_stride_l % 8 != 0 || !al(a->x, 16) || !al(a->out, 16)) return LQ_ERR_SHAPE;
  if (!al(a->weight, 16) || (a->bias && !al(a->bias, 16))) return LQ_ERR_SHAPE;  // taps and bias are read as 16-byte pieces
  const int64_t items = (int64_t)(a->dim / 8) * ((a->seqlen + kTL - 1) / kTL);
  if (items > 0x7fffffff) return LQ_ERR_SHAPE;
  dim3 grid((unsigned)((items + 255) / 256), a->batch);
  const _Float16* x = (const _Float16*)a->x;
  const _Float16* wt = (const _Float16*)a->weight;
  const _Float16* bs = (const _Float16*)a->bias;
  _Float16* out = (_Float16*)a->out;
  switch (a->width) {
    case 2: hipLaunchKernelGGL(causal_conv1d_kernel<2>, grid, dim3(256), 0, stream, x, a->x_stride_b, a->x_stride_l, wt, bs, out, a->seqlen, a->dim, a->silu); break;
    case 3: hipLaunchKernelGGL(causal_conv1d_kernel<3>, grid, dim3(256), 0, stream, x, a->x_stride_b, a->x_stride_l, wt, bs, out, a->seqlen, a->dim, a->silu); break;
    default: hipLaunchKernelGGL(causal_conv1d_kernel<4>, grid, dim3(256), 0, stream, x, a->x_stride_b, a->x_stride_l, wt, bs, out, a->seqlen, a->dim, a->silu); break;
  }
  return lq_check_launch();
}
