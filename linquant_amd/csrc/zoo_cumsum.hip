// Chunk-local cumulative log decay and its per-token envelope.
// Replaces the torch prep inside the reference's zoo wrappers (linquant/kernels/zoo/simple_gla.py:191,
// gla.py:249-251, gated_delta_rule.py:174, kda.py:168-170):
//   gc[b, c*C + t, h(,k)] = sum_{s <= t} g[b, c*C + s, h(,k)]          (fp32 values, accumulated in fp64)
//   logenv[b, t, h] = max_k (gc_last[k] - gc[t, k])                     (diagonal decay only)
// One thread walks one (batch, chunk, head[, channel]) column; threads of a workgroup cover adjacent
// channels, so every step is a coalesced row access.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

__global__ __launch_bounds__(256) void cumsum_scalar_kernel(const float* __restrict__ g, float* __restrict__ gc,
                                                            int T, int H, int C, int64_t total) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (b, chunk, h)
  if (idx >= total) return;
  const int h = idx % H;
  const int64_t bc = idx / H;  // b * NT + chunk
  const int64_t base = bc * C * H + h;
  double run = 0.0;
  for (int t = 0; t < C; ++t) {
    run += (double)g[base + (int64_t)t * H];
    gc[base + (int64_t)t * H] = (float)run;
  }
}

// The same scan for the chunk size every caller uses: all 64 values of a thread are requested before the first is added
// (the loop above waits for each load in turn: 64 round trips), summed in the same order.
__global__ __launch_bounds__(256) void cumsum_scalar64_kernel(const float* __restrict__ g, float* __restrict__ gc, int H,
                                                              int64_t total) {
  const int64_t idx = min((int64_t)blockIdx.x * 256 + threadIdx.x, total - 1);  // (b, chunk, h); the tail repeats the last
  const int h = idx % H;
  const int64_t base = (idx / H) * 64 * H + h;
  float v[64];
#pragma unroll
  for (int t = 0; t < 64; ++t) v[t] = g[base + (int64_t)t * H];
  double run = 0.0;
#pragma unroll
  for (int t = 0; t < 64; ++t) {
    run += (double)v[t];
    gc[base + (int64_t)t * H] = (float)run;
  }
}

// one workgroup per (batch, chunk, head); 4*K threads: thread (k, q) scans tokens q*C/4 .. of channel k (all of its
// loads are independent and issued up front), the four partial totals are combined through LDS; LDS tile [C][K+1]
// for the envelope reduction
__global__ void cumsum_diag_kernel(const float* __restrict__ g, float* __restrict__ gc, float* __restrict__ logenv,
                                   int T, int H, int K, int C) {
  extern __shared__ float tile[];           // [C][K + 1]
  double* part = (double*)(tile + C * (K + 1));  // [4][K] segment totals
  const int k = threadIdx.x % K, q = threadIdx.x / K;
  const int SEG = C / 4;                    // tokens per thread (C is a multiple of 16)
  const int h = blockIdx.x % H;
  const int64_t bc = blockIdx.x / H;
  const int64_t row0 = bc * C;  // global token row of the chunk start (b * T + chunk * C)
  const int64_t base = ((row0 + q * SEG) * H + h) * K + k;
  const int64_t tstride = (int64_t)H * K;
  float v[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    // requested without a branch (a load under `t < SEG` is waited for inside its branch: sixteen round trips in a row);
    // tokens past the segment re-read its last one and count as zero
    const float x = g[base + min(t, SEG - 1) * tstride];
    v[t] = t < SEG ? x : 0.0f;
  }
  double run = 0.0, pre[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    run += (double)v[t];
    pre[t] = run;
  }
  part[q * K + k] = run;
  __syncthreads();
  double off = 0.0, total = 0.0;
#pragma unroll
  for (int qq = 0; qq < 4; ++qq) {
    const double pt = part[qq * K + k];
    if (qq < q) off += pt;
    total += pt;
  }
  const float last = (float)total;
#pragma unroll
  for (int t = 0; t < 16; ++t)
    if (t < SEG) {
      const float c = (float)(off + pre[t]);
      gc[base + t * tstride] = c;
      tile[(q * SEG + t) * (K + 1) + k] = last - c;
    }
  __syncthreads();
  // envelope: 8 lanes per token, each over a contiguous K/8 slice, then a max over the 8 lanes
  const int sub = threadIdx.x & 7, KS = K / 8;
  for (int t = threadIdx.x >> 3; t < C; t += blockDim.x >> 3) {
    const float* row = tile + t * (K + 1) + sub * KS;
    float m = row[0];
    for (int j = 1; j < KS; ++j) m = fmaxf(m, row[j]);
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) m = fmaxf(m, __shfl_xor(m, o));
    if (sub == 0) logenv[(row0 + t) * H + h] = m;
  }
}

}  // namespace

extern "C" int lq_zoo_cumsum(const lq_zoo_cumsum_args* a, hipStream_t stream) {
  if (!a || !a->g || !a->gc) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0 || a->chunk_size <= 0 || a->kdim < 0) return LQ_ERR_SHAPE;
  if (a->seqlen % a->chunk_size != 0) return LQ_ERR_SHAPE;
  const int NT = a->seqlen / a->chunk_size;
  if (a->kdim == 0) {
    const int64_t total = (int64_t)a->batch * NT * a->nheads;
    if (a->chunk_size == 64)
      hipLaunchKernelGGL(cumsum_scalar64_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g, a->gc,
                         a->nheads, total);
    else
      hipLaunchKernelGGL(cumsum_scalar_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g, a->gc,
                         a->seqlen, a->nheads, a->chunk_size, total);
  } else {
    if (!a->logenv) return LQ_ERR_NULL;
    if (a->kdim > 256 || a->kdim % 16 != 0 || a->chunk_size % 16 != 0 || a->chunk_size > 64) return LQ_ERR_SHAPE;
    const size_t lds = (size_t)a->chunk_size * (a->kdim + 1) * sizeof(float) + 4 * (size_t)a->kdim * sizeof(double);
    if (lds > 64 * 1024) return LQ_ERR_SHAPE;
    hipLaunchKernelGGL(cumsum_diag_kernel, dim3((unsigned)((int64_t)a->batch * NT * a->nheads)), dim3(4 * a->kdim), lds,
                       stream, a->g, a->gc, a->logenv, a->seqlen, a->nheads, a->kdim, a->chunk_size);
  }
  return lq_check_launch();
}
