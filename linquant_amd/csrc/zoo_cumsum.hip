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

// one workgroup per (batch, chunk, head); K threads; LDS tile [C][K+1] for the envelope reduction
__global__ void cumsum_diag_kernel(const float* __restrict__ g, float* __restrict__ gc, float* __restrict__ logenv,
                                   int T, int H, int K, int C) {
  extern __shared__ float tile[];
  const int k = threadIdx.x;
  const int h = blockIdx.x % H;
  const int64_t bc = blockIdx.x / H;
  const int64_t row0 = bc * C;  // global token row of the chunk start (b * T + chunk * C)
  const int64_t base = (row0 * H + h) * K + k;
  const int64_t tstride = (int64_t)H * K;
  double run = 0.0;
  for (int t = 0; t < C; ++t) {
    run += (double)g[base + t * tstride];
    const float v = (float)run;
    gc[base + t * tstride] = v;
    tile[t * (K + 1) + k] = v;
  }
  const float last = (float)run;
  for (int t = 0; t < C; ++t) tile[t * (K + 1) + k] = last - tile[t * (K + 1) + k];
  __syncthreads();
  for (int t = threadIdx.x; t < C; t += blockDim.x) {
    float m = tile[t * (K + 1)];
    for (int j = 1; j < K; ++j) m = fmaxf(m, tile[t * (K + 1) + j]);
    logenv[(row0 + t) * H + h] = m;
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
    hipLaunchKernelGGL(cumsum_scalar_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g, a->gc,
                       a->seqlen, a->nheads, a->chunk_size, total);
  } else {
    if (!a->logenv) return LQ_ERR_NULL;
    if (a->kdim > 1024) return LQ_ERR_SHAPE;
    const size_t lds = (size_t)a->chunk_size * (a->kdim + 1) * sizeof(float);
    if (lds > 64 * 1024) return LQ_ERR_SHAPE;
    hipLaunchKernelGGL(cumsum_diag_kernel, dim3((unsigned)((int64_t)a->batch * NT * a->nheads)), dim3(a->kdim), lds,
                       stream, a->g, a->gc, a->logenv, a->seqlen, a->nheads, a->kdim, a->chunk_size);
  }
  return lq_check_launch();
}
