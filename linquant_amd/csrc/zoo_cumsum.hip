// Chunk-local cumulative log decay and its per-token envelope.
// Replaces the torch prep inside the reference's zoo wrappers (linquant/kernels/zoo/simple_gla.py:191,
// gla.py:249-251, gated_delta_rule.py:174, kda.py:168-170):
//   gc[b, c*C + t, h(,k)] = sum_{s <= t} g[b, c*C + s, h(,k)]          (fp32 values, accumulated in fp64)
//   logenv[b, t, h] = max_k (gc_last[k] - gc[t, k])                     (diagonal decay only)
// One thread walks one (batch, chunk, head[, channel]) column; threads of a workgroup cover adjacent
// channels, so every step is a coalesced row access.
#include "zoo_common.h"
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

// The same scan for the chunk sizes the callers use (C = 64, 128, 192 or 256): 64 values of a thread are requested before the first
// is added (the loop above waits for each load in turn: C round trips), summed in the same order.
template <int C>
__global__ __launch_bounds__(256) void cumsum_scalar_fixed_kernel(const float* __restrict__ g, float* __restrict__ gc, int H,
                                                                  int64_t total) {
  const int64_t idx = min((int64_t)blockIdx.x * 256 + threadIdx.x, total - 1);  // (b, chunk, h); the tail repeats the last
  const int h = idx % H;
  const int64_t base = (idx / H) * C * H + h;
  double run = 0.0;
#pragma unroll 1
  for (int t0 = 0; t0 < C; t0 += 64) {
    float v[64];
#pragma unroll
    for (int t = 0; t < 64; ++t) v[t] = g[base + (int64_t)(t0 + t) * H];
#pragma unroll
    for (int t = 0; t < 64; ++t) {
      run += (double)v[t];
      gc[base + (int64_t)(t0 + t) * H] = (float)run;
    }
  }
}

// Write operands of the linear family's state kernel under per-channel decay, made by the cumsum launch from the decay
// tile it holds (what lq_zoo_write_codes would make from the stored gc and logenv; same arithmetic, same bits):
//   kqT[k][t] = q8(key[t][k] * exp(gk_last - gk_t - eta*le_t), 1/skw[k]),  vqT[v][t] = q8(val[t][v] * exp(eta*le_t), 1/svw[v]),
//   ev[t] = exp(eta*le_t),  gam[k] = exp(gk_last).
struct CumsumCodes {
  const uint16_t* k;
  const uint16_t* v;
  int8_t* kqT;
  int8_t* vqT;
  float* ev;
  float* gam;
  const float* skw;
  const float* svw;
  float eta;
  int qmax;
  int V;
  int bf;
};

// one workgroup per (batch, chunk, head); 4*K threads: thread (k, q) scans tokens q*C/4 .. of channel k (all of its
// loads are independent and issued up front), the four partial totals are combined through LDS; LDS tile [C][K+1]
// for the envelope reduction.  CODES (chunk 64 only): a thread's 16 tokens of one channel are one 16-byte piece of that
// channel's row of channel-major codes, so the codes go straight from registers to memory.
// SM = tokens per thread at most: 16 (chunks up to 64 tokens), or 32 (128-token chunks: the envelope tile then holds one half
// of the chunk at a time, so that the workgroup's LDS stays what a 64-token chunk takes).
template <bool CODES, int SM = 16>
__global__ void cumsum_diag_kernel(const float* __restrict__ g, float* __restrict__ gc, float* __restrict__ logenv,
                                   int T, int H, int K, int C, CumsumCodes cc) {
  static_assert(!CODES || SM == 16, "the write codes are made for 64-token chunks");
  constexpr int PH = SM / 16;               // passes over the envelope tile
  const int CT = C / PH;                    // tokens the tile holds at a time
  extern __shared__ float tile[];           // [CT][K + 1]
  double* part = (double*)(tile + CT * (K + 1));  // [4][K] segment totals
  float* le_s = (float*)(part + 4 * K);      // [C] log envelope (CODES)
  const int k = threadIdx.x % K, q = threadIdx.x / K;
  const int SEG = C / 4;                    // tokens per thread (C is a multiple of 16)
  // Workgroups are dealt to the 8 XCDs round-robin in launch order and each XCD has its own L2: workgroup L = x + 8 m takes
  // head m % H of (batch, chunk) number x + 8 (m / H), so that one XCD handles all heads of a (batch, chunk) and writes the
  // (B, T, H) log envelope (four bytes per token and head) as whole lines
  const uint32_t ngroups = gridDim.x / (uint32_t)H;
  int h;
  int64_t bc;
  if ((ngroups & 7u) == 0) {
    const uint32_t m = blockIdx.x >> 3;
    h = (int)(m % (uint32_t)H);
    bc = (int64_t)((blockIdx.x & 7u) + 8u * (m / (uint32_t)H));
  } else {
    h = (int)(blockIdx.x % (uint32_t)H);
    bc = blockIdx.x / (uint32_t)H;
  }
  const int64_t row0 = bc * C;  // global token row of the chunk start (b * T + chunk * C)
  const int64_t base = ((row0 + q * SEG) * H + h) * K + k;
  const int64_t tstride = (int64_t)H * K;
  float v[SM];
#pragma unroll
  for (int t = 0; t < SM; ++t) {
    // requested without a branch (a load under `t < SEG` is waited for inside its branch: sixteen round trips in a row);
    // tokens past the segment re-read its last one and count as zero
    const float x = g[base + min(t, SEG - 1) * tstride];
    v[t] = t < SEG ? x : 0.0f;
  }
  // CODES: this thread's 16 key values (channel k, tokens 16q ..) and its value channels' 16 values, requested now
  uint16_t kraw[CODES ? 16 : 1];
  float inv_skw = 0.0f;
  if constexpr (CODES) {
#pragma unroll
    for (int t = 0; t < 16; ++t) kraw[t] = cc.k[base + t * tstride];
    inv_skw = 1.0f / cc.skw[h * K + k];
  }
  double run = 0.0, pre[SM];
#pragma unroll
  for (int t = 0; t < SM; ++t) {
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
  for (int t = 0; t < SM; ++t)
    if (t < SEG) gc[base + t * tstride] = (float)(off + pre[t]);
#pragma unroll 1
  for (int ph = 0; ph < PH; ++ph) {
    if (ph) __syncthreads();  // the previous pass has been read
#pragma unroll
    for (int t = 0; t < SM; ++t) {
      const int tok = q * SEG + t - ph * CT;  // row of the tile
      if (t < SEG && tok >= 0 && tok < CT) tile[tok * (K + 1) + k] = last - (float)(off + pre[t]);
    }
    __syncthreads();
    // envelope: 8 lanes per token, each over a contiguous K/8 slice, then a max over the 8 lanes
    const int sub = threadIdx.x & 7, KS = K / 8;
    for (int t = threadIdx.x >> 3; t < CT; t += blockDim.x >> 3) {
      const float* row = tile + t * (K + 1) + sub * KS;
      float m = row[0];
      for (int j = 1; j < KS; ++j) m = fmaxf(m, row[j]);
#pragma unroll
      for (int o = 1; o < 8; o <<= 1) m = fmaxf(m, __shfl_xor(m, o));
      if (sub == 0) {
        logenv[(row0 + ph * CT + t) * H + h] = m;
        if constexpr (CODES) {
          le_s[t] = m;
          cc.ev[(row0 + t) * H + h] = zoo_exp(cc.eta * m);
        }
      }
    }
  }
  if constexpr (CODES) {
    __syncthreads();
    const bool bf = cc.bf;
    const int64_t cb = bc * H + h;  // (batch, chunk, head)
    if (q == 0) cc.gam[cb * K + k] = zoo_exp(last);
    // key write codes: 16 tokens of channel k
    int code[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const int tok = 16 * q + t;
      const float el = cc.eta * le_s[tok];
      const float x = zoo_dec1(kraw[t], bf) * zoo_exp(tile[tok * (K + 1) + k] - el);
      code[t] = zoo_q8(x, inv_skw, cc.qmax);
    }
    lq_v4i o;
#pragma unroll
    for (int d = 0; d < 4; ++d) o[d] = (int)zoo_pack_codes(code[4 * d], code[4 * d + 1], code[4 * d + 2], code[4 * d + 3]);
    *(lq_v4i*)(cc.kqT + (cb * K + k) * 64 + 16 * q) = o;
    // value write codes: channel c = k, k + K, ... of the V value channels
    const int V = cc.V;
    for (int c = k; c < V; c += K) {
      const float inv_svw = 1.0f / cc.svw[h * V + c];
      uint16_t vraw[16];
#pragma unroll
      for (int t = 0; t < 16; ++t) vraw[t] = cc.v[((row0 + 16 * q + t) * H + h) * V + c];
#pragma unroll
      for (int t = 0; t < 16; ++t) code[t] = zoo_q8(zoo_dec1(vraw[t], bf) * zoo_exp(cc.eta * le_s[16 * q + t]), inv_svw, cc.qmax);
#pragma unroll
      for (int d = 0; d < 4; ++d) o[d] = (int)zoo_pack_codes(code[4 * d], code[4 * d + 1], code[4 * d + 2], code[4 * d + 3]);
      *(lq_v4i*)(cc.vqT + (cb * V + c) * 64 + 16 * q) = o;
    }
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
      hipLaunchKernelGGL(cumsum_scalar_fixed_kernel<64>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g,
                         a->gc, a->nheads, total);
    else if (a->chunk_size == 128)
      hipLaunchKernelGGL(cumsum_scalar_fixed_kernel<128>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g,
                         a->gc, a->nheads, total);
    else if (a->chunk_size == 192)
      hipLaunchKernelGGL(cumsum_scalar_fixed_kernel<192>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g,
                         a->gc, a->nheads, total);
    else if (a->chunk_size == 256)
      hipLaunchKernelGGL(cumsum_scalar_fixed_kernel<256>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g,
                         a->gc, a->nheads, total);
    else
      hipLaunchKernelGGL(cumsum_scalar_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, a->g, a->gc,
                         a->seqlen, a->nheads, a->chunk_size, total);
  } else {
    if (!a->logenv) return LQ_ERR_NULL;
    const bool big = a->chunk_size == 128;  // two passes over an envelope tile of 64 tokens
    if (a->kdim > 256 || a->kdim % 16 != 0 || a->chunk_size % 16 != 0 || (a->chunk_size > 64 && !big)) return LQ_ERR_SHAPE;
    if (big && a->kqT) return LQ_ERR_SHAPE;
    const int ctile = big ? 64 : a->chunk_size;
    const size_t lds = (size_t)ctile * (a->kdim + 1) * sizeof(float) + 4 * (size_t)a->kdim * sizeof(double) +
                       (size_t)ctile * sizeof(float);
    if (lds > 64 * 1024) return LQ_ERR_SHAPE;
    CumsumCodes cc = {};
    const dim3 grid((unsigned)((int64_t)a->batch * NT * a->nheads)), block(4 * a->kdim);
    if (a->kqT) {
      if (!a->k || !a->v || !a->vqT || !a->ev || !a->gam || !a->skw || !a->svw) return LQ_ERR_NULL;
      if (a->chunk_size != 64 || a->vdim <= 0 || a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
      if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
      if (!zoo_al(a->kqT, 16) || !zoo_al(a->vqT, 16)) return LQ_ERR_SHAPE;
      cc.k = (const uint16_t*)a->k, cc.v = (const uint16_t*)a->v, cc.kqT = a->kqT, cc.vqT = a->vqT, cc.ev = a->ev, cc.gam = a->gam;
      cc.skw = a->skw, cc.svw = a->svw, cc.eta = a->eta, cc.qmax = a->qmax, cc.V = a->vdim, cc.bf = a->act_dtype == LQ_DT_BF16;
      hipLaunchKernelGGL(cumsum_diag_kernel<true>, grid, block, lds, stream, a->g, a->gc, a->logenv, a->seqlen, a->nheads,
                         a->kdim, a->chunk_size, cc);
    } else if (big) {
      hipLaunchKernelGGL((cumsum_diag_kernel<false, 32>), grid, block, lds, stream, a->g, a->gc, a->logenv, a->seqlen,
                         a->nheads, a->kdim, a->chunk_size, cc);
    } else {
      hipLaunchKernelGGL(cumsum_diag_kernel<false>, grid, block, lds, stream, a->g, a->gc, a->logenv, a->seqlen, a->nheads,
                         a->kdim, a->chunk_size, cc);
    }
  }
  return lq_check_launch();
}
