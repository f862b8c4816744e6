// Mamba-2 SSD stage 1: dt pipeline + chunk-local cumulative sum of dt*A.
// Replaces the reference stage linquant/kernels/mamba2/chunk_cumsum.py:27-74 (launcher :77-100).
//
// One 8-wave workgroup per (16 heads, chunk, batch): the (token, head) tile of raw dt is staged through LDS with
// head-contiguous reads (dt is laid out (B, L, H): a head's tokens are H elements apart), then each wavefront
// scans two heads.  Lane l owns the E = Q/64 consecutive positions l*E .. l*E+E-1 of the chunk.  The prefix sum is: sequential inside the lane, Hillis-Steele
// inclusive scan of the lane totals over the wave (offsets 1,2,4,...,32, "t = t + up"), then
// exclusive lane prefix + local prefix.  The CPU checker restates exactly this order.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int kMaxE = 16;  // chunk sizes up to 1024

LQ_DEV float load_dt(const void* p, int64_t off, int dtype) {
  if (dtype == LQ_DT_F16) return (float)((const _Float16*)p)[off];
  if (dtype == LQ_DT_F32) return ((const float*)p)[off];
  return (float)((const int8_t*)p)[off];
}

constexpr int kHG = 16;   // heads per workgroup: one token row of the tile is 16 adjacent heads (32 bytes of fp16 dt)
constexpr int kWaves = 8;  // two heads per wave

// Which (head group, chunk, batch) a workgroup of the flat grid works on.  Workgroups are dealt to the 8 XCDs round-robin
// in launch order, and the head groups of one (chunk, batch) read the same 128-byte lines of dt (a token row of 80 heads
// is 160 bytes): on consecutive workgroups every XCD's L2 fetched those lines from HBM for itself (21 MB read for 5 MB
// of dt).  Workgroup 8 j + x takes head group j % hg of unit 8 (j / hg) + x, so a unit's head groups share one XCD.
struct Where {
  int h0, c, b;
};
LQ_DEV Where where(int hg, int nchunks, int by_xcd) {
  uint32_t unit, grp;
  if (by_xcd) {
    const uint32_t x = blockIdx.x & 7u, j = blockIdx.x >> 3;
    const uint32_t uh = j / (uint32_t)hg;
    grp = j - uh * (uint32_t)hg, unit = uh * 8u + x;
  } else {
    unit = blockIdx.x / (uint32_t)hg, grp = blockIdx.x - unit * (uint32_t)hg;
  }
  Where w;
  w.b = (int)(unit / (uint32_t)nchunks), w.c = (int)(unit - (uint32_t)w.b * (uint32_t)nchunks), w.h0 = (int)grp * kHG;
  return w;
}

__global__ __launch_bounds__(kWaves * 64) void chunk_cumsum_kernel(
    const void* __restrict__ dt_in, int dt_dtype, int64_t sdt_b, int64_t sdt_l, int64_t sdt_h,
    const float* __restrict__ dt_scale_p, const int8_t* __restrict__ a_log, int64_t sa_h,
    const float* __restrict__ a_log_scale_p, const float* __restrict__ dt_bias, int64_t sbias_h,
    float* __restrict__ dt_out, float* __restrict__ dA_cs, int seqlen, int nheads, int nchunks, int Q,
    int softplus, float dt_min, float dt_max, int hg, int by_xcd) {
  extern __shared__ float tile[];  // [Q][kHG + 1] raw dt as float
  const Where wh = where(hg, nchunks, by_xcd);
  const int h0 = wh.h0, c = wh.c, b = wh.b;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int E = Q >> 6;
  const int limit = min(Q, seqlen - c * Q);
  // ---- stage the (token, head) tile: consecutive lanes read consecutive heads of one token
  for (int it = tid; it < Q * kHG; it += kWaves * 64) {
    const int pos = it / kHG, hh = it % kHG;
    float v = 0.0f;
    if (pos < limit && h0 + hh < nheads)
      v = load_dt(dt_in, (int64_t)b * sdt_b + (int64_t)(c * Q + pos) * sdt_l + (int64_t)(h0 + hh) * sdt_h, dt_dtype);
    tile[pos * (kHG + 1) + hh] = v;
  }
  __syncthreads();
  const float dt_scale = *dt_scale_p;
  const float a_scale = *a_log_scale_p;
#pragma unroll
  for (int hw = 0; hw < kHG / kWaves; ++hw) {
    const int hh = wave * (kHG / kWaves) + hw;
    const int h = h0 + hh;
    if (h >= nheads) continue;
    const float A = -lq_expf(a_scale * (float)a_log[(int64_t)h * sa_h]);
    const float bias = dt_bias ? dt_bias[(int64_t)h * sbias_h] : 0.0f;
    float dtv[kMaxE], pre[kMaxE];
    float run = 0.0f;
#pragma unroll
    for (int i = 0; i < kMaxE; ++i) {
      if (i < E) {
        const int pos = lane * E + i;
        float v = 0.0f;
        if (pos < limit) {
          v = dt_scale * tile[pos * (kHG + 1) + hh];
          if (dt_bias) v = v + bias;
          if (softplus) v = (v > 20.0f) ? v : lq_logf(1.0f + lq_expf(v));
          v = fminf(fmaxf(v, dt_min), dt_max);
        }
        dtv[i] = v;
        const float dA = v * A;
        run = (i == 0) ? dA : run + dA;
        pre[i] = run;
      }
    }
    float t = run;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float up = __shfl_up(t, off, 64);
      if (lane >= off) t = t + up;
    }
    float ex = __shfl_up(t, 1, 64);
    if (lane == 0) ex = 0.0f;
    const int64_t base = (((int64_t)b * nheads + h) * nchunks + c) * Q + lane * E;
#pragma unroll
    for (int i = 0; i < kMaxE; ++i) {
      if (i < E) {
        dt_out[base + i] = dtv[i];
        dA_cs[base + i] = ex + pre[i];
      }
    }
  }
}

// The same kernel for chunk sizes of 64 E tokens with E known at compile time (1, 2, 4, 8): every dt of the tile, A_log and
// the bias are requested before the first use, outside any branch (in the generic kernel each staging iteration and each
// head waits for its own load), the element loops have no run-time bounds, and a lane's E outputs leave as one vector
// store when E is 2 or 4.
template <int E>
__global__ __launch_bounds__(kWaves * 64) void chunk_cumsum_fixed_kernel(
    const void* __restrict__ dt_in, int dt_dtype, int64_t sdt_b, int64_t sdt_l, int64_t sdt_h,
    const float* __restrict__ dt_scale_p, const int8_t* __restrict__ a_log, int64_t sa_h,
    const float* __restrict__ a_log_scale_p, const float* __restrict__ dt_bias, int64_t sbias_h,
    float* __restrict__ dt_out, float* __restrict__ dA_cs, int seqlen, int nheads, int nchunks,
    int softplus, float dt_min, float dt_max, int hg, int by_xcd) {
  constexpr int Q = 64 * E, NIT = Q * kHG / (kWaves * 64);
  extern __shared__ float tile[];  // [Q][kHG + 1] raw dt as float
  const Where wh = where(hg, nchunks, by_xcd);
  const int h0 = wh.h0, c = wh.c, b = wh.b;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int limit = min(Q, seqlen - c * Q);
  // ---- requests: the (token, head) tile (consecutive lanes read consecutive heads of one token; positions past the
  // sequence end or the last head re-read a valid neighbour and are zeroed below), then the per-head constants
  float raw[NIT];
  int64_t offs[NIT];
#pragma unroll
  for (int i = 0; i < NIT; ++i) {
    const int it = tid + i * kWaves * 64;
    const int pos = min(it / kHG, limit - 1), hh = min(it % kHG, nheads - 1 - h0);
    offs[i] = (int64_t)b * sdt_b + (int64_t)(c * Q + pos) * sdt_l + (int64_t)(h0 + hh) * sdt_h;
  }
  if (dt_dtype == LQ_DT_F16) {  // one uniform branch around all requests of a dtype, not one per request
    _Float16 r[NIT];
#pragma unroll
    for (int i = 0; i < NIT; ++i) r[i] = ((const _Float16*)dt_in)[offs[i]];
#pragma unroll
    for (int i = 0; i < NIT; ++i) raw[i] = (float)r[i];
  } else if (dt_dtype == LQ_DT_F32) {
#pragma unroll
    for (int i = 0; i < NIT; ++i) raw[i] = ((const float*)dt_in)[offs[i]];
  } else {
    int8_t r[NIT];
#pragma unroll
    for (int i = 0; i < NIT; ++i) r[i] = ((const int8_t*)dt_in)[offs[i]];
#pragma unroll
    for (int i = 0; i < NIT; ++i) raw[i] = (float)r[i];
  }
  int8_t alog[kHG / kWaves];
  float bias[kHG / kWaves];
#pragma unroll
  for (int hw = 0; hw < kHG / kWaves; ++hw) {
    const int h = min(h0 + wave * (kHG / kWaves) + hw, nheads - 1);
    alog[hw] = a_log[(int64_t)h * sa_h];
    bias[hw] = dt_bias ? dt_bias[(int64_t)h * sbias_h] : 0.0f;
  }
  const float dt_scale = *dt_scale_p;
  const float a_scale = *a_log_scale_p;
#pragma unroll
  for (int i = 0; i < NIT; ++i) {
    const int it = tid + i * kWaves * 64;
    const int pos = it / kHG, hh = it % kHG;
    tile[pos * (kHG + 1) + hh] = (pos < limit && h0 + hh < nheads) ? raw[i] : 0.0f;
  }
  __syncthreads();
#pragma unroll
  for (int hw = 0; hw < kHG / kWaves; ++hw) {
    const int hh = wave * (kHG / kWaves) + hw;
    const int h = h0 + hh;
    if (h >= nheads) continue;
    const float A = -lq_expf(a_scale * (float)alog[hw]);
    float dtv[E], pre[E];
    float run = 0.0f;
#pragma unroll
    for (int i = 0; i < E; ++i) {
      const int pos = lane * E + i;
      float v = dt_scale * tile[pos * (kHG + 1) + hh];
      if (dt_bias) v = v + bias[hw];
      if (softplus) v = (v > 20.0f) ? v : lq_logf(1.0f + lq_expf(v));
      v = fminf(fmaxf(v, dt_min), dt_max);
      v = pos < limit ? v : 0.0f;
      dtv[i] = v;
      const float dA = v * A;
      run = (i == 0) ? dA : run + dA;
      pre[i] = run;
    }
    float t = run;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float up = __shfl_up(t, off, 64);
      if (lane >= off) t = t + up;
    }
    float ex = __shfl_up(t, 1, 64);
    if (lane == 0) ex = 0.0f;
    const int64_t base = (((int64_t)b * nheads + h) * nchunks + c) * Q + lane * E;
    if constexpr (E == 4) {
      *(lq_v4f*)(dt_out + base) = lq_v4f{dtv[0], dtv[1], dtv[2], dtv[3]};
      *(lq_v4f*)(dA_cs + base) = lq_v4f{ex + pre[0], ex + pre[1], ex + pre[2], ex + pre[3]};
    } else {
#pragma unroll
      for (int i = 0; i < E; ++i) {
        dt_out[base + i] = dtv[i];
        dA_cs[base + i] = ex + pre[i];
      }
    }
  }
}

}  // namespace

extern "C" int lq_chunk_cumsum(const lq_chunk_cumsum_args* a, hipStream_t stream) {
  if (!a || !a->dt || !a->dt_scale || !a->A_log || !a->A_log_scale || !a->dt_out || !a->dA_cumsum) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0 || a->batch > 65535) return LQ_ERR_SHAPE;
  const int Q = a->chunk_size;
  if (Q < 64 || Q % 64 != 0 || Q > 64 * kMaxE) return LQ_ERR_SHAPE;
  if (a->dt_dtype != LQ_DT_F16 && a->dt_dtype != LQ_DT_F32 && a->dt_dtype != LQ_DT_I8) return LQ_ERR_SHAPE;
  const int nchunks = (a->seqlen + Q - 1) / Q;
  if (nchunks > 65535) return LQ_ERR_SHAPE;
  const int hg = (a->nheads + kHG - 1) / kHG;
  const int64_t units = (int64_t)nchunks * a->batch;
  if (units * hg >= (1ll << 31)) return LQ_ERR_SHAPE;
  const int by_xcd = units % 8 == 0;
  dim3 grid((unsigned)(units * hg));
  const size_t lds = (size_t)Q * (kHG + 1) * sizeof(float);
  if (lds > 65536 && hipFuncSetAttribute(reinterpret_cast<const void*>(&chunk_cumsum_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return LQ_ERR_LAUNCH;
  const bool vec_ok = ((uintptr_t)a->dt_out % 16 == 0) && ((uintptr_t)a->dA_cumsum % 16 == 0);
#define LQ_CUMSUM_FIXED(EE)                                                                                             \
  hipLaunchKernelGGL(chunk_cumsum_fixed_kernel<EE>, grid, dim3(kWaves * 64), lds, stream, a->dt, a->dt_dtype,             \
                     a->dt_stride_b, a->dt_stride_l, a->dt_stride_h, a->dt_scale, a->A_log, a->A_log_stride_h,            \
                     a->A_log_scale, a->dt_bias, a->dt_bias_stride_h, a->dt_out, a->dA_cumsum, a->seqlen, a->nheads,      \
                     nchunks, a->dt_softplus, a->dt_min, a->dt_max, hg, by_xcd)
  if (Q == 64)
    LQ_CUMSUM_FIXED(1);
  else if (Q == 128)
    LQ_CUMSUM_FIXED(2);
  else if (Q == 256 && vec_ok)
    LQ_CUMSUM_FIXED(4);
  else if (Q == 512)
    LQ_CUMSUM_FIXED(8);
  else
    hipLaunchKernelGGL(chunk_cumsum_kernel, grid, dim3(kWaves * 64), lds, stream, a->dt, a->dt_dtype, a->dt_stride_b,
                       a->dt_stride_l, a->dt_stride_h, a->dt_scale, a->A_log, a->A_log_stride_h, a->A_log_scale,
                       a->dt_bias, a->dt_bias_stride_h, a->dt_out, a->dA_cumsum, a->seqlen, a->nheads, nchunks, Q,
                       a->dt_softplus, a->dt_min, a->dt_max, hg, by_xcd);
#undef LQ_CUMSUM_FIXED
  return lq_check_launch();
}
