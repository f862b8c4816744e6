// Mamba-2 SSD stage 5: chunk scan (state read + causal intra-chunk product + D residual) -> fp16.
// Replaces linquant/kernels/mamba2/chunk_scan_v2.py:56-256 (launcher :259-366):
//   acc  = float(C_i8[m,:] . S_i8[p,:]) * sC[g] * ss[h,p] * exp(dA_m)
//   acc += sum_{k<=m} fp16(CB_i8[m,k] * S_cb * exp(dA_m - dA_k) * dt_k) * fp16(x[k,p])    (fp32 accumulate)
//   acc += float(x[m,p]) * (D_scale * float(D_i8[h]))
//
// One workgroup per (64-col P tile, batch*chunk, head) with one wavefront per 64 rows of the chunk.  The
// chunk's x tile, dA and dt are staged once in LDS and shared by all row blocks.  State path: both INT8
// operands are N-contiguous (16-byte loads, INT8 MFMA).  Causal path: CB codes are weighted in registers
// and fed to the fp16 MFMA; x is token-major, so each lane reads, for its 8 tokens, the 4 adjacent
// channels {4*(lane&15)+j} and MFMA call j covers output columns 4*i+j -- every lane then owns 4 adjacent
// fp16 outputs per row (one 8-byte store).  Tiles strictly above the diagonal are skipped.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int kXStride = 72;  // LDS row stride of the x tile in halves (64 + 8): 144 B keeps 16-byte alignment
                              // and puts rows that are 8 apart on disjoint banks for the 8-byte operand reads

struct ScanParams {
  const int8_t* cb;
  const _Float16* x;
  int64_t sx_b, sx_l, sx_h;
  const float* dt;
  const float* dA;
  const int8_t* C;
  int64_t sC_b, sC_l, sC_g;
  const float* C_scale;
  const int8_t* states;
  const float* ss;
  int64_t sss_h, sss_p;
  const int8_t* D;
  int64_t sD_h;
  int D_has_hdim;
  const float* D_scale;
  const float* cb_scale;
  _Float16* out;
  int batch, seqlen, nheads, P, G, N, Q, nchunks;
};

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void chunk_scan_kernel(ScanParams p) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int Q = p.Q;
  _Float16* xs = (_Float16*)lds_raw;                        // [Q][kXStride]
  float* dA2_s = (float*)(lds_raw + (size_t)Q * kXStride * 2);  // dA * log2(e)
  float* w_s = dA2_s + Q;                                   // S_cb * dt

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  const int p0 = blockIdx.x * 64;
  const int b = blockIdx.y / p.nchunks, c = blockIdx.y % p.nchunks;
  const int h = blockIdx.z;
  const int g = h / (p.nheads / p.G);
  const int limit = min(Q, p.seqlen - c * Q);
  const int64_t cs = (((int64_t)b * p.nheads + h) * p.nchunks + c) * Q;
  const float scb = p.cb_scale[g];

  // ---- stage x tile (zero rows past the sequence end), dA*log2e and S_cb*dt
  const _Float16* xg = p.x + (int64_t)b * p.sx_b + (int64_t)c * Q * p.sx_l + (int64_t)h * p.sx_h + p0;
  for (int i = tid; i < Q * 8; i += blockDim.x) {
    const int row = i >> 3, c8 = i & 7;
    lq_v4i v = lq_v4i{0, 0, 0, 0};
    if (row < limit) v = *(const lq_v4i*)(xg + (int64_t)row * p.sx_l + c8 * 8);
    *(lq_v4i*)(xs + row * kXStride + c8 * 8) = v;
  }
  for (int i = tid; i < Q; i += blockDim.x) {
    dA2_s[i] = p.dA[cs + i] * 1.44269504088896340736f;
    w_s[i] = scb * p.dt[cs + i];
  }
  __syncthreads();

  const int mbase = wave * 64;
  if (mbase >= limit) return;

  // ---- state path (INT8 MFMA)
  lq_v4f acc[4][4];  // [m tile][channel call j]
  {
    lq_v4i ai[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) ai[i][j] = lq_v4i{0, 0, 0, 0};
    const int8_t* Cp = p.C + (int64_t)b * p.sC_b + (int64_t)c * Q * p.sC_l + (int64_t)g * p.sC_g;
    const int8_t* Sp = p.states + ((((int64_t)b * p.nchunks + c) * p.nheads + h) * p.P) * p.N;
    for (int n0 = 0; n0 < p.N; n0 += 64) {
      const int nn = n0 + kg * 16;
      lq_v4i cop[4], sop[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = mbase + 16 * i + rl;
        cop[i] = lq_v4i{0, 0, 0, 0};
        if (m < limit) cop[i] = *(const lq_v4i*)(Cp + (int64_t)m * p.sC_l + nn);
        sop[i] = *(const lq_v4i*)(Sp + (int64_t)(p0 + 4 * rl + i) * p.N + nn);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) ai[i][j] = lq_mfma_i8(cop[i], sop[j], ai[i][j]);
    }
    const float gscale = p.C_scale[g];
    float ssv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) ssv[j] = p.ss[(int64_t)h * p.sss_h + (int64_t)(p0 + 4 * rl + j) * p.sss_p];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = mbase + 16 * i + 4 * kg + r;
        const float rg = __builtin_amdgcn_exp2f(dA2_s[m]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float v = (float)ai[i][j][r] * gscale;
          v = v * ssv[j];
          acc[i][j][r] = v * rg;
        }
      }
  }

  // ---- causal intra-chunk path (fp16 MFMA, fp32 accumulate)
  float dAm[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) dAm[i] = dA2_s[mbase + 16 * i + rl];
  const int8_t* cbp = p.cb + ((((int64_t)b * p.nchunks + c) * p.G + g) * Q) * Q;
  const int kmax = min(mbase + 64, limit);
  for (int k0 = 0; k0 < kmax; k0 += 32) {
    const int kb = k0 + 8 * kg;
    // x operand: element t of call j = x[kb + t][4*rl + j]
    lq_v8h xop[4];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const lq_v4h xv = *(const lq_v4h*)(xs + (kb + t) * kXStride + 4 * rl);
#pragma unroll
      for (int j = 0; j < 4; ++j) xop[j][t] = xv[j];
    }
    float a2k[8], wk[8];
    {
      const lq_v4f a0 = *(const lq_v4f*)(dA2_s + kb), a1 = *(const lq_v4f*)(dA2_s + kb + 4);
      const lq_v4f w0 = *(const lq_v4f*)(w_s + kb), w1 = *(const lq_v4f*)(w_s + kb + 4);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        a2k[t] = a0[t], a2k[4 + t] = a1[t];
        wk[t] = w0[t], wk[4 + t] = w1[t];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int mrow0 = mbase + 16 * i;
      if (k0 > mrow0 + 15) continue;  // tile strictly above the diagonal (wave-uniform)
      const int m = mrow0 + rl;
      const lq_v2i cw = *(const lq_v2i*)(cbp + (int64_t)m * Q + kb);
      lq_v8h aop;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float cf = (float)lq_sbyte((uint32_t)cw[t >> 2], t & 3);
        float v = cf * (__builtin_amdgcn_exp2f(dAm[i] - a2k[t]) * wk[t]);
        if (kb + t > m) v = 0.0f;
        aop[t] = (_Float16)v;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = lq_mfma_f16(aop, xop[j], acc[i][j]);
    }
  }

  // ---- D residual + store
  float Dv[4] = {0.f, 0.f, 0.f, 0.f};
  if (p.D) {
    const float dsc = *p.D_scale;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      Dv[j] = dsc * (float)p.D[(int64_t)h * p.sD_h + (p.D_has_hdim ? p0 + 4 * rl + j : 0)];
  }
  _Float16* op = p.out + (((int64_t)b * p.seqlen + (int64_t)c * Q) * p.nheads + h) * p.P + p0 + 4 * rl;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = mbase + 16 * i + 4 * kg + r;
      if (m >= limit) continue;
      const lq_v4h xv = *(const lq_v4h*)(xs + m * kXStride + 4 * rl);
      lq_v4h o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (_Float16)(acc[i][j][r] + (float)xv[j] * Dv[j]);
      *(lq_v4h*)(op + (int64_t)m * p.nheads * p.P) = o;
    }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

}  // namespace

extern "C" int lq_chunk_scan(const lq_chunk_scan_args* a, hipStream_t stream) {
  if (!a || !a->cb || !a->x || !a->dt || !a->dA_cumsum || !a->C || !a->C_scale || !a->states || !a->states_scale ||
      !a->cb_scale || !a->out)
    return LQ_ERR_NULL;
  if (a->D && !a->D_scale) return LQ_ERR_NULL;
  ScanParams p = {};
  p.cb = a->cb, p.x = (const _Float16*)a->x;
  p.sx_b = a->x_stride_b, p.sx_l = a->x_stride_l, p.sx_h = a->x_stride_h;
  p.dt = a->dt, p.dA = a->dA_cumsum, p.C = a->C;
  p.sC_b = a->C_stride_b, p.sC_l = a->C_stride_l, p.sC_g = a->C_stride_g;
  p.C_scale = a->C_scale, p.states = a->states, p.ss = a->states_scale;
  p.sss_h = a->ss_stride_h, p.sss_p = a->ss_stride_p;
  p.D = a->D, p.sD_h = a->D_stride_h, p.D_has_hdim = a->D_has_hdim, p.D_scale = a->D_scale;
  p.cb_scale = a->cb_scale, p.out = (_Float16*)a->out;
  p.batch = a->batch, p.seqlen = a->seqlen, p.nheads = a->nheads, p.P = a->headdim, p.G = a->ngroups;
  p.N = a->dstate, p.Q = a->chunk_size;
  if (p.batch <= 0 || p.seqlen <= 0 || p.nheads <= 0 || p.G <= 0 || p.nheads % p.G != 0) return LQ_ERR_SHAPE;
  if (p.Q < 64 || p.Q % 64 != 0 || p.Q > 512 || p.P % 64 != 0 || p.N % 64 != 0) return LQ_ERR_SHAPE;
  if (p.sx_b % 8 || p.sx_l % 8 || p.sx_h % 8 || !al(p.x, 16)) return LQ_ERR_SHAPE;
  if (p.sC_b % 16 || p.sC_l % 16 || p.sC_g % 16 || !al(p.C, 16) || !al(p.states, 16) || !al(p.cb, 8) || !al(p.out, 8))
    return LQ_ERR_SHAPE;
  p.nchunks = (p.seqlen + p.Q - 1) / p.Q;
  const int64_t by = (int64_t)p.batch * p.nchunks;
  if (by > 65535 || p.nheads > 65535) return LQ_ERR_SHAPE;
  const size_t lds = (size_t)p.Q * kXStride * 2 + (size_t)p.Q * 8;
  dim3 grid(p.P / 64, (unsigned)by, p.nheads);
  switch (p.Q / 64) {
    case 1: hipLaunchKernelGGL(chunk_scan_kernel<1>, grid, dim3(64), lds, stream, p); break;
    case 2: hipLaunchKernelGGL(chunk_scan_kernel<2>, grid, dim3(128), lds, stream, p); break;
    case 4: hipLaunchKernelGGL(chunk_scan_kernel<4>, grid, dim3(256), lds, stream, p); break;
    case 8: hipLaunchKernelGGL(chunk_scan_kernel<8>, grid, dim3(512), lds, stream, p); break;
    default: return LQ_ERR_SHAPE;
  }
  return lq_check_launch();
}
