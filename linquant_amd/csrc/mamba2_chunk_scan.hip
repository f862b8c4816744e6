// Mamba-2 SSD stage 5: chunk scan (state read + causal intra-chunk product + D residual) -> fp16.
// Replaces linquant/kernels/mamba2/chunk_scan_v2.py:56-256 (launcher :259-366):
//   acc  = float(C_i8[m,:] . S_i8[p,:]) * sC[g] * ss[h,p] * exp(dA_m)
//   acc += sum_{k<=m} fp16(CB_i8[m,k] * S_cb * exp(dA_m - dA_k) * dt_k) * fp16(x[k,p])    (fp32 accumulate)
//   acc += float(x[m,p]) * (D_scale * float(D_i8[h]))
//
// One workgroup per (64-col P tile, batch*chunk, head), one wavefront per 32 rows of the chunk.
//
// LDS holds two copies of the chunk's x tile, both "token-pair interleaved" (dword (kp, p) = {x[2kp][p],
// x[2kp+1][p]}) so that an fp16 MFMA operand (8 tokens of one channel) is four 16-byte LDS reads covering the
// four channels {4*(lane&15)+j} of the four MFMA calls at once, with no register shuffling:
//   xP : x as stored
//   xS : x[k] * exp(dA_e(k) - dA_k) * S_cb * dt_k, where e(k) is the last token of k's 64-token block.
// For 64-token blocks strictly before a wave's rows the causal weight factors as
//   exp(dA_m - dA_k) = exp(dA_m - dA_e) * exp(dA_e - dA_k),      both exponents <= 0,
// so those blocks need no per-element exponential: the A operand is the CB code itself (exact int8 -> fp16),
// the B operand is xS, consecutive blocks are chained Horner-style with the scalar exp(dA_e(J) - dA_e(J-1))
// on the fp32 accumulator and the row factor exp(dA_m - dA_e(last)) is applied once.  Only the 64-token block
// that contains the wave's rows evaluates exp(dA_m - dA_k) per element (masked to k <= m).
// State path: both INT8 operands are N-contiguous (16-byte global loads, INT8 MFMA).
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int kRow = 68;  // LDS row stride in dwords: 64 channels + 4 pad (272 B, keeps 16-byte alignment)

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

LQ_DEV float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }

// 4 int8 codes (one dword) -> 4 exact fp16 values as two packed dwords: 0x6400 | (b ^ 0x80) is 1024 + (b + 128).
LQ_DEV void i8x4_to_f16x4(uint32_t w, uint32_t& lo, uint32_t& hi) {
  const uint32_t u = w ^ 0x80808080u;
  const uint32_t a = __builtin_amdgcn_perm(0x64646464u, u, 0x05010400u);
  const uint32_t b = __builtin_amdgcn_perm(0x64646464u, u, 0x05030402u);
  const lq_v2h off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
  lo = __builtin_bit_cast(uint32_t, __builtin_bit_cast(lq_v2h, a) + off);
  hi = __builtin_bit_cast(uint32_t, __builtin_bit_cast(lq_v2h, b) + off);
}

LQ_DEV uint32_t pack_h2(float a, float b) {
  const lq_v2h v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(uint32_t, v);
}

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void chunk_scan_kernel(ScanParams p) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int Q = p.Q;
  uint32_t* xP = (uint32_t*)lds_raw;          // [Q/2][kRow]
  uint32_t* xS = xP + (Q / 2) * kRow;         // [Q/2][kRow]
  float* dA2_s = (float*)(xS + (Q / 2) * kRow);  // dA * log2(e)
  float* w_s = dA2_s + Q;                     // S_cb * dt

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  const int p0 = blockIdx.x * 64;
  const int b = blockIdx.y / p.nchunks, c = blockIdx.y % p.nchunks;
  const int h = blockIdx.z;
  const int g = h / (p.nheads / p.G);
  const int limit = min(Q, p.seqlen - c * Q);
  const int64_t cs = (((int64_t)b * p.nheads + h) * p.nchunks + c) * Q;
  const float scb = p.cb_scale[g];

  // ---- stage dA*log2e, S_cb*dt, then both x tiles
  for (int i = tid; i < Q; i += WAVES * 64) {
    dA2_s[i] = p.dA[cs + i] * 1.44269504088896340736f;
    w_s[i] = scb * p.dt[cs + i];
  }
  const _Float16* xg = p.x + (int64_t)b * p.sx_b + (int64_t)c * Q * p.sx_l + (int64_t)h * p.sx_h + p0;
  lq_v8h r0[2], r1[2];
  int kp_of[2], c8_of[2];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int item = tid + it * WAVES * 64;  // Q*4 items in total, 2 per thread
    const int kp = item >> 3, c8 = item & 7;
    kp_of[it] = kp, c8_of[it] = c8;
    lq_v8h z = {0, 0, 0, 0, 0, 0, 0, 0};
    r0[it] = z, r1[it] = z;
    if (2 * kp < limit) r0[it] = *(const lq_v8h*)(xg + (int64_t)(2 * kp) * p.sx_l + c8 * 8);
    if (2 * kp + 1 < limit) r1[it] = *(const lq_v8h*)(xg + (int64_t)(2 * kp + 1) * p.sx_l + c8 * 8);
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int kp = kp_of[it], c8 = c8_of[it];
    const int k = 2 * kp, ke = (k | 63);
    const float ae = dA2_s[ke];
    const float g0 = fexp2(ae - dA2_s[k]) * w_s[k];
    const float g1 = fexp2(ae - dA2_s[k + 1]) * w_s[k + 1];
    lq_v4i plain[2], scaled[2];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const lq_v2h pr = {r0[it][e], r1[it][e]};
      plain[e >> 2][e & 3] = (int)__builtin_bit_cast(uint32_t, pr);
      scaled[e >> 2][e & 3] = (int)pack_h2((float)r0[it][e] * g0, (float)r1[it][e] * g1);
    }
    uint32_t* d0 = xP + kp * kRow + c8 * 8;
    uint32_t* d1 = xS + kp * kRow + c8 * 8;
    *(lq_v4i*)d0 = plain[0];
    *(lq_v4i*)(d0 + 4) = plain[1];
    *(lq_v4i*)d1 = scaled[0];
    *(lq_v4i*)(d1 + 4) = scaled[1];
  }
  __syncthreads();

  const int mbase = wave * 32;
  if (mbase >= limit) return;

  // ---- state path (INT8 MFMA)
  lq_v4f acc[2][4];  // [16-row tile][channel call j]
  {
    lq_v4i ai[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) ai[i][j] = lq_v4i{0, 0, 0, 0};
    const int8_t* Cp = p.C + (int64_t)b * p.sC_b + (int64_t)c * Q * p.sC_l + (int64_t)g * p.sC_g;
    const int8_t* Sp = p.states + ((((int64_t)b * p.nchunks + c) * p.nheads + h) * p.P) * p.N;
    for (int n0 = 0; n0 < p.N; n0 += 64) {
      const int nn = n0 + kg * 16;
      lq_v4i cop[2], sop[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int m = mbase + 16 * i + rl;
        cop[i] = lq_v4i{0, 0, 0, 0};
        if (m < limit) cop[i] = *(const lq_v4i*)(Cp + (int64_t)m * p.sC_l + nn);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) sop[j] = *(const lq_v4i*)(Sp + (int64_t)(p0 + 4 * rl + j) * p.N + nn);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) ai[i][j] = lq_mfma_i8(cop[i], sop[j], ai[i][j]);
    }
    const float gscale = p.C_scale[g];
    float ssv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) ssv[j] = p.ss[(int64_t)h * p.sss_h + (int64_t)(p0 + 4 * rl + j) * p.sss_p];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float rg = fexp2(dA2_s[mbase + 16 * i + 4 * kg + r]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float v = (float)ai[i][j][r] * gscale;
          v = v * ssv[j];
          acc[i][j][r] = v * rg;
        }
      }
  }

  const int8_t* cbp = p.cb + ((((int64_t)b * p.nchunks + c) * p.G + g) * Q) * Q;
  const int nblk = mbase >> 6;  // 64-token blocks strictly before this wave's rows

  // ---- blocks before the wave's rows: CB codes x anchor-scaled x, Horner chain on the accumulator
  if (nblk > 0) {
    lq_v4f off[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) off[i][j] = lq_v4f{0.f, 0.f, 0.f, 0.f};
    lq_v2i cw[2][2], cwn[2][2];  // [slab][row tile]
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        cw[s2][i] = *(const lq_v2i*)(cbp + (int64_t)(mbase + 16 * i + rl) * Q + 32 * s2 + 8 * kg);
    for (int J = 0; J < nblk; ++J) {
      if (J + 1 < nblk) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int i = 0; i < 2; ++i)
            cwn[s2][i] = *(const lq_v2i*)(cbp + (int64_t)(mbase + 16 * i + rl) * Q + 64 * (J + 1) + 32 * s2 + 8 * kg);
      }
      if (J > 0) {
        const float hs = fexp2(dA2_s[64 * J + 63] - dA2_s[64 * J - 1]);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) off[i][j] = off[i][j] * hs;
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const int kp0 = 32 * J + 16 * s2 + 4 * kg;  // token pair index of this lane's first slot
        lq_v4i xop[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const lq_v4i v = *(const lq_v4i*)(xS + (kp0 + d) * kRow + 4 * rl);
#pragma unroll
          for (int j = 0; j < 4; ++j) xop[j][d] = v[j];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          lq_v4i aw;
          uint32_t lo, hi;
          i8x4_to_f16x4((uint32_t)cw[s2][i][0], lo, hi);
          aw[0] = (int)lo, aw[1] = (int)hi;
          i8x4_to_f16x4((uint32_t)cw[s2][i][1], lo, hi);
          aw[2] = (int)lo, aw[3] = (int)hi;
          const lq_v8h aop = __builtin_bit_cast(lq_v8h, aw);
#pragma unroll
          for (int j = 0; j < 4; ++j) off[i][j] = lq_mfma_f16(aop, __builtin_bit_cast(lq_v8h, xop[j]), off[i][j]);
        }
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int i = 0; i < 2; ++i) cw[s2][i] = cwn[s2][i];
    }
    const float ae = dA2_s[64 * nblk - 1];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float rf = fexp2(dA2_s[mbase + 16 * i + 4 * kg + r] - ae);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j][r] = fmaf(off[i][j][r], rf, acc[i][j][r]);
      }
  }

  // ---- the 64-token block holding the wave's rows: per-element weights, masked to k <= m
  float dAm[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) dAm[i] = dA2_s[mbase + 16 * i + rl];
  const int kend = min(mbase + 32, limit);
  for (int k0 = 64 * nblk; k0 < kend; k0 += 32) {
    const int kb = k0 + 8 * kg;
    lq_v4i xop[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const lq_v4i v = *(const lq_v4i*)(xP + (kb / 2 + d) * kRow + 4 * rl);
#pragma unroll
      for (int j = 0; j < 4; ++j) xop[j][d] = v[j];
    }
    const lq_v4f a0 = *(const lq_v4f*)(dA2_s + kb), a1 = *(const lq_v4f*)(dA2_s + kb + 4);
    const lq_v4f w0 = *(const lq_v4f*)(w_s + kb), w1 = *(const lq_v4f*)(w_s + kb + 4);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = mbase + 16 * i + rl;
      const lq_v2i cw = *(const lq_v2i*)(cbp + (int64_t)m * Q + kb);
      float v[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float cf = (float)lq_sbyte((uint32_t)cw[t >> 2], t & 3);
        const float ak = t < 4 ? a0[t & 3] : a1[t & 3];
        const float wk = t < 4 ? w0[t & 3] : w1[t & 3];
        v[t] = cf * (fexp2(dAm[i] - ak) * wk);
        if (kb + t > m) v[t] = 0.0f;
      }
      lq_v4i aw;
#pragma unroll
      for (int d = 0; d < 4; ++d) aw[d] = (int)pack_h2(v[2 * d], v[2 * d + 1]);
      const lq_v8h aop = __builtin_bit_cast(lq_v8h, aw);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = lq_mfma_f16(aop, __builtin_bit_cast(lq_v8h, xop[j]), acc[i][j]);
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
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = mbase + 16 * i + 4 * kg + r;
      if (m >= limit) continue;
      const lq_v4i xv = *(const lq_v4i*)(xP + (m >> 1) * kRow + 4 * rl);
      lq_v4h o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t wv = (uint32_t)xv[j];
        const _Float16 xr = __builtin_bit_cast(_Float16, (uint16_t)((m & 1) ? (wv >> 16) : (wv & 0xffffu)));
        o[j] = (_Float16)(acc[i][j][r] + (float)xr * Dv[j]);
      }
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
  const size_t lds = (size_t)p.Q * kRow * 4 + (size_t)p.Q * 8;  // two [Q/2][kRow] dword tiles + dA2 + w
  dim3 grid(p.P / 64, (unsigned)by, p.nheads);
  // more than 64 KB of dynamic LDS has to be opted into per kernel
#define LQ_SCAN_LAUNCH(W)                                                                                   \
  do {                                                                                                      \
    if (lds > 65536 && hipFuncSetAttribute(reinterpret_cast<const void*>(&chunk_scan_kernel<W>),            \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
      return LQ_ERR_LAUNCH;                                                                                 \
    hipLaunchKernelGGL(chunk_scan_kernel<W>, grid, dim3(W * 64), lds, stream, p);                           \
  } while (0)
  switch (p.Q / 32) {
    case 2: LQ_SCAN_LAUNCH(2); break;
    case 4: LQ_SCAN_LAUNCH(4); break;
    case 8: LQ_SCAN_LAUNCH(8); break;
    case 16: LQ_SCAN_LAUNCH(16); break;
    default: return LQ_ERR_SHAPE;  // chunk sizes 64, 128, 256, 512
  }
#undef LQ_SCAN_LAUNCH
  return lq_check_launch();
}
