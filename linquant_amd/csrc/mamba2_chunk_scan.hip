// Mamba-2 SSD stage 5: chunk scan (state read + causal intra-chunk product + D residual) -> fp16.
// Replaces linquant/kernels/mamba2/chunk_scan_v2.py:56-256 (launcher :259-366):
//   acc  = float(C_i8[m,:] . S_i8[p,:]) * sC[g] * ss[h,p] * exp(dA_m)
//   acc += sum_{k<=m} fp16(CB_i8[m,k] * S_cb * exp(dA_m - dA_k) * dt_k) * fp16(x[k,p])    (fp32 accumulate)
//   acc += float(x[m,p]) * (D_scale * float(D_i8[h]))
//
// One workgroup per (64-col P tile, batch*chunk, head), one wavefront per two 16-row tiles of the chunk: tile w
// and tile 2*WAVES-1-w, an early and a late one, so every wave carries the same causal work.
//
// LDS holds two copies of the chunk's x tile, both "token-pair interleaved" (dword (kp, p) = {x[2kp][p],
// x[2kp+1][p]}) so that an fp16 MFMA operand (8 tokens of one channel) is four 16-byte LDS reads covering the
// four channels {4*(lane&15)+j} of the four MFMA calls at once, with no register shuffling:
//   xP : x as stored
//   xS : x[k] * exp(dA_e(k) - dA_k) * S_cb * dt_k, where e(k) is the last token of k's 32-token slab.
// For 32-token slabs strictly before a wave's rows the causal weight factors as
//   exp(dA_m - dA_k) = exp(dA_m - dA_E) * exp(dA_E - dA_e) * exp(dA_e - dA_k),   all exponents <= 0,
// (E = last token before the tile's own 32-token slab), so those slabs need no per-element exponential: the B operand is
// xS, the A operand is the CB code times the per-slab scalar exp(dA_E - dA_e), produced by the same packed
// fp16 instruction that finishes the int8 -> fp16 conversion, and the row factor exp(dA_m - dA_E) is applied
// once to the slab accumulator.  Only the tile's own 32-token slab evaluates exp(dA_m - dA_k) per element
// (masked to k <= m).
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
// With (s2, o2) = (s, -1152 s) the result is s * code (one packed fma: exact for s = 1, fp16-rounded otherwise).
LQ_DEV void i8x4_to_f16x4(uint32_t w, lq_v2h s2, lq_v2h o2, uint32_t& lo, uint32_t& hi) {
  const uint32_t u = w ^ 0x80808080u;
  const uint32_t a = __builtin_amdgcn_perm(0x64646464u, u, 0x05010400u);
  const uint32_t b = __builtin_amdgcn_perm(0x64646464u, u, 0x05030402u);
  lo = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(lq_v2h, a), s2, o2));
  hi = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(lq_v2h, b), s2, o2));
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
  // heads vary fastest across consecutive workgroups: the C / CB tiles of a (batch, chunk) are shared by all
  // heads of a group and stay in L2 while they are swept
  const int h = blockIdx.x % p.nheads;
  const int p0 = (blockIdx.x / p.nheads) * 64;
  const int b = blockIdx.y / p.nchunks, c = blockIdx.y % p.nchunks;
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
  // Small per-head operands of the epilogues are fetched now: issued where they are used, each would expose a full
  // memory round trip behind the barriers.
  float ssv[4], Dv[4] = {0.f, 0.f, 0.f, 0.f};
  {
    const float gscale = p.C_scale[g];
#pragma unroll
    for (int j = 0; j < 4; ++j) ssv[j] = gscale * p.ss[(int64_t)h * p.sss_h + (int64_t)(p0 + 4 * rl + j) * p.sss_p];
    if (p.D) {
      const float dsc = *p.D_scale;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        Dv[j] = dsc * (float)p.D[(int64_t)h * p.sD_h + (p.D_has_hdim ? p0 + 4 * rl + j : 0)];
    }
  }
  // Row tiles of this wave: 16w.. and 16(2*WAVES-1-w)..: an early and a late tile, so that every wave has the same
  // number of causal slabs to process.
  int rb[2];
  rb[0] = 16 * wave;
  rb[1] = 16 * (2 * WAVES - 1 - wave);
  // ---- state path (INT8 MFMA), issued before the staging barrier so its global loads overlap the x tile's
  lq_v4i ai[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) ai[i][j] = lq_v4i{0, 0, 0, 0};
  if (rb[0] < limit) {
    const int8_t* Cp = p.C + (int64_t)b * p.sC_b + (int64_t)c * Q * p.sC_l + (int64_t)g * p.sC_g;
    const int8_t* Sp = p.states + ((((int64_t)b * p.nchunks + c) * p.nheads + h) * p.P) * p.N;
    for (int n0 = 0; n0 < p.N; n0 += 64) {
      const int nn = n0 + kg * 16;
      lq_v4i cop[2], sop[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int m = min(rb[i] + rl, limit - 1);
        cop[i] = *(const lq_v4i*)(Cp + (int64_t)m * p.sC_l + nn);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) sop[j] = *(const lq_v4i*)(Sp + (int64_t)(p0 + 4 * rl + j) * p.N + nn);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) ai[i][j] = lq_mfma_i8(cop[i], sop[j], ai[i][j]);
    }
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int kp = kp_of[it], c8 = c8_of[it];
    const int k = 2 * kp, ke = (k | 31);
    const float ae = dA2_s[ke];
    const lq_v2h g2 = {(_Float16)(fexp2(ae - dA2_s[k]) * w_s[k]), (_Float16)(fexp2(ae - dA2_s[k + 1]) * w_s[k + 1])};
    lq_v4i plain[2], scaled[2];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const lq_v2h pr = {r0[it][e], r1[it][e]};
      plain[e >> 2][e & 3] = (int)__builtin_bit_cast(uint32_t, pr);
      scaled[e >> 2][e & 3] = (int)__builtin_bit_cast(uint32_t, pr * g2);
    }
    uint32_t* d0 = xP + kp * kRow + c8 * 8;
    uint32_t* d1 = xS + kp * kRow + c8 * 8;
    *(lq_v4i*)d0 = plain[0];
    *(lq_v4i*)(d0 + 4) = plain[1];
    *(lq_v4i*)d1 = scaled[0];
    *(lq_v4i*)(d1 + 4) = scaled[1];
  }
  __syncthreads();

  if (rb[0] >= limit) return;  // the early tile is past the sequence end, so is the late one

  // ---- state read dequantized and gated: float(acc) * (sC * ss[p]) * exp(dA_m)
  lq_v4f acc[2][4];  // [row tile][channel call j]
  {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float rg = fexp2(dA2_s[rb[i] + 4 * kg + r]);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j][r] = (float)ai[i][j][r] * (ssv[j] * rg);
      }
  }

  const int8_t* cbp = p.cb + ((((int64_t)b * p.nchunks + c) * p.G + g) * Q) * Q;

#pragma unroll
  for (int i = 0; i < 2; ++i) {
    if (rb[i] >= limit) continue;
    const int nslab = rb[i] >> 5;      // 32-token slabs strictly before the slab that holds this tile
    const int sbase = 32 * nslab;      // first token of the tile's own slab
    const int8_t* crow = cbp + (int64_t)(rb[i] + rl) * Q;
    // ---- slabs before the tile's own slab: (scaled CB codes) x (anchor-scaled x), row factor applied once
    if (nslab > 0) {
      lq_v4f off[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) off[j] = lq_v4f{0.f, 0.f, 0.f, 0.f};
      const float aE = dA2_s[sbase - 1];
      lq_v2i cw = *(const lq_v2i*)(crow + 8 * kg), cwn = cw;
      for (int J = 0; J < nslab; ++J) {
        if (J + 1 < nslab) cwn = *(const lq_v2i*)(crow + 32 * (J + 1) + 8 * kg);
        const _Float16 sh = (_Float16)fexp2(aE - dA2_s[32 * J + 31]);
        const lq_v2h s2 = {sh, sh};
        const lq_v2h o2 = s2 * lq_v2h{(_Float16)-1152.0f, (_Float16)-1152.0f};
        const int kp0 = 16 * J + 4 * kg;  // token pair index of this lane's first slot
        lq_v4i xop[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const lq_v4i v = *(const lq_v4i*)(xS + (kp0 + d) * kRow + 4 * rl);
#pragma unroll
          for (int j = 0; j < 4; ++j) xop[j][d] = v[j];
        }
        lq_v4i aw;
        uint32_t lo, hi;
        i8x4_to_f16x4((uint32_t)cw[0], s2, o2, lo, hi);
        aw[0] = (int)lo, aw[1] = (int)hi;
        i8x4_to_f16x4((uint32_t)cw[1], s2, o2, lo, hi);
        aw[2] = (int)lo, aw[3] = (int)hi;
        const lq_v8h aop = __builtin_bit_cast(lq_v8h, aw);
#pragma unroll
        for (int j = 0; j < 4; ++j) off[j] = lq_mfma_f16(aop, __builtin_bit_cast(lq_v8h, xop[j]), off[j]);
        cw = cwn;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float rf = fexp2(dA2_s[rb[i] + 4 * kg + r] - aE);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j][r] = fmaf(off[j][r], rf, acc[i][j][r]);
      }
    }

    // ---- the tile's own 32-token slab: per-element weights exp2(dA2_m - (dA2_k - log2(S_cb dt_k))), k <= m
    {
      const int m = rb[i] + rl;
      const float dAm = dA2_s[m];
      const int kb = sbase + 8 * kg;
      lq_v4i xop[4];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const lq_v4i v = *(const lq_v4i*)(xP + (kb / 2 + d) * kRow + 4 * rl);
#pragma unroll
        for (int j = 0; j < 4; ++j) xop[j][d] = v[j];
      }
      const lq_v4f a0 = *(const lq_v4f*)(dA2_s + kb), a1 = *(const lq_v4f*)(dA2_s + kb + 4);
      const lq_v4f w0 = *(const lq_v4f*)(w_s + kb), w1 = *(const lq_v4f*)(w_s + kb + 4);
      const lq_v2i cw = *(const lq_v2i*)(crow + kb);
      float v[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float akw = (t < 4 ? a0[t & 3] : a1[t & 3]) - __builtin_amdgcn_logf(t < 4 ? w0[t & 3] : w1[t & 3]);
        const float cf = (float)lq_sbyte((uint32_t)cw[t >> 2], t & 3);
        v[t] = cf * fexp2(dAm - akw);
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
  _Float16* op = p.out + (((int64_t)b * p.seqlen + (int64_t)c * Q) * p.nheads + h) * p.P + p0 + 4 * rl;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = rb[i] + 4 * kg + r;
      if (m >= limit) continue;
      const lq_v4i xv = *(const lq_v4i*)(xP + (m >> 1) * kRow + 4 * rl);
      lq_v4h o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t wv = (uint32_t)xv[j];  // rows alternate low / high half: m & 1 == r & 1
        const _Float16 xr = __builtin_bit_cast(_Float16, (uint16_t)((r & 1) ? (wv >> 16) : (wv & 0xffffu)));
        o[j] = (_Float16)fmaf((float)xr, Dv[j], acc[i][j][r]);
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
  dim3 grid((p.P / 64) * p.nheads, (unsigned)by, 1);
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
