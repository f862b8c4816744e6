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
// x[2kp+1][p]}), four token pairs of a channel adjacent, so that an fp16 MFMA operand (8 tokens of one channel) is one
// 16-byte LDS read:
//   xP : x as stored
//   xS : x[k] * exp(dA_e(k) - dA_k) * S_cb * dt_k * 2^-kf, where e(k) is the last token of k's 32-token slab and
//        2^kf is the power-of-two part of S_cb (returned by the row factor).
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

// LDS layout of an x tile: dword (kp, p) = {x[2kp][p], x[2kp+1][p]} lives at [kp >> 2][slot(p)][kp & 3] with
// slot(p) = (p & 3) * 16 + (p >> 2): the four token pairs of one MFMA contraction group are adjacent, so the operand of
// channel 4 * (lane & 15) + j is ONE 16-byte read at slot j * 16 + (lane & 15) (16 lanes = 256 contiguous bytes) and
// lands in four consecutive registers without any move.
constexpr int kQuad = 256;  // dwords per row of four token pairs: 64 channels * 4, unpadded: measured with the LDS
                            // counters, the four 16-lane groups of an operand read (rows kQuad apart) take the
                            // minimum two passes only when kQuad is a multiple of 64 dwords (260 took four)

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
  int64_t sst_b;  // elements between batch rows of states
  const float* ss;
  int64_t sss_h, sss_p;
  const int8_t* D;
  int64_t sD_h;
  int D_has_hdim;
  const float* D_scale;
  const float* cb_scale;
  _Float16* out;
  int batch, seqlen, nheads, P, G, N, Q, nchunks;
  uint32_t hpg_magic, pt_magic;  // floor(2^32 / d) + 1 for d = heads per group, P tiles (0 when d == 1): x / d == umulhi(x, magic) for x, d < 2^16
};

LQ_DEV float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }

// 4 int8 codes (one dword) -> fp16(code * s) as two packed dwords: 0x6400 | (b ^ 0x80) is 1024 + (b + 128), from which
// 1152 is subtracted exactly (the code itself, exact in fp16) before the one rounded multiply by s.  Folding the bias
// into a fused multiply-add as (1152 + code) * s - fp16(1152 s) would shift every weight of the slab by the rounding
// error of fp16(1152 s), up to half a code step: a bias, not noise.
LQ_DEV void i8x4_to_f16x4(uint32_t w, lq_v2h s2, uint32_t& lo, uint32_t& hi) {
  const uint32_t u = w ^ 0x80808080u;
  const uint32_t a = __builtin_amdgcn_perm(0x64646464u, u, 0x05010400u);
  const uint32_t b = __builtin_amdgcn_perm(0x64646464u, u, 0x05030402u);
  const lq_v2h bias = {(_Float16)1152.0f, (_Float16)1152.0f};
  lo = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(lq_v2h, a) - bias) * s2);
  hi = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(lq_v2h, b) - bias) * s2);
}

LQ_DEV uint32_t pack_h2(float a, float b) {
  const lq_v2h v = {(_Float16)a, (_Float16)b};
  return __builtin_bit_cast(uint32_t, v);
}

LQ_DEV lq_v4f mfma_f16_k16(lq_v4h a, lq_v4h b, lq_v4f c) { return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0); }

// base + a 32-bit unsigned byte offset: wave-uniform base, per-lane offset (no 64-bit per-lane arithmetic)
template <typename T>
LQ_DEV const T* at(const void* base, uint32_t byte_off) {
  return (const T*)((const char*)base + byte_off);
}

// WAVES = Q / 32 wavefronts; N64 = N / 64 contraction steps of the state path
template <int WAVES, int N64>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void chunk_scan_kernel(ScanParams p) {
  constexpr int N = 64 * N64;
  constexpr int kSRow = N + 32;  // bytes per state row in LDS: the pitch at which an operand read (16 rows x 4 column
                                 // groups) takes the minimum two passes (measured; N + 16 took four)
  constexpr int kSPieces = (4 * N + WAVES * 64 - 1) / (WAVES * 64);  // 16-byte pieces of the 64 x N state tile per thread
  extern __shared__ __align__(16) unsigned char lds_raw[];
  // Every kernel argument is wanted in scalar registers here, so that all of them are requested in one batch and waited
  // for once: left alone the compiler fetches them in three groups as their first uses come up, each group a full
  // round trip of the scalar cache before the next vector load can be issued.
  asm volatile("" ::"s"(p.cb), "s"(p.x), "s"(p.sx_b), "s"(p.sx_l), "s"(p.sx_h), "s"(p.dt), "s"(p.dA), "s"(p.C), "s"(p.sC_b),
               "s"(p.sC_l), "s"(p.sC_g), "s"(p.C_scale), "s"(p.states), "s"(p.ss), "s"(p.sss_h), "s"(p.sss_p));
  asm volatile("" ::"s"(p.sst_b), "s"(p.D), "s"(p.sD_h), "s"(p.D_has_hdim), "s"(p.D_scale), "s"(p.cb_scale), "s"(p.out), "s"(p.seqlen),
               "s"(p.nheads), "s"(p.P), "s"(p.G), "s"(p.Q), "s"(p.nchunks), "s"(p.hpg_magic), "s"(p.pt_magic));
  const int Q = p.Q;
  uint32_t* xP = (uint32_t*)lds_raw;          // [Q/8][kQuad]
  uint32_t* xS = xP + (Q / 8) * kQuad;        // [Q/8][kQuad]
  float* dA2_s = (float*)(xS + (Q / 8) * kQuad);  // dA * log2(e)
  float* akw_s = dA2_s + Q;                   // dA * log2(e) - log2(S_cb * dt): exp2(dA2_m - akw_k) is the causal weight of (m, k)
  float* ssl_s = akw_s + Q;                   // [64] C scale * state scale of the tile's channels
  float* Dl_s = ssl_s + 64;                   // [64] dequantized D of the tile's channels
  int8_t* S_s = (int8_t*)(Dl_s + 64);           // [64][kSRow] state tile of this (chunk, head), row p at (p & 3) * 16 + (p >> 2)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // known to be wave-uniform: everything derived from it is scalar
  const int rl = lane & 15, kg = lane >> 4;
  // heads vary fastest across consecutive workgroups: the C / CB tiles of a (batch, chunk) are shared by all
  // heads of a group and stay in L2 while they are swept
  // (grid = heads x chunks x (batch * P tiles): no integer division on the way to the first load; the run-time
  // divisions of a flat grid cost four reciprocal sequences between two waits for kernel arguments)
  const int h = blockIdx.x, c = blockIdx.y;
  const int b = p.pt_magic ? (int)__umulhi(blockIdx.z, p.pt_magic) : (int)blockIdx.z;
  const int p0 = ((int)blockIdx.z - b * (p.P >> 6)) * 64;
  const int g = p.hpg_magic ? (int)__umulhi((uint32_t)h, p.hpg_magic) : h;
  const int limit = min(Q, p.seqlen - c * Q);
  const int64_t cs = (((int64_t)b * p.nheads + h) * p.nchunks + c) * Q;
  const float scb = p.cb_scale[g];
  // power-of-two part of S_cb, as an exponent: kept out of the fp16 operand xS (whose values would drift into the
  // fp16 subnormal range with a small S_cb) and returned in fp32 by the row factor of the off-diagonal slabs
  const float kf = (float)(lq_clampi((__float_as_int(scb) >> 23) & 0xff, 2, 252) - 127);

  // Row tiles of this wave: 16w.. and 16(2*WAVES-1-w)..: an early and a late tile, so that every wave has the same
  // number of causal slabs to process.
  int rb[2];
  rb[0] = 16 * wave;
  rb[1] = 16 * (2 * WAVES - 1 - wave);

  // ---- every global load of the prologue is issued here, oldest first in the order it is needed: the state tile
  // (one 16-byte piece per thread, shared through LDS by all waves), this wave's C rows, dA / dt, then the x tile.
  // Addresses are a wave-uniform 64-bit base plus a per-lane unsigned 32-bit byte offset (the launcher checks that every
  // tile fits 32 bits): per-lane 64-bit multiplies and adds ran at a quarter of the rate and made up a tenth of the kernel.
  const int8_t* Sp = p.states + (int64_t)b * p.sst_b + ((((int64_t)c * p.nheads + h) * p.P + p0) * (int64_t)N);
  lq_v4i spiece[kSPieces];
#pragma unroll
  for (int k = 0; k < kSPieces; ++k) {
    const int t = tid + k * WAVES * 64;
    spiece[k] = __builtin_nontemporal_load(at<lq_v4i>(Sp, (uint32_t)min(t, 4 * N - 1) * 16u));  // unconditional: a surplus thread re-reads the last piece
  }
  lq_v4i cop[2][N64];
  {
    const int8_t* Cp = p.C + (int64_t)b * p.sC_b + (int64_t)c * Q * p.sC_l + (int64_t)g * p.sC_g;
    const uint32_t sCl = (uint32_t)p.sC_l;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t coff = __umul24((uint32_t)min(rb[i] + rl, limit - 1), sCl) + (uint32_t)kg * 16u;
#pragma unroll
      for (int n = 0; n < N64; ++n) cop[i][n] = *at<lq_v4i>(Cp, coff + 64u * n);
    }
  }
  // Q <= WAVES * 64: one element per thread; requested without a branch (a conditional request is waited for where
  // the branches join, which here is before the x tile has even been requested)
  const uint32_t qoff = (uint32_t)min(tid, Q - 1) * 4u;
  const float dA_r = *at<float>(p.dA + cs, qoff);
  const float dt_r = *at<float>(p.dt + cs, qoff);
  // per-channel scale and D of channel p0 + (tid & 63): they go through LDS with the other small operands (requested
  // before the bulk of the prologue so that waiting for them does not wait for the x tile: memory operations retire in
  // issue order)
  const float ss_r = *at<float>(p.ss + (int64_t)h * p.sss_h + (int64_t)p0 * p.sss_p, __umul24((uint32_t)lane, (uint32_t)p.sss_p) * 4u);
  // without D the request goes to a valid dummy address and dsc = 0 discards it: no branch around a request
  const int8_t* Dp = p.D ? p.D + (int64_t)h * p.sD_h + (p.D_has_hdim ? p0 : 0) : p.states;
  const int D_r = (int)*at<int8_t>(Dp, (p.D && p.D_has_hdim) ? (uint32_t)lane : 0u);
  const float gscale = p.C_scale[g];
  const float dsc = p.D ? *p.D_scale : 0.0f;
  const _Float16* xg = p.x + (int64_t)b * p.sx_b + (int64_t)c * Q * p.sx_l + (int64_t)h * p.sx_h + p0;
  const uint32_t sxl2 = (uint32_t)p.sx_l * 2u;  // row pitch of x in bytes
  lq_v8h r0[2], r1[2];
  int kp_of[2], c8_of[2];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int item = tid + it * WAVES * 64;  // Q*4 items in total, 2 per thread
    const int kp = item >> 3, c8 = item & 7;
    kp_of[it] = kp, c8_of[it] = c8;
    // rows past the sequence end re-read its last row and are zeroed when staged (no branch around a request)
    // (x and the state tile are streamed: a non-temporal request keeps them from displacing the C / CB tiles that the
    // other heads of the chunk still need; measured 234 -> 217 us)
    r0[it] = __builtin_nontemporal_load(at<lq_v8h>(xg, __umul24((uint32_t)min(2 * kp, limit - 1), sxl2) + (uint32_t)c8 * 16u));
    r1[it] = __builtin_nontemporal_load(at<lq_v8h>(xg, __umul24((uint32_t)min(2 * kp + 1, limit - 1), sxl2) + (uint32_t)c8 * 16u));
  }
  // CB codes of this wave's off-diagonal slabs.  The early tile has ne = rb[0] / 32 of them, the late one the rest of
  // NS = WAVES - 1 (the same total for every wave), so they are walked as one flat list of NS steps whose loads run four
  // steps ahead through a ring of four registers: every request is unconditional and its position in the instruction
  // stream is fixed, which keeps the compiler's wait counts exact (a one-ahead prefetch inside `if (J + 1 < nslab)`
  // was waited for in full at every step).  A slab's address is a scalar (tile row base, slab column) plus the lane's
  // fixed (row, 8-column group) offset.
  constexpr int NS = WAVES - 1;
  const int8_t* cbp = p.cb + ((((int64_t)b * p.nchunks + c) * p.G + g) * Q) * Q;
  const int ne = rb[0] >> 5;
  const uint32_t cb_lane = (uint32_t)(rl * Q + 8 * kg);
  auto cb_slab = [&](int s) {
    const int soff = s < ne ? rb[0] * Q + 32 * s : rb[1] * Q + 32 * (s - ne);  // scalar
    return *at<lq_v2i>(cbp + soff, cb_lane);
  };
  lq_v2i cwr[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) cwr[s] = cb_slab(s < NS ? s : NS - 1);
  if (tid < Q) {
    const float a2 = dA_r * 1.44269504088896340736f;
    dA2_s[tid] = a2;
    akw_s[tid] = a2 - __builtin_amdgcn_logf(scb * dt_r);  // dt = 0 past the sequence end: +inf, weight 0
  }
  if (tid < 64) {
    ssl_s[tid] = gscale * ss_r;
    Dl_s[tid] = dsc * (float)D_r;
  }
#pragma unroll
  for (int k = 0; k < kSPieces; ++k) {
    const int t = tid + k * WAVES * 64;
    const int pr = t / (N / 16), pc = t % (N / 16);
    if (t < 4 * N) *(lq_v4i*)(S_s + ((pr & 3) * 16 + (pr >> 2)) * kSRow + pc * 16) = spiece[k];
  }
  __syncthreads();
  // CB codes of the two 16 x 16 diagonal blocks and of the 16 tokens in front of the tile that sits in the second half
  // of its 32-token slab (exactly one of the wave's two tiles does): one dword (4 codes) per lane each, row rb + rl,
  // columns 4 kg .. 4 kg + 3 of the block.  Needed after the state path and the off-diagonal slabs.
  const int ih = (wave & 1) ? 0 : 1;  // scalar: which tile is the second-half one
  const uint32_t cd_lane = (uint32_t)(rl * Q + 4 * kg);
  int cwd[2];
  cwd[0] = *at<int>(cbp + rb[0] * Q + rb[0], cd_lane);
  cwd[1] = *at<int>(cbp + rb[1] * Q + rb[1], cd_lane);
  const int cwp = *at<int>(cbp + rb[ih] * Q + rb[ih] - 16, cd_lane);
  // ---- state path (INT8 MFMA): C rows from registers, state rows from LDS
  lq_v4i ai[2][4];
#pragma unroll
  for (int n = 0; n < N64; ++n) {
    lq_v4i sop[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sop[j] = *(const lq_v4i*)(S_s + (j * 16 + rl) * kSRow + 64 * n + 16 * kg);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) ai[i][j] = lq_mfma_i8(cop[i][n], sop[j], n == 0 ? lq_v4i{0, 0, 0, 0} : ai[i][j]);
  }
  if (limit < Q) {  // ragged last chunk (wave-uniform): rows past the sequence end are staged as zeros
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const lq_v8h z = {0, 0, 0, 0, 0, 0, 0, 0};
      if (2 * kp_of[it] >= limit) r0[it] = z;
      if (2 * kp_of[it] + 1 >= limit) r1[it] = z;
    }
  }
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int kp = kp_of[it], c8 = c8_of[it];
    const int k = 2 * kp, ke = (k | 31);
    const float ae = dA2_s[ke] - kf;
    const lq_v2h g2 = {(_Float16)fexp2(ae - akw_s[k]), (_Float16)fexp2(ae - akw_s[k + 1])};
    const int base = (kp >> 2) * kQuad + (2 * c8) * 4 + (kp & 3);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const lq_v2h pr = {r0[it][e], r1[it][e]};
      const int off = base + ((e & 3) * 16 + (e >> 2)) * 4;  // x_slot(8 c8 + e) * 4
      xP[off] = __builtin_bit_cast(uint32_t, pr);
      xS[off] = __builtin_bit_cast(uint32_t, pr * g2);
    }
  }
  __syncthreads();

  if (rb[0] >= limit) return;  // the early tile is past the sequence end, so is the late one

  // ---- state read dequantized and gated: float(acc) * (sC * ss[p]) * exp(dA_m)
  lq_v4f acc[2][4];  // [row tile][channel call j]
  {
    const lq_v4f ssv = *(const lq_v4f*)(ssl_s + 4 * rl);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const lq_v4f a4 = *(const lq_v4f*)(dA2_s + rb[i] + 4 * kg);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float rg = fexp2(a4[r]);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j][r] = (float)ai[i][j][r] * (ssv[j] * rg);
      }
    }
  }

  // ---- slabs before each tile's own slab: (scaled CB codes) x (anchor-scaled x), row factor applied once per tile.
  // A tile past the sequence end is processed like any other (its rows are never stored).
  {
    // anchor of a tile = last token before its own slab
    const float aE0 = dA2_s[max(rb[0] & ~31, 1) - 1], aE1 = dA2_s[(rb[1] & ~31) - 1];
    lq_v4f off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) off[j] = lq_v4f{0.f, 0.f, 0.f, 0.f};
    auto flush = [&](int i, float aE) {
      const lq_v4f a4 = *(const lq_v4f*)(dA2_s + rb[i] + 4 * kg);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float rf = fexp2(a4[r] - aE);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j][r] = fmaf(off[j][r], rf, acc[i][j][r]), off[j][r] = 0.0f;
      }
    };
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if (s > 0 && s <= (WAVES - 1) / 2 && s == ne) flush(0, aE0 - kf);  // the early tile's slabs are done (wave-uniform)
      const bool late = s >= ne;
      const int J = late ? s - ne : s;
      const float aE = late ? aE1 : aE0;
      const lq_v2i cw = cwr[s & 3];
      if (s + 4 < NS) cwr[s & 3] = cb_slab(s + 4);
      const _Float16 sh = (_Float16)fexp2(aE - dA2_s[32 * J + 31]);
      // a slab whose factor underflows fp16 (more than 25 octaves of decay between it and the tile) would contribute
      // fp16(code * 0) = 0 to every product: it is left out (wave-uniform; strongly decaying heads skip most slabs)
      if (__builtin_amdgcn_readfirstlane((int)__builtin_bit_cast(uint16_t, sh)) != 0) {
        const lq_v2h s2 = {sh, sh};
        lq_v4i xop[4];  // token pairs 16 J + 4 kg .. + 3 of channel 4 rl + j
#pragma unroll
        for (int j = 0; j < 4; ++j) xop[j] = *(const lq_v4i*)(xS + (4 * J + kg) * kQuad + (j * 16 + rl) * 4);
        lq_v4i aw;
        uint32_t lo, hi;
        i8x4_to_f16x4((uint32_t)cw[0], s2, lo, hi);
        aw[0] = (int)lo, aw[1] = (int)hi;
        i8x4_to_f16x4((uint32_t)cw[1], s2, lo, hi);
        aw[2] = (int)lo, aw[3] = (int)hi;
        const lq_v8h aop = __builtin_bit_cast(lq_v8h, aw);
#pragma unroll
        for (int j = 0; j < 4; ++j) off[j] = lq_mfma_f16(aop, __builtin_bit_cast(lq_v8h, xop[j]), off[j]);
      }
    }
    if (NS > 0) flush(1, aE1 - kf);
  }

  // ---- each tile's own slab, in 16-token blocks on the K = 16 MFMA (4 tokens per lane): the diagonal block
  // [rb, rb + 16) with weights exp2(dA2_m - akw_k) masked to k <= m, and, for the tile in the second half of its slab,
  // the 16 tokens in front of it, all of them before every row of the tile (no mask)
  auto block = [&](int i, int kbase, int codes, bool masked) {
    const float dAm = dA2_s[rb[i] + rl];
    const lq_v4f ak = *(const lq_v4f*)(akw_s + kbase + 4 * kg);
    float v[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      v[t] = (float)lq_sbyte((uint32_t)codes, t) * fexp2(dAm - ak[t]);
      if (masked && 4 * kg + t > rl) v[t] = 0.0f;
    }
    lq_v2i aw;
    aw[0] = (int)pack_h2(v[0], v[1]), aw[1] = (int)pack_h2(v[2], v[3]);
    const lq_v4h aop = __builtin_bit_cast(lq_v4h, aw);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // token pairs kbase / 2 + 2 kg, + 1 of channel 4 rl + j: two adjacent dwords of one quad row
      const lq_v2i xo = *(const lq_v2i*)(xP + ((kbase >> 3) + (kg >> 1)) * kQuad + (j * 16 + rl) * 4 + 2 * (kg & 1));
      acc[i][j] = mfma_f16_k16(aop, __builtin_bit_cast(lq_v4h, xo), acc[i][j]);
    }
  };
  block(0, rb[0], cwd[0], true);
  block(1, rb[1], cwd[1], true);
  if (ih == 0) block(0, rb[0] - 16, cwp, false); else block(1, rb[1] - 16, cwp, false);  // wave-uniform

  // ---- D residual + store
  const lq_v4f Dv = *(const lq_v4f*)(Dl_s + 4 * rl);
  _Float16* op = p.out + (((int64_t)b * p.seqlen + (int64_t)c * Q) * p.nheads + h) * p.P + p0;
  const uint32_t orow = (uint32_t)(p.nheads * p.P) * 2u;  // output row pitch in bytes
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    // x[m][4 rl + j] for the lane's four rows m = rb + 4 kg + r: two adjacent token pairs of one quad row
    lq_v2i xr2[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      xr2[j] = *(const lq_v2i*)(xP + ((rb[i] >> 3) + (kg >> 1)) * kQuad + (j * 16 + rl) * 4 + 2 * (kg & 1));
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = rb[i] + 4 * kg + r;
      if (m >= limit) continue;
      lq_v4h o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const lq_v2h pr = __builtin_bit_cast(lq_v2h, (uint32_t)xr2[j][r >> 1]);
        o[j] = (_Float16)fmaf((float)pr[r & 1], Dv[j], acc[i][j][r]);
      }
      __builtin_nontemporal_store(o, (lq_v4h*)((char*)op + __umul24((uint32_t)m, orow) + (uint32_t)rl * 8u));
    }
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
  p.sst_b = a->states_stride_b ? a->states_stride_b : (int64_t)p.nchunks * p.nheads * p.P * p.N;
  if (p.sst_b % 16 != 0) return LQ_ERR_SHAPE;
  const int ptiles = p.P / 64;
  if ((int64_t)p.batch * ptiles > 65535 || p.nheads > 65535 || p.nchunks > 65535) return LQ_ERR_SHAPE;
  const uint32_t hpg = (uint32_t)(p.nheads / p.G);
  p.hpg_magic = hpg == 1 ? 0u : (uint32_t)(0x100000000ull / hpg) + 1u;
  p.pt_magic = ptiles == 1 ? 0u : (uint32_t)(0x100000000ull / (uint32_t)ptiles) + 1u;
  // per-lane addresses are 32-bit byte offsets from a tile base, row pitches multiplied as 24-bit quantities
  if ((int64_t)p.Q * p.sC_l >= (1ll << 31) || (int64_t)p.P * p.N >= (1ll << 31) || p.sC_l >= (1 << 24) || p.sC_l < 0)
    return LQ_ERR_SHAPE;
  if (p.sx_l < 0 || p.sx_l * 2 >= (1 << 24) || (int64_t)p.Q * p.sx_l * 2 >= (1ll << 31)) return LQ_ERR_SHAPE;
  if ((int64_t)p.nheads * p.P * 2 >= (1 << 24) || (int64_t)p.Q * p.nheads * p.P * 2 >= (1ll << 31)) return LQ_ERR_SHAPE;
  if (p.sss_p < 0 || p.sss_p >= (1 << 24)) return LQ_ERR_SHAPE;
  const size_t lds = (size_t)2 * (p.Q / 8) * kQuad * 4 + (size_t)p.Q * 8 + 512 + (size_t)64 * (p.N + 32);  // x tiles, dA2, akw, per-channel scales, states
  dim3 grid(p.nheads, p.nchunks, p.batch * ptiles);
  // more than 64 KB of dynamic LDS has to be opted into per kernel
#define LQ_SCAN_LAUNCH(W, NN)                                                                                   \
  do {                                                                                                          \
    if (lds > 65536 && hipFuncSetAttribute(reinterpret_cast<const void*>(&chunk_scan_kernel<W, NN>),            \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
      return LQ_ERR_LAUNCH;                                                                                     \
    hipLaunchKernelGGL((chunk_scan_kernel<W, NN>), grid, dim3(W * 64), lds, stream, p);                         \
  } while (0)
#define LQ_SCAN_N(W)                                \
  switch (p.N / 64) {                               \
    case 1: LQ_SCAN_LAUNCH(W, 1); break;            \
    case 2: LQ_SCAN_LAUNCH(W, 2); break;            \
    case 3: LQ_SCAN_LAUNCH(W, 3); break;            \
    case 4: LQ_SCAN_LAUNCH(W, 4); break;            \
    default: return LQ_ERR_SHAPE; /* N 64 .. 256 */    \
  }
  switch (p.Q / 32) {
    case 2: LQ_SCAN_N(2); break;
    case 4: LQ_SCAN_N(4); break;
    case 8: LQ_SCAN_N(8); break;
    case 16: LQ_SCAN_N(16); break;
    default: return LQ_ERR_SHAPE;  // chunk sizes 64, 128, 256, 512
  }
#undef LQ_SCAN_N
#undef LQ_SCAN_LAUNCH
  return lq_check_launch();
}
