// Mamba-2 SSD stage 5: chunk scan (state read + causal intra-chunk product + D residual) -> fp16.
// Replaces linquant/kernels/mamba2/chunk_scan_v2.py:56-256 (launcher :259-366):
//   acc  = float(C_i8[m,:] . S_i8[p,:]) * sC[g] * ss[h,p] * exp(dA_m)
//   acc += sum_{k<=m} fp16(CB_i8[m,k] * S_cb * exp(dA_m - dA_k) * dt_k) * fp16(x[k,p])    (fp32 accumulate)
//   acc += float(x[m,p]) * (D_scale * float(D_i8[h]))
//
// One workgroup per (64-col P tile, batch*chunk, group of heads that share B and C) walks the heads of its group one
// after the other: the C rows and CB codes, which all of them share, are fetched once and stay in registers, and the
// x / state / dA / dt operands of head i + 1 are requested before the products of head i start and land while they
// run (measured at B4 L8192 H80 G8: one head per workgroup 254 us, all ten 180 us, which is the rate at which this
// machine moves the same 128-byte row pieces with no arithmetic at all).  One wavefront per two 16-row tiles of the
// chunk: tile w and tile 2*WAVES-1-w, an early and a late one, so every wave carries the same causal work.
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
  int hpg, hpw, hsplit;          // heads per group, heads per workgroup, workgroups per group (hsplit * hpw >= hpg)
  uint32_t hs_magic, pt_magic;   // floor(2^32 / d) + 1 for d = hsplit, P tiles (0 when d == 1): x / d == umulhi(x, magic) for x, d < 2^16
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

// The value itself, made opaque to the optimizer at this point of the program: whatever is computed from the result is
// computed after this point.  Inside the loop over heads it keeps loop-invariant lane arithmetic (addresses, masks,
// converted codes) from being hoisted into registers that then live through the whole loop and are spilled.
LQ_DEV int fresh(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

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
  constexpr int NS = WAVES - 1;                                      // 32-token slabs in front of a wave's two tiles, in total
  extern __shared__ __align__(16) unsigned char lds_raw[];
  // Every kernel argument is wanted in scalar registers here, so that all of them are requested in one batch and waited
  // for once: left alone the compiler fetches them in groups as their first uses come up, each group a full
  // round trip of the scalar cache before the next vector load can be issued.
  asm volatile("" ::"s"(p.cb), "s"(p.x), "s"(p.sx_b), "s"(p.sx_l), "s"(p.sx_h), "s"(p.dt), "s"(p.dA), "s"(p.C), "s"(p.sC_b),
               "s"(p.sC_l), "s"(p.sC_g), "s"(p.C_scale), "s"(p.states), "s"(p.ss), "s"(p.sss_h), "s"(p.sss_p));
  asm volatile("" ::"s"(p.sst_b), "s"(p.D), "s"(p.sD_h), "s"(p.D_has_hdim), "s"(p.D_scale), "s"(p.cb_scale), "s"(p.out), "s"(p.seqlen),
               "s"(p.nheads), "s"(p.P), "s"(p.G), "s"(p.Q), "s"(p.nchunks), "s"(p.hs_magic), "s"(p.pt_magic), "s"(p.hpg), "s"(p.hpw),
               "s"(p.hsplit));
  const int Q = p.Q;
  uint32_t* xP = (uint32_t*)lds_raw;          // [Q/8][kQuad]
  uint32_t* xS = xP + (Q / 8) * kQuad;        // [Q/8][kQuad]
  // two sets of per-head tables, each: [Q] dA * log2(e); [Q] dA * log2(e) - log2(S_cb * dt), so that exp2(dA2_m - akw_k) is
  // the causal weight of (m, k); [64] C scale * state scale of the tile's channels; [64] dequantized D of the tile's channels
  float* dA2_s = (float*)(xS + (Q / 8) * kQuad);
  int8_t* S_s = (int8_t*)(dA2_s + 2 * (2 * Q + 128));  // [64][kSRow] state tile of this (chunk, head), row p at (p & 3) * 16 + (p >> 2)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // known to be wave-uniform: everything derived from it is scalar
  const int rl = lane & 15, kg = lane >> 4;
  // grid = chunks x (groups x head parts) x (batch * P tiles): no integer division on the way to the first load.  Chunks
  // vary fastest across consecutive workgroups, which are dealt to the 8 XCDs round-robin: the head parts of one (batch,
  // chunk), which read the same C rows and CB codes, then share an XCD's L2 whenever the chunk count is a multiple of 8
  // (with the parts fastest every XCD fetched them from HBM for itself: 75 MB of 527 read).
  const int c = blockIdx.x;
  const int b = p.pt_magic ? (int)__umulhi(blockIdx.z, p.pt_magic) : (int)blockIdx.z;
  const int p0 = ((int)blockIdx.z - b * (p.P >> 6)) * 64;
  const int g = p.hs_magic ? (int)__umulhi(blockIdx.y, p.hs_magic) : (int)blockIdx.y;
  const int part = (int)blockIdx.y - g * p.hsplit;
  const int h0 = g * p.hpg + part * p.hpw;            // this workgroup's heads: h0 .. h0 + nh - 1, all of group g
  const int nh = min(p.hpw, p.hpg - part * p.hpw);
  const int limit = min(Q, p.seqlen - c * Q);
  const float scb = p.cb_scale[g];
  const float gscale = p.C_scale[g];
  const float dsc = p.D ? *p.D_scale : 0.0f;
  // power-of-two part of S_cb, as an exponent: kept out of the fp16 operand xS (whose values would drift into the
  // fp16 subnormal range with a small S_cb) and returned in fp32 by the row factor of the off-diagonal slabs
  const float kf = (float)(lq_clampi((__float_as_int(scb) >> 23) & 0xff, 2, 252) - 127);

  // Row tiles of this wave: 16w.. and 16(2*WAVES-1-w)..: an early and a late tile, so that every wave has the same
  // number of causal slabs to process.
  int rb[2];
  rb[0] = 16 * wave;
  rb[1] = 16 * (2 * WAVES - 1 - wave);

  // ---- operands shared by all heads of the group, fetched once per workgroup and kept in registers: this wave's C rows
  // and its CB codes.  Addresses are a wave-uniform 64-bit base plus a per-lane unsigned 32-bit byte offset (the launcher
  // checks that every tile fits 32 bits): per-lane 64-bit multiplies and adds ran at a quarter of the rate.
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
  // CB codes of this wave's off-diagonal slabs.  The early tile has ne = rb[0] / 32 of them, the late one the rest of
  // NS = WAVES - 1 (the same total for every wave), kept as one flat list.  A slab's address is a scalar (tile row base,
  // slab column) plus the lane's fixed (row, 8-column group) offset.
  const int8_t* cbp = p.cb + ((((int64_t)b * p.nchunks + c) * p.G + g) * Q) * Q;
  const int ne = rb[0] >> 5;
  lq_v2i cwr[NS];
  {
    const uint32_t cb_lane = (uint32_t)(rl * Q + 8 * kg);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int soff = s < ne ? rb[0] * Q + 32 * s : rb[1] * Q + 32 * (s - ne);  // scalar
      cwr[s] = *at<lq_v2i>(cbp + soff, cb_lane);
    }
  }
  // CB codes of the two 16 x 16 diagonal blocks and of the 16 tokens in front of the tile that sits in the second half
  // of its 32-token slab (exactly one of the wave's two tiles does): one dword (4 codes) per lane each, row rb + rl,
  // columns 4 kg .. 4 kg + 3 of the block.
  const int ih = (wave & 1) ? 0 : 1;  // scalar: which tile is the second-half one
  int cwd[2], cwp;
  {
    const uint32_t cd_lane = (uint32_t)(rl * Q + 4 * kg);
    cwd[0] = *at<int>(cbp + rb[0] * Q + rb[0], cd_lane);
    cwd[1] = *at<int>(cbp + rb[1] * Q + rb[1], cd_lane);
    cwp = *at<int>(cbp + rb[ih] * Q + rb[ih] - 16, cd_lane);
  }

  // ---- operands of one head: the state tile (one 16-byte piece per thread), dA / dt (one token per thread), the
  // per-channel state scale and D (one channel per lane), the x tile (8 tokens x 4 channels per thread).  They are
  // requested one head ahead and stay in flight while the previous head is computed; `on` = 0 (no next head) collapses
  // every lane's address onto the first bytes of the head's tile, so that the request is unconditional (a conditional
  // request is waited for where the branches join) and costs one cache line.  All of them are wave-uniform running
  // pointers that advance by one head.
  lq_v4i spiece[kSPieces];
  float dA_r, dt_r, ss_r;
  int D_r;
  lq_v2i xr[8];
  const uint32_t sxl2 = (uint32_t)p.sx_l * 2u;  // row pitch of x in bytes
  const int8_t* rqS = p.states + (int64_t)b * p.sst_b + ((((int64_t)c * p.nheads + h0) * p.P + p0) * (int64_t)N);
  const int64_t cs0 = (((int64_t)b * p.nheads + h0) * p.nchunks + c) * Q;
  const float* rqA = p.dA + cs0;
  const float* rqT = p.dt + cs0;
  const float* rqC = p.ss + (int64_t)h0 * p.sss_h + (int64_t)p0 * p.sss_p;
  // without D the request goes to a valid dummy address and dsc = 0 discards it: no branch around a request
  const int8_t* rqD = p.D ? p.D + (int64_t)h0 * p.sD_h + (p.D_has_hdim ? p0 : 0) : p.states;
  const _Float16* rqX = p.x + (int64_t)b * p.sx_b + (int64_t)c * Q * p.sx_l + (int64_t)h0 * p.sx_h + p0;
  // part 0: the state piece, the per-token and per-channel scalars and the first half of the x rows; part 1: the other half
  // of the x rows; part 2: everything.  The two parts are issued at two places of a head: a wave issues in order, and the
  // thirteen requests in a row held it for as long as the memory pipeline took to accept them (0.7 of a head's 7 us).
  auto request = [&](uint32_t on, int part) {
    const int tid = fresh((int)threadIdx.x), lane = tid & 63;
    if (part != 1) {
#pragma unroll
      for (int k = 0; k < kSPieces; ++k) {
        const int t = tid + k * WAVES * 64;
        // (x and the state tile are streamed: a non-temporal request keeps them from displacing the C / CB tiles that
        // other workgroups still need)
        spiece[k] = __builtin_nontemporal_load(at<lq_v4i>(rqS, ((uint32_t)min(t, 4 * N - 1) * 16u) & on));  // a surplus thread re-reads the last piece
      }
      const uint32_t qoff = ((uint32_t)min(tid, Q - 1) * 4u) & on;
      dA_r = *at<float>(rqA, qoff);
      dt_r = *at<float>(rqT, qoff);
      ss_r = *at<float>(rqC, (__umul24((uint32_t)lane, (uint32_t)p.sss_p) * 4u) & on);
      D_r = (int)*at<int8_t>(rqD, (p.D && p.D_has_hdim) ? ((uint32_t)lane & on) : 0u);
    }
    // tokens 8 q .. 8 q + 7 (the four token pairs of one row of the LDS layout), channels 4 c4 .. 4 c4 + 3
    const int q8 = (tid >> 4) * 8;
    const uint32_t c4b = (uint32_t)(tid & 15) * 8u;
#pragma unroll
    for (int r = 0; r < 8; ++r)
      // rows past the sequence end re-read its last row and are zeroed when staged (no branch around a request)
      if (part == 2 || (r < 4) == (part == 0))
        xr[r] = __builtin_nontemporal_load(at<lq_v2i>(rqX, (__umul24((uint32_t)min(q8 + r, limit - 1), sxl2) + c4b) & on));
  };
  auto advance = [&]() {
    rqS += (int64_t)p.P * N, rqA += (int64_t)p.nchunks * Q, rqT += (int64_t)p.nchunks * Q, rqC += p.sss_h;
    rqD += p.D ? p.sD_h : 0, rqX += p.sx_h;
  };
  // Waits until every operand requested by `request` has arrived.  Loads and stores retire through one in-order
  // counter, and the stores of a head are conditional, so a wait for a request that is older than such stores
  // becomes a wait for the stores as well.  Hence two fixed points: before the loop, and before the last stores of
  // each head (by then the next head's operands have had the whole head to arrive); the top of the loop then never waits.
  auto settle = [&]() {
#pragma unroll
    for (int k = 0; k < kSPieces; ++k) asm volatile("" ::"v"(spiece[k]));
    asm volatile("" ::"v"(dA_r), "v"(dt_r), "v"(ss_r), "v"(D_r), "v"(xr[0]), "v"(xr[1]), "v"(xr[2]), "v"(xr[3]), "v"(xr[4]),
                 "v"(xr[5]), "v"(xr[6]), "v"(xr[7]));
  };
  // The per-token and per-channel tables of a head (2.5 KB) are kept twice: a head's tables are written while the head
  // before it is computed, which leaves two barriers per head.
  const int small_stride = 2 * Q + 128;  // floats
  auto write_small = [&](int buf) {
    const int tid = fresh((int)threadIdx.x);
    float* base = dA2_s + buf * small_stride;
    if (tid < Q) {
      const float a2 = dA_r * 1.44269504088896340736f;
      base[tid] = a2;
      base[Q + tid] = a2 - __builtin_amdgcn_logf(scb * dt_r);  // dt = 0 past the sequence end: +inf, weight 0
    }
    if (tid < 64) {
      base[2 * Q + tid] = gscale * ss_r;
      base[2 * Q + 64 + tid] = dsc * (float)D_r;
    }
  };
  request(0xffffffffu, 2);
  if (nh > 1) advance();
  settle();
  write_small(0);
  _Float16* op = p.out + (((int64_t)b * p.seqlen + (int64_t)c * Q) * p.nheads + h0) * p.P + p0;
  const uint32_t orow = (uint32_t)(p.nheads * p.P) * 2u;  // output row pitch in bytes

  for (int hi = 0; hi < nh; ++hi, op += p.P) {
    __syncthreads();  // every wave is done with the previous head's tiles; this head's tables are in place
    const float* dA2 = dA2_s + (hi & 1) * small_stride;
    const float* akw = dA2 + Q;
    const float* ssl = akw + Q;
    const float* Dl = ssl + 64;
    {
      const int tid = fresh((int)threadIdx.x);
#pragma unroll
      for (int k = 0; k < kSPieces; ++k) {
        const int t = tid + k * WAVES * 64;
        const int pr = t / (N / 16), pc = t % (N / 16);
        if (t < 4 * N) *(lq_v4i*)(S_s + ((pr & 3) * 16 + (pr >> 2)) * kSRow + pc * 16) = spiece[k];
      }
      // x tile: this thread's 8 tokens x 4 channels become, per channel, the four token pairs of one 16-byte group
      const int q = tid >> 4, c4 = tid & 15;
      if (limit < Q) {  // ragged last chunk (wave-uniform): rows past the sequence end are staged as zeros
#pragma unroll
        for (int r = 0; r < 8; ++r)
          if (8 * q + r >= limit) xr[r] = lq_v2i{0, 0};
      }
      const float ae = dA2[(8 * q) | 31] - kf;
      const lq_v4f ak0 = *(const lq_v4f*)(akw + 8 * q), ak1 = *(const lq_v4f*)(akw + 8 * q + 4);
      lq_v2h g2[4];
      g2[0] = lq_v2h{(_Float16)fexp2(ae - ak0[0]), (_Float16)fexp2(ae - ak0[1])};
      g2[1] = lq_v2h{(_Float16)fexp2(ae - ak0[2]), (_Float16)fexp2(ae - ak0[3])};
      g2[2] = lq_v2h{(_Float16)fexp2(ae - ak1[0]), (_Float16)fexp2(ae - ak1[1])};
      g2[3] = lq_v2h{(_Float16)fexp2(ae - ak1[2]), (_Float16)fexp2(ae - ak1[3])};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lq_v4i vp, vs;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const lq_v4h ra = __builtin_bit_cast(lq_v4h, xr[2 * t]), rb2 = __builtin_bit_cast(lq_v4h, xr[2 * t + 1]);
          const lq_v2h pr = {ra[e], rb2[e]};
          vp[t] = (int)__builtin_bit_cast(uint32_t, pr);
          vs[t] = (int)__builtin_bit_cast(uint32_t, pr * g2[t]);
        }
        const int off = q * kQuad + (e * 16 + c4) * 4;  // x_slot(4 c4 + e) * 4
        *(lq_v4i*)(xP + off) = vp;
        *(lq_v4i*)(xS + off) = vs;
      }
    }
    // the next head's operands travel while this one is computed
    const uint32_t on_next = hi + 1 < nh ? 0xffffffffu : 0u;
    request(on_next, 0);
    __syncthreads();

    // One 16-row tile at a time, start to finish (a tile past the sequence end is processed like any other, its rows
    // are never stored).
    auto tile = [&](const int i, const bool last) {
      const int lane = fresh((int)threadIdx.x) & 63, rl = lane & 15, kg = lane >> 4;
      int nes = ne;
      asm volatile("" : "+s"(nes));  // recomputed comparisons instead of a table of them kept in scalar registers
      // ---- slabs before the tile's own slab: (scaled CB codes) x (anchor-scaled x), row factor applied once.
      // anchor of a tile = last token before its own slab
      const float aE = dA2[max(rb[i] & ~31, 1) - 1];
      // factor exp(dA_anchor - dA_end of slab J) of every slab at once: lane J computes slab J's
      const int shb = (int)__builtin_bit_cast(uint16_t, (_Float16)fexp2(aE - dA2[32 * min(lane, NS - 1) + 31]));
      const uint32_t* xs_lane = xS + kg * kQuad + rl * 4;
      lq_v4f off[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) off[j] = lq_v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        if (i == 0 && s >= (WAVES - 1) / 2) continue;  // the early tile has at most (WAVES - 1) / 2 slabs
        const bool mine = i == 0 ? s < nes : s >= nes;  // wave-uniform
        if (!mine) continue;
        const int J = i == 0 ? s : s - nes;
        const uint32_t sb = (uint32_t)__builtin_amdgcn_readlane(shb, J);
        // a slab whose factor underflows fp16 (more than 25 octaves of decay between it and the tile) would contribute
        // fp16(code * 0) = 0 to every product: it is left out (wave-uniform; strongly decaying heads skip most slabs)
        if (sb != 0) {
          lq_v4i xop[4];  // token pairs 16 J + 4 kg .. + 3 of channel 4 rl + j
#pragma unroll
          for (int j = 0; j < 4; ++j) xop[j] = *(const lq_v4i*)(xs_lane + 4 * J * kQuad + j * 64);
          const lq_v2h s2 = __builtin_bit_cast(lq_v2h, sb | (sb << 16));
          lq_v4i aw;
          uint32_t lo, hi2;
          i8x4_to_f16x4((uint32_t)fresh(cwr[s][0]), s2, lo, hi2);
          aw[0] = (int)lo, aw[1] = (int)hi2;
          i8x4_to_f16x4((uint32_t)fresh(cwr[s][1]), s2, lo, hi2);
          aw[2] = (int)lo, aw[3] = (int)hi2;
          const lq_v8h aop = __builtin_bit_cast(lq_v8h, aw);
#pragma unroll
          for (int j = 0; j < 4; ++j) off[j] = lq_mfma_f16(aop, __builtin_bit_cast(lq_v8h, xop[j]), off[j]);
        }
      }
      // ---- state path (INT8 MFMA): C rows from registers, state rows from LDS
      lq_v4i ai[4];
#pragma unroll
      for (int n = 0; n < N64; ++n)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const lq_v4i sop = *(const lq_v4i*)(S_s + (j * 16 + rl) * kSRow + 64 * n + 16 * kg);
          ai[j] = lq_mfma_i8(cop[i][n], sop, n == 0 ? lq_v4i{0, 0, 0, 0} : ai[j]);
        }
      // ---- state read dequantized and gated, float(acc) * (sC * ss[p]) * exp(dA_m), plus the slabs' sum times its
      // row factor exp(dA_m - dA_anchor) * 2^kf
      lq_v4f acc[4];
      {
        const lq_v4f ssv = *(const lq_v4f*)(ssl + 4 * rl);
        const lq_v4f a4 = *(const lq_v4f*)(dA2 + rb[i] + 4 * kg);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float rg = fexp2(a4[r]);
          const float rf = fexp2(a4[r] - (aE - kf));
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            acc[j][r] = (float)ai[j][r] * (ssv[j] * rg);
            if (NS > 0 && (i == 1 || ne > 0)) acc[j][r] = fmaf(off[j][r], rf, acc[j][r]);
          }
        }
      }
      // ---- the tile's own slab, in 16-token blocks on the K = 16 MFMA (4 tokens per lane): the diagonal block
      // [rb, rb + 16) with weights exp2(dA2_m - akw_k) masked to k <= m, and, for the tile in the second half of its
      // slab, the 16 tokens in front of it, all of them before every row of the tile (no mask)
      const float dAm = dA2[rb[i] + rl];
      auto block = [&](int kbase, int codes, bool masked) {
        const lq_v4f ak = *(const lq_v4f*)(akw + kbase + 4 * kg);
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
          acc[j] = mfma_f16_k16(aop, __builtin_bit_cast(lq_v4h, xo), acc[j]);
        }
      };
      block(rb[i], fresh(cwd[i]), true);
      if (i == ih) block(rb[i] - 16, fresh(cwp), false);  // wave-uniform
      // ---- D residual + store
      const lq_v4f Dv = *(const lq_v4f*)(Dl + 4 * rl);
      // x[m][4 rl + j] for the lane's four rows m = rb + 4 kg + r: two adjacent token pairs of one quad row
      lq_v2i xr2[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        xr2[j] = *(const lq_v2i*)(xP + ((rb[i] >> 3) + (kg >> 1)) * kQuad + (j * 16 + rl) * 4 + 2 * (kg & 1));
      if (last) {
        settle();
        write_small((hi + 1) & 1);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = rb[i] + 4 * kg + r;
        if (m >= limit) continue;
        lq_v4h o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const lq_v2h pr = __builtin_bit_cast(lq_v2h, (uint32_t)xr2[j][r >> 1]);
          o[j] = (_Float16)fmaf((float)pr[r & 1], Dv[j], acc[j][r]);
        }
        __builtin_nontemporal_store(o, (lq_v4h*)((char*)op + __umul24((uint32_t)m, orow) + (uint32_t)rl * 8u));
      }
    };
    if (rb[0] < limit) {  // else the early tile is past the sequence end, and so is the late one (wave-uniform)
      tile(0, false);
      request(on_next, 1);
      if (hi + 2 < nh) advance();
      tile(1, true);
    } else {
      request(on_next, 1);
      if (hi + 2 < nh) advance();
      settle();
      write_small((hi + 1) & 1);
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
  // Heads of a group per workgroup: as many as leave about two workgroups for each of the 512 slots of the chip (256
  // compute units x 2 resident workgroups), since a workgroup fetches its C rows and CB codes once and overlaps each
  // head's loads with the previous head's arithmetic.
  p.hpg = p.nheads / p.G;
  {
    const int64_t tiles = (int64_t)p.G * p.nchunks * p.batch * ptiles;
    int64_t split = (1024 + tiles - 1) / tiles;
    if (split > p.hpg) split = p.hpg;
    if (a->heads_hint > 0) split = (p.hpg + a->heads_hint - 1) / a->heads_hint;
    if (a->heads_hint < 0) return LQ_ERR_SHAPE;
    p.hpw = (int)((p.hpg + split - 1) / split);
    p.hsplit = (p.hpg + p.hpw - 1) / p.hpw;
  }
  if ((int64_t)p.G * p.hsplit > 65535) return LQ_ERR_SHAPE;
  p.hs_magic = p.hsplit == 1 ? 0u : (uint32_t)(0x100000000ull / (uint32_t)p.hsplit) + 1u;
  p.pt_magic = ptiles == 1 ? 0u : (uint32_t)(0x100000000ull / (uint32_t)ptiles) + 1u;
  // per-lane addresses are 32-bit byte offsets from a tile base, row pitches multiplied as 24-bit quantities
  if ((int64_t)p.Q * p.sC_l >= (1ll << 31) || (int64_t)p.P * p.N >= (1ll << 31) || p.sC_l >= (1 << 24) || p.sC_l < 0)
    return LQ_ERR_SHAPE;
  if (p.sx_l < 0 || p.sx_l * 2 >= (1 << 24) || (int64_t)p.Q * p.sx_l * 2 >= (1ll << 31)) return LQ_ERR_SHAPE;
  if ((int64_t)p.nheads * p.P * 2 >= (1 << 24) || (int64_t)p.Q * p.nheads * p.P * 2 >= (1ll << 31)) return LQ_ERR_SHAPE;
  if (p.sss_p < 0 || p.sss_p >= (1 << 24)) return LQ_ERR_SHAPE;
  const size_t lds = (size_t)2 * (p.Q / 8) * kQuad * 4 + 2 * ((size_t)p.Q * 8 + 512) + (size_t)64 * (p.N + 32);  // x tiles, two sets of dA2 / akw / per-channel tables, states
  dim3 grid(p.nchunks, p.G * p.hsplit, p.batch * ptiles);
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
