// Mamba-2 SSD stage 2: INT8 chunk states, value-side and key-side scale absorption.
// Replaces linquant/kernels/mamba2/chunk_state.py:72-255 (value side) and
// linquant/kernels/mamba2/chunk_state_keyside.py:163-330 (key side).
//
//   value side: xq = clamp(rha(x * (1/alpha[p]) * gate[k]), +-127),  acc = xq^T . B_i8
//               state = clamp(rha(float(acc) * ((alpha[p]/S_out[p]) * bscale_g)), +-127)
//   key side  : x_i8 = clamp(rint(x * (1/max(x_scale[p],1e-10))), +-127)
//               B'   = clamp(rint((B_fp * gate[k]) * (127/b_gate[n])), +-127),  acc = x_i8^T . B'
//               state = clamp(rint(float(acc) * (b_gate[n]/127) * (x_scale[p]/S_out[p])), +-127)
//   gate[k] = exp(dA_last - dA[k]) * dt[k]
//
// One 4-wave workgroup per (64-row P tile, <=128-col N tile, batch*chunk, head).  The per-element
// quantization is the expensive part (VALU), so it is done exactly once per element: for every 64-token
// slab the workgroup quantizes the x slab and the B slab cooperatively into LDS, double-buffered against the
// next slab's global loads.  A thread handles 4 consecutive tokens of a few adjacent channels and emits, per
// channel, one dword holding the 4 token codes; LDS is laid out [token quad][channel] in dwords, so those
// stores are contiguous 16-byte writes and an MFMA operand (16 token codes of one channel) is 4 dword reads
// at consecutive banks across the lanes.  Wave w owns the 16 P rows 16w..16w+15 and all N columns of
// the tile (transposed product: accumulator rows are N, so each lane holds 4 adjacent N of one P row and
// stores them as one dword).  The gates of the whole chunk are evaluated once per workgroup.
// Round-half-even + clamp + int conversion is one fp32 add of 1.5*2^23 after the clamp (the low byte of the
// sum's bit pattern is the two's-complement code).
// Key side, zero-slab elision: the gate exp(dA_last - dA_k) * dt_k decays towards the start of the chunk, and a gated key
// code rint((B * gate) * 127 / b_gate) is exactly zero once gate_k * max_n |B[k, n]| * max_n (127 / b_gate[n]) < 0.5.  A
// 64-token slab all of whose tokens satisfy that bound contributes nothing to the INT32 product, so neither its x rows nor
// its B rows are fetched or quantized; the per-token max_n |B| comes from a small pre-pass over B (shared by all heads).
// The result is bit-identical; the saving depends on the data (none for slowly decaying heads, three slabs of four for
// per-token decays of 0.1 and more at chunk 256).  Slabs are walked from the end of the chunk backwards, so the last one
// (live whenever anything is) can be requested before the gates are known.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

typedef uint32_t lq_v2u __attribute__((ext_vector_type(2)));

constexpr int kXW = 64 + 4;    // dwords per token-quad row of the x slab (64 channels + pad: the four lane groups of an
constexpr int kPad = 4;       // operand read land on bank offsets 0,16,32,48)

struct Params {
  const _Float16* x;
  int64_t sx_b, sx_l, sx_h;
  const void* B;
  int64_t sB_b, sB_l, sB_g;
  const float* dt;
  const float* dA;
  const float* xs;  // alpha_hp (value) or x_scale_hp (key)
  int64_t sxs_h, sxs_p;
  const float* bscale_g;
  int64_t sbs_g;
  const float* oqs;
  int64_t soq_h, soq_p;
  const float* bgs;
  int64_t sbg_b, sbg_c, sbg_h, sbg_n;
  const float* rowmax;  // key side, optional: (B,L,G) max_n |B|, filled by row_absmax_kernel
  int rowmax_ready;     // the table is already filled (by the prologue that produced B)
  int8_t* states;
  int64_t sst_b;        // elements between batch rows of states
  int batch, seqlen, nheads, P, G, N, Q, nchunks, n_ntiles;
  // floor(2^32 / d) + 1 for d = heads per group, tiles per (batch, chunk, head), N tiles per P tile; 0 when d == 1:
  // x / d == umulhi(x, magic) for x, d < 2^16
  uint32_t hpg_magic, tiles_magic, nt_magic;
};

LQ_DEV int div_magic(uint32_t x, uint32_t magic) { return magic ? (int)__umulhi(x, magic) : (int)x; }

// clamp to [-127, 127] then round half even; returns a dword whose low byte is the INT8 code
LQ_DEV uint32_t rint_code(float y) {
  const float c = __builtin_amdgcn_fmed3f(y, -127.0f, 127.0f);
  return __float_as_uint(c + 12582912.0f);
}

LQ_DEV uint32_t pack_low_bytes(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uint32_t lo = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);  // {a.b0, b.b0, 0, 0}
  const uint32_t hi = __builtin_amdgcn_perm(d, c, 0x04000c0cu);  // {0, 0, c.b0, d.b0}
  return lo | hi;
}

// float(half of the packed fp16 pair w) * f in one instruction: the mixed-precision fma converts the selected half
// exactly and rounds the product once, so the result equals the separate convert-then-multiply bit for bit.
template <int HI>
LQ_DEV float mul_half(uint32_t w, float f) {
  // an explicit fma with a +0 addend selects v_fma_mix_f32 and leaves the hazard bookkeeping to the compiler
  const lq_v2h h = __builtin_bit_cast(lq_v2h, w);
  return __builtin_fmaf((float)h[HI], f, 0.0f);
}

// NSLAB = number of 64-token slabs of a chunk when it is one of the unrolled counts (2, 4), else 0 (run-time loop).
// With a known count the slab loop is fully unrolled over two register sets: the next slab is requested before the
// current one is quantized, no request sits inside a run-time branch, and the compiler's wait counts stay exact.
// Measured at B4 L8192 H80 P64 N128 Q256: value side 115 -> 108 us; key side 146 -> 150 us, and 123 -> 128 us after the
// prologue was slimmed (its slabs are bound by the per-head quantization arithmetic of B, not by the loads), so the key
// side keeps the run-time loop.
template <bool KEYSIDE, int NT, int NSLAB>
__global__ __launch_bounds__(256, 2) void chunk_state_kernel(Params p) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int Q = p.Q;
  float* gate_s = (float*)lds_raw;                    // [Q]
  float* bdeq_s = gate_s + Q;                         // [NT] b_gate / 127 (key side)
  float* binv_s = bdeq_s + NT;                        // [NT] 127 / b_gate (key side)
  float* xinv_s = binv_s + NT;                        // [64] reciprocal operand scale of the tile's P rows
  float* req_s = xinv_s + 64;                         // [64] epilogue factor of the tile's P rows
  constexpr int kBW = NT + kPad;
  uint32_t* xq = (uint32_t*)(req_s + 64);             // [2][16][kXW]
  uint32_t* bq = xq + 2 * 16 * kXW;                   // [2][16][kBW]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  // grid = chunks x heads x (batch * tiles): no run-time integer division in front of the first request.  Chunks vary
  // fastest across consecutive workgroups, which are dealt to the 8 XCDs round-robin: the heads of one (batch, chunk),
  // which share its B tile, then meet in one XCD's L2 whenever the chunk count is a multiple of 8 (with the heads fastest
  // every XCD fetched the tile from HBM for itself)
  const int h = blockIdx.y, c = blockIdx.x;
  const int b = div_magic(blockIdx.z, p.tiles_magic);
  const int tile = (int)blockIdx.z - b * (p.P >> 6) * p.n_ntiles;
  const int ptile = div_magic((uint32_t)tile, p.nt_magic), ntile = tile - ptile * p.n_ntiles;
  const int g = div_magic((uint32_t)h, p.hpg_magic);
  const int p0 = ptile * 64, n0 = ntile * NT;
  const int limit = min(Q, p.seqlen - c * Q);
  const int64_t cs = (((int64_t)b * p.nheads + h) * p.nchunks + c) * Q;

  // ---- Every global request of the prologue is issued first, oldest first in the order of first use, and none sits
  // inside a branch: memory operations retire in issue order, a request inside a branch is waited for where the branches
  // join, and arithmetic on a loaded value is a wait for it.  (The gates were computed by a loop that waited for dA and
  // for dt in turn, followed by a wait for the B scales: three memory round trips before the first slab was requested.)
  // Tokens past the sequence end carry a zero gate, which zeroes the gated operand's codes; their loads are redirected
  // to the last valid token so no access leaves the tensor.
  const float dA_last = p.dA[cs + Q - 1];
  const int kg0 = min(tid, Q - 1);  // gate of token kg0 (threads past a short chunk repeat its last token)
  const float dA_k = p.dA[cs + kg0];
  const float dt_k = p.dt[cs + kg0];
  // Scales: every distinct value of the tile is requested by one thread and turned into its reciprocal / ratio once,
  // then shared through LDS (each thread used to fetch and divide its own 4 + 8 + 2 copies: fourteen IEEE divisions and as
  // many 64-bit address computations per thread, a quarter of the kernel's instructions).
  float bg_t = 1.0f;
  if (KEYSIDE)
    bg_t = p.bgs[(int64_t)b * p.sbg_b + (int64_t)c * p.sbg_c + (int64_t)h * p.sbg_h + (int64_t)(n0 + (tid & (NT - 1))) * p.sbg_n];
  const int prow = p0 + (tid & 63);
  const float xs_t = p.xs[(int64_t)h * p.sxs_h + (int64_t)prow * p.sxs_p];
  const float so_t = p.oqs[(int64_t)h * p.soq_h + (int64_t)prow * p.soq_p];
  // per-token max |B| of the first four slabs before the last (slabs further out, in chunks longer than 320 tokens, are
  // fetched when they are tested); clamped rows, dead data when the elision is off
  const bool elide = KEYSIDE && p.rowmax != nullptr;
  const int nslab_all = Q >> 6;
  float rmv[4];
  {
    const float* rmp = elide ? p.rowmax + ((int64_t)b * p.seqlen + (int64_t)c * Q) * p.G + g : p.dt + cs;
    const int rstride = elide ? p.G : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) rmv[i] = rmp[(int64_t)min(max(64 * (nslab_all - 2 - i), 0) + lane, limit - 1) * rstride];
  }
  const float bs_t = KEYSIDE ? 0.0f : p.bscale_g[(int64_t)g * p.sbs_g];

  // fixed thread -> work mapping of the quantize phase: x slab = 16 token quads x 16 groups of 4 channels (all 256
  // threads), B slab = 16 token quads x NT/8 groups of 8 channels (threads without a B item load a clamped address)
  const int kqx = tid >> 4, c4x = tid & 15;
  constexpr int kBItems = NT / 8;
  const bool has_b = (NT == 128) || (tid < 16 * kBItems);
  const int kqb = (NT == 128) ? (tid >> 4) : (tid / kBItems);
  const int cb8 = (NT == 128) ? (tid & 15) : (tid % kBItems);

  const int pr = p0 + 16 * wave + rl;

  const int last = limit - 1;
  // wave-uniform 64-bit bases; the lane's own channel offset goes into the 32-bit part
  const _Float16* xg = p.x + (int64_t)b * p.sx_b + (int64_t)c * Q * p.sx_l + (int64_t)h * p.sx_h + p0;
  const char* bg0 = (const char*)p.B + ((int64_t)b * p.sB_b + (int64_t)c * Q * p.sB_l + (int64_t)g * p.sB_g + n0) * (KEYSIDE ? 2 : 1);
  const uint32_t xlane = (uint32_t)c4x * 8u, blane = (uint32_t)cb8 * (KEYSIDE ? 16u : 8u);
  const int64_t bstep = p.sB_l * (KEYSIDE ? 2 : 1);  // bytes per token
  lq_v2i xrA[4], xrB[4];  // x: 4 tokens x 4 fp16 (two sets: the slab being quantized and the one in flight)
  lq_v4i brA[4], brB[4];  // key side: 4 tokens x 8 fp16; value side: only [t][0..1] used (8 int8)

  // token * stride stays below 2^31 and both factors below 2^23 (checked by the launcher): a full-rate 24-bit multiply
  // instead of the quarter-rate 64-bit one.  A full chunk needs no clamping of the token index, so its row offsets are
  // formed once and advanced by a scalar per slab; a ragged last chunk (wave-uniform) multiplies the clamped index.
  const int sxl = (int)p.sx_l, bst = (int)bstep;
  const bool ragged = limit < Q;
  uint32_t xo[4], bo4[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    xo[t] = (uint32_t)__mul24(4 * kqx + t, sxl) * 2u + xlane;
    bo4[t] = (uint32_t)__mul24(4 * kqb + t, bst) + blane;
  }
  auto load_slab = [&](int k0, lq_v2i (&xr)[4], lq_v4i (&br)[4]) {
    const uint32_t xk = (uint32_t)(k0 * sxl) * 2u, bk = (uint32_t)(k0 * bst);  // scalar
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t ox = ragged ? (uint32_t)__mul24(min(k0 + 4 * kqx + t, last), sxl) * 2u + xlane : xo[t] + xk;
      const uint32_t ob = ragged ? (uint32_t)__mul24(min(k0 + 4 * kqb + t, last), bst) + blane : bo4[t] + bk;
      xr[t] = *(const lq_v2i*)((const char*)xg + ox);
      if (KEYSIDE) {
        br[t] = *(const lq_v4i*)(bg0 + ob);
      } else {
        const lq_v2i v = *(const lq_v2i*)(bg0 + ob);
        br[t][0] = v[0], br[t][1] = v[1];
      }
    }
  };
  load_slab(NSLAB > 0 ? 0 : 64 * (nslab_all - 1), xrA, brA);  // the run-time loop starts at the last slab

  // ---- gates of the whole chunk, dequantization scales of B, reciprocal operand scales
  // (written by every thread, duplicates included: a store under `if (tid < Q)` lets the compiler sink the requests
  // above into that branch, which puts their round trip back on the critical path)
  {
    const float gv = lq_expf(dA_last - dA_k) * dt_k;
    gate_s[kg0] = kg0 < limit ? gv : 0.0f;
  }
  for (int k = tid + 256; k < Q; k += 256)  // chunks longer than the workgroup
    gate_s[k] = k < limit ? lq_expf(dA_last - p.dA[cs + k]) * p.dt[cs + k] : 0.0f;
  if (KEYSIDE) {
    bdeq_s[tid & (NT - 1)] = bg_t / 127.0f;
    binv_s[tid & (NT - 1)] = 127.0f / bg_t;
  }
  xinv_s[tid & 63] = KEYSIDE ? 1.0f / fmaxf(xs_t, 1e-10f) : 1.0f / xs_t;
  {
    const float ratio = xs_t / so_t;
    req_s[tid & 63] = KEYSIDE ? ratio : ratio * bs_t;
  }

  lq_v4i acc[NT / 16];
#pragma unroll
  for (int q = 0; q < NT / 16; ++q) acc[q] = lq_v4i{0, 0, 0, 0};

  __syncthreads();  // gates and scale tables visible
  float xinv[4], binv[8];
  {
    const lq_v4f xv = *(const lq_v4f*)(xinv_s + 4 * c4x);
#pragma unroll
    for (int e = 0; e < 4; ++e) xinv[e] = xv[e];
    if (KEYSIDE) {
      const lq_v4f b0 = *(const lq_v4f*)(binv_s + 8 * cb8), b1 = *(const lq_v4f*)(binv_s + 8 * cb8 + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) binv[e] = e < 4 ? b0[e & 3] : b1[e & 3];
    }
  }

  const int nslab = Q >> 6;
  auto slab = [&](int s, int par, lq_v2i (&xr)[4], lq_v4i (&br)[4], auto post) {
    const int k0 = s * 64;
    uint32_t* xb = xq + (par & 1) * 16 * kXW;
    uint32_t* bb = bq + (par & 1) * 16 * kBW;
    // ---- quantize this slab into LDS (codes of 4 consecutive tokens of one channel form one dword)
    {
      float gt[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) gt[t] = gate_s[k0 + 4 * kqx + t];
      lq_v4i xo;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t cd[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t w = (uint32_t)xr[t][e >> 1];
          float y = (e & 1) ? mul_half<1>(w, xinv[e]) : mul_half<0>(w, xinv[e]);
          if (KEYSIDE) {
            cd[t] = rint_code(y);
          } else {
            y = y * gt[t];
            cd[t] = (uint32_t)lq_q_rha(y, 127);
          }
        }
        xo[e] = (int)pack_low_bytes(cd[0], cd[1], cd[2], cd[3]);
      }
      *(lq_v4i*)(xb + kqx * kXW + 4 * c4x) = xo;
    }
    if (has_b) {
      lq_v4i bo[2];
      if (KEYSIDE) {
        float gt[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) gt[t] = gate_s[k0 + 4 * kqb + t];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          uint32_t cd[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const uint32_t w = (uint32_t)br[t][e >> 1];
            float y = (e & 1) ? mul_half<1>(w, gt[t]) : mul_half<0>(w, gt[t]);
            y = y * binv[e];
            cd[t] = rint_code(y);
          }
          bo[e >> 2][e & 3] = (int)pack_low_bytes(cd[0], cd[1], cd[2], cd[3]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          // byte e of the four token rows -> one dword
          const uint32_t s0 = (uint32_t)br[0][e >> 2], s1 = (uint32_t)br[1][e >> 2];
          const uint32_t s2 = (uint32_t)br[2][e >> 2], s3 = (uint32_t)br[3][e >> 2];
          const uint32_t sel = 0x0c0c0400u + 0x0101u * (e & 3);
          const uint32_t lo = __builtin_amdgcn_perm(s1, s0, sel);
          const uint32_t hi = __builtin_amdgcn_perm(s3, s2, sel);
          bo[e >> 2][e & 3] = (int)(lo | (hi << 16));
        }
      }
      uint32_t* dst = bb + kqb * kBW + 8 * cb8;
      *(lq_v4i*)dst = bo[0];
      *(lq_v4i*)(dst + 4) = bo[1];
    }
    post();  // the run-time loop requests the next slab here, into the registers just consumed
    __syncthreads();
    // ---- MFMA from LDS: rows = N (this tile), cols = the wave's 16 P rows
    lq_v4i xop;
#pragma unroll
    for (int i = 0; i < 4; ++i) xop[i] = (int)xb[(4 * kg + i) * kXW + 16 * wave + rl];
#pragma unroll
    for (int q = 0; q < NT / 16; ++q) {
      lq_v4i bop;
#pragma unroll
      for (int i = 0; i < 4; ++i) bop[i] = (int)bb[(4 * kg + i) * kBW + 16 * q + rl];
      acc[q] = lq_mfma_i8(bop, xop, acc[q]);
    }
  };
  if constexpr (NSLAB > 0) {
#pragma unroll
    for (int s = 0; s < NSLAB; ++s) {
      if (s & 1) {
        if (s + 1 < NSLAB) load_slab(64 * (s + 1), xrA, brA);
        asm volatile("" ::: "memory");  // the requests stay ahead of the LDS traffic below
        slab(s, s, xrB, brB, [] {});
      } else {
        if (s + 1 < NSLAB) load_slab(64 * (s + 1), xrB, brB);
        asm volatile("" ::: "memory");
        slab(s, s, xrA, brA, [] {});
      }
    }
  } else {
    // which slabs before the last can be left out (bit s of `live`; wave-uniform, every wave evaluates all of them)
    uint64_t live = nslab >= 64 ? ~0ull : ((1ull << nslab) - 1);
    if (elide) {
      float bmax = 0.0f;
      for (int n = lane; n < NT; n += 64) bmax = fmaxf(bmax, fabsf(binv_s[n]));
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) bmax = fmaxf(bmax, __shfl_xor(bmax, o));
      live = 1ull << (nslab - 1);
      for (int i = 0; i < nslab - 1; ++i) {
        const int sidx = nslab - 2 - i, k = 64 * sidx + lane;
        float rm = rmv[i & 3];
        if (i >= 4) rm = p.rowmax[((int64_t)b * p.seqlen + (int64_t)c * Q + min(k, limit - 1)) * p.G + g];
        // not provably zero (NaN / Inf in B keep the slab); magnitudes, so that a negative gate (dt_min < 0 without
        // softplus) or a negative gate scale cannot make the bound negative
        const bool keep = !((fabsf(gate_s[k]) * rm) * bmax < 0.499f);
        if (__ballot(keep)) live |= 1ull << sidx;
      }
    }
    int cur = nslab - 1;
    for (int it = 0; cur >= 0; ++it) {
      const uint64_t below = live & ((1ull << cur) - 1);
      const int next = below ? 63 - __builtin_clzll(below) : -1;
      slab(cur, it, xrA, brA, [&] { if (next >= 0) load_slab(64 * next, xrA, brA); });
      cur = next;
    }
  }

  // ---- epilogue: lane holds N = n0 + 16q + 4kg + {0..3} of P row p0 + 16*wave + rl
  const float ratio = req_s[16 * wave + rl];  // key side: x_scale / S_out; value side: (alpha / S_out) * bscale
  const float req = ratio;
  int8_t* sp = p.states + (int64_t)b * p.sst_b + ((((int64_t)c * p.nheads + h) * p.P + pr) * p.N + n0);
  uint32_t dq[NT / 16];  // dword q of this lane: codes of N = n0 + 16 q + 4 kg + {0..3}
#pragma unroll
  for (int q = 0; q < NT / 16; ++q) {
    uint32_t cd[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float a = (float)acc[q][r];
      if (KEYSIDE) {
        float y = a * bdeq_s[16 * q + 4 * kg + r];
        y = y * ratio;
        cd[r] = rint_code(y);
      } else {
        cd[r] = (uint32_t)lq_q_rha(a * req, 127);
      }
    }
    dq[q] = pack_low_bytes(cd[0], cd[1], cd[2], cd[3]);
  }
  // The four lanes kg = 0..3 of one P row hold the four dwords of every 16-byte piece q of the row.  A 4 x 4 transpose
  // between register index and lane group (two row-swap instructions per register pair) leaves lane kg with the whole
  // piece q = 4 i + kg, stored as 16 bytes: a fourth of the store instructions, 64 contiguous bytes per row and store.
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) {
    uint32_t r0 = dq[4 * i], r1 = dq[4 * i + 1], r2 = dq[4 * i + 2], r3 = dq[4 * i + 3];
    lq_v2u t;
    t = __builtin_amdgcn_permlane32_swap(r0, r2, false, false), r0 = t[0], r2 = t[1];
    t = __builtin_amdgcn_permlane32_swap(r1, r3, false, false), r1 = t[0], r3 = t[1];
    t = __builtin_amdgcn_permlane16_swap(r0, r1, false, false), r0 = t[0], r1 = t[1];
    t = __builtin_amdgcn_permlane16_swap(r2, r3, false, false), r2 = t[0], r3 = t[1];
    *(lq_v4i*)(sp + 16 * (4 * i + kg)) = lq_v4i{(int)r0, (int)r1, (int)r2, (int)r3};
  }
}

// max_n |B[b, l, g, n]| of the fp16 key tensor -> (B, L, G) fp32; N / 8 lanes per row, 16 bytes per lane
template <int N>
__global__ __launch_bounds__(256) void row_absmax_kernel(const _Float16* __restrict__ B, int64_t s_b, int64_t s_l, int64_t s_g,
                                                         float* __restrict__ out, int L, int G, int64_t rows) {
  constexpr int LPR = N / 8, RPB = 256 / LPR;
  const int sub = threadIdx.x % LPR;
  const int64_t row = min((int64_t)blockIdx.x * RPB + threadIdx.x / LPR, rows - 1);  // the tail repeats the last row
  const int g = (int)(row % G);
  const int64_t bl = row / G;
  const int64_t bb = bl / L, l = bl % L;
  const lq_v8h v = *(const lq_v8h*)(B + bb * s_b + l * s_l + (int64_t)g * s_g + 8 * sub);
  float m = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float a = __builtin_fabsf((float)v[e]);
    m = (a > m || a != a) ? a : m;  // NaN propagates, so a row holding one is never elided
  }
#pragma unroll
  for (int o = 1; o < LPR; o <<= 1) {
    const float t = __shfl_xor(m, o);
    m = (t > m || t != t) ? t : m;
  }
  if (sub == 0) out[row] = m;
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

template <bool KEYSIDE>
int launch(const Params& p, hipStream_t stream) {
  if (p.batch <= 0 || p.seqlen <= 0 || p.nheads <= 0 || p.G <= 0 || p.nheads % p.G != 0) return LQ_ERR_SHAPE;
  if (p.P % 64 != 0 || p.N % 64 != 0 || p.Q % 64 != 0 || p.Q < 64 || p.Q > 4096) return LQ_ERR_SHAPE;
  if (p.sx_b % 4 || p.sx_l % 4 || p.sx_h % 4 || !al(p.x, 8)) return LQ_ERR_SHAPE;
  const int bmod = KEYSIDE ? 8 : 8, balign = KEYSIDE ? 16 : 8;
  if (p.sB_b % bmod || p.sB_l % bmod || p.sB_g % bmod || !al(p.B, balign)) return LQ_ERR_SHAPE;
  if (!al(p.states, 16)) return LQ_ERR_SHAPE;
  if (p.nchunks > 65535 || p.nheads > 65535) return LQ_ERR_SHAPE;
  auto magic = [](uint32_t d) { return d == 1 ? 0u : (uint32_t)(0x100000000ull / d) + 1u; };
  if (p.sx_l < 0 || p.sB_l < 0 || p.sx_l >= (1 << 22) || p.sB_l >= (1 << 22) || (int64_t)p.Q * p.sx_l >= (1ll << 30) ||
      (int64_t)p.Q * p.sB_l >= (1ll << 30))
    return LQ_ERR_SHAPE;  // 24-bit token * stride products in the slab loads
  Params q = p;
  if (q.sst_b == 0) q.sst_b = (int64_t)p.nchunks * p.nheads * p.P * p.N;
  if (q.sst_b % 16 != 0) return LQ_ERR_SHAPE;
  if (KEYSIDE && p.rowmax) {
    if (p.rowmax_ready) {
      // nothing to do: the caller's table is used as it is
    } else if (p.N != 64 && p.N != 128 && p.N != 256) {
      q.rowmax = nullptr;  // no pre-pass for this width: every slab is processed
    } else {
      const int64_t rows = (int64_t)p.batch * p.seqlen * p.G;
      const int rpb = 256 / (p.N / 8);
      const dim3 rgrid((unsigned)((rows + rpb - 1) / rpb));
      float* out = const_cast<float*>(p.rowmax);
      const _Float16* Bp = (const _Float16*)p.B;
      if (p.N == 64)
        hipLaunchKernelGGL((row_absmax_kernel<64>), rgrid, dim3(256), 0, stream, Bp, p.sB_b, p.sB_l, p.sB_g, out, p.seqlen, p.G, rows);
      else if (p.N == 128)
        hipLaunchKernelGGL((row_absmax_kernel<128>), rgrid, dim3(256), 0, stream, Bp, p.sB_b, p.sB_l, p.sB_g, out, p.seqlen, p.G, rows);
      else
        hipLaunchKernelGGL((row_absmax_kernel<256>), rgrid, dim3(256), 0, stream, Bp, p.sB_b, p.sB_l, p.sB_g, out, p.seqlen, p.G, rows);
    }
  }
  if (p.N % 128 == 0) {
    q.n_ntiles = p.N / 128;
    const size_t lds = (size_t)p.Q * 4 + (2 * 128 + 128) * 4 + (2 * 16 * kXW + 2 * 16 * (128 + kPad)) * 4;
    const int tiles = (p.P / 64) * q.n_ntiles;
    if ((int64_t)p.batch * tiles > 65535) return LQ_ERR_SHAPE;
    q.hpg_magic = magic((uint32_t)(p.nheads / p.G)), q.tiles_magic = magic((uint32_t)tiles), q.nt_magic = magic((uint32_t)q.n_ntiles);
    dim3 grid(p.nchunks, p.nheads, p.batch * tiles);
    if (!KEYSIDE && p.Q == 256)
      hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 128, 4>), grid, dim3(256), lds, stream, q);
    else if (!KEYSIDE && p.Q == 128)
      hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 128, 2>), grid, dim3(256), lds, stream, q);
    else
      hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 128, 0>), grid, dim3(256), lds, stream, q);
  } else {
    q.n_ntiles = p.N / 64;
    const size_t lds = (size_t)p.Q * 4 + (2 * 64 + 128) * 4 + (2 * 16 * kXW + 2 * 16 * (64 + kPad)) * 4;
    const int tiles = (p.P / 64) * q.n_ntiles;
    if ((int64_t)p.batch * tiles > 65535) return LQ_ERR_SHAPE;
    q.hpg_magic = magic((uint32_t)(p.nheads / p.G)), q.tiles_magic = magic((uint32_t)tiles), q.nt_magic = magic((uint32_t)q.n_ntiles);
    dim3 grid(p.nchunks, p.nheads, p.batch * tiles);
    if (!KEYSIDE && p.Q == 256)
      hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 64, 4>), grid, dim3(256), lds, stream, q);
    else if (!KEYSIDE && p.Q == 128)
      hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 64, 2>), grid, dim3(256), lds, stream, q);
    else
      hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 64, 0>), grid, dim3(256), lds, stream, q);
  }
  return lq_check_launch();
}

}  // namespace

extern "C" int lq_chunk_state_value(const lq_chunk_state_value_args* a, hipStream_t stream) {
  if (!a || !a->x || !a->B || !a->dt || !a->dA_cumsum || !a->alpha_hp || !a->bscale_g || !a->out_qscale || !a->states)
    return LQ_ERR_NULL;
  Params p = {};
  p.x = (const _Float16*)a->x;
  p.sx_b = a->x_stride_b, p.sx_l = a->x_stride_l, p.sx_h = a->x_stride_h;
  p.B = a->B;
  p.sB_b = a->B_stride_b, p.sB_l = a->B_stride_l, p.sB_g = a->B_stride_g;
  p.dt = a->dt, p.dA = a->dA_cumsum;
  p.xs = a->alpha_hp, p.sxs_h = a->alpha_stride_h, p.sxs_p = a->alpha_stride_p;
  p.bscale_g = a->bscale_g, p.sbs_g = a->bscale_stride_g;
  p.oqs = a->out_qscale, p.soq_h = a->oqs_stride_h, p.soq_p = a->oqs_stride_p;
  p.states = a->states, p.sst_b = a->states_stride_b;
  p.batch = a->batch, p.seqlen = a->seqlen, p.nheads = a->nheads, p.P = a->headdim, p.G = a->ngroups, p.N = a->dstate;
  p.Q = a->chunk_size;
  if (p.Q <= 0) return LQ_ERR_SHAPE;
  p.nchunks = (p.seqlen + p.Q - 1) / p.Q;
  return launch<false>(p, stream);
}

extern "C" int lq_chunk_state_key(const lq_chunk_state_key_args* a, hipStream_t stream) {
  if (!a || !a->x || !a->B || !a->dt || !a->dA_cumsum || !a->x_scale_hp || !a->out_qscale || !a->b_gate_scale || !a->states)
    return LQ_ERR_NULL;
  Params p = {};
  p.x = (const _Float16*)a->x;
  p.sx_b = a->x_stride_b, p.sx_l = a->x_stride_l, p.sx_h = a->x_stride_h;
  p.B = a->B;
  p.sB_b = a->B_stride_b, p.sB_l = a->B_stride_l, p.sB_g = a->B_stride_g;
  p.dt = a->dt, p.dA = a->dA_cumsum;
  p.xs = a->x_scale_hp, p.sxs_h = a->xs_stride_h, p.sxs_p = a->xs_stride_p;
  p.oqs = a->out_qscale, p.soq_h = a->oqs_stride_h, p.soq_p = a->oqs_stride_p;
  p.bgs = a->b_gate_scale;
  p.rowmax = a->b_rowmax;
  p.rowmax_ready = a->b_rowmax_ready;
  if (p.rowmax_ready != 0 && p.rowmax_ready != 1) return LQ_ERR_SHAPE;
  p.sbg_b = a->bgs_stride_b, p.sbg_c = a->bgs_stride_c, p.sbg_h = a->bgs_stride_h, p.sbg_n = a->bgs_stride_n;
  p.states = a->states, p.sst_b = a->states_stride_b;
  p.batch = a->batch, p.seqlen = a->seqlen, p.nheads = a->nheads, p.P = a->headdim, p.G = a->ngroups, p.N = a->dstate;
  p.Q = a->chunk_size;
  if (p.Q <= 0) return LQ_ERR_SHAPE;
  p.nchunks = (p.seqlen + p.Q - 1) / p.Q;
  return launch<true>(p, stream);
}
