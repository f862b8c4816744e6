// Canonical-storage variants of the zoo state and output kernels (value rotation R_V with in-kernel un-rotation).
// Replaces _state_kernel_unrot / _output_kernel_unrot (linquant/kernels/zoo/simple_gla.py:86-95, 165-172 with
// USE_UNROT in _state_body :67-70 and _output_body :147-150), _gla_state_kernel_unrot / _gla_output_kernel_unrot
// (gla.py), _delta_state_kernel_unrot (gated_delta_rule.py:60-63, 93-95, 107-109) and _kda_state_kernel_unrot (kda.py):
// v (or U) arrives in the rotated value basis, the carried and stored state stay canonical.
//   state:  h += fp16(dequantized write product) . Ru                 Ru = R_V^T, (V,V) fp16
//           delta family: the dequantized state read is rotated first, ws = fp16(ws) . Ru^T, so E stays rotated
//   output: o = state read (canonical) + fp16(local product * svl) . Ru
// One workgroup spans all V value channels (V = 64 or 128).  Every product is computed transposed (value channel
// on the accumulator rows): a lane then holds, for one token or one key channel, the value channels
// 16*vt + 4*(lane >> 4) + r, which is exactly a B operand of the fp16 rotation product when the rotation matrix
// rows are read with the matching channel -> slot map.  Nothing is transposed through LDS except the INT8 codes.
#include "zoo_params.h"
#include "../../include/linquant_hip.h"

namespace {

// out[v'][c] = sum_v Rs[v'][v] * x[v][c] for one 16-column tile c: x arrives as accumulator fragments
// d[vt][r] (rows v = 16vt + 4kg + r); slot e of step sg is channel 16*(2sg + (e >> 2)) + 4kg + (e & 3).
// VO output rows v' (the rows Rs holds): all V of them, or the slice a workgroup owns.
template <int V, int VO = V>
LQ_DEV void rotate_tile(const _Float16* Rs, const float (&d)[V / 16][4], lq_v4f (&out)[VO / 16], int rl, int kg) {
  constexpr int RS = V + 8;
  lq_v8h bop[V / 32];
#pragma unroll
  for (int sg = 0; sg < V / 32; ++sg)
#pragma unroll
    for (int e = 0; e < 8; ++e) bop[sg][e] = (_Float16)d[2 * sg + (e >> 2)][e & 3];
#pragma unroll
  for (int vt = 0; vt < VO / 16; ++vt) {
    lq_v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sg = 0; sg < V / 32; ++sg) {
      const lq_v4h a0 = *(const lq_v4h*)(Rs + (16 * vt + rl) * RS + 32 * sg + 4 * kg);
      const lq_v4h a1 = *(const lq_v4h*)(Rs + (16 * vt + rl) * RS + 32 * sg + 16 + 4 * kg);
      lq_v8h aop;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        aop[e] = a0[e];
        aop[4 + e] = a1[e];
      }
      acc = lq_mfma_f16(aop, bop[sg], acc);
    }
    out[vt] = acc;
  }
}

// Rs[m][n] = R[n][m0 + m] (transposed copy, lanes walk m) or Rs[m][n] = R[m][n]; VO rows m (a slice starting at row m0
// in the transposed form)
template <int V, bool TRANSPOSE, int VO = V, int NTHR = 256>
LQ_DEV void stage_rotation(_Float16* Rs, const _Float16* R, int tid, int m0 = 0) {
  constexpr int RS = V + 8;
  for (int it = tid; it < VO * (V / 8); it += NTHR) {
    if (TRANSPOSE) {
      const int m = it % VO, n8 = it / VO;
      lq_v8h rv;
#pragma unroll
      for (int e = 0; e < 8; ++e) rv[e] = R[(8 * n8 + e) * V + m0 + m];
      *(lq_v8h*)(Rs + m * RS + 8 * n8) = rv;
    } else {
      const int m = it / (V / 8), n8 = it % (V / 8);
      *(lq_v8h*)(Rs + m * RS + 8 * n8) = *(const lq_v8h*)(R + m * V + 8 * n8);
    }
  }
}

template <bool DELTA, int K, int V>
struct UStepOps {
  lq_v4i kop[K / 64];
  float gam[K / 64];
  lq_v4i vop[DELTA ? 1 : V / 16];
  lq_v4i wop[DELTA ? K / 64 : 1];
  lq_v2i u[DELTA ? V / 16 : 1];
  float fw, ev;
};

// KP: workgroups per (batch, head) along K.  The key rows of the linear family are independent recurrences, so a
// workgroup may own K / KP of them (the delta family reads the whole state per step: KP = 1).
// VS: workgroups per (batch, head, key part) along the canonical value axis, linear family only.  The un-rotation mixes
// all rotated value channels into every canonical one, but the canonical channels are independent of each other: a
// workgroup forms the whole rotated product of its key rows (eight INT8 products, repeated by its VS - 1 siblings) and
// un-rotates it into its own V / VS canonical columns only, which is where the step's time goes (a quarter of the fp16
// products and of the carry at VS = 4).  The delta family rotates the state read back into the basis of U, which needs
// every canonical column: VS = 1.
// NW: wavefronts per workgroup, 4 or 8.  Each owns KW / NW key rows of the carry.  The state read and E are per token
// tile (four of them per chunk): with eight waves, two share a token tile, both form its whole state read (the rotation
// back into the basis of U contracts over all canonical channels) and each rotates it into, and finishes E for, one half
// of the value channels.  The delta family's single workgroup per (batch, head) runs one dependent chain of chunk steps,
// so halving what a wave does per step is what shortens it.
// PAIR: 128-token chunks walked as two 64-token halves: the state is quantized and stored at the first half only (both
// halves of the delta family read that copy), the INT8 write product of the first half stays in the accumulators the second
// half's product adds to, and the sum over the 128 tokens is dequantized, un-rotated and added to the carry once.
template <bool DELTA, int K, int V, int KP, int VS = 1, int NW = 4, bool PAIR = false>
__global__ __launch_bounds__(NW * 64) void zoo_state_unrot_kernel(ZooStateParams p) {
  static_assert(KP == 1 || !DELTA, "the delta family needs all of K in one workgroup");
  static_assert(VS == 1 || !DELTA, "the delta family needs all of V in one workgroup");
  static_assert(NW == 4 || (NW == 8 && DELTA), "eight waves: delta family only");
  constexpr int NTHR = NW * 64;
  constexpr int VH = NW / 4;               // waves per token tile = parts of the value axis of E
  constexpr int VE = V / VH, VET = VE / 16;  // value channels (and tiles) of E one wave finishes
  constexpr int KW = K / KP, KR = KW / NW, KT = KR / 16, VT = V / 16;
  constexpr int VO = V / VS, VOT = VO / 16;  // canonical value channels (and 16-row tiles of them) of this workgroup
  static_assert(KT >= 1, "a wave owns at least one 16-row tile");
  static_assert(VOT >= 1, "a workgroup owns at least one 16-channel tile");
  constexpr int HS = KW + 16, ES = 64 + 16, RS = V + 8;
  __shared__ __align__(16) unsigned char hT[VO * HS];
  __shared__ __align__(16) unsigned char eT[DELTA ? V * ES : 16];
  __shared__ __align__(16) _Float16 RuT_s[VO * RS];         // RuT_s[v'][v] = Ru[v][v0 + v']: x . Ru
  __shared__ __align__(16) _Float16 Ru_s[DELTA ? V * RS : 8];  // Ru_s[v'][v] = Ru[v'][v]: x . Ru^T
  __shared__ __align__(16) float ss_s[V], inv_ss_s[V], svw_s[V], inv_svw_s[V];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tt = wave & 3;                 // token tile of the state read / E
  const int ve0 = (wave >> 2) * VE;        // first value channel of the part of E this wave finishes
  const int rl = lane & 15, kg = lane >> 4;
  const int b = blockIdx.x / p.H, h = blockIdx.x % p.H;
  const int kb = blockIdx.y * KW;  // first key row of this workgroup
  const int v0 = VS == 1 ? 0 : (int)blockIdx.z * VO;  // first canonical value channel of this workgroup
  const int H = p.H, T = p.T, NT = p.NT;
  const int qmax = p.qmax;
  const bool bf = p.bf != 0;

  stage_rotation<V, true, VO, NTHR>(RuT_s, p.unrot, tid, v0);
  if (DELTA) stage_rotation<V, false, V, NTHR>(Ru_s, p.unrot, tid);
  if (tid < V) {
    const float s = p.ss[h * V + tid], w = p.svw[h * V + tid];
    ss_s[tid] = s, inv_ss_s[tid] = 1.0f / s, svw_s[tid] = w, inv_svw_s[tid] = 1.0f / w;
  }
  float skw_c[KT];
#pragma unroll
  for (int kt = 0; kt < KT; ++kt) skw_c[kt] = p.skw[h * K + kb + KR * wave + 16 * kt + rl];
  const float sw = DELTA ? p.sw[h] : 0.0f;

  auto load_step = [&](int ct, UStepOps<DELTA, K, V>& o) {
    const int64_t cb = ((int64_t)b * NT + ct) * H + h;
    const int64_t t0 = (int64_t)b * T + (int64_t)ct * 64;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      o.kop[kt] = *(const lq_v4i*)(p.kqT + (cb * K + kb + KR * wave + 16 * kt + rl) * 64 + 16 * kg);
      o.gam[kt] = p.gam[cb * K + kb + KR * wave + 16 * kt + rl];
    }
    if constexpr (!DELTA) {
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) o.vop[vt] = *(const lq_v4i*)(p.vqT + (cb * V + 16 * vt + rl) * 64 + 16 * kg);
    } else {
      const int64_t tr = (t0 + 16 * tt + rl) * H + h;
#pragma unroll
      for (int ks = 0; ks < K / 64; ++ks) o.wop[ks] = *(const lq_v4i*)(p.wq + tr * K + 64 * ks + 16 * kg);
#pragma unroll
      for (int vt = 0; vt < VET; ++vt) o.u[vt] = *(const lq_v2i*)(p.u + tr * V + ve0 + 16 * vt + 4 * kg);
      o.fw = p.fw[tr];
      o.ev = p.ev[tr];
    }
  };

  // carry, transposed: rows v = v0 + 16vt + 4kg + r, column k = KR*wave + 16kt + rl
  float hc[VOT][KT][4];
#pragma unroll
  for (int vt = 0; vt < VOT; ++vt)
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int r = 0; r < 4; ++r) hc[vt][kt][r] = 0.0f;

  UStepOps<DELTA, K, V> cur, nxt;
  load_step(0, cur);
  nxt = cur;
  __syncthreads();

  lq_v4i pend[PAIR ? KT : 1][PAIR ? VT : 1];  // PAIR: the first half's write product
  for (int ct = 0; ct < NT; ++ct) {
    const int64_t t0 = (int64_t)b * T + (int64_t)ct * 64;
    const bool second = PAIR && (ct & 1);  // wave-uniform
    // the next step's operands are requested first and without a condition (the last step asks for its own again): a
    // request inside a branch is waited for where the paths join, in front of the products below
    load_step(min(ct + 1, NT - 1), nxt);
    // ---- stored copy of the incoming state -> LDS (V-major), one byte per (v, k)
    if (!second) {
#pragma unroll
      for (int vt = 0; vt < VOT; ++vt) {
        const lq_v4f is4 = *(const lq_v4f*)(inv_ss_s + v0 + 16 * vt + 4 * kg);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            hT[(16 * vt + 4 * kg + r) * HS + KR * wave + 16 * kt + rl] = (unsigned char)zoo_q8(hc[vt][kt][r], is4[r], 127);
      }
    }
    __syncthreads();
    if (!second) {
      int8_t* dst = p.h_i8 + ((((int64_t)b * (PAIR ? NT >> 1 : NT) + (PAIR ? ct >> 1 : ct)) * H + h) * V + v0) * K + kb;
      constexpr int SEG = KW / 16;
      for (int it = tid; it < VO * SEG; it += NTHR) {
        const int vr = it / SEG, sg = it % SEG;
        *(lq_v4i*)(dst + vr * K + sg * 16) = *(const lq_v4i*)(hT + vr * HS + sg * 16);
      }
    }

    if constexpr (DELTA) {
      // ---- state read (transposed: rows v, columns = the wave's 16 tokens), rotated into the value basis of U
      float ws[VT][4];
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        lq_v4i acc = {0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < K / 64; ++ks)
          acc = lq_mfma_i8(*(const lq_v4i*)(hT + (16 * vt + rl) * HS + 64 * ks + 16 * kg), cur.wop[ks], acc);
        const lq_v4f s4 = *(const lq_v4f*)(ss_s + 16 * vt + 4 * kg);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float x = (float)acc[r] * sw;
          ws[vt][r] = x * s4[r];
        }
      }
      lq_v4f wsr[VET];
      rotate_tile<V, VE>(Ru_s + ve0 * RS, ws, wsr, rl, kg);
      const int64_t eoff = ((t0 + 16 * tt + rl) * H + h) * V + ve0;
#pragma unroll
      for (int vt = 0; vt < VET; ++vt) {
        const lq_v4f iw4 = *(const lq_v4f*)(inv_svw_s + ve0 + 16 * vt + 4 * kg);
        float ef[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float u = zoo_dec1(((uint32_t)cur.u[vt][r >> 1] >> (16 * (r & 1))) & 0xffffu, bf);
          ef[r] = (u - wsr[vt][r]) * cur.fw;
          eT[(ve0 + 16 * vt + 4 * kg + r) * ES + 16 * tt + rl] = (unsigned char)zoo_q8(ef[r] * cur.ev, iw4[r], qmax);
        }
        lq_v2i eo;
        eo[0] = (int)zoo_enc2(ef[0], ef[1], bf);
        eo[1] = (int)zoo_enc2(ef[2], ef[3], bf);
        *(lq_v2i*)(p.e_out + eoff + 16 * vt + 4 * kg) = eo;
      }
      __syncthreads();
    }

    // ---- write product (transposed), dequantized, un-rotated, added to the canonical carry
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      float d[VT][4];
      if constexpr (PAIR) {
        if (!second) {  // first half: the product waits for the second half's
#pragma unroll
          for (int vt = 0; vt < VT; ++vt) {
            lq_v4i aop;
            if constexpr (DELTA)
              aop = *(const lq_v4i*)(eT + (16 * vt + rl) * ES + 16 * kg);
            else
              aop = cur.vop[vt];
            pend[kt][vt] = lq_mfma_i8(aop, cur.kop[kt], lq_v4i{0, 0, 0, 0});
          }
          continue;
        }
      }
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        lq_v4i aop;
        if constexpr (DELTA)
          aop = *(const lq_v4i*)(eT + (16 * vt + rl) * ES + 16 * kg);
        else
          aop = cur.vop[vt];
        const lq_v4i a = lq_mfma_i8(aop, cur.kop[kt], PAIR ? pend[kt][vt] : lq_v4i{0, 0, 0, 0});
        const lq_v4f w4 = *(const lq_v4f*)(svw_s + 16 * vt + 4 * kg);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float x = (float)a[r] * skw_c[kt];
          d[vt][r] = x * w4[r];
        }
      }
      lq_v4f rot[VOT];
      rotate_tile<V, VO>(RuT_s, d, rot, rl, kg);
#pragma unroll
      for (int vt = 0; vt < VOT; ++vt)
#pragma unroll
        for (int r = 0; r < 4; ++r) hc[vt][kt][r] = hc[vt][kt][r] * cur.gam[kt] + rot[vt][r];
    }
    cur = nxt;
  }

  if (p.ht) {
#pragma unroll
    for (int vt = 0; vt < VOT; ++vt)
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
        *(lq_v4f*)(p.ht + (((int64_t)b * H + h) * K + kb + KR * wave + 16 * kt + rl) * V + v0 + 16 * vt + 4 * kg) =
            lq_v4f{hc[vt][kt][0], hc[vt][kt][1], hc[vt][kt][2], hc[vt][kt][3]};
  }
}

constexpr int kAS = 72;  // halves per row of the fp16 A tile in LDS

template <bool GLA, bool USE_G, int K, int V>
__global__ __launch_bounds__(256, 2) void zoo_output_unrot_kernel(ZooOutParams p) {
  constexpr int QS = K + 16, VT = V / 16, RS = V + 8, VW = V + 4;
  __shared__ __align__(16) unsigned char qc[GLA ? 16 : 64 * QS];
  __shared__ __align__(16) unsigned char kc[GLA ? 16 : 64 * QS];
  __shared__ __align__(16) _Float16 Afl[GLA ? 8 : 64 * kAS];
  __shared__ __align__(16) uint32_t vP[32 * VW];
  __shared__ __align__(16) _Float16 RuT_s[V * RS];
  __shared__ __align__(16) float g_s[64], ss_s[V], svl_s[V];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  const int ct = blockIdx.x;
  const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
  const int H = p.H;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)ct * 64;
  const float sq = p.sq[h];
  const float inv_sq = 1.0f / sq;
  const float sk = GLA ? 1.0f : p.sk[h];
  const float inv_sk = 1.0f / sk;
  const int qmax = p.qmax;
  const bool bf = p.bf != 0;

  // state-read operands (and the stored query codes) are requested first: they are not needed before phase 2 and
  // arrive while phase 1 stages the codes
  // (128-token chunks: one stored state per chunk, read by both halves)
  const int8_t* hp = p.h_i8 + (((int64_t)b * (p.NT / p.S) + ct / p.S) * H + h) * V * K;
  lq_v4i hop[K / 64][VT];
  lq_v4i qgop[GLA ? K / 64 : 1];
#pragma unroll
  for (int ks = 0; ks < K / 64; ++ks) {
    if constexpr (GLA) qgop[ks] = *(const lq_v4i*)(p.qg + ((t0 + 16 * wave + rl) * H + h) * K + 64 * ks + 16 * kg);
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) hop[ks][vt] = *(const lq_v4i*)(hp + (16 * vt + rl) * K + 64 * ks + 16 * kg);
  }

  // ---- phase 1: codes and tables -> LDS
  stage_rotation<V, true>(RuT_s, p.unrot, tid);
  if (tid < V) ss_s[tid] = p.ss[h * V + tid], svl_s[tid] = p.svl[h * V + tid];
  if (!GLA)
  for (int it = tid; it < 64 * (K / 8); it += 256) {
    const int t = it / (K / 8), c8 = it % (K / 8);
    const int64_t off = ((t0 + t) * H + h) * K + 8 * c8;
    float qv[8];
    zoo_ld8(p.q + off, bf, qv);
    int cq[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) cq[e] = zoo_q8(qv[e] * p.scale, inv_sq, qmax);
    lq_v2i o;
    o[0] = (int)zoo_pack_codes(cq[0], cq[1], cq[2], cq[3]);
    o[1] = (int)zoo_pack_codes(cq[4], cq[5], cq[6], cq[7]);
    *(lq_v2i*)(qc + t * QS + 8 * c8) = o;
    {
      float kv[8];
      zoo_ld8(p.k + off, bf, kv);
      int ck[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) ck[e] = zoo_q8(kv[e], inv_sk, qmax);
      o[0] = (int)zoo_pack_codes(ck[0], ck[1], ck[2], ck[3]);
      o[1] = (int)zoo_pack_codes(ck[4], ck[5], ck[6], ck[7]);
      *(lq_v2i*)(kc + t * QS + 8 * c8) = o;
    }
  }
  for (int it = tid; it < 32 * (V / 8); it += 256) {
    const int tp = it / (V / 8), c8 = it % (V / 8);  // token pair, group of 8 value channels
    const int64_t off = ((t0 + 2 * tp) * H + h) * V + 8 * c8;
    float va[8];
    zoo_ld8(p.v + off, bf, va);
    float vb[8];
    zoo_ld8(p.v + off + (int64_t)H * V, bf, vb);
    const lq_v4f s0 = *(const lq_v4f*)(p.svl + h * V + 8 * c8), s1 = *(const lq_v4f*)(p.svl + h * V + 8 * c8 + 4);
    lq_v4i o0, o1;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float inv = 1.0f / (e < 4 ? s0[e & 3] : s1[e & 3]);
      const int w = (int)zoo_pack_h2((float)zoo_q8(va[e], inv, qmax), (float)zoo_q8(vb[e], inv, qmax));
      if (e < 4) o0[e] = w; else o1[e - 4] = w;
    }
    *(lq_v4i*)(vP + tp * VW + 8 * c8) = o0;
    *(lq_v4i*)(vP + tp * VW + 8 * c8 + 4) = o1;
  }
  if (USE_G && !GLA && tid < 64) g_s[tid] = p.g[(t0 + tid) * H + h];
  __syncthreads();

  // ---- phase 2: INT8 contractions of this wave's 16 tokens (state read transposed: rows v, columns tokens)
  lq_v4i o32[VT];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) o32[vt] = lq_v4i{0, 0, 0, 0};
  lq_v4i a32[4];
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) a32[jt] = lq_v4i{0, 0, 0, 0};
#pragma unroll
  for (int ks = 0; ks < K / 64; ++ks) {
    lq_v4i qop;
    if constexpr (GLA)
      qop = qgop[ks];
    else
      qop = *(const lq_v4i*)(qc + (16 * wave + rl) * QS + 64 * ks + 16 * kg);
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) o32[vt] = lq_mfma_i8(hop[ks][vt], qop, o32[vt]);
    if (!GLA) {
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
        if (jt > wave) continue;
        const lq_v4i kop = *(const lq_v4i*)(kc + (16 * jt + rl) * QS + 64 * ks + 16 * kg);
        a32[jt] = lq_mfma_i8(qop, kop, a32[jt]);
      }
    }
  }

  // ---- phase 3: A -> fp16 in operand layout
  if (!GLA) {
    const float sqk = sq * sk;
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) {
      if (jt > wave + 1) continue;
      const int j = 16 * jt + rl;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * wave + 4 * kg + r;
        float x = 0.0f;
        if (jt <= wave && j <= i) {
          x = (float)a32[jt][r] * sqk;
          if (USE_G) x = x * zoo_exp(g_s[i] - g_s[j]);
        }
        Afl[i * kAS + j] = (_Float16)x;
      }
    }
    __syncthreads();
  }

  // ---- phase 4: local product (transposed), scaled, un-rotated; output = state read + rotated local product
  float d[VT][4];
  {
    lq_v4f loc[VT];
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) loc[vt] = lq_v4f{0.f, 0.f, 0.f, 0.f};
    if (p.cross && (ct % p.S) != 0) {
      // second half of a 128-token chunk: the local product with the first half's tokens, left by the cross launch of the
      // rotated-storage output kernel (the local product is in the rotated basis either way); lane (rl = token, kg) holds
      // channels 16vt + 4kg + r
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) loc[vt] = *(const lq_v4f*)(p.cross + ((t0 + 16 * wave + rl) * H + h) * V + 16 * vt + 4 * kg);
    }
    const int nslab = (16 * wave + 15) / 32 + 1;
    for (int js = 0; js < nslab; ++js) {
      lq_v8h aop;
      if (GLA) {
        aop = *(const lq_v8h*)(p.A + ((t0 + 16 * wave + rl) * H + h) * 64 + 32 * js + 8 * kg);
      } else {
        aop = *(const lq_v8h*)(Afl + (16 * wave + rl) * kAS + 32 * js + 8 * kg);
      }
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        lq_v4i vv;
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) vv[dd] = (int)vP[(16 * js + 4 * kg + dd) * VW + 16 * vt + rl];
        loc[vt] = lq_mfma_f16(__builtin_bit_cast(lq_v8h, vv), aop, loc[vt]);
      }
    }
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) {
      const lq_v4f s4 = *(const lq_v4f*)(svl_s + 16 * vt + 4 * kg);
#pragma unroll
      for (int r = 0; r < 4; ++r) d[vt][r] = loc[vt][r] * s4[r];
    }
  }
  lq_v4f rot[VT];
  rotate_tile<V>(RuT_s, d, rot, rl, kg);
  const float eg = (USE_G && !GLA) ? zoo_exp(g_s[16 * wave + rl]) : 1.0f;
  const int64_t ooff = ((t0 + 16 * wave + rl) * H + h) * V;
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) {
    const lq_v4f s4 = *(const lq_v4f*)(ss_s + 16 * vt + 4 * kg);
    float res[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = (float)o32[vt][r] * sq;
      x = x * s4[r];
      if (USE_G && !GLA) x = x * eg;
      res[r] = x + rot[vt][r];
    }
    if (p.o_is_f32) {
      *(lq_v4f*)((float*)p.o + ooff + 16 * vt + 4 * kg) = lq_v4f{res[0], res[1], res[2], res[3]};
    } else {
      lq_v2i w;
      w[0] = (int)zoo_enc2(res[0], res[1], bf);
      w[1] = (int)zoo_enc2(res[2], res[3], bf);
      *(lq_v2i*)((_Float16*)p.o + ooff + 16 * vt + 4 * kg) = w;
    }
  }
}

template <bool DELTA, int K, bool PAIR>
int launch_state(const ZooStateParams& p, int batch, hipStream_t stream) {
  constexpr int KP = (!DELTA && K == 128) ? 2 : 1;
  // canonical value slices of 32 (V = 128) or 16 (V = 64) channels; measured at B4 T4096 H16 K = V = 128, no decay: one
  // slice 158 us, two 107, four 101, eight 167 (the rotated product every sibling repeats starts to dominate)
  constexpr int VS = DELTA ? 1 : 4;
  // delta family at K = 128: eight waves, one 16-row key tile each (four waves carry two)
  constexpr int NW = (DELTA && K == 128) ? 8 : 4;
  dim3 grid(batch * p.H, KP, VS);
  if (p.V == 128)
    hipLaunchKernelGGL((zoo_state_unrot_kernel<DELTA, K, 128, KP, VS, NW, PAIR>), grid, dim3(NW * 64), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_state_unrot_kernel<DELTA, K, 64, KP, VS, NW, PAIR>), grid, dim3(NW * 64), 0, stream, p);
  return lq_check_launch();
}

template <bool GLA, bool USE_G, int K>
int launch_output(const ZooOutParams& p, hipStream_t stream) {
  dim3 grid(p.NT, p.B * p.H);
  if (p.V == 128)
    hipLaunchKernelGGL((zoo_output_unrot_kernel<GLA, USE_G, K, 128>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_output_unrot_kernel<GLA, USE_G, K, 64>), grid, dim3(256), 0, stream, p);
  return lq_check_launch();
}

}  // namespace

int zoo_state_unrot_launch(const ZooStateParams& p, bool delta, int K, int batch, bool pair, hipStream_t stream) {
  if (p.V != 64 && p.V != 128) return LQ_ERR_SHAPE;
  if (pair) {
    if (delta) return K == 128 ? launch_state<true, 128, true>(p, batch, stream) : launch_state<true, 64, true>(p, batch, stream);
    return K == 128 ? launch_state<false, 128, true>(p, batch, stream) : launch_state<false, 64, true>(p, batch, stream);
  }
  if (delta) return K == 128 ? launch_state<true, 128, false>(p, batch, stream) : launch_state<true, 64, false>(p, batch, stream);
  return K == 128 ? launch_state<false, 128, false>(p, batch, stream) : launch_state<false, 64, false>(p, batch, stream);
}

int zoo_output_unrot_launch(const ZooOutParams& p, int decay, int K, hipStream_t stream) {
  if (p.V != 64 && p.V != 128) return LQ_ERR_SHAPE;
  if (decay == LQ_DECAY_DIAGONAL)
    return K == 128 ? launch_output<true, true, 128>(p, stream) : launch_output<true, true, 64>(p, stream);
  if (decay == LQ_DECAY_SCALAR)
    return K == 128 ? launch_output<false, true, 128>(p, stream) : launch_output<false, true, 64>(p, stream);
  return K == 128 ? launch_output<false, false, 128>(p, stream) : launch_output<false, false, 64>(p, stream);
}
