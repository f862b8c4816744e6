// Zoo state kernels: sequential chunk loop with an fp32 carry and an INT8 stored copy per chunk.
// Replaces _state_body (linquant/kernels/zoo/simple_gla.py:23-75), _gla_state_body (gla.py:102-148),
// _delta_state_body (gated_delta_rule.py:50-115) and _kda_state_body (kda.py:68-130).
//
// Per chunk, in the reference's order:
//   1. hq = q8(h, 1/ss, 127) is stored: the state entering the chunk (read by the output kernel and, delta
//      family, by this chunk's state read);
//   2. delta family: ws = (q8(W) . hq) * sw * ss[v];  E = (U - ws) * fw[t], stored fp16 (pre-decay);
//   3. decay split: key operand *= exp((1-eta) d) (scalar) or exp(gk_last - gk - eta*le) (diagonal),
//      value operand *= exp(eta d) or exp(eta*le);  h *= exp(g_last);
//   4. h += (q8(key)^T . q8(value)) * skw[k] * svw[v].
//
// One 4-wave workgroup per (64-column V tile, batch*head) holding the whole K axis (the delta state read
// needs the full contraction).  The carry lives in registers: wave w owns K/4 rows.  All operands of the
// two INT8 contractions are quantized exactly once per chunk; the write operands go to LDS as
// [token quad][channel] dwords (4 token codes each), the stored state goes to LDS V-major so that it can be
// copied out coalesced and read back as the K-contiguous operand of the state read.
#include "zoo_common.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int BV = 64;
constexpr int kPad = 4;

struct StateParams {
  const _Float16* k;
  const _Float16* v;
  const _Float16* w;
  const float* fw;
  const float* g;
  const float* logenv;
  int8_t* h_i8;
  _Float16* e_out;
  float* ht;
  const float* skw;
  const float* svw;
  const float* sw;
  const float* ss;
  float eta;
  int qmax;
  int B, T, H, V, NT;
};

template <bool DELTA, int DECAY, int K>
__global__ __launch_bounds__(256) void zoo_state_kernel(StateParams p) {
  constexpr int KR = K / 4;       // carry rows per wave
  constexpr int KT = KR / 16;     // 16-row tiles per wave
  constexpr int VT = BV / 16;     // 16-col tiles
  constexpr int HS = K + 16;      // byte stride of a stored-state row in LDS
  constexpr int KW = K + kPad;    // dword stride of a key-code row
  constexpr int EW = BV + kPad;   // dword stride of a value-code row
  constexpr int CK = K / 16;      // channels per thread in the key quantize phase (16 groups)

  __shared__ __align__(16) unsigned char hT[BV * HS];
  __shared__ __align__(16) uint32_t kb[16 * KW];
  __shared__ __align__(16) uint32_t eb[16 * EW];
  __shared__ float ek_s[64], ev_s[64], fw_s[64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  const int v0 = blockIdx.x * BV;
  const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
  const int H = p.H, V = p.V, T = p.T;
  const float eta = p.eta;
  const int qmax = p.qmax;

  // per-lane scales of the carry tile: rows k = KR*wave + 16kt + 4kg + r, cols v = v0 + 16vt + rl
  float skw_r[KT][4], svw_c[VT], inv_ss_c[VT], ss_c[VT];
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int r = 0; r < 4; ++r) skw_r[kt][r] = p.skw[h * K + KR * wave + 16 * kt + 4 * kg + r];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) {
    svw_c[vt] = p.svw[h * V + v0 + 16 * vt + rl];
    ss_c[vt] = p.ss[h * V + v0 + 16 * vt + rl];
    inv_ss_c[vt] = 1.0f / ss_c[vt];
  }
  // quantize-phase constants: key channels kc0..kc0+CK-1, value channels 4*(tid&15)..+3, token quad tid>>4
  const int tq = tid >> 4, cg = tid & 15;
  float inv_skw_q[CK], inv_svw_q[4];
#pragma unroll
  for (int e = 0; e < CK; ++e) inv_skw_q[e] = 1.0f / p.skw[h * K + CK * cg + e];
#pragma unroll
  for (int e = 0; e < 4; ++e) inv_svw_q[e] = 1.0f / p.svw[h * V + v0 + 4 * cg + e];
  // delta state read: value columns 4*rl + jj of this V tile
  float ss_d[4], inv_ew_d[4], inv_sw = 0.f, sw = 0.f;
  if (DELTA) {
    sw = p.sw[h];
    inv_sw = 1.0f / sw;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      ss_d[jj] = p.ss[h * V + v0 + 4 * rl + jj];
      inv_ew_d[jj] = 1.0f / p.svw[h * V + v0 + 4 * rl + jj];
    }
  }

  float hc[KT][VT][4];
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int r = 0; r < 4; ++r) hc[kt][vt][r] = 0.0f;

  for (int ct = 0; ct < p.NT; ++ct) {
    const int64_t t0 = (int64_t)b * T + (int64_t)ct * 64;  // global token row of the chunk start
    // ---- phase A: stored copy of the incoming state -> LDS (V-major), per-token decay factors
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        int cd[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) cd[r] = zoo_q8(hc[kt][vt][r], inv_ss_c[vt], 127);
        *(uint32_t*)(hT + (16 * vt + rl) * HS + KR * wave + 16 * kt + 4 * kg) = zoo_pack_codes(cd[0], cd[1], cd[2], cd[3]);
      }
    float g_last = 0.0f;
    if (DECAY == LQ_DECAY_SCALAR) g_last = p.g[(t0 + 63) * H + h];
    if (tid < 64) {
      float ekv = 1.0f, evv = 1.0f;
      if (DECAY == LQ_DECAY_SCALAR) {
        const float d = g_last - p.g[(t0 + tid) * H + h];
        ekv = lq_expf((1.0f - eta) * d);
        evv = lq_expf(eta * d);
      } else if (DECAY == LQ_DECAY_DIAGONAL) {
        const float le = p.logenv[(t0 + tid) * H + h];
        ekv = eta * le;  // the key factor is per element: exp(gk_last - gk - eta*le)
        evv = lq_expf(eta * le);
      }
      ek_s[tid] = ekv;
      ev_s[tid] = evv;
      if (DELTA) fw_s[tid] = p.fw[(t0 + tid) * H + h];
    }
    __syncthreads();

    // ---- phase B: copy the stored state out, coalesced: h_i8[b][ct][h][v0 + v][k]
    {
      int8_t* dst = p.h_i8 + ((((int64_t)b * p.NT + ct) * H + h) * V + v0) * K;
      constexpr int SEG = K / 16;
      for (int it = tid; it < BV * SEG; it += 256) {
        const int vr = it / SEG, sg = it % SEG;
        *(lq_v4i*)(dst + vr * K + sg * 16) = *(const lq_v4i*)(hT + vr * HS + sg * 16);
      }
    }

    // ---- phase C (delta): state read against the stored copy, pseudo-values E, their write codes
    if (DELTA) {
      lq_v4i aw[4];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) aw[jj] = lq_v4i{0, 0, 0, 0};
      const _Float16* wp = p.w + ((t0 + 16 * wave + rl) * H + h) * K + 16 * kg;
#pragma unroll
      for (int ks = 0; ks < K / 64; ++ks) {
        const lq_v8h w0 = *(const lq_v8h*)(wp + 64 * ks);
        const lq_v8h w1 = *(const lq_v8h*)(wp + 64 * ks + 8);
        int cd[16];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          cd[e] = zoo_q8((float)w0[e], inv_sw, qmax);
          cd[8 + e] = zoo_q8((float)w1[e], inv_sw, qmax);
        }
        lq_v4i wop;
#pragma unroll
        for (int d = 0; d < 4; ++d) wop[d] = (int)zoo_pack_codes(cd[4 * d], cd[4 * d + 1], cd[4 * d + 2], cd[4 * d + 3]);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const lq_v4i hop = *(const lq_v4i*)(hT + (4 * rl + jj) * HS + 64 * ks + 16 * kg);
          aw[jj] = lq_mfma_i8(wop, hop, aw[jj]);
        }
      }
      // lane holds tokens 16*wave + 4kg + r, value columns v0 + 4rl + jj
      uint32_t ecode[4][4];  // [jj][r]
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int tl = 16 * wave + 4 * kg + r;
        const int64_t off = ((t0 + tl) * H + h) * V + v0 + 4 * rl;
        const lq_v2i uu = *(const lq_v2i*)(p.v + off);
        const float fwt = fw_s[tl], evt = ev_s[tl];
        lq_v2i eo;
        float ef[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          float ws = (float)aw[jj][r] * sw;
          ws = ws * ss_d[jj];
          const float u = (float)zoo_half_of((uint32_t)uu[jj >> 1], jj & 1);
          ef[jj] = (u - ws) * fwt;
        }
        eo[0] = (int)zoo_pack_h2(ef[0], ef[1]);
        eo[1] = (int)zoo_pack_h2(ef[2], ef[3]);
        *(lq_v2i*)(p.e_out + off) = eo;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const float ed = (DECAY == LQ_DECAY_NONE) ? ef[jj] : ef[jj] * evt;
          ecode[jj][r] = (uint32_t)zoo_q8(ed, inv_ew_d[jj], qmax);
        }
      }
      lq_v4i ev4;
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) ev4[jj] = (int)zoo_pack_codes((int)ecode[jj][0], (int)ecode[jj][1], (int)ecode[jj][2], (int)ecode[jj][3]);
      *(lq_v4i*)(eb + (4 * wave + kg) * EW + 4 * rl) = ev4;
    }

    // ---- phase D: quantize the key slab (and, linear family, the value slab) into LDS
    {
      const _Float16* kp = p.k + ((t0 + 4 * tq) * H + h) * K + CK * cg;
      uint32_t kcode[CK][4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int tl = 4 * tq + t;
        const _Float16* kr = kp + (int64_t)t * H * K;
        float kv[CK];
        if constexpr (CK == 8) {
          const lq_v8h v8 = *(const lq_v8h*)kr;
#pragma unroll
          for (int e = 0; e < 8; ++e) kv[e] = (float)v8[e];
        } else {
          const lq_v4h v4 = *(const lq_v4h*)kr;
#pragma unroll
          for (int e = 0; e < 4; ++e) kv[e] = (float)v4[e];
        }
        if (DECAY == LQ_DECAY_SCALAR) {
          const float f = ek_s[tl];
#pragma unroll
          for (int e = 0; e < CK; ++e) kv[e] = kv[e] * f;
        } else if (DECAY == LQ_DECAY_DIAGONAL) {
          const float* gr = p.g + ((t0 + tl) * H + h) * K + CK * cg;
          const float* gl = p.g + ((t0 + 63) * H + h) * K + CK * cg;
          const float el = ek_s[tl];
#pragma unroll
          for (int e = 0; e < CK; ++e) kv[e] = kv[e] * lq_expf(gl[e] - gr[e] - el);
        }
#pragma unroll
        for (int e = 0; e < CK; ++e) kcode[e][t] = (uint32_t)zoo_q8(kv[e], inv_skw_q[e], qmax);
      }
#pragma unroll
      for (int e = 0; e < CK; e += 4) {
        lq_v4i o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (int)zoo_pack_codes((int)kcode[e + i][0], (int)kcode[e + i][1], (int)kcode[e + i][2], (int)kcode[e + i][3]);
        *(lq_v4i*)(kb + tq * KW + CK * cg + e) = o;
      }
      if (!DELTA) {
        const _Float16* vp = p.v + ((t0 + 4 * tq) * H + h) * V + v0 + 4 * cg;
        uint32_t vcode[4][4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const lq_v4h v4 = *(const lq_v4h*)(vp + (int64_t)t * H * V);
          const float f = ev_s[4 * tq + t];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float x = (DECAY == LQ_DECAY_NONE) ? (float)v4[e] : (float)v4[e] * f;
            vcode[e][t] = (uint32_t)zoo_q8(x, inv_svw_q[e], qmax);
          }
        }
        lq_v4i o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (int)zoo_pack_codes((int)vcode[e][0], (int)vcode[e][1], (int)vcode[e][2], (int)vcode[e][3]);
        *(lq_v4i*)(eb + tq * EW + 4 * cg) = o;
      }
    }
    __syncthreads();

    // ---- phase E: write product and carry update
    {
      const float gamma_s = (DECAY == LQ_DECAY_SCALAR) ? lq_expf(g_last) : 1.0f;
      lq_v4i vop[VT];
#pragma unroll
      for (int vt = 0; vt < VT; ++vt)
#pragma unroll
        for (int i = 0; i < 4; ++i) vop[vt][i] = (int)eb[(4 * kg + i) * EW + 16 * vt + rl];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        lq_v4i kop;
#pragma unroll
        for (int i = 0; i < 4; ++i) kop[i] = (int)kb[(4 * kg + i) * KW + KR * wave + 16 * kt + rl];
        float gam[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (DECAY == LQ_DECAY_SCALAR)
            gam[r] = gamma_s;
          else if (DECAY == LQ_DECAY_DIAGONAL)
            gam[r] = lq_expf(p.g[((t0 + 63) * H + h) * K + KR * wave + 16 * kt + 4 * kg + r]);
          else
            gam[r] = 1.0f;
        }
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
          const lq_v4i a = lq_mfma_i8(kop, vop[vt], lq_v4i{0, 0, 0, 0});
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float prod = (float)a[r] * skw_r[kt][r];
            prod = prod * svw_c[vt];
            float hv = hc[kt][vt][r];
            if (DECAY != LQ_DECAY_NONE) hv = hv * gam[r];
            hc[kt][vt][r] = hv + prod;
          }
        }
      }
    }
  }

  if (p.ht) {
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int vt = 0; vt < VT; ++vt)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          p.ht[(((int64_t)b * H + h) * K + KR * wave + 16 * kt + 4 * kg + r) * V + v0 + 16 * vt + rl] = hc[kt][vt][r];
  }
}

template <bool DELTA, int DECAY>
int launch_k(const StateParams& p, int K, dim3 grid, hipStream_t stream) {
  if (K == 128)
    hipLaunchKernelGGL((zoo_state_kernel<DELTA, DECAY, 128>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_state_kernel<DELTA, DECAY, 64>), grid, dim3(256), 0, stream, p);
  return lq_check_launch();
}

template <bool DELTA>
int launch_d(const StateParams& p, int K, int decay, dim3 grid, hipStream_t stream) {
  switch (decay) {
    case LQ_DECAY_NONE: return launch_k<DELTA, LQ_DECAY_NONE>(p, K, grid, stream);
    case LQ_DECAY_SCALAR: return launch_k<DELTA, LQ_DECAY_SCALAR>(p, K, grid, stream);
    case LQ_DECAY_DIAGONAL: return launch_k<DELTA, LQ_DECAY_DIAGONAL>(p, K, grid, stream);
  }
  return LQ_ERR_SHAPE;
}

}  // namespace

extern "C" int lq_zoo_state(const lq_zoo_state_args* a, hipStream_t stream) {
  if (!a || !a->k || !a->v || !a->h_i8 || !a->skw || !a->svw || !a->ss) return LQ_ERR_NULL;
  const bool delta = a->family == LQ_FAMILY_DELTA;
  if (a->family != LQ_FAMILY_LINEAR && !delta) return LQ_ERR_SHAPE;
  if (delta && (!a->w || !a->fw || !a->e_out || !a->sw)) return LQ_ERR_NULL;
  if (a->decay != LQ_DECAY_NONE && !a->g) return LQ_ERR_NULL;
  if (a->decay == LQ_DECAY_DIAGONAL && !a->logenv) return LQ_ERR_NULL;
  if (a->unrot) return LQ_ERR_SHAPE;  // canonical storage (in-kernel un-rotation) is not built yet
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  if (a->chunk_size != 64 || a->seqlen % 64 != 0) return LQ_ERR_SHAPE;
  if ((a->kdim != 64 && a->kdim != 128) || a->vdim % 64 != 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  if (a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
  if (!zoo_al(a->k, 16) || !zoo_al(a->v, 8) || !zoo_al(a->h_i8, 16) || (delta && (!zoo_al(a->w, 16) || !zoo_al(a->e_out, 8))))
    return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  StateParams p = {};
  p.k = (const _Float16*)a->k, p.v = (const _Float16*)a->v, p.w = (const _Float16*)a->w;
  p.fw = a->fw, p.g = a->g, p.logenv = a->logenv, p.h_i8 = a->h_i8, p.e_out = (_Float16*)a->e_out, p.ht = a->ht;
  p.skw = a->skw, p.svw = a->svw, p.sw = a->sw, p.ss = a->ss;
  p.eta = a->eta, p.qmax = a->qmax;
  p.B = a->batch, p.T = a->seqlen, p.H = a->nheads, p.V = a->vdim, p.NT = a->seqlen / 64;
  dim3 grid(a->vdim / BV, a->batch * a->nheads);
  return delta ? launch_d<true>(p, a->kdim, a->decay, grid, stream) : launch_d<false>(p, a->kdim, a->decay, grid, stream);
}
