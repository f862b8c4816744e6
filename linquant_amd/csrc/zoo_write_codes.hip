// Write-operand pre-pass of the zoo state kernels: every operand of the chunk recurrence that does not depend on
// the carried state is quantized here, fully parallel over (chunk, batch*head), and stored in the layout the
// sequential state kernel consumes as plain 16-byte INT8 MFMA operands.
// Covers the operand preparation inside _state_body (linquant/kernels/zoo/simple_gla.py:55-66), _gla_state_body
// (gla.py:124-141), _delta_state_body (gated_delta_rule.py:85-105) and _kda_state_body (kda.py:100-124):
//   key write codes   kqT[b][c][h][k][t] = q8(key[t][k] * fk(t,k), 1/skw[k])        (channel-major inside the chunk)
//       fk = 1 | exp((1-eta)(g_last - g_t)) | exp(gk_last - gk_t - eta*le_t)
//   value write codes vqT[b][c][h][v][t] = q8(val[t][v] * fv(t), 1/svw[v])          (linear family)
//       fv = 1 | exp(eta (g_last - g_t)) | exp(eta*le_t)
//   state-read codes  wq[b][t][h][k]     = q8(W[t][k], 1/sw)                        (delta family)
//   ev[b][t][h] = fv(t)  (the delta kernels scale their pseudo-values with it),  gam[b][c][h][k] = exp(g_last(k))
// One 4-wave workgroup per (chunk, batch*head); the code tiles are transposed through LDS.
#include "zoo_common.h"
#include "../../include/linquant_hip.h"

namespace {

struct CodesParams {
  const _Float16* key;
  const _Float16* val;
  const _Float16* w;
  const float* g;
  const float* logenv;
  int8_t* kqT;
  int8_t* vqT;
  int8_t* wq;
  float* ev;
  float* gam;
  const float* skw;
  const float* svw;
  const float* sw;
  float eta;
  int qmax;
  int bf;
  int T, H, V, NT;
  int span;  // tokens per chunk: 64, or 128 (two workgroups per chunk, the decays reach to the end of the chunk)
};

template <int DECAY, int K, bool BF>
__global__ __launch_bounds__(256) void zoo_write_codes_kernel(CodesParams p) {
  constexpr int CK = K / 16;  // key channels per thread
  constexpr int TS = 20;      // dwords per channel row of the transposed tile (16 token quads + pad)
  __shared__ __align__(16) uint32_t cT[K * TS];
  __shared__ float ek_s[64], ev_s[64];

  const int tid = threadIdx.x;
  const int ct = blockIdx.x;
  const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
  const int H = p.H, V = p.V, T = p.T;
  const int64_t t0 = (int64_t)b * T + (int64_t)ct * 64;
  const int64_t cb = ((int64_t)b * p.NT + ct) * H + h;  // (batch, chunk, head) index
  // last token of the chunk: of these 64 tokens, or, when they are one piece of a chunk of 128 .. 256 tokens, of that chunk
  const int pieces = p.span / 64;
  const int64_t tlast = t0 + 63 + (int64_t)(pieces - 1 - ct % pieces) * 64;
  const float eta = p.eta;
  const int qmax = p.qmax;
  constexpr bool bf = BF;

  if (tid < 64) {
    float ekv = 1.0f, evv = 1.0f;
    if (DECAY == LQ_DECAY_SCALAR) {
      const float d = p.g[tlast * H + h] - p.g[(t0 + tid) * H + h];
      ekv = zoo_exp((1.0f - eta) * d);
      evv = zoo_exp(eta * d);
    } else if (DECAY == LQ_DECAY_DIAGONAL) {
      const float le = p.logenv[(t0 + tid) * H + h];
      ekv = eta * le;  // the key factor is per element: exp(gk_last - gk - eta*le)
      evv = zoo_exp(eta * le);
    }
    ek_s[tid] = ekv;
    ev_s[tid] = evv;
    p.ev[(t0 + tid) * H + h] = evv;
  }
  if (tid < K) {
    float gm = 1.0f;
    if (DECAY == LQ_DECAY_SCALAR) gm = zoo_exp(p.g[tlast * H + h]);
    if (DECAY == LQ_DECAY_DIAGONAL) gm = zoo_exp(p.g[(tlast * H + h) * K + tid]);
    p.gam[cb * K + tid] = gm;
  }
  __syncthreads();

  const int tq = tid >> 4, cg = tid & 15;  // token quad, channel group
  // ---- key write codes (and the state-read codes of W, token-major, straight from registers)
  {
    float inv_skw[CK];
#pragma unroll
    for (int e = 0; e < CK; ++e) inv_skw[e] = 1.0f / p.skw[h * K + CK * cg + e];
    const float inv_sw = p.w ? 1.0f / p.sw[h] : 0.0f;
    // every request of the thread's four tokens is issued before the first is used (with the loads inside the token
    // loop, next to a run-time `if (p.w)`, each token cost its own memory round trips)
    typedef int raw_t __attribute__((ext_vector_type(CK / 2)));  // CK half-precision values
    typedef float gf_t __attribute__((ext_vector_type(4)));
    raw_t kraw[4], wraw[4];
    gf_t graw[4][CK / 4], glast[CK / 4];
    int64_t offs[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      offs[t] = ((t0 + 4 * tq + t) * H + h) * K + CK * cg;
      kraw[t] = *(const raw_t*)(p.key + offs[t]);
      if (DECAY == LQ_DECAY_DIAGONAL) {
#pragma unroll
        for (int d = 0; d < CK / 4; ++d) graw[t][d] = *(const gf_t*)(p.g + offs[t] + 4 * d);
      }
    }
    if (DECAY == LQ_DECAY_DIAGONAL) {
#pragma unroll
      for (int d = 0; d < CK / 4; ++d) glast[d] = *(const gf_t*)(p.g + (tlast * H + h) * K + CK * cg + 4 * d);
    }
    if (p.w) {
#pragma unroll
      for (int t = 0; t < 4; ++t) wraw[t] = *(const raw_t*)(p.w + offs[t]);
    }
    uint32_t kcode[CK][4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int tl = 4 * tq + t;
      float kv[CK];
#pragma unroll
      for (int d = 0; d < CK / 2; ++d) zoo_dec2((uint32_t)kraw[t][d], bf, kv[2 * d], kv[2 * d + 1]);
      if (DECAY == LQ_DECAY_SCALAR) {
        const float f = ek_s[tl];
#pragma unroll
        for (int e = 0; e < CK; ++e) kv[e] = kv[e] * f;
      } else if (DECAY == LQ_DECAY_DIAGONAL) {
        const float el = ek_s[tl];
#pragma unroll
        for (int e = 0; e < CK; ++e) kv[e] = kv[e] * zoo_exp(glast[e >> 2][e & 3] - graw[t][e >> 2][e & 3] - el);
      }
#pragma unroll
      for (int e = 0; e < CK; ++e) kcode[e][t] = (uint32_t)zoo_q8(kv[e], inv_skw[e], qmax);
    }
    if (p.w) {
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        int wc[CK];
#pragma unroll
        for (int d = 0; d < CK / 2; ++d) {
          float w0, w1;
          zoo_dec2((uint32_t)wraw[t][d], bf, w0, w1);
          wc[2 * d] = zoo_q8(w0, inv_sw, qmax), wc[2 * d + 1] = zoo_q8(w1, inv_sw, qmax);
        }
        if constexpr (CK == 8) {
          lq_v2i o;
          o[0] = (int)zoo_pack_codes(wc[0], wc[1], wc[2], wc[3]);
          o[1] = (int)zoo_pack_codes(wc[4], wc[5], wc[6], wc[7]);
          *(lq_v2i*)(p.wq + offs[t]) = o;
        } else {
          *(uint32_t*)(p.wq + offs[t]) = zoo_pack_codes(wc[0], wc[1], wc[2], wc[3]);
        }
      }
    }
#pragma unroll
    for (int e = 0; e < CK; ++e)
      cT[(CK * cg + e) * TS + tq] = zoo_pack_codes((int)kcode[e][0], (int)kcode[e][1], (int)kcode[e][2], (int)kcode[e][3]);
  }
  __syncthreads();
  for (int it = tid; it < K * 4; it += 256) {
    const int row = it >> 2, seg = it & 3;
    *(lq_v4i*)(p.kqT + (cb * K + row) * 64 + seg * 16) = *(const lq_v4i*)(cT + row * TS + 4 * seg);
  }

  // ---- value write codes (linear family), 64 value channels per pass
  if (p.val) {
    for (int vc = 0; vc < V; vc += 64) {
      __syncthreads();
      float inv_svw[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) inv_svw[e] = 1.0f / p.svw[h * V + vc + 4 * cg + e];
      uint32_t vcode[4][4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        float v4[4];
        zoo_ld4(p.val + ((t0 + 4 * tq + t) * H + h) * V + vc + 4 * cg, bf, v4);
        const float f = ev_s[4 * tq + t];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x = (DECAY == LQ_DECAY_NONE) ? v4[e] : v4[e] * f;
          vcode[e][t] = (uint32_t)zoo_q8(x, inv_svw[e], qmax);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
        cT[(4 * cg + e) * TS + tq] = zoo_pack_codes((int)vcode[e][0], (int)vcode[e][1], (int)vcode[e][2], (int)vcode[e][3]);
      __syncthreads();
      {
        const int row = tid >> 2, seg = tid & 3;
        *(lq_v4i*)(p.vqT + (cb * V + vc + row) * 64 + seg * 16) = *(const lq_v4i*)(cT + row * TS + 4 * seg);
      }
    }
  }
}

template <int DECAY, int K>
void launch_bf(const CodesParams& p, dim3 grid, hipStream_t stream) {
  if (p.bf)
    hipLaunchKernelGGL((zoo_write_codes_kernel<DECAY, K, true>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_write_codes_kernel<DECAY, K, false>), grid, dim3(256), 0, stream, p);
}

template <int K>
int launch(const CodesParams& p, int decay, dim3 grid, hipStream_t stream) {
  switch (decay) {
    case LQ_DECAY_NONE: launch_bf<LQ_DECAY_NONE, K>(p, grid, stream); break;
    case LQ_DECAY_SCALAR: launch_bf<LQ_DECAY_SCALAR, K>(p, grid, stream); break;
    case LQ_DECAY_DIAGONAL: launch_bf<LQ_DECAY_DIAGONAL, K>(p, grid, stream); break;
    default: return LQ_ERR_SHAPE;
  }
  return lq_check_launch();
}

}  // namespace

extern "C" int lq_zoo_write_codes(const lq_zoo_write_codes_args* a, hipStream_t stream) {
  if (!a || !a->key || !a->kqT || !a->ev || !a->gam || !a->skw) return LQ_ERR_NULL;
  if ((a->val != nullptr) != (a->vqT != nullptr) || (a->val && !a->svw)) return LQ_ERR_NULL;
  if ((a->w != nullptr) != (a->wq != nullptr) || (a->w && !a->sw)) return LQ_ERR_NULL;
  if (a->decay != LQ_DECAY_NONE && !a->g) return LQ_ERR_NULL;
  if (a->decay == LQ_DECAY_DIAGONAL && !a->logenv) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  // 128-token chunks: the state kernel walks them as pairs of 64-token halves (linear family, no / scalar decay: also 192, 256)
  const bool pair = a->chunk_size == 128 || a->chunk_size == 192 || a->chunk_size == 256;
  if (a->chunk_size > 128 && (a->w || a->decay == LQ_DECAY_DIAGONAL)) return LQ_ERR_SHAPE;
  if ((a->chunk_size != 64 && !pair) || a->seqlen % a->chunk_size != 0) return LQ_ERR_SHAPE;
  if ((a->kdim != 64 && a->kdim != 128) || a->vdim % 64 != 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  if (a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
  if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  if (!zoo_al(a->key, 16) || !zoo_al(a->kqT, 16) || (a->val && (!zoo_al(a->val, 8) || !zoo_al(a->vqT, 16))) ||
      (a->w && (!zoo_al(a->w, 16) || !zoo_al(a->wq, 8))) || (a->g && !zoo_al(a->g, 16)))
    return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  CodesParams p = {};
  p.key = (const _Float16*)a->key, p.val = (const _Float16*)a->val, p.w = (const _Float16*)a->w;
  p.g = a->g, p.logenv = a->logenv, p.kqT = a->kqT, p.vqT = a->vqT, p.wq = a->wq, p.ev = a->ev, p.gam = a->gam;
  p.skw = a->skw, p.svw = a->svw, p.sw = a->sw, p.eta = a->eta, p.qmax = a->qmax, p.bf = a->act_dtype == LQ_DT_BF16;
  p.T = a->seqlen, p.H = a->nheads, p.V = a->vdim, p.NT = a->seqlen / 64;
  p.span = a->chunk_size;
  dim3 grid(p.NT, a->batch * a->nheads);
  return a->kdim == 128 ? launch<128>(p, a->decay, grid, stream) : launch<64>(p, a->decay, grid, stream);
}
