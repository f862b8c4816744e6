// Fused operand prologue of the linear family (no / scalar decay): rotation + rescaling + quantization of q, k, v in one
// launch, straight to the INT8 operands the state kernel and the output kernel consume.
// Covers, for a call that would otherwise run them one after the other,
//   the operand rotations q @ R_QK, k @ R_QK, v @ R_V of bench/zoo_kernels.py:135-140 ("not fused yet") and the D_QK
//     rescaling of linquant/harness.py:68-88                                   (lq_zoo_rotate_qkv),
//   the write-operand preparation inside _state_body, linquant/kernels/zoo/simple_gla.py:55-66   (lq_zoo_write_codes),
//   the operand quantization at the top of _output_body, simple_gla.py:125-140                   (lq_zoo_output),
// with the same arithmetic in the same order on the same rounded values, so every code equals what the three launches
// would have made from the rotated activations stored in between; those activations need not be stored at all.
//
// One 256-thread workgroup per (tensor, chunk, batch*head).  A row of D channels is spread over D / 8 lanes (16 bytes per
// lane); a thread takes four consecutive tokens of its eight channels, so the channel-major write codes of a token quad
// are one dword per channel; they are transposed through LDS into 64-byte rows.  The rotation R = H_D / sqrt(D) .
// diag(signs) is a fast Walsh-Hadamard transform in fp32 (butterflies 1, 2, 4 in registers, the rest through lane
// exchanges), rounded once to the activation dtype exactly as lq_zoo_rotate_qkv rounds it.
#include "zoo_common.h"
#include "../../include/linquant_hip.h"

namespace {

struct RqParams {
  const uint16_t* src[3];   // q, k, v; nullptr: that tensor is not part of the call
  uint16_t* dst[3];         // rotated activations, or nullptr: not stored
  int8_t* loc[3];           // token-major local codes (B,T,H,D)
  int8_t* wrT[3];           // channel-major write codes (B,NT,H,D,64) of k and v ([0] unused)
  const float* mul[3];      // (H,D) multiplier (q: D_QK; k: its reciprocal), or nullptr
  const float* divd[3];     // (H,D) divisor of k (the row is divided, rounded once), or nullptr
  const float* signs[3];    // (D,) column signs of the rotation, or nullptr: no rotation
  const float* sloc[3];     // local scales: q, k (H,); v (H,D)
  const float* swr[3];      // write scales (H,D) of k and v
  const float* g;           // (B,T,H) chunk-local cumulative log decay, or nullptr
  float* ev;                // (B,T,H)
  float* gam;               // (B,NT,H,K)
  float eta, scale, rsqrt_n;
  int qmax;
  int T, H, NT;
  int first;                // tensor index of blockIdx.z == 0
};

// clamp(rha(x * inv), -qmax, qmax) with the clamp as one median instruction (same value as zoo_q8)
LQ_DEV int rq_q8(float x, float inv, int qmax) {
  int r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(lq_rha_i32(x * inv)), "v"(-qmax), "v"(qmax));
  return r;
}

constexpr int kTS = 20;  // dwords per channel row of the transposed tile (16 token quads + pad)

// WHICH: 0 = q, 1 = k, 2 = v (compile-time, so that what only one of them needs costs the others nothing)
template <int D, bool BF, int WHICH>
LQ_DEV void rotate_quant_body(const RqParams& p, uint32_t* cT, float* f_s, float* inv_s) {
  constexpr int LPR = D / 8;  // lanes per row
  constexpr int TS = kTS;
  constexpr int which = WHICH;
  const uint16_t* src = p.src[which];
  if (!src) return;  // block-uniform
  const int tid = threadIdx.x;
  const int ct = blockIdx.x;
  const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
  const int H = p.H;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)ct * 64;
  const int64_t cb = ((int64_t)b * p.NT + ct) * H + h;
  constexpr bool writes = which > 0;
  constexpr bool bf = BF;
  // reciprocal scales, one IEEE division per channel and workgroup: [0, D) local (per channel for v), [D, 2D) write
  if (tid < D) {
    if (which == 2) inv_s[tid] = 1.0f / p.sloc[2][(int64_t)h * D + tid];
    if (writes) inv_s[D + tid] = 1.0f / p.swr[which][(int64_t)h * D + tid];
  }

  // ---- per-token factor of the write operand (key: exp((1-eta)(g_last - g_t)); value: exp(eta (g_last - g_t))), the
  // per-token value factor and the chunk decay, as lq_zoo_write_codes forms them
  if (writes && tid < 64) {
    float ekv = 1.0f, evv = 1.0f;
    if (p.g) {
      const float d = p.g[(t0 + 63) * H + h] - p.g[(t0 + tid) * H + h];
      ekv = zoo_exp((1.0f - p.eta) * d);
      evv = zoo_exp(p.eta * d);
    }
    f_s[tid] = which == 1 ? ekv : evv;
    if (which == 2) p.ev[(t0 + tid) * H + h] = evv;
  }
  if (which == 1 && tid >= 64 && tid < 64 + D) {
    float gm = 1.0f;
    if (p.g) gm = zoo_exp(p.g[(t0 + 63) * H + h]);
    p.gam[cb * D + (tid - 64)] = gm;
  }

  const int tq = tid / LPR, sub = tid % LPR;  // token quad, group of eight channels
  const bool active = tid < 16 * LPR;         // wave-uniform: 16 * LPR is a multiple of 64
  if (active) {
    const float* mul = p.mul[which];
    const float* divd = p.divd[which];
    const float* signs = p.signs[which];
    // every request before the first use; absent operands are read from a valid address and ignored
    lq_v4i raw[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = *(const lq_v4i*)(src + ((t0 + 4 * tq + i) * H + h) * D + 8 * sub);
    const float* any = (const float*)src;
    const float* sp = signs ? signs + 8 * sub : any;
    const lq_v4f s0 = *(const lq_v4f*)sp, s1 = *(const lq_v4f*)(signs ? sp + 4 : sp);
    const float* mp = mul ? mul + (int64_t)h * D + 8 * sub : any;
    const lq_v4f m0 = *(const lq_v4f*)mp, m1 = *(const lq_v4f*)(mul ? mp + 4 : mp);
    const float* dp = divd ? divd + (int64_t)h * D + 8 * sub : any;
    const lq_v4f e0 = *(const lq_v4f*)dp, e1 = *(const lq_v4f*)(divd ? dp + 4 : dp);
    constexpr bool loc_pc = which == 2;  // the value's local scale is per channel
    const float inv_head = loc_pc ? 0.0f : 1.0f / p.sloc[which][h];
    if (writes) __syncthreads();  // f_s, inv_s (threads that are not active meet this barrier in the other branch)
    float inv_loc[8], inv_wr[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      inv_loc[e] = loc_pc ? inv_s[8 * sub + e] : inv_head;
      inv_wr[e] = writes ? inv_s[D + 8 * sub + e] : 0.0f;
    }
    int wc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v[8];
#pragma unroll
      for (int d = 0; d < 4; ++d) zoo_dec2((uint32_t)raw[i][d], bf, v[2 * d], v[2 * d + 1]);
      if (divd) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = zoo_div_rn(v[e], e < 4 ? e0[e & 3] : e1[e & 3], e < 4 ? m0[e & 3] : m1[e & 3]);
      } else if (mul) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = zoo_mul_rn(v[e], e < 4 ? m0[e & 3] : m1[e & 3]);
      }
      if (signs) {
        zoo_fwht<LPR>(v, sub);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (v[e] * p.rsqrt_n) * (e < 4 ? s0[e & 3] : s1[e & 3]);
      }
      // the activation as it would have been stored, and back
      lq_v4i enc;
#pragma unroll
      for (int d = 0; d < 4; ++d) enc[d] = (int)zoo_enc2(v[2 * d], v[2 * d + 1], bf);
      const int64_t off = ((t0 + 4 * tq + i) * H + h) * D + 8 * sub;
      if (p.dst[which]) *(lq_v4i*)(p.dst[which] + off) = enc;
#pragma unroll
      for (int d = 0; d < 4; ++d) zoo_dec2((uint32_t)enc[d], bf, v[2 * d], v[2 * d + 1]);
      int lc[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) lc[e] = rq_q8(which == 0 ? v[e] * p.scale : v[e], inv_loc[e], p.qmax);
      lq_v2i lo;
      lo[0] = (int)zoo_pack_codes(lc[0], lc[1], lc[2], lc[3]);
      lo[1] = (int)zoo_pack_codes(lc[4], lc[5], lc[6], lc[7]);
      *(lq_v2i*)(p.loc[which] + off) = lo;
      if (writes) {
        const float f = f_s[4 * tq + i];
#pragma unroll
        for (int e = 0; e < 8; ++e) wc[i][e] = rq_q8(p.g ? v[e] * f : v[e], inv_wr[e], p.qmax);
      }
    }
    if (writes) {
#pragma unroll
      for (int e = 0; e < 8; ++e) cT[(8 * sub + e) * TS + tq] = zoo_pack_codes(wc[0][e], wc[1][e], wc[2][e], wc[3][e]);
    }
  } else if (writes) {
    __syncthreads();  // pairs with the barrier of the active threads
  }
  if (!writes) return;
  __syncthreads();
  for (int it = tid; it < D * 4; it += 256) {
    const int row = it >> 2, seg = it & 3;
    *(lq_v4i*)(p.wrT[which] + (cb * D + row) * 64 + seg * 16) = *(const lq_v4i*)(cT + row * TS + 4 * seg);
  }
}

template <int D, bool BF>
__global__ __launch_bounds__(256) void zoo_rotate_quant_kernel(RqParams p) {
  __shared__ __align__(16) uint32_t cT[D * kTS];
  __shared__ float f_s[64], inv_s[2 * D];
  switch (p.first + blockIdx.z) {  // block-uniform
    case 0: rotate_quant_body<D, BF, 0>(p, cT, f_s, inv_s); break;
    case 1: rotate_quant_body<D, BF, 1>(p, cT, f_s, inv_s); break;
    default: rotate_quant_body<D, BF, 2>(p, cT, f_s, inv_s); break;
  }
}

bool al16(const void* q) { return ((uintptr_t)q % 16) == 0; }

template <int D>
int launch(const RqParams& p, bool bf, dim3 grid, hipStream_t stream) {
  if (bf)
    hipLaunchKernelGGL((zoo_rotate_quant_kernel<D, true>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_rotate_quant_kernel<D, false>), grid, dim3(256), 0, stream, p);
  return lq_check_launch();
}

}  // namespace

extern "C" int lq_zoo_rotate_quant(const lq_zoo_rotate_quant_args* a, hipStream_t stream) {
  if (!a || !a->q || !a->k || !a->v) return LQ_ERR_NULL;
  if (!a->qc || !a->kc || !a->vc || !a->kqT || !a->vqT || !a->ev || !a->gam) return LQ_ERR_NULL;
  if (!a->sq || !a->sk || !a->svl || !a->skw || !a->svw) return LQ_ERR_NULL;
  if (a->dk && !a->dq) return LQ_ERR_NULL;  // k is divided by dq; dk is its reciprocal
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  if (a->chunk_size != 64 || a->seqlen % 64 != 0) return LQ_ERR_SHAPE;
  const int K = a->kdim, V = a->vdim;
  if ((K != 64 && K != 128) || (V != 64 && V != 128)) return LQ_ERR_SHAPE;
  if (a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
  if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  const void* ptrs[] = {a->q, a->k, a->v, a->q_out, a->k_out, a->v_out, a->qc, a->kc, a->vc, a->kqT, a->vqT,
                        a->dq, a->dk, a->signs_qk, a->signs_v, a->svl, a->skw, a->svw};
  for (const void* q : ptrs)
    if (q && !al16(q)) return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535 || a->seqlen / 64 > 0x7fffffff) return LQ_ERR_SHAPE;
  RqParams p = {};
  p.src[0] = (const uint16_t*)a->q, p.src[1] = (const uint16_t*)a->k, p.src[2] = (const uint16_t*)a->v;
  p.dst[0] = (uint16_t*)a->q_out, p.dst[1] = (uint16_t*)a->k_out, p.dst[2] = (uint16_t*)a->v_out;
  p.loc[0] = a->qc, p.loc[1] = a->kc, p.loc[2] = a->vc;
  p.wrT[1] = a->kqT, p.wrT[2] = a->vqT;
  p.mul[0] = a->dq, p.mul[1] = a->dk, p.divd[1] = a->dk ? a->dq : nullptr;
  p.signs[0] = a->signs_qk, p.signs[1] = a->signs_qk, p.signs[2] = a->signs_v;
  p.sloc[0] = a->sq, p.sloc[1] = a->sk, p.sloc[2] = a->svl;
  p.swr[1] = a->skw, p.swr[2] = a->svw;
  p.g = a->g, p.ev = a->ev, p.gam = a->gam;
  p.eta = a->eta, p.scale = a->scale, p.qmax = a->qmax;
  p.T = a->seqlen, p.H = a->nheads, p.NT = a->seqlen / 64;
  const bool bf = a->act_dtype == LQ_DT_BF16;
  const unsigned nt = (unsigned)p.NT, bh = (unsigned)(a->batch * a->nheads);
  // one launch per distinct row width: q and k share K, v joins them when V == K
  int rc;
  p.first = 0;
  p.rsqrt_n = (float)(1.0 / sqrt((double)K));
  rc = K == 128 ? launch<128>(p, bf, dim3(nt, bh, V == K ? 3 : 2), stream) : launch<64>(p, bf, dim3(nt, bh, V == K ? 3 : 2), stream);
  if (rc != LQ_OK || V == K) return rc;
  p.first = 2;
  p.rsqrt_n = (float)(1.0 / sqrt((double)V));
  return V == 128 ? launch<128>(p, bf, dim3(nt, bh, 1), stream) : launch<64>(p, bf, dim3(nt, bh, 1), stream);
}
