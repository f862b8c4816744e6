// Intra-chunk product under per-channel (diagonal) decay for 128-token chunks: the blocks that pair a row of the chunk's
// second half with a token of its first half.  (The blocks inside either half are the 64-token kernel's: the decay enters
// only through differences of the cumulative log decay, which do not care where the cumulation started.)
// Follows _gla_A_inter (linquant/kernels/zoo/gla.py:27-63) with BT = 128: block (I, J), I in 4..7, J in 0..3, anchored at
// the first row of sub-block I:
//     qg = q * exp(g_i - a) * scale,  kg = k * exp(a - g_j),  a[n] = g[first row of I][n]
//     A[i][j] = float(q8(qg, 1/sq) . q8(kg, 1/sk)) * (sq*sk)
// and with a local R_QK both anchored operands are rounded to fp16 and rotated on the fp16 MFMA before quantization.
// One 4-wave workgroup per (chunk, batch*head); wave w owns sub-block I = 4 + w: its anchored query codes are made once
// and stay in registers, the key rows of the four first-half sub-blocks are fetched and anchored in turn.  Lane (rl, kg)
// holds token rl, channels 32ks + 8kg + e; after the rotation channels 16mt + 4kg + r; query and key operand share the
// channel -> slot map, so the INT8 dot is exact.  Output: Ax (B,T,H,64) fp16, rows of the second halves only, column j =
// token j of the chunk's first half.
#include "zoo_params.h"
#include "../../include/linquant_hip.h"

namespace {

template <int K, bool ROT, bool BF>
__global__ __launch_bounds__(256) void zoo_gla_A_cross_kernel(ZooACrossParams p) {
  constexpr int RS = K + 8;  // halves per row of the transposed rotation
  __shared__ __align__(16) _Float16 RT[ROT ? K * RS : 8];  // RT[m][n] = R[n][m]
  constexpr int KS = K / 32, MT = K / 16;
  constexpr bool bf = BF;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  const int H = p.H;
  const int b = blockIdx.y / H, h = blockIdx.y % H;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)blockIdx.x * 128;  // first token of the chunk
  const int64_t r0 = t0 + 64 + 16 * wave;                           // first row of this wave's sub-block
  const float sq = p.sq[h], sk = p.sk[h];
  const float inv_sq = 1.0f / sq, inv_sk = 1.0f / sk;
  const int qmax = p.qmax;

  if constexpr (ROT) {
    for (int it = tid; it < K * (K / 8); it += 256) {
      const int m = it % K, n8 = it / K;
      lq_v8h rv;
#pragma unroll
      for (int e = 0; e < 8; ++e) rv[e] = p.rot[(int64_t)(8 * n8 + e) * K + m];
      *(lq_v8h*)(RT + m * RS + 8 * n8) = rv;
    }
    __syncthreads();
  }
  auto unpack = [&](const lq_v4i& raw, float (&o)[8]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) zoo_dec2((uint32_t)raw[d], bf, o[2 * d], o[2 * d + 1]);
  };
  // one sweep over R^T for one operand; codes of token rl, dword mt = channels 16mt + 4kg + r
  auto sweep = [&](const lq_v8h (&x0)[KS], float inv0, uint32_t (&c0)[MT]) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      lq_v4f r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const lq_v8h rop = *(const lq_v8h*)(RT + (16 * mt + rl) * RS + 32 * ks + 8 * kg);
        r = lq_mfma_f16(rop, x0[ks], r);
      }
      c0[mt] = zoo_pack_codes(zoo_q8(r[0], inv0, qmax), zoo_q8(r[1], inv0, qmax), zoo_q8(r[2], inv0, qmax), zoo_q8(r[3], inv0, qmax));
    }
  };

  // ---- own rows: the query operand anchored at the sub-block's first row; the anchor row stays in registers
  lq_v4f an[KS][2];
  lq_v8h x[KS];
  uint32_t cq[MT], ck[MT];
  {
    const int64_t roff = ((r0 + rl) * H + h) * K + 8 * kg, aoff = (r0 * H + h) * K + 8 * kg;
    lq_v4i qraw[KS];
    lq_v4f gown[KS][2];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qraw[ks] = *(const lq_v4i*)(p.q + roff + 32 * ks);
      gown[ks][0] = *(const lq_v4f*)(p.g + roff + 32 * ks), gown[ks][1] = *(const lq_v4f*)(p.g + roff + 32 * ks + 4);
      an[ks][0] = *(const lq_v4f*)(p.g + aoff + 32 * ks), an[ks][1] = *(const lq_v4f*)(p.g + aoff + 32 * ks + 4);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      float qf[8];
      unpack(qraw[ks], qf);
      if (p.dq) {  // D_QK at load: q' = act(q * D)
        const float* dp = p.dq + h * K + 32 * ks + 8 * kg;
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[e] = zoo_round_act(zoo_mul_rn(qf[e], dp[e]), bf);
      }
      int iq[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = gown[ks][e >> 2][e & 3] - an[ks][e >> 2][e & 3];
        float xv = qf[e] * zoo_exp(d);
        xv = xv * p.scale;
        if constexpr (ROT)
          x[ks][e] = (_Float16)xv;
        else
          iq[e] = zoo_q8(xv, inv_sq, qmax);
      }
      if constexpr (!ROT)
        cq[2 * ks] = zoo_pack_codes(iq[0], iq[1], iq[2], iq[3]), cq[2 * ks + 1] = zoo_pack_codes(iq[4], iq[5], iq[6], iq[7]);
    }
    if constexpr (ROT) sweep(x, inv_sq, cq);
  }

  // ---- the four sub-blocks of the first half, anchored at this sub-block's first row
  const float sqk = sq * sk;
#pragma unroll 1
  for (int J = 0; J < 4; ++J) {
    const int64_t koff = ((t0 + 16 * J + rl) * H + h) * K + 8 * kg;
    lq_v4i kraw[KS];
    lq_v4f gk[KS][2];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kraw[ks] = *(const lq_v4i*)(p.k + koff + 32 * ks);
      gk[ks][0] = *(const lq_v4f*)(p.g + koff + 32 * ks), gk[ks][1] = *(const lq_v4f*)(p.g + koff + 32 * ks + 4);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      float kf[8];
      unpack(kraw[ks], kf);
      int ic[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float v = kf[e] * zoo_exp(an[ks][e >> 2][e & 3] - gk[ks][e >> 2][e & 3]);
        if constexpr (ROT)
          x[ks][e] = (_Float16)v;
        else
          ic[e] = zoo_q8(v, inv_sk, qmax);
      }
      if constexpr (!ROT)
        ck[2 * ks] = zoo_pack_codes(ic[0], ic[1], ic[2], ic[3]), ck[2 * ks + 1] = zoo_pack_codes(ic[4], ic[5], ic[6], ic[7]);
    }
    if constexpr (ROT) sweep(x, inv_sk, ck);
    lq_v4i acc = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < K / 64; ++s) {
      lq_v4i qop, kop;
#pragma unroll
      for (int d = 0; d < 4; ++d) qop[d] = (int)cq[4 * s + d], kop[d] = (int)ck[4 * s + d];
      acc = lq_mfma_i8(qop, kop, acc);
    }
    // lane holds column j = 16J + rl, rows 4kg + r of the sub-block
#pragma unroll
    for (int r = 0; r < 4; ++r) p.Ax[((r0 + 4 * kg + r) * H + h) * 64 + 16 * J + rl] = (_Float16)((float)acc[r] * sqk);
  }
}

template <int K, bool ROT>
void launch_bf(const ZooACrossParams& p, dim3 grid, hipStream_t stream) {
  if (p.bf)
    hipLaunchKernelGGL((zoo_gla_A_cross_kernel<K, ROT, true>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_gla_A_cross_kernel<K, ROT, false>), grid, dim3(256), 0, stream, p);
}

}  // namespace

int zoo_gla_A_cross_launch(const ZooACrossParams& p, int K, hipStream_t stream) {
  const dim3 grid(p.T / 128, p.B * p.H);
  if (K == 128) {
    if (p.rot) launch_bf<128, true>(p, grid, stream); else launch_bf<128, false>(p, grid, stream);
  } else {
    if (p.rot) launch_bf<64, true>(p, grid, stream); else launch_bf<64, false>(p, grid, stream);
  }
  return lq_check_launch();
}
