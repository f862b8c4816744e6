// Intra-chunk product under per-channel (diagonal) decay, 16-token sub-blocks.
// Replaces _gla_A_inter (linquant/kernels/zoo/gla.py:27-63) and _gla_A_intra (gla.py:66-99):
//   off-diagonal block (I > J), anchor a[n] = g[first row of block I][n]:
//     qg = q * exp(g_i - a) * scale,  kg = k * exp(a - g_j)
//     A[i][j] = float(q8(qg, 1/sq) . q8(kg, 1/sk)) * (sq*sk)
//   diagonal block: A[i][j] = sum_n qh[i][n] * kh[j][n] * exp(g[i][n] - g[j][n]),  j <= i,
//     with qh = q8(q*scale, 1/sq) * sq and kh = q8(k, 1/sk) * sk  (fp32 reduction over the dequantized codes)
//   entries above the diagonal are written as zero.
//
// One 4-wave workgroup per (chunk, batch*head); wave w owns the 16 rows of sub-block w.  Off-diagonal
// operands are K-contiguous, so each lane builds its own 16-slot INT8 MFMA operand from plain global loads
// (no LDS).  The diagonal block stages INT8 codes and the decay rows of its 16 tokens in LDS and lets lane
// (i = lane & 15, j-group = lane >> 4) accumulate four (i, j) pairs.
#include "zoo_common.h"
#include "../../include/linquant_hip.h"

namespace {

struct AParams {
  const _Float16* q;
  const _Float16* k;
  const float* g;
  float* A;
  const float* sq;
  const float* sk;
  float scale;
  int qmax;
  int B, T, H;
};

template <int K>
__global__ __launch_bounds__(256) void zoo_gla_A_kernel(AParams p) {
  __shared__ float g_s[4][16][K + 1];
  __shared__ int8_t qd_s[4][16][K + 4];
  __shared__ int8_t kd_s[4][16][K + 4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  const int ct = blockIdx.x;
  const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
  const int H = p.H;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)ct * 64;
  const float sq = p.sq[h], sk = p.sk[h];
  const float inv_sq = 1.0f / sq, inv_sk = 1.0f / sk;
  const int qmax = p.qmax;
  const int i0 = 16 * wave;

  // ---- stage the diagonal block: codes of q*scale and k, decay rows
  for (int it = lane; it < 16 * (K / 8); it += 64) {
    const int r = it / (K / 8), c8 = it % (K / 8);
    const int64_t off = ((t0 + i0 + r) * H + h) * K + 8 * c8;
    const lq_v8h qv = *(const lq_v8h*)(p.q + off);
    const lq_v8h kv = *(const lq_v8h*)(p.k + off);
    const lq_v4f g0 = *(const lq_v4f*)(p.g + off), g1 = *(const lq_v4f*)(p.g + off + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      qd_s[wave][r][8 * c8 + e] = (int8_t)zoo_q8((float)qv[e] * p.scale, inv_sq, qmax);
      kd_s[wave][r][8 * c8 + e] = (int8_t)zoo_q8((float)kv[e], inv_sk, qmax);
      g_s[wave][r][8 * c8 + e] = e < 4 ? g0[e & 3] : g1[e & 3];
    }
  }

  // ---- off-diagonal blocks J < wave (INT8 MFMA on anchored operands)
  lq_v4i acc[3];
#pragma unroll
  for (int J = 0; J < 3; ++J) acc[J] = lq_v4i{0, 0, 0, 0};
  if (wave > 0) {
#pragma unroll
    for (int ks = 0; ks < K / 64; ++ks) {
      const int kk = 64 * ks + 16 * kg;
      float an[16];
      {
        const float* ap = p.g + ((t0 + i0) * H + h) * K + kk;
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
          const lq_v4f a4 = *(const lq_v4f*)(ap + 4 * e4);
#pragma unroll
          for (int e = 0; e < 4; ++e) an[4 * e4 + e] = a4[e];
        }
      }
      lq_v4i qop;
      {
        const int64_t off = ((t0 + i0 + rl) * H + h) * K + kk;
        const lq_v8h q0 = *(const lq_v8h*)(p.q + off), q1 = *(const lq_v8h*)(p.q + off + 8);
        int cd[16];
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
          const lq_v4f g4 = *(const lq_v4f*)(p.g + off + 4 * e4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int n = 4 * e4 + e;
            const float qf = n < 8 ? (float)q0[n & 7] : (float)q1[n & 7];
            float x = qf * lq_expf(g4[e] - an[n]);
            x = x * p.scale;
            cd[n] = zoo_q8(x, inv_sq, qmax);
          }
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) qop[d] = (int)zoo_pack_codes(cd[4 * d], cd[4 * d + 1], cd[4 * d + 2], cd[4 * d + 3]);
      }
#pragma unroll
      for (int J = 0; J < 3; ++J) {
        if (J >= wave) continue;
        const int64_t off = ((t0 + 16 * J + rl) * H + h) * K + kk;
        const lq_v8h k0 = *(const lq_v8h*)(p.k + off), k1 = *(const lq_v8h*)(p.k + off + 8);
        int cd[16];
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
          const lq_v4f g4 = *(const lq_v4f*)(p.g + off + 4 * e4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int n = 4 * e4 + e;
            const float kf = n < 8 ? (float)k0[n & 7] : (float)k1[n & 7];
            cd[n] = zoo_q8(kf * lq_expf(an[n] - g4[e]), inv_sk, qmax);
          }
        }
        lq_v4i kop;
#pragma unroll
        for (int d = 0; d < 4; ++d) kop[d] = (int)zoo_pack_codes(cd[4 * d], cd[4 * d + 1], cd[4 * d + 2], cd[4 * d + 3]);
        acc[J] = lq_mfma_i8(qop, kop, acc[J]);
      }
    }
  }
  const float sqk = sq * sk;
#pragma unroll
  for (int J = 0; J < 3; ++J) {
    if (J >= wave) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r)
      p.A[((t0 + i0 + 4 * kg + r) * H + h) * 64 + 16 * J + rl] = (float)acc[J][r] * sqk;
  }
  // zero blocks above the diagonal
  for (int J = wave + 1; J < 4; ++J)
#pragma unroll
    for (int r = 0; r < 4; ++r) p.A[((t0 + i0 + 4 * kg + r) * H + h) * 64 + 16 * J + rl] = 0.0f;

  __syncthreads();  // staged diagonal rows visible (each wave only reads its own block)

  // ---- diagonal block: lane (i = rl, j = 4kg + jj)
  {
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (int n = 0; n < K; ++n) {
      const float qi = (float)qd_s[wave][rl][n] * sq;
      const float gi = g_s[wave][rl][n];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int j = 4 * kg + jj;
        const float kj = (float)kd_s[wave][j][n] * sk;
        const float w = (j <= rl) ? lq_expf(gi - g_s[wave][j][n]) : 0.0f;
        s[jj] = s[jj] + (qi * kj) * w;
      }
    }
    lq_v4f o;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) o[jj] = (4 * kg + jj <= rl) ? s[jj] : 0.0f;
    *(lq_v4f*)(p.A + ((t0 + i0 + rl) * H + h) * 64 + i0 + 4 * kg) = o;
  }
}

}  // namespace

extern "C" int lq_zoo_gla_A(const lq_zoo_gla_A_args* a, hipStream_t stream) {
  if (!a || !a->q || !a->k || !a->g || !a->A || !a->sq || !a->sk) return LQ_ERR_NULL;
  if (a->rot) return LQ_ERR_SHAPE;  // local R_QK rotation of the anchored operands is not built yet
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  if (a->chunk_size != 64 || a->seqlen % 64 != 0) return LQ_ERR_SHAPE;
  if (a->kdim != 64 && a->kdim != 128) return LQ_ERR_SHAPE;
  if (a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
  if (!zoo_al(a->q, 16) || !zoo_al(a->k, 16) || !zoo_al(a->g, 16) || !zoo_al(a->A, 16)) return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  AParams p = {};
  p.q = (const _Float16*)a->q, p.k = (const _Float16*)a->k, p.g = a->g, p.A = a->A;
  p.sq = a->sq, p.sk = a->sk, p.scale = a->scale, p.qmax = a->qmax;
  p.B = a->batch, p.T = a->seqlen, p.H = a->nheads;
  dim3 grid(a->seqlen / 64, a->batch * a->nheads);
  if (a->kdim == 128)
    hipLaunchKernelGGL(zoo_gla_A_kernel<128>, grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(zoo_gla_A_kernel<64>, grid, dim3(256), 0, stream, p);
  return lq_check_launch();
}
