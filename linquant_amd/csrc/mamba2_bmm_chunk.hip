// Mamba-2 SSD stage 4: INT8 C.B^T per (batch, chunk, group), requantized to INT8 on a static scale.
// Replaces linquant/kernels/mamba2/bmm_chunk.py:49-139 (launcher :142-217):
//   acc = C_i8[m,:] . B_i8[k,:]        (key side: B_i8 = clamp(rint(B_fp * (1/sB)), +-127) in-loop)
//   CB_i8[m,k] = clamp(rint(float(acc) * ((sC*sB)/S_cb)), +-127)      full QxQ, no causal mask here.
//
// Both operands are contraction-contiguous (N is the unit-stride axis), so MFMA operands are plain
// 16-byte loads.  One wavefront computes a 64x64 output tile as the transposed product (rows = B tokens,
// cols = C tokens) so that every lane ends up with 4 consecutive k of one m: one 32-bit store each.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

template <bool B_IS_FP>
__global__ __launch_bounds__(64, 2) void bmm_chunk_kernel(const int8_t* __restrict__ a, int64_t sa_b, int64_t sa_l,
                                                       int64_t sa_g, const void* __restrict__ bv, int64_t sb_b,
                                                       int64_t sb_l, int64_t sb_g, const float* __restrict__ a_scale,
                                                       const float* __restrict__ b_scale,
                                                       const float* __restrict__ cb_scale, int8_t* __restrict__ out,
                                                       int seqlen, int G, int N, int Q, int nchunks) {
  const int lane = threadIdx.x, rl = lane & 15, kg = lane >> 4;
  const int tiles = Q >> 6;
  const int mt64 = blockIdx.x / tiles, kt64 = blockIdx.x % tiles;
  const int b = blockIdx.y;
  const int c = blockIdx.z / G, g = blockIdx.z % G;
  const int limit = min(Q, seqlen - c * Q);
  const float a_sc = a_scale[g], b_sc = b_scale[g];
  const float b_inv = 1.0f / b_sc;

  lq_v4i acc[4][4];  // [k tile][m tile]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = lq_v4i{0, 0, 0, 0};

  const int8_t* ap = a + (int64_t)b * sa_b + (int64_t)c * Q * sa_l + (int64_t)g * sa_g;
  for (int n0 = 0; n0 < N; n0 += 64) {
    const int nn = n0 + kg * 16;
    lq_v4i cop[4], bop[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = mt64 * 64 + i * 16 + rl;
      cop[i] = lq_v4i{0, 0, 0, 0};
      if (m < limit) cop[i] = *(const lq_v4i*)(ap + (int64_t)m * sa_l + nn);
      const int k = kt64 * 64 + i * 16 + rl;
      bop[i] = lq_v4i{0, 0, 0, 0};
      if (k < limit) {
        if (B_IS_FP) {
          const _Float16* bp = (const _Float16*)bv + (int64_t)b * sb_b + ((int64_t)c * Q + k) * sb_l + (int64_t)g * sb_g + nn;
          const lq_v8h h0 = *(const lq_v8h*)bp;
          const lq_v8h h1 = *(const lq_v8h*)(bp + 8);
          int code[16];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            code[e] = lq_q_rint((float)h0[e] * b_inv, -127, 127);
            code[8 + e] = lq_q_rint((float)h1[e] * b_inv, -127, 127);
          }
#pragma unroll
          for (int d = 0; d < 4; ++d)
            bop[i][d] = (int)lq_pack4(code[4 * d], code[4 * d + 1], code[4 * d + 2], code[4 * d + 3]);
        } else {
          const int8_t* bp = (const int8_t*)bv + (int64_t)b * sb_b + ((int64_t)c * Q + k) * sb_l + (int64_t)g * sb_g + nn;
          bop[i] = *(const lq_v4i*)bp;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = lq_mfma_i8(bop[i], cop[j], acc[i][j]);
  }

  const float inv_scb = (a_sc * b_sc) / cb_scale[g];
  int8_t* op = out + ((((int64_t)b * nchunks + c) * G + g) * Q) * Q;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // accumulator rows = k (4 consecutive per lane), column = m
      const int m = mt64 * 64 + j * 16 + rl;
      const int k = kt64 * 64 + i * 16 + 4 * kg;
      int code[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) code[r] = lq_q_rint((float)acc[i][j][r] * inv_scb, -127, 127);
      *(uint32_t*)(op + (int64_t)m * Q + k) = lq_pack4(code[0], code[1], code[2], code[3]);
    }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

}  // namespace

extern "C" int lq_bmm_chunk(const lq_bmm_chunk_args* a, hipStream_t stream) {
  if (!a || !a->a || !a->b || !a->a_scale || !a->b_scale || !a->cb_scale || !a->out) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->ngroups <= 0 || a->batch > 65535) return LQ_ERR_SHAPE;
  const int Q = a->chunk_size, N = a->dstate;
  if (Q < 64 || Q % 64 != 0 || N < 64 || N % 64 != 0) return LQ_ERR_SHAPE;
  if (a->a_stride_b % 16 || a->a_stride_l % 16 || a->a_stride_g % 16 || !al(a->a, 16)) return LQ_ERR_SHAPE;
  const int bal = 16;  // 16 int8 or 8 fp16 per vector load
  const int bmod = a->b_is_fp ? 8 : 16;
  if (a->b_stride_b % bmod || a->b_stride_l % bmod || a->b_stride_g % bmod || !al(a->b, bal) || !al(a->out, 4))
    return LQ_ERR_SHAPE;
  const int nchunks = (a->seqlen + Q - 1) / Q;
  if ((int64_t)nchunks * a->ngroups > 65535) return LQ_ERR_SHAPE;
  dim3 grid((Q / 64) * (Q / 64), a->batch, nchunks * a->ngroups);
  if (a->b_is_fp)
    hipLaunchKernelGGL((bmm_chunk_kernel<true>), grid, dim3(64), 0, stream, a->a, a->a_stride_b, a->a_stride_l,
                       a->a_stride_g, a->b, a->b_stride_b, a->b_stride_l, a->b_stride_g, a->a_scale, a->b_scale,
                       a->cb_scale, a->out, a->seqlen, a->ngroups, N, Q, nchunks);
  else
    hipLaunchKernelGGL((bmm_chunk_kernel<false>), grid, dim3(64), 0, stream, a->a, a->a_stride_b, a->a_stride_l,
                       a->a_stride_g, a->b, a->b_stride_b, a->b_stride_l, a->b_stride_g, a->a_scale, a->b_scale,
                       a->cb_scale, a->out, a->seqlen, a->ngroups, N, Q, nchunks);
  return lq_check_launch();
}
