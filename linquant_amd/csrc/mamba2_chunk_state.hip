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
// One wavefront per (64-row P tile, <=128-col N tile, batch*chunk, head); the whole K = chunk loop runs in
// registers.  Both operands are stored token-major in HBM while the MFMA wants 16 contraction slots per
// lane, so each lane loads, for its 16 tokens, the 4 adjacent channels {4*(lane&15)+j}: 16 lanes cover one
// contiguous 128-byte row, and packing "along tokens" yields the operand of MFMA call j directly.  Tile
// row i of call j is therefore channel 4*i+j; the accumulator layout then gives every lane 4 adjacent
// output columns, which are packed into one 32-bit store.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

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
  int8_t* states;
  int batch, seqlen, nheads, P, G, N, Q, nchunks, n_ntiles;
};

template <bool KEYSIDE, int NH>
__global__ __launch_bounds__(64) void chunk_state_kernel(Params p) {
  const int lane = threadIdx.x, rl = lane & 15, kg = lane >> 4;
  const int ptile = blockIdx.x / p.n_ntiles, ntile = blockIdx.x % p.n_ntiles;
  const int b = blockIdx.y / p.nchunks, c = blockIdx.y % p.nchunks;
  const int h = blockIdx.z;
  const int g = h / (p.nheads / p.G);
  const int p0 = ptile * 64, n0 = ntile * (64 * NH);
  const int Q = p.Q;
  const int limit = min(Q, p.seqlen - c * Q);

  const _Float16* xp = p.x + (int64_t)b * p.sx_b + (int64_t)c * Q * p.sx_l + (int64_t)h * p.sx_h + p0 + 4 * rl;
  const int64_t tok0 = (int64_t)c * Q;
  const int64_t cs = (((int64_t)b * p.nheads + h) * p.nchunks + c) * Q;
  const float* dtp = p.dt + cs;
  const float* dAp = p.dA + cs;
  const float dA_last = dAp[Q - 1];

  // per-lane operand scales for the 4 channels p0 + 4*rl + j
  float xinv[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float s = p.xs[(int64_t)h * p.sxs_h + (int64_t)(p0 + 4 * rl + j) * p.sxs_p];
    xinv[j] = KEYSIDE ? 1.0f / fmaxf(s, 1e-10f) : 1.0f / s;
  }
  float bgate[NH][4], binv[NH][4];
  if (KEYSIDE) {
#pragma unroll
    for (int hf = 0; hf < NH; ++hf)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int n = n0 + 64 * hf + 4 * rl + jj;
        bgate[hf][jj] = p.bgs[(int64_t)b * p.sbg_b + (int64_t)c * p.sbg_c + (int64_t)h * p.sbg_h + (int64_t)n * p.sbg_n];
        binv[hf][jj] = 127.0f / bgate[hf][jj];
      }
  }

  lq_v4i acc[4][NH * 4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int q = 0; q < NH * 4; ++q) acc[j][q] = lq_v4i{0, 0, 0, 0};

  for (int k0 = 0; k0 < Q; k0 += 64) {
    const int kb = k0 + kg * 16;
    float gate[16];
#pragma unroll
    for (int t4 = 0; t4 < 4; ++t4) {
      const float4 a4 = *(const float4*)(dAp + kb + 4 * t4);
      const float4 d4 = *(const float4*)(dtp + kb + 4 * t4);
      gate[4 * t4 + 0] = lq_expf(dA_last - a4.x) * d4.x;
      gate[4 * t4 + 1] = lq_expf(dA_last - a4.y) * d4.y;
      gate[4 * t4 + 2] = lq_expf(dA_last - a4.z) * d4.z;
      gate[4 * t4 + 3] = lq_expf(dA_last - a4.w) * d4.w;
    }
    // ---- x operand: 16 tokens x 4 channels per lane
    lq_v2i xw[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      xw[t] = lq_v2i{0, 0};
      if (kb + t < limit) xw[t] = *(const lq_v2i*)(xp + (int64_t)(kb + t) * p.sx_l);
    }
    lq_v4i aop[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int code[16];
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const uint32_t w = (uint32_t)xw[t][j >> 1];
        const _Float16 hv = __builtin_bit_cast(_Float16, (uint16_t)(j & 1 ? w >> 16 : w & 0xffff));
        float y = (float)hv * xinv[j];
        if (KEYSIDE) {
          code[t] = lq_q_rint(y, -127, 127);
        } else {
          y = y * gate[t];
          code[t] = lq_q_rha(y, 127);
        }
      }
#pragma unroll
      for (int d = 0; d < 4; ++d) aop[j][d] = (int)lq_pack4(code[4 * d], code[4 * d + 1], code[4 * d + 2], code[4 * d + 3]);
    }
    // ---- B operand per 64-column half
#pragma unroll
    for (int hf = 0; hf < NH; ++hf) {
      lq_v4i bop[4];
      if (KEYSIDE) {
        const _Float16* bp = (const _Float16*)p.B + (int64_t)b * p.sB_b + (int64_t)g * p.sB_g + n0 + 64 * hf + 4 * rl;
        lq_v2i bw[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          bw[t] = lq_v2i{0, 0};
          if (kb + t < limit) bw[t] = *(const lq_v2i*)(bp + (tok0 + kb + t) * p.sB_l);
        }
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          int code[16];
#pragma unroll
          for (int t = 0; t < 16; ++t) {
            const uint32_t w = (uint32_t)bw[t][jj >> 1];
            const _Float16 hv = __builtin_bit_cast(_Float16, (uint16_t)(jj & 1 ? w >> 16 : w & 0xffff));
            float y = (float)hv * gate[t];
            y = y * binv[hf][jj];
            code[t] = lq_q_rint(y, -127, 127);
          }
#pragma unroll
          for (int d = 0; d < 4; ++d)
            bop[jj][d] = (int)lq_pack4(code[4 * d], code[4 * d + 1], code[4 * d + 2], code[4 * d + 3]);
        }
      } else {
        const int8_t* bp = (const int8_t*)p.B + (int64_t)b * p.sB_b + (int64_t)g * p.sB_g + n0 + 64 * hf + 4 * rl;
        uint32_t bw[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
          bw[t] = 0;
          if (kb + t < limit) bw[t] = *(const uint32_t*)(bp + (tok0 + kb + t) * p.sB_l);
        }
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            // byte jj of four consecutive tokens -> one operand dword
            const uint32_t lo = __builtin_amdgcn_perm(bw[4 * d + 1], bw[4 * d + 0], 0x0c0c0400u + 0x0101u * jj);
            const uint32_t hi = __builtin_amdgcn_perm(bw[4 * d + 3], bw[4 * d + 2], 0x0c0c0400u + 0x0101u * jj);
            bop[jj][d] = (int)(lo | (hi << 16));
          }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) acc[j][hf * 4 + jj] = lq_mfma_i8(aop[j], bop[jj], acc[j][hf * 4 + jj]);
    }
  }

  // ---- epilogue: requantize and store 4 adjacent columns per 32-bit store
  int8_t* sp = p.states + ((((int64_t)b * p.nchunks + c) * p.nheads + h) * p.P) * p.N;
  const float bscale = KEYSIDE ? 0.0f : p.bscale_g[(int64_t)g * p.sbs_g];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int pr = p0 + 16 * kg + 4 * r + j;
      const float xs = p.xs[(int64_t)h * p.sxs_h + (int64_t)pr * p.sxs_p];
      const float so = p.oqs[(int64_t)h * p.soq_h + (int64_t)pr * p.soq_p];
      const float ratio = xs / so;
#pragma unroll
      for (int hf = 0; hf < NH; ++hf) {
        int code[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const float a = (float)acc[j][hf * 4 + jj][r];
          if (KEYSIDE) {
            float y = a * (bgate[hf][jj] / 127.0f);
            y = y * ratio;
            code[jj] = lq_q_rint(y, -127, 127);
          } else {
            code[jj] = lq_q_rha(a * (ratio * bscale), 127);
          }
        }
        *(uint32_t*)(sp + (int64_t)pr * p.N + n0 + 64 * hf + 4 * rl) = lq_pack4(code[0], code[1], code[2], code[3]);
      }
    }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

template <bool KEYSIDE>
int launch(const Params& p, hipStream_t stream) {
  if (p.batch <= 0 || p.seqlen <= 0 || p.nheads <= 0 || p.G <= 0 || p.nheads % p.G != 0) return LQ_ERR_SHAPE;
  if (p.P % 64 != 0 || p.N % 64 != 0 || p.Q % 64 != 0 || p.Q < 64) return LQ_ERR_SHAPE;
  if (p.sx_b % 4 || p.sx_l % 4 || p.sx_h % 4 || !al(p.x, 8)) return LQ_ERR_SHAPE;
  const int balign = KEYSIDE ? 8 : 4;
  if (p.sB_b % 4 || p.sB_l % 4 || p.sB_g % 4 || !al(p.B, balign)) return LQ_ERR_SHAPE;
  if (!al(p.dt, 16) || !al(p.dA, 16) || !al(p.states, 4)) return LQ_ERR_SHAPE;
  const int64_t by = (int64_t)p.batch * p.nchunks;
  if (by > 65535 || p.nheads > 65535) return LQ_ERR_SHAPE;
  Params q = p;
  if (p.N % 128 == 0) {
    q.n_ntiles = p.N / 128;
    dim3 grid((p.P / 64) * q.n_ntiles, (unsigned)by, p.nheads);
    hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 2>), grid, dim3(64), 0, stream, q);
  } else {
    q.n_ntiles = p.N / 64;
    dim3 grid((p.P / 64) * q.n_ntiles, (unsigned)by, p.nheads);
    hipLaunchKernelGGL((chunk_state_kernel<KEYSIDE, 1>), grid, dim3(64), 0, stream, q);
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
  p.states = a->states;
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
  p.sbg_b = a->bgs_stride_b, p.sbg_c = a->bgs_stride_c, p.sbg_h = a->bgs_stride_h, p.sbg_n = a->bgs_stride_n;
  p.states = a->states;
  p.batch = a->batch, p.seqlen = a->seqlen, p.nheads = a->nheads, p.P = a->headdim, p.G = a->ngroups, p.N = a->dstate;
  p.Q = a->chunk_size;
  if (p.Q <= 0) return LQ_ERR_SHAPE;
  p.nchunks = (p.seqlen + p.Q - 1) / p.Q;
  return launch<true>(p, stream);
}
