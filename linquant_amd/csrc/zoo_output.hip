// Zoo output kernels: o = state read + intra-chunk local product, fully parallel over chunks.
// Replaces _output_body (linquant/kernels/zoo/simple_gla.py:98-153) and _gla_output_body (gla.py:170-213).
//
//   no / scalar decay:  qq = q8(q*scale, 1/sq), kq = q8(k, 1/sk)
//                       of = float(qq . h_i8) * sq * ss[v] [* exp(g_i)]
//                       Af = float(qq . kq^T) * (sq*sk) [* exp(g_i - g_j)], zero above the diagonal
//   diagonal decay:     qq = q8(q*exp(g)*scale, 1/sq);  of = float(qq . h_i8) * sq * ss[v];  Af = A (fp32 input)
//   both:               o  = of + (fp16(Af) . fp16(q8(v, 1/svl))) * svl[v]
//
// One 4-wave workgroup per (one or two 64-column V tiles, chunk, batch*head); wave w owns rows 16w..16w+15 of the
// chunk.  With two tiles (V a multiple of 128) the q / k codes and the A tile are made once for both.
// q / k codes are produced once per workgroup into LDS (K-contiguous rows: plain 16-byte INT8 MFMA operands);
// the stored state is V-major in HBM, so its operand is a plain 16-byte global load.  The local value
// operand goes to LDS as token-pair interleaved fp16 (dword = two consecutive tokens of one channel), the
// same layout trick as the Mamba-2 chunk scan: four 16-byte reads give the operands of the four MFMA calls
// that cover channels {4*(lane&15)+j}, and every lane ends up with 4 adjacent output channels.
#include "zoo_params.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int BV = 64;
constexpr int kAS = 72;  // halves per row of the fp16 A tile in LDS
constexpr int kVW = 68;  // dwords per token-pair row of the value tile

using OutParams = ZooOutParams;

// NV: 64-column V tiles per workgroup (2 when V is a multiple of 128: the q / k codes and the A tile are then made once
// for both tiles)
// CIN: the local codes of q, k, v arrive ready-made (lq_zoo_rotate_quant made them): they are copied into the same LDS
// tiles instead of being quantized here.
// CROSS (chunks of S = 2..4 pieces of 64 tokens; described for S = 2, where it runs once: launch j of S - 1 gives piece
// s >= j its product with the tokens of piece j - 1, adding to what launch j - 1 left, oldest tokens first): this launch
// makes, for the second half of every chunk,
// the part of the local product that reaches back into the first half -- fp16(Af[i][j]) . fp16(q8(v_j)) over the 64 tokens j
// of the first half, no causal mask, no state read; under per-channel decay Af comes from p.Ax -- and leaves it as fp32 in p.cross; the ordinary launch that follows
// starts its local accumulators from it (one fp32 accumulation over the 128 tokens, oldest first, as a 128-token tile has).
template <bool GLA, bool USE_G, int K, bool BF, int NV, bool CIN, bool CROSS = false>
__global__ __launch_bounds__(256, 2) void zoo_output_kernel(OutParams p) {
  static_assert(!CROSS || !CIN, "the cross launch exists for raw operands");
  constexpr int QS = K + 16;  // byte stride of a code row
  __shared__ __align__(16) unsigned char qc[GLA ? 16 : 64 * QS];
  __shared__ __align__(16) unsigned char kc[GLA ? 16 : 64 * QS];
  __shared__ __align__(16) _Float16 Afl[GLA ? 8 : 64 * kAS];
  __shared__ __align__(16) uint32_t vP[NV * 32 * kVW];
  __shared__ float g_s[64];
  __shared__ float gk_s[CROSS ? 64 : 1];  // cross launch: cumulative log decay of the first half's tokens

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  // Workgroups go to the 8 XCDs round-robin by linear id and each XCD has its own L2: the V tiles of one (chunk,
  // batch, head) read the same q / k / A rows, so they are renumbered onto one XCD when the grid divides evenly.
  int vtile = blockIdx.x, ct = blockIdx.y, bh = blockIdx.z;
  {
    const int nv = gridDim.x, total = gridDim.x * gridDim.y * gridDim.z;
    if (nv > 1 && total % 8 == 0 && (total / 8) % nv == 0) {
      const int lid = blockIdx.x + nv * (blockIdx.y + gridDim.y * blockIdx.z);
      const int vid = (lid % 8) * (total / 8) + lid / 8;
      vtile = vid % nv;
      ct = (vid / nv) % gridDim.y;
      bh = vid / (nv * gridDim.y);
    }
  }
  const int piece = ct % p.S;  // which 64-token piece of its chunk
  if constexpr (CROSS) {
    if (piece < p.cross_j) return;  // (uniform over the workgroup, in front of every barrier)
  }
  const int v0 = vtile * BV * NV;
  const int b = bh / p.H, h = bh % p.H;
  const int H = p.H, V = p.V;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)ct * 64;
  // first token of the keys / values this launch contracts against
  const int64_t tk0 = CROSS ? t0 - (int64_t)(piece - p.cross_j + 1) * 64 : t0;
  const float sq = p.sq[h];
  const float inv_sq = 1.0f / sq;
  const float sk = GLA ? 1.0f : p.sk[h];
  const float inv_sk = 1.0f / sk;
  const int qmax = p.qmax;
  constexpr bool bf = BF;

  // ---- every global request of the workgroup is issued here, before the first use and outside any branch, oldest first
  // in the order of use.  (Issued where they were used they formed a chain of about nine exposed round trips: one per
  // iteration of the code loop, one for v, one per contraction step of the state read, one per scale vector.)
  constexpr int NQ = K / 32;  // 16-byte pieces of q (and of k) per thread: 64 tokens x K / 8 pieces over 256 threads
  lq_v4i qraw[GLA ? 1 : NQ], kraw[GLA ? 1 : NQ];
  if constexpr (!GLA && !CIN) {
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
      const int it = tid + 256 * i;
      const int t = it / (K / 8), c8 = it % (K / 8);
      const int64_t off = ((t0 + t) * H + h) * K + 8 * c8;
      qraw[i] = *(const lq_v4i*)(p.q + off);
      kraw[i] = *(const lq_v4i*)(p.k + off + (tk0 - t0) * H * K);
    }
  }
  if constexpr (!GLA && CIN) {  // 16 codes per piece: half as many pieces
#pragma unroll
    for (int i = 0; i < NQ / 2; ++i) {
      const int it = tid + 256 * i;
      const int t = it / (K / 16), c16 = it % (K / 16);
      const int64_t off = ((t0 + t) * H + h) * K + 16 * c16;
      qraw[i] = *(const lq_v4i*)(p.qc + off);
      kraw[i] = *(const lq_v4i*)(p.kc + off);
    }
  }
  const int tp = tid >> 3, c8v = tid & 7;  // value tile: 32 token pairs x 8 groups of 8 channels
  const int64_t voff = ((tk0 + 2 * tp) * H + h) * V + v0 + 8 * c8v;
  lq_v4i va_raw[NV], vb_raw[NV];
  lq_v4f sv0[NV], sv1[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    if constexpr (CIN) {  // eight codes per token: the low two dwords of the raw registers
      const lq_v2i ca = *(const lq_v2i*)(p.vc + voff + BV * n), cb2 = *(const lq_v2i*)(p.vc + voff + BV * n + (int64_t)H * V);
      va_raw[n] = lq_v4i{ca[0], ca[1], 0, 0}, vb_raw[n] = lq_v4i{cb2[0], cb2[1], 0, 0};
    } else {
      va_raw[n] = *(const lq_v4i*)(p.v + voff + BV * n), vb_raw[n] = *(const lq_v4i*)(p.v + voff + BV * n + (int64_t)H * V);
      sv0[n] = *(const lq_v4f*)(p.svl + h * V + v0 + BV * n + 8 * c8v), sv1[n] = *(const lq_v4f*)(p.svl + h * V + v0 + BV * n + 8 * c8v + 4);
    }
  }
  const float g_raw = (USE_G && !GLA) ? p.g[(t0 + (tid & 63)) * H + h] : 0.0f;
  const float gk_raw = (USE_G && CROSS) ? p.g[(tk0 + (tid & 63)) * H + h] : 0.0f;
  // (128-token chunks: one stored state per chunk, read by both halves)
  const int8_t* hp = p.h_i8 + ((((int64_t)b * (p.NT / p.S) + ct / p.S) * H + h) * V + v0) * K;
  lq_v4i hop[CROSS ? 1 : NV][K / 64][4];
  lq_v4i qgop[GLA ? K / 64 : 1];
#pragma unroll
  for (int ks = 0; ks < K / 64; ++ks) {
    if constexpr (GLA && !CROSS) qgop[ks] = *(const lq_v4i*)(p.qg + ((t0 + 16 * wave + rl) * H + h) * K + 64 * ks + 16 * kg);
    if constexpr (!CROSS) {
#pragma unroll
      for (int n = 0; n < NV; ++n)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) hop[n][ks][jj] = *(const lq_v4i*)(hp + (BV * n + 4 * rl + jj) * K + 64 * ks + 16 * kg);
    }
  }
  lq_v4f ss4[NV], svl4[NV];
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    ss4[n] = *(const lq_v4f*)(p.ss + h * V + v0 + BV * n + 4 * rl);
    svl4[n] = *(const lq_v4f*)(p.svl + h * V + v0 + BV * n + 4 * rl);
  }

  // ---- phase 1: q (and k) codes -> LDS, value codes -> LDS (fp16, token-pair interleaved)
  if constexpr (!GLA && CIN) {
#pragma unroll
    for (int i = 0; i < NQ / 2; ++i) {
      const int it = tid + 256 * i;
      const int t = it / (K / 16), c16 = it % (K / 16);
      *(lq_v4i*)(qc + t * QS + 16 * c16) = qraw[i];
      *(lq_v4i*)(kc + t * QS + 16 * c16) = kraw[i];
    }
  }
  if constexpr (!GLA && !CIN) {
#pragma unroll
    for (int i = 0; i < NQ; ++i) {
      const int it = tid + 256 * i;
      const int t = it / (K / 8), c8 = it % (K / 8);
      lq_v2i oq, ok;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        int cq[4], ck[4];
#pragma unroll
        for (int d = 0; d < 2; ++d) {
          float q0, q1, k0, k1;
          zoo_dec2((uint32_t)qraw[i][2 * hf + d], bf, q0, q1);
          zoo_dec2((uint32_t)kraw[i][2 * hf + d], bf, k0, k1);
          cq[2 * d] = zoo_q8(q0 * p.scale, inv_sq, qmax), cq[2 * d + 1] = zoo_q8(q1 * p.scale, inv_sq, qmax);
          ck[2 * d] = zoo_q8(k0, inv_sk, qmax), ck[2 * d + 1] = zoo_q8(k1, inv_sk, qmax);
        }
        oq[hf] = (int)zoo_pack_codes(cq[0], cq[1], cq[2], cq[3]);
        ok[hf] = (int)zoo_pack_codes(ck[0], ck[1], ck[2], ck[3]);
      }
      *(lq_v2i*)(qc + t * QS + 8 * c8) = oq;
      *(lq_v2i*)(kc + t * QS + 8 * c8) = ok;
    }
  }
#pragma unroll
  for (int n = 0; n < NV; ++n) {
    lq_v4i o0, o1;
    if constexpr (CIN) {  // codes -> exact fp16, token pair per dword
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int ca = lq_sbyte((uint32_t)va_raw[n][e >> 2], e & 3), cb2 = lq_sbyte((uint32_t)vb_raw[n][e >> 2], e & 3);
        const int w = (int)zoo_pack_h2((float)ca, (float)cb2);
        if (e < 4) o0[e] = w; else o1[e - 4] = w;
      }
    } else {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      float a0, a1, b0, b1;
      zoo_dec2((uint32_t)va_raw[n][d], bf, a0, a1);
      zoo_dec2((uint32_t)vb_raw[n][d], bf, b0, b1);
      const float s0 = d < 2 ? sv0[n][2 * d] : sv1[n][2 * d - 4], s1 = d < 2 ? sv0[n][2 * d + 1] : sv1[n][2 * d - 3];
      const float i0 = 1.0f / s0, i1 = 1.0f / s1;
      const int w0 = (int)zoo_pack_h2((float)zoo_q8(a0, i0, qmax), (float)zoo_q8(b0, i0, qmax));
      const int w1 = (int)zoo_pack_h2((float)zoo_q8(a1, i1, qmax), (float)zoo_q8(b1, i1, qmax));
      if (d < 2) o0[2 * d] = w0, o0[2 * d + 1] = w1; else o1[2 * d - 4] = w0, o1[2 * d - 3] = w1;
    }
    }
    *(lq_v4i*)(vP + (32 * n + tp) * kVW + 8 * c8v) = o0;
    *(lq_v4i*)(vP + (32 * n + tp) * kVW + 8 * c8v + 4) = o1;
  }
  if (USE_G && !GLA) g_s[tid & 63] = g_raw;  // four threads per token write the same value
  if constexpr (USE_G && CROSS) gk_s[tid & 63] = gk_raw;
  __syncthreads();

  // ---- phase 2: INT8 contractions of this wave's 16 rows
  lq_v4i o32[CROSS ? 1 : NV][4];
  if constexpr (!CROSS) {
#pragma unroll
    for (int n = 0; n < NV; ++n)
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) o32[n][jj] = lq_v4i{0, 0, 0, 0};
  }
  lq_v4i a32[4];
#pragma unroll
  for (int jt = 0; jt < 4; ++jt) a32[jt] = lq_v4i{0, 0, 0, 0};
#pragma unroll
  for (int ks = 0; ks < K / 64; ++ks) {
    lq_v4i qop = {0, 0, 0, 0};
    if constexpr (GLA && CROSS)
      break;  // nothing to contract: A arrives ready-made, the state is not read
    else if constexpr (GLA)
      qop = qgop[ks];
    else
      qop = *(const lq_v4i*)(qc + (16 * wave + rl) * QS + 64 * ks + 16 * kg);
    if constexpr (!CROSS) {
#pragma unroll
      for (int n = 0; n < NV; ++n)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) o32[n][jj] = lq_mfma_i8(qop, hop[n][ks][jj], o32[n][jj]);
    }
    if (!GLA) {
#pragma unroll
      for (int jt = 0; jt < 4; ++jt) {
        if (!CROSS && jt > wave) continue;  // strictly above the diagonal (wave-uniform)
        const lq_v4i kop = *(const lq_v4i*)(kc + (16 * jt + rl) * QS + 64 * ks + 16 * kg);
        a32[jt] = lq_mfma_i8(qop, kop, a32[jt]);
      }
    }
  }

  // ---- phase 3: dequantize; A -> fp16 in operand layout
  float of[CROSS ? 1 : NV][4][4];  // [tile][jj][r]: rows 16w + 4kg + r, channels v0 + 64 tile + 4rl + jj
  if constexpr (!CROSS) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float eg = (USE_G && !GLA) ? zoo_exp(g_s[16 * wave + 4 * kg + r]) : 1.0f;
#pragma unroll
      for (int n = 0; n < NV; ++n)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          float x = (float)o32[n][jj][r] * sq;
          x = x * ss4[n][jj];
          of[n][jj][r] = (USE_G && !GLA) ? x * eg : x;
        }
    }
  }
  if (!GLA) {
    const float sqk = sq * sk;
#pragma unroll
    for (int jt = 0; jt < 4; ++jt) {
      if (!CROSS && jt > wave + 1) continue;
      const int j = 16 * jt + rl;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * wave + 4 * kg + r;
        float x = 0.0f;
        if constexpr (CROSS) {  // every token of the first half precedes every row: the whole block, its decay from gk_s
          x = (float)a32[jt][r] * sqk;
          if (USE_G) x = x * zoo_exp(g_s[i] - gk_s[j]);
        } else if (jt <= wave && j <= i) {
          x = (float)a32[jt][r] * sqk;
          if (USE_G) x = x * zoo_exp(g_s[i] - g_s[j]);
        }
        Afl[i * kAS + j] = (_Float16)x;
      }
    }
    __syncthreads();
  }

  // ---- phase 4: local product on the fp16 MFMA and store
  lq_v4f loc[NV][4];
#pragma unroll
  for (int n = 0; n < NV; ++n)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) loc[n][jj] = lq_v4f{0.f, 0.f, 0.f, 0.f};
  {
    // later piece of a chunk: what the cross launch(es) left for these rows
    if (CROSS ? p.cross_j > 1 : (p.cross != nullptr && piece != 0)) {
#pragma unroll
      for (int n = 0; n < NV; ++n)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const lq_v4f c4 = *(const lq_v4f*)(p.cross + ((t0 + 16 * wave + 4 * kg + r) * H + h) * V + v0 + BV * n + 4 * rl);
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) loc[n][jj][r] = c4[jj];
        }
    }
  }
  const int nslab = CROSS ? 2 : (16 * wave + 15) / 32 + 1;
  for (int js = 0; js < nslab; ++js) {
    lq_v8h aop;
    if (GLA) {
      aop = *(const lq_v8h*)((CROSS ? p.Ax : p.A) + ((t0 + 16 * wave + rl) * H + h) * 64 + 32 * js + 8 * kg);
    } else {
      aop = *(const lq_v8h*)(Afl + (16 * wave + rl) * kAS + 32 * js + 8 * kg);
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      lq_v4i xop[4];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const lq_v4i vv = *(const lq_v4i*)(vP + (32 * n + 16 * js + 4 * kg + d) * kVW + 4 * rl);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) xop[jj][d] = vv[jj];
      }
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) loc[n][jj] = lq_mfma_f16(aop, __builtin_bit_cast(lq_v8h, xop[jj]), loc[n][jj]);
    }
  }
#pragma unroll
  for (int n = 0; n < NV; ++n)
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int64_t off = ((t0 + 16 * wave + 4 * kg + r) * H + h) * V + v0 + BV * n + 4 * rl;
    if constexpr (CROSS) {
      *(lq_v4f*)(p.cross + off) = lq_v4f{loc[n][0][r], loc[n][1][r], loc[n][2][r], loc[n][3][r]};
    } else {
      float res[4];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) res[jj] = of[n][jj][r] + loc[n][jj][r] * svl4[n][jj];
      if (p.o_is_f32) {
        __builtin_nontemporal_store(lq_v4f{res[0], res[1], res[2], res[3]}, (lq_v4f*)((float*)p.o + off));
      } else {
        lq_v2i w;
        w[0] = (int)zoo_enc2(res[0], res[1], bf);
        w[1] = (int)zoo_enc2(res[2], res[3], bf);
        __builtin_nontemporal_store(w, (lq_v2i*)((_Float16*)p.o + off));
      }
    }
  }
}

template <bool GLA, bool USE_G, int K, int NV>
void launch_cross(const OutParams& p, dim3 grid, hipStream_t stream) {
  if (p.bf)
    hipLaunchKernelGGL((zoo_output_kernel<GLA, USE_G, K, true, NV, false, true>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_output_kernel<GLA, USE_G, K, false, NV, false, true>), grid, dim3(256), 0, stream, p);
}

template <bool GLA, bool USE_G, int K, int NV>
void launch_bf(const OutParams& p, dim3 grid, hipStream_t stream) {
  if (p.cross) {
    OutParams c = p;
    for (c.cross_j = 1; c.cross_j < p.S; ++c.cross_j) launch_cross<GLA, USE_G, K, NV>(c, grid, stream);
  }
  if constexpr (!GLA) {
    if (p.qc) {  // ready-made codes: the activation dtype only matters for a 16-bit output
      if (p.bf)
        hipLaunchKernelGGL((zoo_output_kernel<GLA, USE_G, K, true, NV, true>), grid, dim3(256), 0, stream, p);
      else
        hipLaunchKernelGGL((zoo_output_kernel<GLA, USE_G, K, false, NV, true>), grid, dim3(256), 0, stream, p);
      return;
    }
  }
  if (p.bf)
    hipLaunchKernelGGL((zoo_output_kernel<GLA, USE_G, K, true, NV, false>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_output_kernel<GLA, USE_G, K, false, NV, false>), grid, dim3(256), 0, stream, p);
}

// the cross launch alone (canonical storage: the local product is formed in the rotated basis there too, so its first-half
// part comes from this kernel and the un-rotating kernel starts from it)
template <bool GLA, bool USE_G>
int launch_cross_only(const OutParams& p, int K, hipStream_t stream) {
  const bool two = p.V % (2 * BV) == 0;
  const dim3 grid(p.V / (two ? 2 * BV : BV), p.NT, p.B * p.H);
  OutParams c = p;
  c.cross_j = 1;  // (canonical storage: two pieces per chunk)
  if (K == 128) {
    if (two) launch_cross<GLA, USE_G, 128, 2>(c, grid, stream); else launch_cross<GLA, USE_G, 128, 1>(c, grid, stream);
  } else {
    if (two) launch_cross<GLA, USE_G, 64, 2>(c, grid, stream); else launch_cross<GLA, USE_G, 64, 1>(c, grid, stream);
  }
  return lq_check_launch();
}

template <bool GLA, bool USE_G>
int launch(const OutParams& p, int K, hipStream_t stream) {
  const bool two = p.V % (2 * BV) == 0;  // two V tiles per workgroup
  const dim3 grid(p.V / (two ? 2 * BV : BV), p.NT, p.B * p.H);
  if (K == 128) {
    if (two)
      launch_bf<GLA, USE_G, 128, 2>(p, grid, stream);
    else
      launch_bf<GLA, USE_G, 128, 1>(p, grid, stream);
  } else {
    if (two)
      launch_bf<GLA, USE_G, 64, 2>(p, grid, stream);
    else
      launch_bf<GLA, USE_G, 64, 1>(p, grid, stream);
  }
  return lq_check_launch();
}

}  // namespace

extern "C" int lq_zoo_output(const lq_zoo_output_args* a, hipStream_t stream) {
  if (!a || !a->h_i8 || !a->o || !a->sq || !a->svl || !a->ss) return LQ_ERR_NULL;
  const bool gla = a->decay == LQ_DECAY_DIAGONAL;
  const bool cin = a->qc != nullptr;  // ready-made local codes of q, k, v (no / scalar decay, rotated storage)
  if (cin && (gla || a->unrot || !a->kc || !a->vc || !a->sk)) return LQ_ERR_NULL;
  if (!cin && !a->v) return LQ_ERR_NULL;
  if (gla && (!a->A || !a->qg)) return LQ_ERR_NULL;
  if (!gla && !cin && (!a->q || !a->k || !a->sk)) return LQ_ERR_NULL;
  if (a->decay == LQ_DECAY_SCALAR && !a->g) return LQ_ERR_NULL;
  if (a->decay < 0 || a->decay > 2) return LQ_ERR_SHAPE;
  if (a->unrot && ((a->vdim != 64 && a->vdim != 128) || !zoo_al(a->unrot, 16))) return LQ_ERR_SHAPE;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  // chunks of 128 tokens (raw operands) run as pairs of 64-token halves; no / scalar decay in rotated storage also as
  // three or four pieces (192, 256 tokens)
  const bool pair = a->chunk_size == 128 || a->chunk_size == 192 || a->chunk_size == 256;
  if (pair && cin) return LQ_ERR_SHAPE;
  if (a->chunk_size > 128 && (gla || a->unrot)) return LQ_ERR_SHAPE;
  if (pair && (!a->cross || (gla && !a->A_cross))) return LQ_ERR_NULL;
  if (pair && (!zoo_al(a->cross, 16) || (gla && !zoo_al(a->A_cross, 16)))) return LQ_ERR_SHAPE;
  if ((a->chunk_size != 64 && !pair) || a->seqlen % a->chunk_size != 0) return LQ_ERR_SHAPE;
  if ((a->kdim != 64 && a->kdim != 128) || a->vdim % 64 != 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  if (a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
  if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  if ((a->q && !zoo_al(a->q, 16)) || (a->qg && !zoo_al(a->qg, 16)) || (a->A && !zoo_al(a->A, 16)) || (a->k && !zoo_al(a->k, 16)) || (a->v && !zoo_al(a->v, 16)) || !zoo_al(a->h_i8, 16) || !zoo_al(a->o, 16) || !zoo_al(a->ss, 16) || !zoo_al(a->svl, 16))
    return LQ_ERR_SHAPE;
  if (cin && (!zoo_al(a->qc, 16) || !zoo_al(a->kc, 16) || !zoo_al(a->vc, 8))) return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535 || a->seqlen / 64 > 65535) return LQ_ERR_SHAPE;
  OutParams p = {};
  p.q = (const _Float16*)a->q, p.k = (const _Float16*)a->k, p.v = (const _Float16*)a->v;
  p.h_i8 = a->h_i8, p.g = a->g, p.A = (const _Float16*)a->A, p.qg = a->qg, p.o = a->o, p.o_is_f32 = a->o_is_f32;
  p.sq = a->sq, p.sk = a->sk, p.svl = a->svl, p.ss = a->ss, p.scale = a->scale, p.qmax = a->qmax, p.bf = a->act_dtype == LQ_DT_BF16;
  p.B = a->batch, p.T = a->seqlen, p.H = a->nheads, p.V = a->vdim, p.NT = a->seqlen / 64;
  p.unrot = (const _Float16*)a->unrot;
  p.qc = a->qc, p.kc = a->kc, p.vc = a->vc;
  p.cross = pair ? a->cross : nullptr, p.S = a->chunk_size / 64, p.cross_j = 0;
  p.Ax = pair ? (const _Float16*)a->A_cross : nullptr;
  if (a->unrot) {
    if (pair) {
      const int rc = gla ? launch_cross_only<true, true>(p, a->kdim, stream)
                         : (a->decay == LQ_DECAY_SCALAR ? launch_cross_only<false, true>(p, a->kdim, stream)
                                                        : launch_cross_only<false, false>(p, a->kdim, stream));
      if (rc) return rc;
    }
    return zoo_output_unrot_launch(p, a->decay, a->kdim, stream);
  }
  if (gla) return launch<true, true>(p, a->kdim, stream);
  if (a->decay == LQ_DECAY_SCALAR) return launch<false, true>(p, a->kdim, stream);
  return launch<false, false>(p, a->kdim, stream);
}
