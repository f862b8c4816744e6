// Intra-chunk product under per-channel (diagonal) decay, 16-token sub-blocks.
// Replaces _gla_A_inter (linquant/kernels/zoo/gla.py:27-63) and _gla_A_intra (gla.py:66-99):
//   off-diagonal block (I > J), anchor a[n] = g[first row of block I][n]:
//     qg = q * exp(g_i - a) * scale,  kg = k * exp(a - g_j)
//     A[i][j] = float(q8(qg, 1/sq) . q8(kg, 1/sk)) * (sq*sk)
//   diagonal block: A[i][j] = sum_n qh[i][n] * kh[j][n] * exp(g[i][n] - g[j][n]),  j <= i,
//     with qh = q8(q*scale, 1/sq) * sq and kh = q8(k, 1/sk) * sk  (fp32 reduction over the dequantized codes)
//   entries above the diagonal are written as zero.
//
// One 4-wave workgroup per (pair of chunks, batch*head); wave w owns sub-block w of the first chunk and then sub-block
// 3 - w of the second one, so every wave does the same amount of off-diagonal work and the rotation is staged once
// for both chunks.  The diagonal block factorizes the decay weight around the block's first row whenever the decay
// spread inside the block allows it and then runs as an fp32 MFMA product; otherwise lane (i = lane & 15, j-group =
// lane >> 4) accumulates four (i, j) pairs with one exponential per (i, j, channel).
// Column-wise: the wave of sub-block J fetches its own rows once (the k and g rows then stay in registers for the whole
// chunk), hands its anchored query codes to the other waves through LDS and builds its key operand once per later
// sub-block I (anchored at I's first row, one operand and one sweep over the rotation at a time), meeting I's query codes
// from LDS on the INT8 MFMA; a lane's 16 INT8 slots per contraction step hold the same channels in the query and the key
// operand, so the dot product is exact whatever the channel -> slot map.
// With a local R_QK (rot, (K,K) fp16, x -> x.R) the anchored off-diagonal operands are rounded to fp16 and rotated
// on the fp16 MFMA before quantization (gla.py:53-57); without one they are quantized as they are built.  The diagonal
// blocks are never rotated.
#include <type_traits>

#include "zoo_params.h"
#include "../../include/linquant_hip.h"

namespace {

struct AParams {
  const _Float16* q;
  const _Float16* k;
  const float* g;
  _Float16* A;
  int8_t* qg;
  const float* sq;
  const float* sk;
  const _Float16* rot;
  const float* dq;  // (H,K) D_QK applied to q at load (q' = act(q * dq)), or nullptr
  float scale;
  int qmax;
  int bf;
  int B, T, H;
};

LQ_DEV float wave_max(float m) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  return m;
}

// Diagonal block, every (i, j, n) weight evaluated on its own and masked before use (any decay spread):
// lane (i = rl, j = 4kg + jj), 8 channels per step.
template <int K, bool BF>
LQ_DEV void diag_exact(const AParams& p, float sq, float sk, float inv_sq, float inv_sk, int rl, int kg, int64_t row0, int h,
                       int i0) {
  const int H = p.H, qmax = p.qmax;
  constexpr bool bf = BF;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  const int64_t irow = ((row0 + rl) * H + h) * K;
  for (int n8 = 0; n8 < K; n8 += 8) {
    float qv[8];
    zoo_ld8(p.q + irow + n8, bf, qv);
    if (p.dq) {
#pragma unroll
      for (int e = 0; e < 8; ++e) qv[e] = zoo_round_act(zoo_mul_rn(qv[e], p.dq[h * K + n8 + e]), bf);
    }
    const lq_v4f gi0 = *(const lq_v4f*)(p.g + irow + n8), gi1 = *(const lq_v4f*)(p.g + irow + n8 + 4);
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int j = 4 * kg + jj;
      const int64_t jrow = ((row0 + j) * H + h) * K;
      float kv[8];
      zoo_ld8(p.k + jrow + n8, bf, kv);
      const lq_v4f gj0 = *(const lq_v4f*)(p.g + jrow + n8), gj1 = *(const lq_v4f*)(p.g + jrow + n8 + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float qh = (float)zoo_q8(qv[e] * p.scale, inv_sq, qmax) * sq;
        const float kh = (float)zoo_q8(kv[e], inv_sk, qmax) * sk;
        const float gi = e < 4 ? gi0[e & 3] : gi1[e & 3], gj = e < 4 ? gj0[e & 3] : gj1[e & 3];
        const float w = (j <= rl) ? zoo_exp(gi - gj) : 0.0f;
        s[jj] = s[jj] + (qh * kh) * w;
      }
    }
  }
  lq_v4f o;
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) o[jj] = (4 * kg + jj <= rl) ? s[jj] : 0.0f;
  {
    lq_v2i oh;
    oh[0] = (int)zoo_pack_h2(o[0], o[1]);
    oh[1] = (int)zoo_pack_h2(o[2], o[3]);
    *(lq_v2i*)(p.A + ((row0 + rl) * H + h) * 64 + i0 + 4 * kg) = oh;
  }
}

// QG: the state-read codes are wanted (p.qg is set); a compile-time flag keeps the own-rows loop
// one basic block.
// DQ: q is rescaled per (head, channel) as it is loaded (a compile-time flag: the kernel sits at its register limit).
template <int K, bool ROT, bool BF, bool QG, bool DQ>
__global__ __launch_bounds__(256, 3) void zoo_gla_A_kernel(AParams p) {
  constexpr int RS = K + 8;  // halves per row of the transposed rotation
  __shared__ __align__(16) _Float16 RT[ROT ? K * RS : 8];  // RT[m][n] = R[n][m]
  // rotated query codes of sub-blocks 1..3 of both chunks: [pass][I - 1][lane][dword]
  __shared__ __align__(16) uint32_t QC[2 * 3 * 64 * (K / 16)];
  __shared__ __align__(16) float DQs[DQ ? K : 4];
  __shared__ __align__(16) float AN[2 * 2 * K];  // first g rows of sub-blocks 2 and 3 of both chunks: [pass][I - 2][channel]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: branches on the sub-block index are scalar
  // Flat grid.  Workgroups are dealt to the 8 XCDs round-robin in launch order and each XCD has its own L2.  Workgroup
  // L = x + 8 m (x = its XCD) takes head m % H of (batch, chunk pair) number x + 8 (m / H): the workgroups resident on one
  // XCD at a time then cover all heads of a few (batch, chunk pair)s, whose rows lie next to each other in memory, and
  // the eight XCDs work on neighbouring chunks at the same time.
  const int npairs = (p.T / 64 + 1) / 2;
  const uint32_t ngroups = (uint32_t)p.B * (uint32_t)npairs;
  uint32_t group, hh;
  if ((ngroups & 7u) == 0) {
    const uint32_t m = blockIdx.x >> 3;
    hh = m % (uint32_t)p.H;
    group = (blockIdx.x & 7u) + 8u * (m / (uint32_t)p.H);
  } else {
    hh = blockIdx.x % (uint32_t)p.H;
    group = blockIdx.x / (uint32_t)p.H;
  }
  const int h = (int)hh;
  const int pair = (int)(group % (uint32_t)npairs), b = (int)(group / (uint32_t)npairs);
  const int H = p.H;
  const float sq = p.sq[h], sk = p.sk[h];
  const float inv_sq = 1.0f / sq, inv_sk = 1.0f / sk;
  const int qmax = p.qmax;
  constexpr bool bf = BF;
  const int nchunks = p.T / 64;

  if constexpr (DQ) {
    if (tid < K) DQs[tid] = p.dq[h * K + tid];
    if constexpr (!ROT) __syncthreads();
  }
  if constexpr (ROT) {
    // lanes walk m (coalesced rows of R), each thread gathers 8 consecutive n and writes one 16-byte piece of a row
    for (int it = tid; it < K * (K / 8); it += 256) {
      const int m = it % K, n8 = it / K;
      lq_v8h rv;
#pragma unroll
      for (int e = 0; e < 8; ++e) rv[e] = p.rot[(int64_t)(8 * n8 + e) * K + m];
      *(lq_v8h*)(RT + m * RS + 8 * n8) = rv;
    }
  }

#pragma unroll 1
  for (int pass = 0; pass < 2; ++pass) {
  const int ct = 2 * pair + pass;
  if (ct >= nchunks) break;  // uniform over the workgroup
  const int blk = pass ? 3 - wave : wave;  // sub-block of this wave in this chunk
  // lane coordinates, made opaque per pass: left visible, every address derived from them is computed once in front of
  // the loop over the two chunks and kept in registers through both (spilled)
  int lane_o = lane;
  asm volatile("" : "+v"(lane_o));
  const int rl = lane_o & 15, kg = lane_o >> 4;
  const int i0 = 16 * blk;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)ct * 64;

  {
    // ---- The wave loads its own sub-block (q, k, g rows) once, in the layout of the rotation
    // operand (lane (rl, kg) = token rl, channels 32ks + 8kg + e), and takes everything that needs those rows from
    // the registers: the state-read codes q*exp(g)*scale, the diagonal block, the query operand anchored at this
    // sub-block's first row (rotated, quantized, handed to the other waves through LDS) and the key operands anchored
    // at the first row of each later sub-block I (rotated, quantized, met with sub-block I's query codes from LDS).
    // The rotation is the transposed product R^T . X^T: lane (rl, kg) receives, for token rl, channels 16mt + 4kg + r,
    // which it packs as dword mt of its INT8 operand; q and k operands share that channel -> slot map, so the INT8
    // dot is exact and a consumer lane needs exactly the dwords the same lane of the producer wave holds.
    constexpr int KS = K / 32, MT = K / 16;
    if (ROT && pass == 0) __syncthreads();  // R^T staged
    const int64_t roff = ((t0 + i0 + rl) * H + h) * K + 8 * kg;
    // One step = 32 channels, 8 per lane, requested one step ahead of its use.  The k and g rows of the sub-block stay in
    // registers for the whole chunk (every key operand of this sub-block, one per later sub-block, is built from them); q
    // and the own anchor row are dropped after their step.  The anchor rows of sub-blocks 2 and 3 pass through LDS (AN) to
    // the waves that need them after the rendezvous.
    lq_v4i kraw[KS];
    lq_v4f gown[KS][2];
    struct Step {
      lq_v4i q;
      lq_v4f a[2];
    };
    auto request = [&](int ks, Step& r) {
      r.q = *(const lq_v4i*)(p.q + roff + 32 * ks);
      kraw[ks] = *(const lq_v4i*)(p.k + roff + 32 * ks);
      const float* gp = p.g + roff + 32 * ks;
      gown[ks][0] = *(const lq_v4f*)gp, gown[ks][1] = *(const lq_v4f*)(gp + 4);
      const float* ap = p.g + ((t0 + i0) * H + h) * K + 32 * ks + 8 * kg;
      r.a[0] = *(const lq_v4f*)ap, r.a[1] = *(const lq_v4f*)(ap + 4);
    };
    auto unpack = [&](const lq_v4i& raw, float (&o)[8]) {
#pragma unroll
      for (int d = 0; d < 4; ++d) zoo_dec2((uint32_t)raw[d], bf, o[2 * d], o[2 * d + 1]);
    };
    // key rows of this sub-block anchored at the first row of a later sub-block (anchor row `an`): fp16 rotation operand
    // x, or, without a rotation, the codes themselves
    auto build_k = [&](auto anchor, lq_v8h (&x)[KS], uint32_t (&c)[MT]) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        lq_v4f an[2];
        anchor(ks, an);
        float kf[8];
        unpack(kraw[ks], kf);
        int ic[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float v = kf[e] * zoo_exp(an[e >> 2][e & 3] - gown[ks][e >> 2][e & 3]);
          if constexpr (ROT)
            x[ks][e] = (_Float16)v;
          else
            ic[e] = zoo_q8(v, inv_sk, qmax);
        }
        if constexpr (!ROT) {
          c[2 * ks] = zoo_pack_codes(ic[0], ic[1], ic[2], ic[3]), c[2 * ks + 1] = zoo_pack_codes(ic[4], ic[5], ic[6], ic[7]);
          // the codes are next used after the loop: without this anchor their arithmetic sinks there and every step's
          // operands stay in registers
          asm volatile("" : "+v"(c[2 * ks]), "+v"(c[2 * ks + 1]));
        }
        __builtin_amdgcn_sched_barrier(0);  // one step after the other
      }
    };
    // one sweep over R^T for one operand; codes of token rl, dword mt = channels 16mt + 4kg + r
    auto sweep = [&](const lq_v8h (&x0)[KS], float inv0, uint32_t (&c0)[MT]) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        lq_v4f r0 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const lq_v8h rop = *(const lq_v8h*)(RT + (16 * mt + rl) * RS + 32 * ks + 8 * kg);
          r0 = lq_mfma_f16(rop, x0[ks], r0);
        }
        c0[mt] = zoo_pack_codes(zoo_q8(r0[0], inv0, qmax), zoo_q8(r0[1], inv0, qmax), zoo_q8(r0[2], inv0, qmax),
                                zoo_q8(r0[3], inv0, qmax));
      }
    };
    const float sqk = sq * sk;
    // key codes of this sub-block against the query codes of sub-block I (from LDS) -> A[rows of I][columns of blk]
    auto meet = [&](int I, const uint32_t (&ck)[MT]) {
      const uint32_t* qc = QC + (((pass * 3 + I - 1) * 64 + lane) * MT);
      lq_v4i acc = {0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < K / 64; ++s) {
        const lq_v4i qop = *(const lq_v4i*)(qc + 4 * s);
        lq_v4i kop;
#pragma unroll
        for (int d = 0; d < 4; ++d) kop[d] = (int)ck[4 * s + d];
        acc = lq_mfma_i8(qop, kop, acc);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        p.A[((t0 + 16 * I + 4 * kg + r) * H + h) * 64 + i0 + rl] = (_Float16)((float)acc[r] * sqk);
    };

    // own rows, fetched once: state-read codes, diagonal block (factorized around the first row while the spread is
    // measured) and the query operand anchored at the sub-block's first row
    lq_v8h x[KS];
    uint32_t cq[MT], ck[MT];
    float spread = 0.0f;
    lq_v4f dacc = {0.f, 0.f, 0.f, 0.f};
    Step st[2];
    request(0, st[0]);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks + 1 < KS) request(ks + 1, st[(ks + 1) & 1]);
      const Step& r = st[ks & 1];
      const lq_v4f(&aown)[2] = r.a;
      float qf[8], kf[8];
      unpack(r.q, qf);
      unpack(kraw[ks], kf);
      if constexpr (DQ) {  // D_QK at load: q' = act(q * D), what the stand-alone rescaling launch would have stored
        const lq_v4f d0 = *(const lq_v4f*)(DQs + 32 * ks + 8 * kg), d1 = *(const lq_v4f*)(DQs + 32 * ks + 8 * kg + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[e] = zoo_round_act(zoo_mul_rn(qf[e], e < 4 ? d0[e & 3] : d1[e & 3]), bf);
      }
      int cs[8], iq[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float gg = gown[ks][e >> 2][e & 3];
        const float d = gg - aown[e >> 2][e & 3];
        spread = fmaxf(spread, __builtin_fabsf(d));
        const float ed = zoo_exp(d);
        const float qh = (float)zoo_q8(qf[e] * p.scale, inv_sq, qmax) * sq;
        const float kh = (float)zoo_q8(kf[e], inv_sk, qmax) * sk;
        dacc = __builtin_amdgcn_mfma_f32_16x16x4f32(qh * ed, kh * zoo_exp(-d), dacc, 0, 0, 0);
        float xv = qf[e] * ed;
        xv = xv * p.scale;
        if constexpr (ROT)
          x[ks][e] = (_Float16)xv;
        else
          iq[e] = zoo_q8(xv, inv_sq, qmax);
        float y = qf[e] * zoo_exp(gg);
        y = y * p.scale;
        cs[e] = zoo_q8(y, inv_sq, qmax);
      }
      if constexpr (QG) {
        lq_v2i o;
        o[0] = (int)zoo_pack_codes(cs[0], cs[1], cs[2], cs[3]);
        o[1] = (int)zoo_pack_codes(cs[4], cs[5], cs[6], cs[7]);
        *(lq_v2i*)(p.qg + roff + 32 * ks) = o;
      }
      if constexpr (!ROT) {
        cq[2 * ks] = zoo_pack_codes(iq[0], iq[1], iq[2], iq[3]), cq[2 * ks + 1] = zoo_pack_codes(iq[4], iq[5], iq[6], iq[7]);
        asm volatile("" : "+v"(cq[2 * ks]), "+v"(cq[2 * ks + 1]));  // as in build_k
      }
      // the diagonal block's accumulator is next used at the end of the chunk: unpinned, its products sink there and
      // their operands wait in registers
      asm volatile("" : "+v"(dacc), "+v"(spread));  // (the running maximum of the decay spread likewise)
      __builtin_amdgcn_sched_barrier(0);  // one step after the other
    }
    if (blk >= 2 && rl == 0) {  // this sub-block's first g row: the anchor of the key operands other waves build later
      float* an = AN + ((pass * 2 + blk - 2) * K + 8 * kg);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) *(lq_v4f*)(an + 32 * ks) = gown[ks][0], *(lq_v4f*)(an + 32 * ks + 4) = gown[ks][1];
    }
    // before the rendezvous: the query codes of this sub-block (none for sub-block 0) go to LDS, and the key codes for
    // the next sub-block (none for sub-block 3) are made, so that every wave arrives with about the same work done
    if (blk > 0) {
      if constexpr (ROT) sweep(x, inv_sq, cq);
      uint32_t* qc = QC + (((pass * 3 + blk - 1) * 64 + lane) * MT);
#pragma unroll
      for (int s = 0; s < MT / 4; ++s) {
        lq_v4i o;
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = (int)cq[4 * s + d];
        *(lq_v4i*)(qc + 4 * s) = o;
      }
    }
    if (blk < 3) {
      // (anchor row from memory, one step ahead: the sub-block that owns it has not been through the rendezvous yet)
      const float* ap = p.g + ((t0 + 16 * (blk + 1)) * H + h) * K + 8 * kg;
      lq_v4f nx[2][2];
      nx[0][0] = *(const lq_v4f*)ap, nx[0][1] = *(const lq_v4f*)(ap + 4);
      build_k(
          [&](int ks, lq_v4f (&an)[2]) {
            if (ks + 1 < KS) nx[(ks + 1) & 1][0] = *(const lq_v4f*)(ap + 32 * (ks + 1)), nx[(ks + 1) & 1][1] = *(const lq_v4f*)(ap + 32 * (ks + 1) + 4);
            an[0] = nx[ks & 1][0], an[1] = nx[ks & 1][1];
          },
          x, ck);
      if constexpr (ROT) sweep(x, inv_sk, ck);
    }
    __syncthreads();  // query codes of the chunk are in LDS (the two passes use separate buffers)
    if (blk < 3) meet(blk + 1, ck);
    // key operands for the sub-blocks after the next one, from the rows still in registers
#pragma unroll 1
    for (int I = blk + 2; I < 4; ++I) {
      const float* an_s = AN + ((pass * 2 + I - 2) * K + 8 * kg);
      build_k([&](int ks, lq_v4f (&an)[2]) { an[0] = *(const lq_v4f*)(an_s + 32 * ks), an[1] = *(const lq_v4f*)(an_s + 32 * ks + 4); }, x, ck);
      if constexpr (ROT) sweep(x, inv_sk, ck);
      meet(I, ck);
    }
    // diagonal block, last: its rare exact path is kept away from the registers of the sweeps
    spread = wave_max(spread);
    if (spread <= 40.0f) {
      // lane holds column j = rl, rows i = 4kg + r
#pragma unroll
      for (int r = 0; r < 4; ++r)
        p.A[((t0 + i0 + 4 * kg + r) * H + h) * 64 + i0 + rl] = (_Float16)((rl <= 4 * kg + r) ? dacc[r] : 0.0f);
    } else {
      diag_exact<K, BF>(p, sq, sk, inv_sq, inv_sk, rl, kg, t0 + i0, h, i0);  // (applies p.dq itself)
    }
  }
  // zero blocks above the diagonal
  for (int J = blk + 1; J < 4; ++J)
#pragma unroll
    for (int r = 0; r < 4; ++r) p.A[((t0 + i0 + 4 * kg + r) * H + h) * 64 + 16 * J + rl] = (_Float16)0.0f;
  }  // pass
}

}  // namespace

extern "C" int lq_zoo_gla_A(const lq_zoo_gla_A_args* a, hipStream_t stream) {
  if (!a || !a->q || !a->k || !a->g || !a->A || !a->sq || !a->sk) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  // 128-token chunks: the blocks inside either half are those of 64-token chunks (g cumulated over the 128 tokens), the
  // blocks between the halves come from a second launch into A_cross
  const bool pair = a->chunk_size == 128;
  if (pair && !a->A_cross) return LQ_ERR_NULL;
  if (pair && !zoo_al(a->A_cross, 16)) return LQ_ERR_SHAPE;
  if ((a->chunk_size != 64 && !pair) || a->seqlen % a->chunk_size != 0) return LQ_ERR_SHAPE;
  if (a->kdim != 64 && a->kdim != 128) return LQ_ERR_SHAPE;
  if (a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
  if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  if (!zoo_al(a->q, 16) || !zoo_al(a->k, 16) || !zoo_al(a->g, 16) || !zoo_al(a->A, 16) || (a->qg && !zoo_al(a->qg, 8)))
    return LQ_ERR_SHAPE;
  if (a->rot && !zoo_al(a->rot, 16)) return LQ_ERR_SHAPE;
  if (a->dq && !zoo_al(a->dq, 16)) return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  AParams p = {};
  p.q = (const _Float16*)a->q, p.k = (const _Float16*)a->k, p.g = a->g, p.A = (_Float16*)a->A, p.qg = a->qg;
  p.dq = a->dq;
  p.sq = a->sq, p.sk = a->sk, p.rot = (const _Float16*)a->rot, p.scale = a->scale, p.qmax = a->qmax, p.bf = a->act_dtype == LQ_DT_BF16;
  p.B = a->batch, p.T = a->seqlen, p.H = a->nheads;
  if ((int64_t)((a->seqlen / 64 + 1) / 2) * a->batch * a->nheads > 0x7fffffff) return LQ_ERR_SHAPE;
  dim3 grid((uint32_t)(((a->seqlen / 64 + 1) / 2) * a->batch * a->nheads));
#define LQ_A_LAUNCH3(KV, ROTV, BFV, QGV)                                                                   \
  do {                                                                                                     \
    if (p.dq)                                                                                              \
      hipLaunchKernelGGL((zoo_gla_A_kernel<KV, ROTV, BFV, QGV, true>), grid, dim3(256), 0, stream, p);     \
    else                                                                                                   \
      hipLaunchKernelGGL((zoo_gla_A_kernel<KV, ROTV, BFV, QGV, false>), grid, dim3(256), 0, stream, p);    \
  } while (0)
#define LQ_A_LAUNCH2(KV, ROTV, QGV)                                                                        \
  do {                                                                                                     \
    if (p.bf)                                                                                              \
      LQ_A_LAUNCH3(KV, ROTV, true, QGV);                                                                   \
    else                                                                                                   \
      LQ_A_LAUNCH3(KV, ROTV, false, QGV);                                                                  \
  } while (0)
#define LQ_A_LAUNCH(KV)                 \
  do {                                  \
    if (a->rot && p.qg)                 \
      LQ_A_LAUNCH2(KV, true, true);     \
    else if (a->rot)                    \
      LQ_A_LAUNCH2(KV, true, false);    \
    else if (p.qg)                      \
      LQ_A_LAUNCH2(KV, false, true);    \
    else                                \
      LQ_A_LAUNCH2(KV, false, false);   \
  } while (0)
  if (a->kdim == 128)
    LQ_A_LAUNCH(128);
  else
    LQ_A_LAUNCH(64);
#undef LQ_A_LAUNCH3
#undef LQ_A_LAUNCH2
#undef LQ_A_LAUNCH
  if (pair) {
    const int rc = lq_check_launch();
    if (rc) return rc;
    ZooACrossParams c = {};
    c.q = p.q, c.k = p.k, c.g = p.g, c.Ax = (_Float16*)a->A_cross, c.sq = p.sq, c.sk = p.sk, c.rot = p.rot, c.dq = p.dq;
    c.scale = p.scale, c.qmax = p.qmax, c.bf = p.bf, c.B = p.B, c.T = p.T, c.H = p.H;
    return zoo_gla_A_cross_launch(c, a->kdim, stream);
  }
  return lq_check_launch();
}
