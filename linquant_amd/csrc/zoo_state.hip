// Zoo state kernels: sequential chunk loop with an fp32 carry and an INT8 stored copy per chunk.
// Replaces the chunk loops of _state_body (linquant/kernels/zoo/simple_gla.py:23-75), _gla_state_body
// (gla.py:102-148), _delta_state_body (gated_delta_rule.py:50-115) and _kda_state_body (kda.py:68-130).
//
// Everything that does not depend on the carried state is prepared by the write-operand pre-pass
// (lq_zoo_write_codes): key write codes kqT (channel-major inside the chunk), value write codes vqT (linear
// family), state-read codes wq (delta family), per-token value factors ev and per-row chunk decays gam.
// Per chunk, in the reference's order:
//   1. hq = q8(h, 1/ss, 127) is stored: the state entering the chunk (read by the output kernel and, delta
//      family, by this chunk's state read);
//   2. delta family: ws = (wq . hq) * sw * ss[v];  E = (U - ws) * fw[t], stored fp16;  eq = q8(E * ev[t], 1/ew[v]);
//   3. h = h * gam[k] + (kqT . eq|vqT) * skw[k] * svw[v].
//
// One 4-wave workgroup per (BV-column V tile, batch*head) holding the whole K axis (the delta state read needs
// the full contraction).  The carry lives in registers: wave w owns K/4 rows.  The stored state goes through
// LDS V-major so that it is copied out coalesced and read back as the K-contiguous operand of the state read;
// the pseudo-value codes go through LDS channel-major so that they are the token-contiguous operand of the
// write product.  All global operands of chunk c+2 are fetched into registers while chunk c is computed.
#include "zoo_params.h"
#include "../../include/linquant_hip.h"

namespace {

using StateParams = ZooStateParams;

template <bool DELTA, int K, int BV>
struct StepOps {
  lq_v4i kop[K / 64];                  // key write codes: rows of this wave, 16 token slots of the lane's group
  lq_v4i vop[DELTA ? 1 : BV / 16];     // linear: value write codes
  lq_v4i wop[DELTA ? K / 64 : 1];      // delta: state-read codes of token 16*wave + (lane & 15)
  uint32_t uraw[DELTA ? BV / 8 : 1];   // delta: U of token 16*wave + (lane >> 2), columns BV/4 * (lane & 3) .. + BV/4 - 1
  // one value per lane of what the wave needs per token and per carry row: lanes 0..15 fw of tokens 16*wave + lane, lanes
  // 16..31 ev of the same tokens (delta family), lanes 32.. the chunk decay of carry rows K/4*wave + lane - 32.  One request
  // instead of ten (each of which every lane of a row group repeated); the values reach the lanes that use them through
  // a wave-private piece of LDS.
  float misc;
};

// BF (bf16 activations) is a template parameter: as a run-time flag every decode / encode of U and E in the chunk loop
// became a branch of its own.
// PAIR (chunks of S = 2 pieces of 64 tokens; the linear family also S = 3, 4, where "first half" below reads "first piece"
// and "second half" "last piece", the pieces between only adding their product): the chunk loop still walks 64-token halves,
// whose operands the pre-pass wrote with the decay to the end of the chunk.  The state is quantized and stored at the first half only (index ct / 2; the delta
// family's second half reads that same stored copy: its W and U come from a WY transform over the 128 tokens), the INT8
// write product of the first half stays in the accumulators that the second half's product adds to, and the carry takes
// decay and product once per chunk: the integer sum over 128 tokens that one 128-token tile gives.
template <bool DELTA, int K, int BV, bool BF, bool PAIR = false>
__global__ __launch_bounds__(256, DELTA ? 1 : 2) void zoo_state_kernel(StateParams p) {
  constexpr int KR = K / 4;     // carry rows per wave
  constexpr int KT = KR / 16;   // 16-row tiles per wave (= K / 64)
  constexpr int VT = BV / 16;   // 16-col tiles
  constexpr int NJ = BV / 16;   // adjacent value columns per lane in the state read
  constexpr int HS = K + 16;    // byte stride of a stored-state row in LDS
  constexpr int ES = 64 + 16;   // byte stride of a pseudo-value code row in LDS
  static_assert(KT == K / 64, "row tiling");

  __shared__ __align__(16) unsigned char hT[(DELTA ? 1 : 2) * BV * HS];
  __shared__ __align__(16) unsigned char eT[DELTA ? BV * ES : 16];
  __shared__ __align__(16) float misc_lds[256];  // 64 floats per wave, written and read by that wave only
  constexpr int US = 2 * BV + 16;  // byte stride of a token row of the wave-private U / E tile (bank-conflict-free column reads)
  __shared__ __align__(16) unsigned char ue_lds[DELTA ? 4 * 16 * US : 16];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  // Workgroups are dealt to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  The V tiles of one
  // (batch, head) read the same key, state-read and decay operands at the same time, so they are renumbered onto one
  // XCD (consecutive slots of it) whenever the grid divides evenly; otherwise each tile fetches its own copy from HBM.
  int vtile = blockIdx.x, bh = blockIdx.y;
  {
    const int nv = gridDim.x, total = gridDim.x * gridDim.y;
    if (total % 8 == 0 && (total / 8) % nv == 0) {
      const int lid = blockIdx.x + nv * blockIdx.y;
      const int vid = (lid % 8) * (total / 8) + lid / 8;
      vtile = vid % nv, bh = vid / nv;
    }
  }
  const int v0 = vtile * BV;
  const int b = bh / p.H, h = bh % p.H;
  const int H = p.H, V = p.V, T = p.T, NT = p.NT;
  const int qmax = p.qmax;
  constexpr bool bf = BF;

  // per-lane scales of the carry tile: rows k = KR*wave + 16kt + 4kg + r, cols v = v0 + 16vt + rl
  float skw_r[KT][4], svw_c[VT], inv_ss_c[VT];
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int r = 0; r < 4; ++r) skw_r[kt][r] = p.skw[h * K + KR * wave + 16 * kt + 4 * kg + r];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) {
    svw_c[vt] = p.svw[h * V + v0 + 16 * vt + rl];
    inv_ss_c[vt] = 1.0f / p.ss[h * V + v0 + 16 * vt + rl];
  }
  // delta state read: value columns v0 + NJ*rl + jj
  float ss_d[NJ], inv_ew_d[NJ], sw = 0.f;
  if (DELTA) {
    sw = p.sw[h];
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj) {
      ss_d[jj] = p.ss[h * V + v0 + NJ * rl + jj];
      inv_ew_d[jj] = 1.0f / p.svw[h * V + v0 + NJ * rl + jj];
    }
  }

  // part: 0 = everything, 1 = key codes, chunk decays and (delta family) per-token factors, 2 = state-read codes and U
  auto load_part = [&](auto part_c, int ct, StepOps<DELTA, K, BV>& o) {
    constexpr int part = decltype(part_c)::value;
    const int64_t cb = ((int64_t)b * NT + ct) * H + h;
    const int64_t t0 = (int64_t)b * T + (int64_t)ct * 64;
    if constexpr (part == 0 || part == 1) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const int row = KR * wave + 16 * kt;
        o.kop[kt] = *(const lq_v4i*)(p.kqT + (cb * K + row + rl) * 64 + 16 * kg);
      }
      if constexpr (!DELTA) o.misc = p.gam[cb * K + KR * wave + min(max(lane - 32, 0), KR - 1)];
      if constexpr (DELTA) {
        const int64_t tr = (t0 + 16 * wave + (lane & 15)) * H + h;
        const float* src = lane < 16 ? p.fw + tr : lane < 32 ? p.ev + tr : p.gam + cb * K + KR * wave + min(lane - 32, KR - 1);
        if (p.pack) {  // the same values, contiguous per (batch, chunk, head): fw[64] | ev[64] | gam[K]
          const float* pk = p.pack + cb * (128 + K);
          src = lane < 32 ? pk + 64 * (lane >> 4) + 16 * wave + (lane & 15) : pk + 128 + KR * wave + min(lane - 32, KR - 1);
        }
        o.misc = *src;
      }
    }
    if constexpr (!DELTA) {
      if constexpr (part == 0 || part == 1)
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) o.vop[vt] = *(const lq_v4i*)(p.vqT + (cb * V + v0 + 16 * vt + rl) * 64 + 16 * kg);
    } else {
      if constexpr (part == 0 || part == 2) {
#pragma unroll
        for (int ks = 0; ks < K / 64; ++ks)
          o.wop[ks] = *(const lq_v4i*)(p.wq + ((t0 + 16 * wave + rl) * H + h) * K + 64 * ks + 16 * kg);
      }
      if constexpr (part == 0 || part == 2) {
        // the wave's 16 x BV tile of U, whole row pieces: lane -> token lane / 4, a quarter of the tile's columns (one request
        // where four requests of a few bytes per lane stood); it reaches the lanes that use it through wave-private LDS
        const _Float16* up = p.u + ((t0 + 16 * wave + (lane >> 2)) * H + h) * V + v0 + (BV / 4) * (lane & 3);
        if constexpr (BV == 64) {
          const lq_v4i a = *(const lq_v4i*)up, c = *(const lq_v4i*)(up + 8);
#pragma unroll
          for (int d = 0; d < 4; ++d) o.uraw[d] = (uint32_t)a[d], o.uraw[4 + d] = (uint32_t)c[d];
        } else if constexpr (BV == 32) {
          const lq_v4i a = *(const lq_v4i*)up;
#pragma unroll
          for (int d = 0; d < 4; ++d) o.uraw[d] = (uint32_t)a[d];
        } else {
          const lq_v2i a = *(const lq_v2i*)up;
          o.uraw[0] = (uint32_t)a[0], o.uraw[1] = (uint32_t)a[1];
        }
      }
    }
  };
  auto load_step = [&](int ct, StepOps<DELTA, K, BV>& o) { load_part(std::integral_constant<int, 0>{}, ct, o); };

  float hc[KT][VT][4];
#pragma unroll
  for (int kt = 0; kt < KT; ++kt)
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int r = 0; r < 4; ++r) hc[kt][vt][r] = 0.0f;

  // One chunk step; the operands of chunk ct + 2 are requested into `pre` at its start.  Vector memory operations
  // retire in issue order, loads and stores alike, so a load issued behind the stores of the previous step is not seen
  // complete before those stores are acknowledged: with one step of look-ahead that acknowledgement sat on the critical
  // path of every step, with two it has a whole step to arrive.
  lq_v4i pend[PAIR ? KT : 1][PAIR ? VT : 1];  // PAIR: the first half's write product
  auto do_step = [&](int ct, StepOps<DELTA, K, BV>& cur, StepOps<DELTA, K, BV>& pre) {
    const int64_t t0 = (int64_t)b * T + (int64_t)ct * 64;
    const int S = PAIR ? p.S : 1;
    const int piece = PAIR ? ct % S : 0;
    const bool second = piece != 0;       // PAIR: a later piece of a chunk (nothing is stored)
    const bool last = piece == S - 1;     // PAIR: the piece after which the carry is updated
    unsigned char* hTb = hT + (DELTA ? 0 : ((PAIR ? ct / S : ct) & 1) * BV * HS);
    float* misc_s = misc_lds + 64 * wave;
    unsigned char* ue_s = ue_lds + wave * 16 * US;
    misc_s[lane] = cur.misc;
    if constexpr (DELTA) {
      unsigned char* ud = ue_s + (lane >> 2) * US + (BV / 2) * (lane & 3);
      if constexpr (BV == 64) {
        *(lq_v4i*)ud = lq_v4i{(int)cur.uraw[0], (int)cur.uraw[1], (int)cur.uraw[2], (int)cur.uraw[3]};
        *(lq_v4i*)(ud + 16) = lq_v4i{(int)cur.uraw[4], (int)cur.uraw[5], (int)cur.uraw[6], (int)cur.uraw[7]};
      } else if constexpr (BV == 32) {
        *(lq_v4i*)ud = lq_v4i{(int)cur.uraw[0], (int)cur.uraw[1], (int)cur.uraw[2], (int)cur.uraw[3]};
      } else {
        *(lq_v2i*)ud = lq_v2i{(int)cur.uraw[0], (int)cur.uraw[1]};
      }
    }
    // ---- stored copy of the incoming state -> LDS (V-major)
    if (!second) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
          int cd[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) cd[r] = zoo_q8(hc[kt][vt][r], inv_ss_c[vt], 127);
          *(uint32_t*)(hTb + (16 * vt + rl) * HS + KR * wave + 16 * kt + 4 * kg) = zoo_pack_codes(cd[0], cd[1], cd[2], cd[3]);
        }
    }
    // requested unconditionally (the last chunks re-request the final one): a branch around the loads would make the
    // compiler's count of outstanding memory operations path-dependent, and it then waits for the newest loads as well
    const int ctn = min(ct + 2, NT - 1);
    if constexpr (DELTA)
      load_part(std::integral_constant<int, 1>{}, ctn, pre);  // (the delta family spreads its requests over the step, below)
    else
      load_step(ctn, pre);
    __syncthreads();

    // the stored state leaves coalesced: h_i8[b][ct][h][v0 + v][k]
    auto copy_out = [&]() {
      int8_t* dst = p.h_i8 + ((((int64_t)b * (PAIR ? NT / S : NT) + (PAIR ? ct / S : ct)) * H + h) * V + v0) * K;
      constexpr int SEG = K / 16;
      if constexpr (BV * SEG % 256 == 0) {
#pragma unroll
        for (int i = 0; i < BV * SEG / 256; ++i) {
          const int it = tid + 256 * i;
          const int vr = it / SEG, sg = it % SEG;
          *(lq_v4i*)(dst + vr * K + sg * 16) = *(const lq_v4i*)(hTb + vr * HS + sg * 16);
        }
      } else {
        for (int it = tid; it < BV * SEG; it += 256) {
          const int vr = it / SEG, sg = it % SEG;
          *(lq_v4i*)(dst + vr * K + sg * 16) = *(const lq_v4i*)(hTb + vr * HS + sg * 16);
        }
      }
    };

    if constexpr (DELTA) {
      // ---- state read against the stored copy, pseudo-values E, their write codes
      lq_v4i aw[NJ];
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) aw[jj] = lq_v4i{0, 0, 0, 0};
#pragma unroll
      for (int ks = 0; ks < K / 64; ++ks)
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) {
          const lq_v4i hop = *(const lq_v4i*)(hTb + (NJ * rl + jj) * HS + 64 * ks + 16 * kg);
          aw[jj] = lq_mfma_i8(cur.wop[ks], hop, aw[jj]);
        }
      // the rest of chunk ct + 2's operands are requested while the matrix unit and then the vector ALU are busy: one wave
      // per SIMD issues in order, and 18 requests in a row held it for as long as the memory pipeline took to accept them
      load_part(std::integral_constant<int, 2>{}, ctn, pre);
      if (!second) copy_out();  // behind the products and the requests: nothing in this step waits for it
      // lane holds tokens 16*wave + 4kg + r, value columns v0 + NJ*rl + jj
      uint32_t ecode[NJ][4];
      const lq_v4f fw4 = *(const lq_v4f*)(misc_s + 4 * kg), ev4 = *(const lq_v4f*)(misc_s + 16 + 4 * kg);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        // U of (token 4kg + r, columns NJ*rl ..) from the wave's tile; E goes back to the same place
        unsigned char* cell = ue_s + (4 * kg + r) * US + 2 * NJ * rl;
        uint32_t uw[2] = {0u, 0u};
        if constexpr (NJ == 4) {
          const lq_v2i uu = *(const lq_v2i*)cell;
          uw[0] = (uint32_t)uu[0], uw[1] = (uint32_t)uu[1];
        } else if constexpr (NJ == 2) {
          uw[0] = *(const uint32_t*)cell;
        } else {
          uw[0] = *(const uint16_t*)cell;
        }
        float ef[NJ];
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj) {
          float ws = (float)aw[jj][r] * sw;
          ws = ws * ss_d[jj];
          const float u = zoo_dec1((uw[jj >> 1] >> (16 * (jj & 1))) & 0xffffu, bf);
          ef[jj] = (u - ws) * fw4[r];
          ecode[jj][r] = (uint32_t)zoo_q8(ef[jj] * ev4[r], inv_ew_d[jj], qmax);
        }
        if constexpr (NJ == 4) {
          lq_v2i eo;
          eo[0] = (int)zoo_enc2(ef[0], ef[1], bf);
          eo[1] = (int)zoo_enc2(ef[2], ef[3], bf);
          *(lq_v2i*)cell = eo;
        } else if constexpr (NJ == 2) {
          *(uint32_t*)cell = zoo_enc2(ef[0], ef[1], bf);
        } else {
          *(uint16_t*)cell = zoo_enc1(ef[0], bf);
        }
      }
      {
        // the wave's E tile leaves as whole row pieces, the way U came in
        const unsigned char* es = ue_s + (lane >> 2) * US + (BV / 2) * (lane & 3);
        _Float16* ep = p.e_out + ((t0 + 16 * wave + (lane >> 2)) * H + h) * V + v0 + (BV / 4) * (lane & 3);
        if constexpr (BV == 64) {
          *(lq_v4i*)ep = *(const lq_v4i*)es;
          *(lq_v4i*)(ep + 8) = *(const lq_v4i*)(es + 16);
        } else if constexpr (BV == 32) {
          *(lq_v4i*)ep = *(const lq_v4i*)es;
        } else {
          *(lq_v2i*)ep = *(const lq_v2i*)es;
        }
      }
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj)
        *(uint32_t*)(eT + (NJ * rl + jj) * ES + 16 * wave + 4 * kg) =
            zoo_pack_codes((int)ecode[jj][0], (int)ecode[jj][1], (int)ecode[jj][2], (int)ecode[jj][3]);
      __syncthreads();
    }

    if constexpr (!DELTA) {
      if (!second) copy_out();
    }

    // ---- write product and carry update
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) {
      lq_v4i bop;
      if constexpr (DELTA)
        bop = *(const lq_v4i*)(eT + (16 * vt + rl) * ES + 16 * kg);
      else
        bop = cur.vop[vt];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        lq_v4i a;
        if constexpr (PAIR) {
          a = lq_mfma_i8(cur.kop[kt], bop, second ? pend[kt][vt] : lq_v4i{0, 0, 0, 0});
          if (!last) {
            pend[kt][vt] = a;
            continue;
          }
        } else {
          a = lq_mfma_i8(cur.kop[kt], bop, lq_v4i{0, 0, 0, 0});
        }
        const lq_v4f gam4 = *(const lq_v4f*)(misc_s + 32 + 16 * kt + 4 * kg);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float prod = (float)a[r] * skw_r[kt][r];
          prod = prod * svw_c[vt];
          hc[kt][vt][r] = hc[kt][vt][r] * gam4[r] + prod;
        }
      }
    }
  };

  StepOps<DELTA, K, BV> s0, s1, s2;
  load_step(0, s0);
  s2 = s1 = s0;
  load_step(min(1, NT - 1), s1);
  // Everything requested so far (scales, the first two operand sets) is waited for here, once.  The compiler places its
  // waits from a count of the memory operations issued after a load; a load still outstanding at loop entry has few
  // operations behind it on the entry path, and the merged count would make every iteration wait until almost nothing
  // is in flight, the look-ahead loads included.
  asm volatile("" ::: "memory");  // keeps the requests above on this side of the wait
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), as an instruction the compiler's own wait placement accounts for
  asm volatile("" ::: "memory");
  // Six steps per trip.  The operand sets rotate with period three; what the compiler cannot do is carry a set that is
  // still being loaded across the loop's back edge without copying it (the copy waits for loads issued only a step
  // earlier), so the back edge is met every sixth step (every twelfth was slower again: instruction cache).
#define LQ_STEP3(base)                   \
  do_step(ct + (base), s0, s2);          \
  if (ct + (base) + 1 >= NT) break;      \
  do_step(ct + (base) + 1, s1, s0);      \
  if (ct + (base) + 2 >= NT) break;      \
  do_step(ct + (base) + 2, s2, s1);      \
  if (ct + (base) + 3 >= NT) break;
  for (int ct = 0; ct < NT; ct += 6) {
    LQ_STEP3(0)
    LQ_STEP3(3)
  }
#undef LQ_STEP3

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

template <bool DELTA, int K>
int launch_bv(const StateParams& p, int BV, int B, hipStream_t stream, bool pair = false) {
  dim3 grid(p.V / BV, B * p.H);
  constexpr bool D = DELTA;  // the linear family touches no half-precision tensor: one instantiation serves both dtypes
#define LQ_STATE_LAUNCH(BVV)                                                                                  \
  do {                                                                                                        \
    if (pair) {                                                                                               \
      if (D && p.bf)                                                                                          \
        hipLaunchKernelGGL((zoo_state_kernel<DELTA, K, BVV, D, true>), grid, dim3(256), 0, stream, p);        \
      else                                                                                                    \
        hipLaunchKernelGGL((zoo_state_kernel<DELTA, K, BVV, false, true>), grid, dim3(256), 0, stream, p);    \
      break;                                                                                                  \
    }                                                                                                         \
    if (D && p.bf)                                                                                            \
      hipLaunchKernelGGL((zoo_state_kernel<DELTA, K, BVV, D>), grid, dim3(256), 0, stream, p);                \
    else                                                                                                      \
      hipLaunchKernelGGL((zoo_state_kernel<DELTA, K, BVV, false>), grid, dim3(256), 0, stream, p);            \
  } while (0)
  if (BV == 64)
    LQ_STATE_LAUNCH(64);
  else if (BV == 32)
    LQ_STATE_LAUNCH(32);
  else
    LQ_STATE_LAUNCH(16);
#undef LQ_STATE_LAUNCH
  return lq_check_launch();
}

}  // namespace

extern "C" int lq_zoo_state(const lq_zoo_state_args* a, hipStream_t stream) {
  if (!a || !a->kqT || !a->gam || !a->h_i8 || !a->skw || !a->svw || !a->ss) return LQ_ERR_NULL;
  const bool delta = a->family == LQ_FAMILY_DELTA;
  if (a->family != LQ_FAMILY_LINEAR && !delta) return LQ_ERR_SHAPE;
  if (delta && (!a->wq || !a->u || !a->fw || !a->ev || !a->e_out || !a->sw)) return LQ_ERR_NULL;
  if (!delta && !a->vqT) return LQ_ERR_NULL;
  if (a->unrot && ((a->vdim != 64 && a->vdim != 128) || !zoo_al(a->unrot, 16))) return LQ_ERR_SHAPE;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  // 128-token chunks run as pairs of 64-token halves; the linear family in rotated storage also takes 192 and 256 tokens
  const bool pair = a->chunk_size == 128 || a->chunk_size == 192 || a->chunk_size == 256;
  if (a->chunk_size > 128 && (delta || a->unrot)) return LQ_ERR_SHAPE;
  if ((a->chunk_size != 64 && !pair) || a->seqlen % a->chunk_size != 0) return LQ_ERR_SHAPE;
  if ((a->kdim != 64 && a->kdim != 128) || a->vdim % 64 != 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  if (a->qmax < 1 || a->qmax > 127) return LQ_ERR_SHAPE;
  if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  if (a->vtile != 0 && a->vtile != 16 && a->vtile != 32 && a->vtile != 64) return LQ_ERR_SHAPE;
  if (!zoo_al(a->kqT, 16) || !zoo_al(a->gam, 16) || !zoo_al(a->h_i8, 16) || (!delta && !zoo_al(a->vqT, 16)) ||
      (delta && (!zoo_al(a->wq, 16) || !zoo_al(a->u, 16) || !zoo_al(a->e_out, 16))))
    return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  StateParams p = {};
  p.kqT = a->kqT, p.vqT = a->vqT, p.wq = a->wq, p.u = (const _Float16*)a->u, p.fw = a->fw, p.ev = a->ev, p.gam = a->gam;
  p.h_i8 = a->h_i8, p.e_out = (_Float16*)a->e_out, p.ht = a->ht;
  p.skw = a->skw, p.svw = a->svw, p.sw = a->sw, p.ss = a->ss, p.qmax = a->qmax, p.bf = a->act_dtype == LQ_DT_BF16;
  p.unrot = (const _Float16*)a->unrot;
  p.pack = a->pack;
  p.T = a->seqlen, p.H = a->nheads, p.V = a->vdim, p.NT = a->seqlen / 64;
  p.S = a->chunk_size / 64;
  if (a->unrot) return zoo_state_unrot_launch(p, delta, a->kdim, a->batch, pair, stream);
  // narrower V tiles when batch*head alone cannot fill the 256 compute units
  int BV = a->vtile;
  if (BV == 0) {
    // measured on 256 compute units: the delta family (two barriers and two dependent products per chunk) is fastest
    // with 32 columns, the linear family with 16, until the grid alone fills the chip
    const int64_t wg64 = (int64_t)a->batch * a->nheads * (a->vdim / 64);
    if (delta)
      BV = wg64 >= 512 ? 64 : 32;
    else
      BV = wg64 >= 1024 ? 64 : (wg64 >= 512 ? 32 : 16);
  }
  if (delta) return a->kdim == 128 ? launch_bv<true, 128>(p, BV, a->batch, stream, pair) : launch_bv<true, 64>(p, BV, a->batch, stream, pair);
  return a->kdim == 128 ? launch_bv<false, 128>(p, BV, a->batch, stream, pair) : launch_bv<false, 64>(p, BV, a->batch, stream, pair);
}
