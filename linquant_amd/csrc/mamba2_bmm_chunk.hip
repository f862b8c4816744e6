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

typedef uint32_t lq_v2u __attribute__((ext_vector_type(2)));

// clamp to [-127, 127] then round half even; returns a dword whose low byte is the INT8 code
LQ_DEV uint32_t rint_code(float y) {
  const float c = __builtin_amdgcn_fmed3f(y, -127.0f, 127.0f);
  return __float_as_uint(c + 12582912.0f);
}

LQ_DEV uint32_t pack_low_bytes(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uint32_t lo = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);  // {a.b0, b.b0, 0, 0}
  const uint32_t hi = __builtin_amdgcn_perm(d, c, 0x04000c0cu);  // {0, 0, c.b0, d.b0}
  return lo | hi;
}

// One wavefront per 64 x 64 output tile.  N64 = N / 64 contraction steps, all of whose operands are requested before
// the first is used, from clamped (always valid) rows: a request inside `if (row < limit)` is waited for where the
// branches join, and a run-time loop over N put a second memory round trip behind the first.  Rows past the sequence
// end are zeroed after the fact.  The epilogue transposes each lane's 4 x 4 block of code dwords across the four lane
// groups so that a lane stores 16 contiguous bytes: 4 stores per lane instead of 16, 64 contiguous bytes per row.
template <bool B_IS_FP, int N64>
__global__ __launch_bounds__(64, 2) void bmm_chunk_kernel(const int8_t* __restrict__ a, int64_t sa_b, int64_t sa_l,
                                                       int64_t sa_g, const void* __restrict__ bv, int64_t sb_b,
                                                       int64_t sb_l, int64_t sb_g, const float* __restrict__ a_scale,
                                                       const float* __restrict__ b_scale,
                                                       const float* __restrict__ cb_scale, int8_t* __restrict__ out,
                                                       int seqlen, int G, int Q, int nchunks, uint32_t tiles_magic,
                                                       uint32_t g_magic, uint32_t tpc, uint32_t tpc_magic, uint32_t ncg,
                                                       uint32_t ncg_magic, int by_xcd) {
  const int lane = threadIdx.x, rl = lane & 15, kg = lane >> 4;
  // floor(2^32 / d) + 1 multipliers (0 for d == 1) stand in for the run-time divisions (exact while x * d < 2^32, which
  // the launcher checks).
  // Workgroups are dealt to the 8 XCDs round-robin in launch order, and the tpc tiles of one (batch, chunk, group) read
  // the same C and B rows: with consecutive workgroups on consecutive tiles every XCD's L2 fetched those rows from HBM
  // for itself (33.7 MB read for 12.6 MB of operands).  Workgroup 8 j + x takes tile j % tpc of unit 8 (j / tpc) + x, so
  // a unit's tiles run on one XCD, one after the other.
  uint32_t unit, tile;
  if (by_xcd) {
    const uint32_t x = blockIdx.x & 7u, j = blockIdx.x >> 3;
    const uint32_t uh = tpc_magic ? __umulhi(j, tpc_magic) : j;
    tile = j - uh * tpc, unit = uh * 8u + x;
  } else {
    unit = tpc_magic ? __umulhi(blockIdx.x, tpc_magic) : blockIdx.x;
    tile = blockIdx.x - unit * tpc;
  }
  const int mt64 = tiles_magic ? (int)__umulhi(tile, tiles_magic) : (int)tile;
  const int kt64 = (int)tile - mt64 * (Q >> 6);
  const int b = ncg_magic ? (int)__umulhi(unit, ncg_magic) : (int)unit;
  const uint32_t cg = unit - (uint32_t)b * ncg;
  const int c = g_magic ? (int)__umulhi(cg, g_magic) : (int)cg;
  const int g = (int)cg - c * G;
  const int limit = min(Q, seqlen - c * Q);
  const float a_sc = a_scale[g], b_sc = b_scale[g], cb_sc = cb_scale[g];

  const int8_t* ap = a + (int64_t)b * sa_b + (int64_t)c * Q * sa_l + (int64_t)g * sa_g;
  const char* bp = (const char*)bv + ((int64_t)b * sb_b + (int64_t)c * Q * sb_l + (int64_t)g * sb_g) * (B_IS_FP ? 2 : 1);
  const uint32_t sal = (uint32_t)sa_l, sbl = (uint32_t)sb_l * (B_IS_FP ? 2u : 1u);
  lq_v4i cop[N64][4], braw[N64][4][B_IS_FP ? 2 : 1];
  bool mlive[4], klive[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = mt64 * 64 + i * 16 + rl, k = kt64 * 64 + i * 16 + rl;
    mlive[i] = m < limit, klive[i] = k < limit;
    const uint32_t mo = __umul24((uint32_t)min(m, limit - 1), sal) + (uint32_t)kg * 16u;
    const uint32_t ko = __umul24((uint32_t)min(k, limit - 1), sbl) + (uint32_t)kg * (B_IS_FP ? 32u : 16u);
#pragma unroll
    for (int n = 0; n < N64; ++n) {
      cop[n][i] = *(const lq_v4i*)(ap + mo + 64u * n);
      braw[n][i][0] = *(const lq_v4i*)(bp + ko + (B_IS_FP ? 128u : 64u) * n);
      if (B_IS_FP) braw[n][i][1] = *(const lq_v4i*)(bp + ko + 128u * n + 16u);
    }
  }
  const float b_inv = 1.0f / b_sc;
  const float inv_scb = (a_sc * b_sc) / cb_sc;

  lq_v4i acc[4][4];  // [k tile][m tile]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = lq_v4i{0, 0, 0, 0};
#pragma unroll
  for (int n = 0; n < N64; ++n) {
    lq_v4i bop[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (!mlive[i]) cop[n][i] = lq_v4i{0, 0, 0, 0};
      if (B_IS_FP) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const lq_v8h hv = __builtin_bit_cast(lq_v8h, braw[n][i][d >> 1]);
          uint32_t cd[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) cd[e] = rint_code((float)hv[4 * (d & 1) + e] * b_inv);
          bop[i][d] = (int)pack_low_bytes(cd[0], cd[1], cd[2], cd[3]);
        }
      } else {
        bop[i] = braw[n][i][0];
      }
      if (!klive[i]) bop[i] = lq_v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = lq_mfma_i8(bop[i], cop[n][j], acc[i][j]);
  }

  int8_t* op = out + ((((int64_t)b * nchunks + c) * G + g) * Q) * Q + (int64_t)(mt64 * 64) * Q + kt64 * 64;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    // accumulator rows = k (4 consecutive per lane: k = 16 i + 4 kg + r), column = m = 16 j + rl
    uint32_t d[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t cd[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) cd[r] = rint_code((float)acc[i][j][r] * inv_scb);
      d[i] = pack_low_bytes(cd[0], cd[1], cd[2], cd[3]);
    }
    // dword i of lane group kg covers k = 16 i + 4 kg ..: transposing register index with lane group leaves lane group
    // kg with the four dwords of k = 16 kg .. 16 kg + 15
    lq_v2u t;
    t = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false), d[0] = t[0], d[2] = t[1];
    t = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false), d[1] = t[0], d[3] = t[1];
    t = __builtin_amdgcn_permlane16_swap(d[0], d[1], false, false), d[0] = t[0], d[1] = t[1];
    t = __builtin_amdgcn_permlane16_swap(d[2], d[3], false, false), d[2] = t[0], d[3] = t[1];
    *(lq_v4i*)(op + (uint32_t)((16 * j + rl) * Q + 16 * kg)) = lq_v4i{(int)d[0], (int)d[1], (int)d[2], (int)d[3]};
  }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

}  // namespace

extern "C" int lq_bmm_chunk(const lq_bmm_chunk_args* a, hipStream_t stream) {
  if (!a || !a->a || !a->b || !a->a_scale || !a->b_scale || !a->cb_scale || !a->out) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->ngroups <= 0 || a->batch > 65535) return LQ_ERR_SHAPE;
  const int Q = a->chunk_size, N = a->dstate;
  if (Q < 64 || Q % 64 != 0 || Q > 4096 || N < 64 || N % 64 != 0 || N > 256) return LQ_ERR_SHAPE;
  if (a->a_stride_b % 16 || a->a_stride_l % 16 || a->a_stride_g % 16 || !al(a->a, 16)) return LQ_ERR_SHAPE;
  const int bal = 16;  // 16 int8 or 8 fp16 per vector load
  const int bmod = a->b_is_fp ? 8 : 16;
  if (a->b_stride_b % bmod || a->b_stride_l % bmod || a->b_stride_g % bmod || !al(a->b, bal) || !al(a->out, 16))
    return LQ_ERR_SHAPE;
  // 24-bit row * pitch products and 32-bit lane offsets inside a chunk
  if (a->a_stride_l < 0 || a->b_stride_l < 0 || a->a_stride_l >= (1 << 23) || a->b_stride_l >= (1 << 22) ||
      (int64_t)Q * a->a_stride_l >= (1ll << 31) || (int64_t)Q * a->b_stride_l * 2 >= (1ll << 31))
    return LQ_ERR_SHAPE;
  const int nchunks = (a->seqlen + Q - 1) / Q;
  if ((int64_t)nchunks * a->ngroups > 65535) return LQ_ERR_SHAPE;
  const uint32_t shift = Q == 64 ? 0u : (uint32_t)(0x100000000ull / (uint32_t)(Q / 64)) + 1u;  // tiles per row, as a multiplier
  const uint32_t g_magic = a->ngroups == 1 ? 0u : (uint32_t)(0x100000000ull / (uint32_t)a->ngroups) + 1u;
  const uint32_t tpc = (uint32_t)((Q / 64) * (Q / 64)), ncg = (uint32_t)(nchunks * a->ngroups);
  const uint64_t units = (uint64_t)a->batch * ncg, total = units * tpc;
  if (total >= (1ull << 31) || total * tpc >= (1ull << 32) || units * ncg >= (1ull << 32)) return LQ_ERR_SHAPE;
  auto magic = [](uint32_t d) { return d == 1 ? 0u : (uint32_t)(0x100000000ull / d) + 1u; };
  const int by_xcd = units % 8 == 0;
  dim3 grid((unsigned)total);
#define LQ_BMM_LAUNCH(FP, NN)                                                                                              \
  hipLaunchKernelGGL((bmm_chunk_kernel<FP, NN>), grid, dim3(64), 0, stream, a->a, a->a_stride_b, a->a_stride_l,            \
                     a->a_stride_g, a->b, a->b_stride_b, a->b_stride_l, a->b_stride_g, a->a_scale, a->b_scale, a->cb_scale, \
                     a->out, a->seqlen, a->ngroups, Q, nchunks, shift, g_magic, tpc, magic(tpc), ncg, magic(ncg), by_xcd)
  switch (N / 64) {
    case 1: if (a->b_is_fp) LQ_BMM_LAUNCH(true, 1); else LQ_BMM_LAUNCH(false, 1); break;
    case 2: if (a->b_is_fp) LQ_BMM_LAUNCH(true, 2); else LQ_BMM_LAUNCH(false, 2); break;
    case 3: if (a->b_is_fp) LQ_BMM_LAUNCH(true, 3); else LQ_BMM_LAUNCH(false, 3); break;
    default: if (a->b_is_fp) LQ_BMM_LAUNCH(true, 4); else LQ_BMM_LAUNCH(false, 4); break;
  }
#undef LQ_BMM_LAUNCH
  return lq_check_launch();
}
