// Stages behind the Mamba-2 SSD: gated RMSNorm and the Hadamard + INT8 quantizer of the out_proj input.
//   lq_rmsnorm_gated       replaces `self.norm(y, z)` at linquant/quantized_mamba2.py:354-358 (RMSNormGated,
//                          norm_before_gate = False, group_size = d_ssm / ngroups, fp16 gate)
//   lq_qhad_transform      replaces qhad_transform (linquant/hadamard_utils.py:9-19): Hadamard of the row, scale,
//                          round half away, saturate to +-127 (patches/ssdi8.patch:101-112)
//   lq_rmsnorm_gated_qhad  both in one launch (linquant/quantized_mamba2.py:354-364 with d_mlp = 0)
//
// One wave per row, one row per workgroup.  A row of dim = 128 g channels is a g x 128 matrix X (chunk c, position
// i); the transform is had (g x g, any +-1 matrix) across chunks times the Sylvester H_128 inside a chunk:
//   stage 0  16-byte loads; optional gate + group RMS statistics in fp32; the fp16 row goes to LDS with the values of two
//            adjacent chunks at one position sharing a dword (v_permlane16_swap pairs them up in registers)
//   stage 1  D1[i, c'] = sum_c X[c, i] had[c', c]      fp16 MFMA 16x16x32, fp32 accumulate (+-1 times fp16 is exact)
//   stage 2  D2 = H_16 . D1 over the low four bits of i  fp32 MFMA 16x16x4: the accumulator layout of stage 1 (column
//            = lane & 15, rows 4 (lane >> 4) + r) is the B-operand layout of this product with contraction slot 4 kg + r
//            in step r, so nothing moves between lanes
//   stage 3  H_8 over the high three bits of i: the eight 16-row tiles of one lane, butterflies in registers
//   stage 4  * scale, round half away, clamp, four adjacent positions per dword -> LDS -> 16-byte coalesced stores
// HBM-bound: 2 (or 4 with the gate) bytes in and 1 byte out per channel.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

typedef uint32_t lq_v2u __attribute__((ext_vector_type(2)));

constexpr int kLS = 132;    // halves per chunk in LDS
constexpr int kPS = 132;    // dwords per chunk pair in LDS (4 kPS = 16 mod 64: the four contraction groups read distinct banks)
constexpr int kOS = 144;    // bytes per chunk in the INT8 staging tile (36 dwords: the 64 lanes of one write hit 64 banks)
constexpr int kMaxG = 64;
constexpr int kWaves = 1;  // rows (waves) per workgroup: single-wave workgroups keep the rows independent of each other

struct EpiParams {
  const _Float16* x;
  int64_t x_stride;
  const _Float16* z;
  int64_t z_stride;
  const void* weight;
  int weight_f32;
  _Float16* norm_out;
  const int8_t* had;
  int8_t* out;
  int rows, dim, g, group_size;
  float eps, scale;
};

// roundf as one add: y + copysign(0.5 - 2^-25, y) lands on the next integer exactly when |y| has a fraction >= 0.5
// (the sum of a tie k + 0.5 is k + 1 - 2^-25, which rounds to k + 1; anything below the tie stays below k + 1), and the
// float -> int conversion truncates toward zero and saturates.
LQ_DEV int round_half_away(float y) { return (int)(y + __builtin_copysignf(0x1.fffffep-2f, y)); }

// float(h) * f as an explicit fma with a +0 addend: the compiler selects the mixed-precision fma, which converts the
// half exactly and rounds the product once, as a conversion followed by a multiply would (a -0 product comes out +0)
LQ_DEV float mul_half(_Float16 h, float f) { return __builtin_fmaf((float)h, f, 0.0f); }

LQ_DEV float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, 64);
  return v;
}

// A 16-byte global load issued as an instruction (the compiler neither moves nor repeats it), and the wait that makes
// its result usable: every value requested this way passes through arrived() before its first use.
LQ_DEV void request16(lq_v4i& dst, const void* ptr) {
  asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(ptr) : "memory");  // streamed once
}
LQ_DEV void arrived(lq_v4i& v) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(v)::"memory"); }

// IT = 16-byte pieces per lane (g <= 4 IT); NT = 16-column tiles of had, KS = 32-chunk contraction steps that follow
// NORM: gate + RMSNorm in front; QHAD: Hadamard + INT8 behind (false: the kernel ends after storing the normalized row)
// GATE: z is given; EXACT: g = 4 IT, every lane owns IT whole pieces and no access needs a guard
template <int IT, bool NORM, bool QHAD, bool GATE, bool EXACT>
__global__ __launch_bounds__(64 * kWaves) __attribute__((amdgpu_waves_per_eu(IT <= 10 ? 3 : 2, IT <= 10 ? 3 : 2))) void epilogue_kernel(
    EpiParams p) {
  constexpr int kIt = IT, NT = (IT + 3) / 4, KS = (IT + 7) / 8;
  extern __shared__ __align__(16) unsigned char smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = EXACT ? 4 * IT : p.g, g8 = (g + 7) & ~7;
  const int wave_bytes = g8 * kLS * 2;  // >= g * kOS and >= 16 g * 4
  _Float16* Xs = (_Float16*)(smem + (size_t)wave * wave_bytes);
  float* Ps = (float*)Xs;               // per-piece sums of squares (before X is written)
  unsigned char* Os = (unsigned char*)Xs;  // INT8 staging (after the last operand read)
  const int row_raw = blockIdx.x * kWaves + wave;
  const bool live = row_raw < p.rows;
  const int row = live ? row_raw : p.rows - 1;  // surplus waves redo the last row and store nothing
  const int pieces = 16 * g;

  // every load is issued before the first use; a piece past the row re-reads the last one and is zeroed in registers
  bool valid[kIt];
  int pcc[kIt];
#pragma unroll
  for (int it = 0; it < kIt; ++it) {
    const int pc = it * 64 + lane;
    valid[it] = EXACT || pc < pieces;
    pcc[it] = EXACT ? pc : min(pc, pieces - 1);
  }
  // The row's requests are written as instructions: as plain loads the compiler sinks them next to their uses (or drops
  // and repeats them) to save registers, and the row then arrives two pieces at a time, one memory round trip after the
  // other.  All of them are issued back to back and waited for once; no other vector memory operation is outstanding at
  // this point, and the compiler's own wait counts are unaffected by operations older than the ones it tracks.
  lq_v8h xv[kIt];
  lq_v8h zv[(NORM && GATE) ? kIt : 1];
  {
    lq_v4i xraw[kIt], zraw[(NORM && GATE) ? kIt : 1];
    const _Float16* xr = p.x + (int64_t)row * p.x_stride;
#pragma unroll
    for (int it = 0; it < kIt; ++it) request16(xraw[it], xr + pcc[it] * 8);
    if constexpr (NORM && GATE) {
      const _Float16* zr = p.z + (int64_t)row * p.z_stride;
#pragma unroll
      for (int it = 0; it < kIt; ++it) request16(zraw[it], zr + pcc[it] * 8);
    }
#pragma unroll
    for (int it = 0; it < kIt; ++it) arrived(xraw[it]);
    if constexpr (NORM && GATE) {
#pragma unroll
      for (int it = 0; it < kIt; ++it) arrived(zraw[it]);
    }
#pragma unroll
    for (int it = 0; it < kIt; ++it) xv[it] = __builtin_bit_cast(lq_v8h, xraw[it]);
    if constexpr (NORM && GATE) {
#pragma unroll
      for (int it = 0; it < kIt; ++it) zv[it] = __builtin_bit_cast(lq_v8h, zraw[it]);
    }
  }

  if constexpr (NORM) {
    // The gated value is evaluated twice, for the sum of squares and again for the normalized output, instead of being
    // kept: an fp32 copy of the row (8 IT registers) next to the packed x and z made the scheduler sink the row's
    // requests next to their uses, and the row then arrived two pieces at a time, one memory round trip after the other.
    // Without the copy all 2 IT requests are in flight together; the second evaluation costs 2 IT quarter-rate
    // instructions per lane and returns the same bits.
    auto gated = [&](int it, int e) -> float {
      float a;
      if constexpr (GATE) {
        const float sg = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(mul_half(zv[it][e], -1.44269504088896340736f)));
        a = mul_half(xv[it][e], mul_half(zv[it][e], sg));
      } else {
        a = (float)xv[it][e];
      }
      return valid[it] ? a : 0.0f;
    };
    float part[kIt];
#pragma unroll
    for (int it = 0; it < kIt; ++it) {
      float s = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float a = gated(it, e);
        s = __builtin_fmaf(a, a, s);
      }
      part[it] = s;
    }
    const int ngroups = p.dim / p.group_size;
    const int ppg = p.group_size >> 3;  // pieces per group
    float rstd[kIt];
    if (ngroups == 1) {
      float s = 0.0f;
#pragma unroll
      for (int it = 0; it < kIt; ++it) s = s + part[it];
      s = wave_sum(s);
      const float r = 1.0f / __builtin_sqrtf(s / (float)p.group_size + p.eps);
#pragma unroll
      for (int it = 0; it < kIt; ++it) rstd[it] = r;
    } else {
      int grp[kIt];
#pragma unroll
      for (int it = 0; it < kIt; ++it) {
        const int pc = it * 64 + lane;
        if (valid[it]) Ps[pc] = part[it];
        grp[it] = pc / ppg;
        rstd[it] = 0.0f;
      }
      __syncthreads();
      for (int gi = 0; gi < ngroups; ++gi) {
        float s = 0.0f;
        for (int t = lane; t < ppg; t += 64) s = s + Ps[gi * ppg + t];
        s = wave_sum(s);
        const float r = 1.0f / __builtin_sqrtf(s / (float)p.group_size + p.eps);
#pragma unroll
        for (int it = 0; it < kIt; ++it)
          if (grp[it] == gi) rstd[it] = r;
      }
      __syncthreads();
    }
    // Weights without a branch on their dtype (a load inside a branch is waited for inside it: one memory round trip per
    // piece): two 16-byte requests per piece, the whole fp16 piece twice or the two halves of the fp32 piece, and a
    // select per element.  (float)h * f rounds once either way, so both dtypes share y = (a * rstd) * w.
    const bool wf32 = p.weight_f32;
    const char* wbase = (const char*)p.weight;
#pragma unroll
    for (int it = 0; it < kIt; ++it) {
      const char* wp = wbase + (int64_t)pcc[it] * (wf32 ? 32 : 16);
      const lq_v4i wa = *(const lq_v4i*)wp;
      const lq_v4i wb = *(const lq_v4i*)(wp + (wf32 ? 16 : 0));
      const lq_v8h wh = __builtin_bit_cast(lq_v8h, wa);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float w32 = __int_as_float(e < 4 ? wa[e & 3] : wb[e & 3]);
        const float w = wf32 ? w32 : (float)wh[e];
        float y = (gated(it, e) * rstd[it]) * w;
        asm("" : "+v"(y));  // keeps the fp32 rounding of the product: no multiply fused into the fp16 conversion
        xv[it][e] = (_Float16)y;
      }
    }
    if (p.norm_out && live) {
#pragma unroll
      for (int it = 0; it < kIt; ++it)
        if (valid[it]) __builtin_nontemporal_store(xv[it], (lq_v8h*)(p.norm_out + (int64_t)row * p.dim + (it * 64 + lane) * 8));
    }
  } else if constexpr (!EXACT) {
#pragma unroll
    for (int it = 0; it < kIt; ++it)
      if (!valid[it]) xv[it] = lq_v8h{0, 0, 0, 0, 0, 0, 0, 0};
  }

  if constexpr (QHAD) {
    // ---- stage 0: the fp16 row into LDS as dwords (X[2 cp][i], X[2 cp + 1][i]) at [cp][i]: the lanes of an even and
    // an odd 16-lane row hold the same eight positions of two adjacent chunks; two row swaps give each lane four
    // positions of both chunks, which it interleaves and stores with one 16-byte write ----
    uint32_t* Xp = (uint32_t*)Xs;
    const int n = lane & 15, kg = lane >> 4;
#pragma unroll
    for (int it = 0; it < kIt; ++it) {
      const lq_v4i d = __builtin_bit_cast(lq_v4i, xv[it]);  // zero for the pieces past the row
      const lq_v2u s02 = __builtin_amdgcn_permlane16_swap((uint32_t)d[0], (uint32_t)d[2], false, false);
      const lq_v2u s13 = __builtin_amdgcn_permlane16_swap((uint32_t)d[1], (uint32_t)d[3], false, false);
      lq_v4i w;
      w[0] = (int)__builtin_amdgcn_perm(s02[1], s02[0], 0x05040100u);
      w[1] = (int)__builtin_amdgcn_perm(s02[1], s02[0], 0x07060302u);
      w[2] = (int)__builtin_amdgcn_perm(s13[1], s13[0], 0x05040100u);
      w[3] = (int)__builtin_amdgcn_perm(s13[1], s13[0], 0x07060302u);
      const int cp = 2 * it + (lane >> 5);
      if (2 * cp < g8) *(lq_v4i*)(Xp + cp * kPS + n * 8 + 4 * (kg & 1)) = w;
    }
    for (int t = lane; t < (g8 / 2 - 2 * kIt) * 32; t += 64)  // chunk pairs past the last piece (g8 > 4 kIt)
      *(lq_v4i*)(Xp + (2 * kIt + (t >> 5)) * kPS + (t & 31) * 4) = lq_v4i{0, 0, 0, 0};

    // operands that do not depend on the row: had^T as the B operand of stage 1, H_16 as the A operand of stage 2
    lq_v8h bop[NT][KS];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int cp = 16 * nt + n, c0 = 32 * ks + 8 * kg;
        if ((g & 3) == 0) {
          // +-1 bytes -> fp16 bits: 0x3C00 with the byte's sign bit on top
          lq_v4i hb;
#pragma unroll
          for (int hw = 0; hw < 2; ++hw) {
            const bool ok = cp < g && c0 + 4 * hw < g;
            // requested without a branch (entries outside the matrix read a clamped address and are zeroed below)
            const uint32_t wd = *(const uint32_t*)(p.had + min(cp, g - 1) * g + min(c0 + 4 * hw, g - 4));
            const uint32_t lo = 0x3C003C00u | ((wd & 0x80u) << 8) | ((wd & 0x8000u) << 16);
            const uint32_t hi = 0x3C003C00u | ((wd & 0x800000u) >> 8) | (wd & 0x80000000u);
            hb[2 * hw] = ok ? (int)lo : 0;
            hb[2 * hw + 1] = ok ? (int)hi : 0;
          }
          bop[nt][ks] = __builtin_bit_cast(lq_v8h, hb);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            bop[nt][ks][j] = (cp < g && c0 + j < g) ? (_Float16)(float)p.had[cp * g + c0 + j] : (_Float16)0.0f;
        }
      }
    float h16[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) h16[r] = (__builtin_popcount(n & (4 * kg + r)) & 1) ? -1.0f : 1.0f;
    // pair-row base of this lane's contraction slots; lanes whose eight chunks lie past g8 feed zeros
    int pbase[KS];
    bool kvalid[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c0 = 32 * ks + 8 * kg;
      kvalid[ks] = c0 < g8;
      pbase[ks] = (kvalid[ks] ? c0 / 2 : 0) * kPS + n;
    }
    __syncthreads();

    // ---- stage 1 ----
    lq_v4f acc[8][NT];
#pragma unroll
    for (int mt = 0; mt < 8; ++mt) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = lq_v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        lq_v4i ad;
#pragma unroll
        for (int jp = 0; jp < 4; ++jp) ad[jp] = (int)Xp[pbase[ks] + jp * kPS + 16 * mt];
        if (!(EXACT && 32 * ks + 24 < ((4 * IT + 7) & ~7)) && !kvalid[ks]) ad = lq_v4i{0, 0, 0, 0};
        const lq_v8h a = __builtin_bit_cast(lq_v8h, ad);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = lq_mfma_f16(a, bop[nt][ks], acc[mt][nt]);
      }
    }
    __syncthreads();  // every operand read is done: the buffer becomes the INT8 staging tile

    // ---- stage 2: H_16 over the 16 rows of each tile ----
#pragma unroll
    for (int mt = 0; mt < 8; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        lq_v4f d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int r = 0; r < 4; ++r) d = __builtin_amdgcn_mfma_f32_16x16x4f32(h16[r], acc[mt][nt][r], d, 0, 0, 0);
        acc[mt][nt] = d;
      }

    // ---- stage 3: H_8 across the tiles (bits 4..6 of the position) ----
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
      for (int mt = 0; mt < 8; ++mt)
        if ((mt & h) == 0)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const lq_v4f a = acc[mt][nt], b = acc[mt + h][nt];
            acc[mt][nt] = a + b;
            acc[mt + h][nt] = a - b;
          }

    // ---- stage 4 ----
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int cp = 16 * nt + n;
      if (cp < g) {
#pragma unroll
        for (int mt = 0; mt < 8; ++mt) {
          int q[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) q[r] = lq_clampi(round_half_away(acc[mt][nt][r] * p.scale), -127, 127);
          *(uint32_t*)(Os + cp * kOS + 16 * mt + 4 * kg) = lq_pack4(q[0], q[1], q[2], q[3]);
        }
      }
    }
    __syncthreads();
    if (live) {
#pragma unroll
      for (int it = 0; it < (kIt + 1) / 2; ++it) {
        const int pc = it * 64 + lane;  // 16-byte pieces of the INT8 row: 8 per chunk
        if (pc < 8 * g) {
          const lq_v4i o = *(const lq_v4i*)(Os + (pc >> 3) * kOS + (pc & 7) * 16);
          __builtin_nontemporal_store(o, (lq_v4i*)(p.out + (int64_t)row * p.dim + pc * 16));
        }
      }
    }
  }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

template <bool NORM, bool QHAD, bool GATE>
int launch(const EpiParams& p, hipStream_t stream) {
  const int g = p.g, g8 = (g + 7) & ~7;
  const size_t lds = QHAD || (NORM && p.dim / p.group_size > 1) ? (size_t)kWaves * g8 * kLS * 2 : 0;
  const dim3 grid((unsigned)((p.rows + kWaves - 1) / kWaves)), block(64 * kWaves);
#define LQ_EPI_LAUNCH_(IT_, EX_)                                                                                  \
  do {                                                                                                            \
    auto kern = &epilogue_kernel<IT_, NORM, QHAD, GATE, EX_>;                                                     \
    if (lds > 65536 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                   \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)   \
      return LQ_ERR_LAUNCH;                                                                                       \
    hipLaunchKernelGGL(kern, grid, block, lds, stream, p);                                                        \
  } while (0)
  // sizes with g = 4 IT run the guard-free kernel; any other g runs the guarded kernel of the next multiple of 16
#define LQ_EPI_EXACT(IT_) case IT_: LQ_EPI_LAUNCH_(IT_, true); break
  if (g % 4 == 0 && (g / 4 <= 8 || g / 4 == 10 || g / 4 == 12 || g / 4 == 14 || g / 4 == 16)) {
    switch (g / 4) {
      LQ_EPI_EXACT(1); LQ_EPI_EXACT(2); LQ_EPI_EXACT(3); LQ_EPI_EXACT(4); LQ_EPI_EXACT(5); LQ_EPI_EXACT(6);
      LQ_EPI_EXACT(7); LQ_EPI_EXACT(8); LQ_EPI_EXACT(10); LQ_EPI_EXACT(12); LQ_EPI_EXACT(14); LQ_EPI_EXACT(16);
    }
  } else if (g <= 16) LQ_EPI_LAUNCH_(4, false);
  else if (g <= 32) LQ_EPI_LAUNCH_(8, false);
  else if (g <= 48) LQ_EPI_LAUNCH_(12, false);
  else LQ_EPI_LAUNCH_(16, false);
#undef LQ_EPI_EXACT
#undef LQ_EPI_LAUNCH_
  return lq_check_launch();
}

int check_row_tensor(const void* x, int64_t stride, int dim) {
  if (!x) return LQ_ERR_NULL;
  if (stride < dim || stride % 8 != 0 || !al(x, 16)) return LQ_ERR_SHAPE;
  return LQ_OK;
}

int check_dims(int rows, int dim) {
  if (rows <= 0 || dim < 128 || dim % 128 != 0 || dim / 128 > kMaxG) return LQ_ERR_SHAPE;
  return LQ_OK;
}

int check_norm(const void* weight, int weight_dtype, int dim, int group_size, float eps) {
  if (!weight) return LQ_ERR_NULL;
  if (weight_dtype != LQ_DT_F16 && weight_dtype != LQ_DT_F32) return LQ_ERR_SHAPE;
  if (!al(weight, 16)) return LQ_ERR_SHAPE;
  if (group_size <= 0 || group_size % 8 != 0 || dim % group_size != 0) return LQ_ERR_SHAPE;
  if (!(eps >= 0.0f)) return LQ_ERR_SHAPE;
  return LQ_OK;
}

}  // namespace

extern "C" int lq_rmsnorm_gated(const lq_rmsnorm_gated_args* a, hipStream_t stream) {
  if (!a || !a->out) return LQ_ERR_NULL;
  int rc = check_dims(a->rows, a->dim);
  if (rc) return rc;
  if ((rc = check_row_tensor(a->x, a->x_stride, a->dim))) return rc;
  if (a->z && (rc = check_row_tensor(a->z, a->z_stride, a->dim))) return rc;
  if ((rc = check_norm(a->weight, a->weight_dtype, a->dim, a->group_size, a->eps))) return rc;
  if (!al(a->out, 16)) return LQ_ERR_SHAPE;
  EpiParams p{};
  p.x = (const _Float16*)a->x; p.x_stride = a->x_stride;
  p.z = (const _Float16*)a->z; p.z_stride = a->z_stride;
  p.weight = a->weight; p.weight_f32 = a->weight_dtype == LQ_DT_F32;
  p.norm_out = (_Float16*)a->out;
  p.rows = a->rows; p.dim = a->dim; p.g = a->dim / 128; p.group_size = a->group_size; p.eps = a->eps;
  return a->z ? launch<true, false, true>(p, stream) : launch<true, false, false>(p, stream);
}

extern "C" int lq_qhad_transform(const lq_qhad_transform_args* a, hipStream_t stream) {
  if (!a || !a->had || !a->out) return LQ_ERR_NULL;
  int rc = check_dims(a->rows, a->dim);
  if (rc) return rc;
  if ((rc = check_row_tensor(a->x, a->x_stride, a->dim))) return rc;
  if (!al(a->out, 16) || !al(a->had, 4) || !(a->scale == a->scale)) return LQ_ERR_SHAPE;
  EpiParams p{};
  p.x = (const _Float16*)a->x; p.x_stride = a->x_stride;
  p.had = a->had; p.out = a->out; p.scale = a->scale;
  p.rows = a->rows; p.dim = a->dim; p.g = a->dim / 128; p.group_size = a->dim;
  return launch<false, true, false>(p, stream);
}

extern "C" int lq_rmsnorm_gated_qhad(const lq_rmsnorm_gated_qhad_args* a, hipStream_t stream) {
  if (!a || !a->had || !a->out) return LQ_ERR_NULL;
  int rc = check_dims(a->rows, a->dim);
  if (rc) return rc;
  if ((rc = check_row_tensor(a->x, a->x_stride, a->dim))) return rc;
  if (a->z && (rc = check_row_tensor(a->z, a->z_stride, a->dim))) return rc;
  if ((rc = check_norm(a->weight, a->weight_dtype, a->dim, a->group_size, a->eps))) return rc;
  if (!al(a->out, 16) || !al(a->had, 4) || (a->norm_out && !al(a->norm_out, 16)) || !(a->scale == a->scale))
    return LQ_ERR_SHAPE;
  EpiParams p{};
  p.x = (const _Float16*)a->x; p.x_stride = a->x_stride;
  p.z = (const _Float16*)a->z; p.z_stride = a->z_stride;
  p.weight = a->weight; p.weight_f32 = a->weight_dtype == LQ_DT_F32;
  p.norm_out = (_Float16*)a->norm_out;
  p.had = a->had; p.out = a->out; p.scale = a->scale;
  p.rows = a->rows; p.dim = a->dim; p.g = a->dim / 128; p.group_size = a->group_size; p.eps = a->eps;
  return a->z ? launch<true, true, true>(p, stream) : launch<true, true, false>(p, stream);
}
