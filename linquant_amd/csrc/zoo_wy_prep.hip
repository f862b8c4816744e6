// WY / UT transform of the delta family, per chunk, in fp32.
// Replaces the torch prep linquant/kernels/zoo/gated_delta_rule.py:20-47 (no / scalar decay) and
// linquant/kernels/zoo/kda.py:22-53 (per-channel decay); the reference's default route through fla-core's
// prep kernels for sigma = tau = 1 is served by the same native prep.
//   L = beta^sigma k,  Hg = beta^(1-sigma) k
//   G[i][j] = sum_n L[i][n] Hg[j][n] * decay(i,j,n)  for i > j, decay = 1 | exp(g_i - g_j) | exp(g_in - g_jn)
//   T = (I + G)^-1  (unit lower triangular, forward substitution)
//   W = T (L * exp(g)),  U = T (beta^sigma v),  Hw = beta^((1-sigma) tau) k,  fw = beta^((1-sigma)(1-tau))
//
// One 4-wave workgroup per (chunk, batch*head); the Gram and the inverse run on the fp32 MFMA (16x16x4).
//   Gram: both operands are staged once per token as fp32 in LDS and the ten lower 16x16 blocks are spread 3/3/2/2
//     over the waves.  Per-channel decay is factorized around the chunk's middle row; when the decay spread over the
//     chunk is too large for that, each wave redoes its row block around the block's first row straight from global
//     memory (diagonal block: one exponential per (i, j, channel) when even that spread is too large).
//   Inverse: the four 16x16 diagonal blocks by forward substitution (lane per column), then block rows 1..3:
//     T_IJ = -T_II . sum_{J <= M < I} G_IM . T_MJ.
//   W, U: T . X on the bf16 MFMA with T and X each split in three bf16 pieces (six products per step); X is staged
//     transposed in LDS, each wave takes row block w for the first half of the column tiles and row block 3 - w for
//     the second half (equal work), and stores four adjacent channels per lane.
#include "zoo_common.h"
#include "../../include/linquant_hip.h"

namespace {

struct WyParams {
  const _Float16* k;
  const _Float16* v;
  const float* beta;
  const float* g;
  _Float16* Hw;
  _Float16* W;
  _Float16* U;
  float* fw;
  float sigma, tau;
  int bf;
  int B, T, H, V;
  // write-operand codes of the state kernel, made here when kqT is set (otherwise lq_zoo_write_codes makes them from the
  // stored Hw and W)
  int8_t* kqT;
  int8_t* wq;
  float* ev;
  float* gam;
  const float* logenv;
  const float* skw;
  const float* sw;
  float eta;
  int qmax;
  int NT;
  const float* dk_div;  // (H,K) D_QK applied to k at load (k' = act(k / D)), with its reciprocal; or nullptr
  const float* dk_rcp;
  float* pack;  // fw | ev | gam per (batch, chunk, head), 64 + 64 + K floats, or nullptr
};

LQ_DEV float powb(float b, float e) {
  if (e == 0.0f) return 1.0f;
  if (e == 1.0f) return b;
  return __builtin_amdgcn_exp2f(e * __builtin_amdgcn_logf(b));
}

typedef float wy_v2f __attribute__((ext_vector_type(2)));

// D_QK at load: k' = act(k / D) for the eight adjacent channels n .. n + 7 (the quotient rounded once to fp32, then to
// the activation dtype: what the stand-alone rescaling launch would have stored).  tab: D at [n], RN(1 / D) at [128 + n],
// staged per head in LDS.  DK is a compile-time flag: the kernels sit at their register limit, and a run-time test
// around this arithmetic spilled dozens of registers in the variants that never rescale.
template <bool BF, bool DK>
LQ_DEV void wy_dk8(const float* tab, int n, float (&kv)[8]) {
  if constexpr (DK) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {  // two channels at a time: the table entries are short-lived
      const wy_v2f dd = *(const wy_v2f*)(tab + n + 2 * d), rr = *(const wy_v2f*)(tab + 128 + n + 2 * d);
      kv[2 * d] = zoo_round_act(zoo_div_rn(kv[2 * d], dd[0], rr[0]), BF);
      kv[2 * d + 1] = zoo_round_act(zoo_div_rn(kv[2 * d + 1], dd[1], rr[1]), BF);
    }
  }
}

LQ_DEV lq_v4f mfma_f32(float a, float b, lq_v4f c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

LQ_DEV float wy_wave_max(float m) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  return m;
}

constexpr int kGS = 70;  // floats per row of the G / T tiles: measured, an A-operand read (16 rows, 4 adjacent slots) takes one LDS pass when the pitch is 2 mod 4 (68 took two)

// ---- T . X on the bf16 MFMA with both factors split in three bf16 pieces, x = hi + mid + lo (each the upper 16 bits
// of what the pieces before it leave, so hi + mid + lo has 24 significant bits): the six products down to 2^-16 of the
// leading one (hi.hi, hi.mid, mid.hi, mid.mid, hi.lo, lo.hi) reproduce the fp32 product to about 2^-23 at 3/8 of the
// fp32 MFMA's issue time.  (Two pieces per factor, 2^-16, moved stored state codes by two steps in places.)
typedef __bf16 wy_v8bf __attribute__((ext_vector_type(8)));

LQ_DEV lq_v4f mfma_bf16(lq_v4i a, lq_v4i b, lq_v4f c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(wy_v8bf, a), __builtin_bit_cast(wy_v8bf, b), c, 0, 0, 0);
}

// two fp32 values -> one dword each of their hi, mid and lo pieces (first value in the low half)
LQ_DEV void split3(float x0, float x1, uint32_t& hi, uint32_t& mid, uint32_t& lo) {
  const uint32_t b0 = __float_as_uint(x0), b1 = __float_as_uint(x1);
  hi = __builtin_amdgcn_perm(b1, b0, 0x07060302u);
  const float r0 = x0 - __uint_as_float(b0 & 0xffff0000u), r1 = x1 - __uint_as_float(b1 & 0xffff0000u);  // exact
  const uint32_t c0 = __float_as_uint(r0), c1 = __float_as_uint(r1);
  mid = __builtin_amdgcn_perm(c1, c0, 0x07060302u);
  const float q0 = r0 - __uint_as_float(c0 & 0xffff0000u), q1 = r1 - __uint_as_float(c1 & 0xffff0000u);  // exact
  lo = __builtin_amdgcn_perm(__float_as_uint(q1), __float_as_uint(q0), 0x07060302u);
}

constexpr int kXP = 36;  // dwords per column of the transposed X tiles (32 token pairs + pad)
constexpr int kXT = 64 * kXP;  // dwords per tile (64 columns)

// X tiles in LDS: one tile per piece, [column][token pair] dwords (even token in the low half), 64 columns; the token-pair index is
// XOR-ed with 8 * ((column >> 4) & 3) so that the transposing writes of one wave (8 pairs x 8 column groups) spread
// over all banks while a 16-byte operand piece (4 pairs) stays whole.
LQ_DEV int xt_index(int col, int pair) { return col * kXP + (pair ^ (((col >> 4) & 3) << 3)); }

// T operand of row block I for contraction step st (tokens 32st + 8kg .. + 7): lane (rl, kg) holds T[16I + rl][those],
// zero where the block column lies right of the diagonal block (never written)
LQ_DEV void t_operand(const float* T_s, int I, int st, int rl, int kg, lq_v4i& th, lq_v4i& tm, lq_v4i& tl) {
  const int m0 = 32 * st + 8 * kg;
  const float* tp = T_s + (16 * I + rl) * kGS + m0;
  const bool live = m0 < 16 * (I + 1);
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const wy_v2f t2 = *(const wy_v2f*)(tp + 2 * d);
    uint32_t h, m, l;
    split3(live ? t2[0] : 0.0f, live ? t2[1] : 0.0f, h, m, l);
    th[d] = (int)h, tm[d] = (int)m, tl[d] = (int)l;
  }
}

// D^T tile of T . X for row block I and the 16 columns of tile nt: lane (rl = token, kg) gets columns 16nt + 4kg + r
LQ_DEV lq_v4f tx_tile(const uint32_t* Xt, const lq_v4i (&th)[2], const lq_v4i (&tm)[2], const lq_v4i (&tl)[2], int I,
                      int nt, int rl, int kg) {
  lq_v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < 2; ++st) {
    if (st > (I >> 1)) continue;
    const int at = xt_index(16 * nt + rl, 16 * st + 4 * kg);
    const lq_v4i xh = *(const lq_v4i*)(Xt + at), xm = *(const lq_v4i*)(Xt + kXT + at), xl = *(const lq_v4i*)(Xt + 2 * kXT + at);
    acc = mfma_bf16(xl, th[st], acc);
    acc = mfma_bf16(xh, tl[st], acc);
    acc = mfma_bf16(xm, tm[st], acc);
    acc = mfma_bf16(xm, th[st], acc);
    acc = mfma_bf16(xh, tm[st], acc);
    acc = mfma_bf16(xh, th[st], acc);
  }
  return acc;
}

// Gram of row block I = wave with the per-channel decay factorized around the first row of the row block (used when
// the decay spread over the whole chunk is too large for one anchor): operands straight from global memory, lane
// (rl, kg) supplies 16 contiguous channels of token rl per 64-channel pass; off-diagonal blocks: both factors <= 1;
// diagonal block: only when the spread inside the block is small, otherwise one exponential per (i, j, channel).
// NB = row blocks of the chunk (4, or 8 for the 128-token kernel), GS = floats per row of the G tile.
template <int DECAY, int K, bool BF, bool DK, int NB = 4, int GS = kGS>
LQ_DEV void gram_rowblock(const WyParams& p, float* G_s, const float* bs_s, const float* bh_s, const float* gs_s, int I,
                          int rl, int kg, int64_t t0, int h, const float* dk_s) {
  const int H = p.H;
  constexpr bool bf = BF;
    const int64_t irow = ((t0 + 16 * I + rl) * H + h) * K;
    const int64_t arow = ((t0 + 16 * I) * H + h) * K;
    const float bs_i = bs_s[16 * I + rl];
    lq_v4f acc[NB];
#pragma unroll
    for (int J = 0; J < NB; ++J) acc[J] = lq_v4f{0.f, 0.f, 0.f, 0.f};
    bool exact_diag = false;
    if (DECAY == LQ_DECAY_DIAGONAL) {
      float spread = 0.0f;
      for (int c = 16 * kg; c < K; c += 64)
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
          const lq_v4f g4 = *(const lq_v4f*)(p.g + irow + c + 4 * e4), a4 = *(const lq_v4f*)(p.g + arow + c + 4 * e4);
#pragma unroll
          for (int e = 0; e < 4; ++e) spread = fmaxf(spread, __builtin_fabsf(g4[e] - a4[e]));
        }
      exact_diag = wy_wave_max(spread) > 40.0f;
    }
#pragma unroll
    for (int ps = 0; ps < K / 64; ++ps) {
      const int c0 = 64 * ps + 16 * kg;
      float Lr[16], gi[16], an[16];
      {
        float k0[8];
        zoo_ld8(p.k + irow + c0, bf, k0);
        float k1[8];
        zoo_ld8(p.k + irow + c0 + 8, bf, k1);
        wy_dk8<BF, DK>(dk_s, c0, k0);
        wy_dk8<BF, DK>(dk_s, c0 + 8, k1);
#pragma unroll
        for (int e = 0; e < 16; ++e) Lr[e] = bs_i * (float)(e < 8 ? k0[e & 7] : k1[e & 7]);
        if (DECAY == LQ_DECAY_DIAGONAL) {
#pragma unroll
          for (int e4 = 0; e4 < 4; ++e4) {
            const lq_v4f g4 = *(const lq_v4f*)(p.g + irow + c0 + 4 * e4), a4 = *(const lq_v4f*)(p.g + arow + c0 + 4 * e4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              gi[4 * e4 + e] = g4[e];
              an[4 * e4 + e] = a4[e];
            }
          }
#pragma unroll
          for (int e = 0; e < 16; ++e) Lr[e] = Lr[e] * zoo_exp(gi[e] - an[e]);
        }
      }
#pragma unroll
      for (int J = 0; J < NB; ++J) {
        if (J > I) continue;
        if (DECAY == LQ_DECAY_DIAGONAL && J == I && exact_diag) continue;
        const int64_t jrow = ((t0 + 16 * J + rl) * H + h) * K;
        const float bh_j = bh_s[16 * J + rl];
        float k0[8];
        zoo_ld8(p.k + jrow + c0, bf, k0);
        float k1[8];
        zoo_ld8(p.k + jrow + c0 + 8, bf, k1);
        wy_dk8<BF, DK>(dk_s, c0, k0);
        wy_dk8<BF, DK>(dk_s, c0 + 8, k1);
        float Hr[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) Hr[e] = bh_j * (float)(e < 8 ? k0[e & 7] : k1[e & 7]);
        if (DECAY == LQ_DECAY_DIAGONAL) {
#pragma unroll
          for (int e4 = 0; e4 < 4; ++e4) {
            const lq_v4f g4 = *(const lq_v4f*)(p.g + jrow + c0 + 4 * e4);
#pragma unroll
            for (int e = 0; e < 4; ++e) Hr[4 * e4 + e] = Hr[4 * e4 + e] * zoo_exp(an[4 * e4 + e] - g4[e]);
          }
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[J] = mfma_f32(Lr[e], Hr[e], acc[J]);
      }
    }
    // lane holds column j = rl of block J, rows i = 4kg + r of block I
#pragma unroll
    for (int J = 0; J < NB; ++J) {
      if (J > I) continue;
      if (DECAY == LQ_DECAY_DIAGONAL && J == I && exact_diag) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * I + 4 * kg + r, j = 16 * J + rl;
        float v = 0.0f;
        if (i > j) {
          v = acc[J][r];
          if (DECAY == LQ_DECAY_SCALAR) v = v * zoo_exp(gs_s[i] - gs_s[j]);
        }
        G_s[i * GS + j] = v;
      }
    }
    if (DECAY == LQ_DECAY_DIAGONAL && exact_diag) {
      // lane (i = rl, j = 4kg + jj) of the diagonal block, one exponential per (i, j, channel)
      float sacc[4] = {0.f, 0.f, 0.f, 0.f};
      for (int n8 = 0; n8 < K; n8 += 8) {
        float ki[8];
        zoo_ld8(p.k + irow + n8, bf, ki);
        wy_dk8<BF, DK>(dk_s, n8, ki);
        const lq_v4f gi0 = *(const lq_v4f*)(p.g + irow + n8), gi1 = *(const lq_v4f*)(p.g + irow + n8 + 4);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int j = 4 * kg + jj;
          const int64_t jrow = ((t0 + 16 * I + j) * H + h) * K;
          float kj[8];
          zoo_ld8(p.k + jrow + n8, bf, kj);
          wy_dk8<BF, DK>(dk_s, n8, kj);
          const lq_v4f gj0 = *(const lq_v4f*)(p.g + jrow + n8), gj1 = *(const lq_v4f*)(p.g + jrow + n8 + 4);
          const float bh_j = bh_s[16 * I + j];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float gi_ = e < 4 ? gi0[e & 3] : gi1[e & 3], gj_ = e < 4 ? gj0[e & 3] : gj1[e & 3];
            const float w = (rl > j) ? zoo_exp(gi_ - gj_) : 0.0f;
            sacc[jj] = fmaf((bs_i * ki[e]) * (bh_j * kj[e]), w, sacc[jj]);
          }
        }
      }
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) G_s[(16 * I + rl) * GS + 16 * I + 4 * kg + jj] = (rl > 4 * kg + jj) ? sacc[jj] : 0.0f;
    }
}

// CODES: the kernel also emits what lq_zoo_write_codes would make from the stored Hw and W (same arithmetic on the same
// rounded values, so the same bits): channel-major key write codes, token-major state-read codes of W, the per-token
// value factor and the per-channel chunk decay.  W itself is then stored only when p.W is set.
template <int DECAY, int K, bool BF, bool CODES, bool DK>
__global__ __launch_bounds__(256, 4) void zoo_wy_prep_kernel(WyParams p) {
  constexpr int LS = 64 + 16;  // floats per row of the buffer that holds the Gram tile and then the X tiles
  static_assert(LS >= kGS, "the Gram tile lives in the X buffer until the inverse is done");
  static_assert(3 * kXT <= 64 * kGS + 64 * LS, "the three bf16 pieces of a 64-column X tile overlay the T and X buffers");
  __shared__ __align__(16) float lds_f[64 * kGS + 64 * LS];  // 38 KB of LDS: four workgroups per compute unit
  float* T_s = lds_f;
  float* X_s = lds_f + 64 * kGS;
  float* G_s = X_s;
  uint32_t* Xt = (uint32_t*)lds_f;  // overlays T once its operands sit in registers
  constexpr int kOP = 72;  // floats per row of the staged Gram operands: a 16-byte read of 16 rows x 4 adjacent pieces takes the minimum two LDS passes at 40 or 72
  static_assert(2 * 64 * kOP <= 64 * kGS + 64 * LS, "the Gram operands live in the T / X buffers until G is written");
  float* Lg_s = lds_f;
  float* Hg_s = lds_f + 64 * kOP;
  __shared__ float gs_s[DECAY == LQ_DECAY_SCALAR ? 64 : 1], bs_s[64], bh_s[64];
  __shared__ float iskw_s[CODES ? K : 1], bw_s[CODES ? 64 : 1], el_s[CODES ? 64 : 1];
  // the last 1.5 KB of the big buffer lie beyond the Gram operands, the G / T tiles and the X tiles alike: the per-head
  // tables live there for the whole kernel (D_QK and its reciprocal, 128 floats each; the chunk's last decay row)
  static_assert(2 * 64 * kOP + 384 <= 64 * kGS + 64 * LS && 2 * 64 * kGS + 384 <= 64 * kGS + 64 * LS &&
                3 * kXT + 384 <= 64 * kGS + 64 * LS, "table space behind every overlay");
  float* dk_s = lds_f + 64 * kGS + 64 * LS - 384;
  float* glast_s = dk_s + 256;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  // Flat grid.  Workgroups are dealt to the 8 XCDs round-robin in launch order and each XCD has its own L2.  Workgroup
  // L = x + 8 m (x = its XCD) takes head m % H of (batch, chunk) number x + 8 (m / H): the workgroups resident on one XCD
  // at a time then cover all heads of a few (batch, chunk)s, so the (B, T, H) tensors (beta, the log envelope, fw, ev:
  // four bytes per token and head, a head's values 4 H bytes apart) are fetched and written as whole lines by that XCD
  // instead of one line per value, and the eight XCDs work on neighbouring chunks at the same time.
  const uint32_t ngroups = (uint32_t)p.B * (uint32_t)p.NT;
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
  const int ct = (int)(group % (uint32_t)p.NT), b = (int)(group / (uint32_t)p.NT);
  const int H = p.H, V = p.V;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)ct * 64;
  const float sigma = p.sigma, tau = p.tau;
  constexpr bool bf = BF;

  if (DK && tid < K) {
    dk_s[tid] = p.dk_div[h * K + tid];
    dk_s[128 + tid] = p.dk_rcp[h * K + tid];
  }
  // ---- per-token factors; fw is written straight out
  if (tid < 64) {
    const float bt = p.beta[(t0 + tid) * H + h];
    bs_s[tid] = powb(bt, sigma);
    bh_s[tid] = powb(bt, 1.0f - sigma);
    const float fwv = powb(bt, (1.0f - sigma) * (1.0f - tau));
    p.fw[(t0 + tid) * H + h] = fwv;
    if constexpr (CODES) {
      if (p.pack) p.pack[(((int64_t)b * p.NT + ct) * H + h) * (128 + K) + tid] = fwv;
    }
    if (DECAY == LQ_DECAY_SCALAR) gs_s[tid] = p.g[(t0 + tid) * H + h];
  }
  if constexpr (CODES) {
    // per-token value factor and per-channel chunk decay, as lq_zoo_write_codes writes them
    if (tid < 64) {
      float evv = 1.0f;
      if (DECAY == LQ_DECAY_SCALAR) evv = zoo_exp(p.eta * (p.g[(t0 + 63) * H + h] - p.g[(t0 + tid) * H + h]));
      if (DECAY == LQ_DECAY_DIAGONAL) evv = zoo_exp(p.eta * p.logenv[(t0 + tid) * H + h]);
      p.ev[(t0 + tid) * H + h] = evv;
      if (p.pack) p.pack[(((int64_t)b * p.NT + ct) * H + h) * (128 + K) + 64 + tid] = evv;
    }
    if (tid < K) {
      float gm = 1.0f, gl = 0.0f;
      if (DECAY == LQ_DECAY_SCALAR) gm = zoo_exp(p.g[(t0 + 63) * H + h]);
      if (DECAY == LQ_DECAY_DIAGONAL) {
        gl = p.g[((t0 + 63) * H + h) * K + tid];
        gm = zoo_exp(gl);
      }
      p.gam[(((int64_t)b * p.NT + ct) * H + h) * K + tid] = gm;
      if (p.pack) p.pack[(((int64_t)b * p.NT + ct) * H + h) * (128 + K) + 128 + tid] = gm;
      if (DECAY == LQ_DECAY_DIAGONAL) glast_s[tid] = gl;
      iskw_s[tid] = 1.0f / p.skw[h * K + tid];
    }
    if (tid >= 128 && tid < 192) {
      // per token: the factor of Hw and the key-side factor of the write codes (scalar decay: exp((1-eta)(g_last - g_t));
      // per-channel decay: eta * log envelope, subtracted in the exponent per element)
      const int t = tid - 128;
      bw_s[t] = powb(p.beta[(t0 + t) * H + h], (1.0f - sigma) * tau);
      float e = 1.0f;
      if (DECAY == LQ_DECAY_SCALAR) e = zoo_exp((1.0f - p.eta) * (p.g[(t0 + 63) * H + h] - p.g[(t0 + t) * H + h]));
      if (DECAY == LQ_DECAY_DIAGONAL) e = p.eta * p.logenv[(t0 + t) * H + h];
      el_s[t] = e;
    }
  }
  __syncthreads();

  // ---- Gram G[i][j] for i > j.  Operands are staged once per token, 64 channels at a time, as fp32 in LDS:
  //   Lg = beta^sigma k e^(g - a),  Hg = beta^(1-sigma) k e^(a - g),  a = g of the chunk's middle row (one anchor for the
  //   whole chunk: |g - a| <= 40 keeps every factor and product a normal fp32 number; checked, see below),
  // and the ten 16x16 blocks are spread 3/3/2/2 over the waves.  An operand read is 16 bytes: lane (rl, kg) takes
  // channels 16s + 4kg .. + 3 of row rl, and its element e feeds MFMA step e of both operands alike.
  {
    // wave 0: (3,0) (3,1) (3,2); wave 1: (2,0) (2,1) (2,2); wave 2: (1,0) (1,1); wave 3: (3,3) (0,0)
    const int nb = wave < 2 ? 3 : 2;
    auto blk_i = [&](int q) { return wave < 3 ? 3 - wave : (q == 0 ? 3 : 0); };
    auto blk_j = [&](int q) { return wave < 3 ? q : (q == 0 ? 3 : 0); };
    lq_v4f acc[3];
#pragma unroll
    for (int q = 0; q < 3; ++q) acc[q] = lq_v4f{0.f, 0.f, 0.f, 0.f};
    float spread = 0.0f;
    const int64_t arow = ((t0 + 32) * H + h) * K;
#pragma unroll 1
    for (int ps = 0; ps < K / 64; ++ps) {
      if (ps > 0) __syncthreads();
      uint32_t c03[2], c47[2];  // CODES: the thread's write codes, channels 0..3 / 4..7 of its eight, per token
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int it = tid + 256 * q;
        // with CODES a thread takes two adjacent tokens, so that a token quad of a channel sits in two lanes
        const int r = CODES ? 2 * (tid >> 3) + q : it >> 3, c8 = it & 7;
        const int64_t off = ((t0 + r) * H + h) * K + 64 * ps + 8 * c8;
        float kv[8];
        zoo_ld8(p.k + off, bf, kv);
        wy_dk8<BF, DK>(dk_s, 64 * ps + 8 * c8, kv);
        const float bs = bs_s[r], bh = bh_s[r];
        lq_v4f l0, l1, h0, h1;
        lq_v4f g0 = {0.f, 0.f, 0.f, 0.f}, g1 = g0;
        if (DECAY == LQ_DECAY_DIAGONAL) {
          g0 = *(const lq_v4f*)(p.g + off), g1 = *(const lq_v4f*)(p.g + off + 4);
          const lq_v4f a0 = *(const lq_v4f*)(p.g + arow + 64 * ps + 8 * c8), a1 = *(const lq_v4f*)(p.g + arow + 64 * ps + 8 * c8 + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float d0 = g0[e] - a0[e], d1 = g1[e] - a1[e];
            spread = fmaxf(spread, fmaxf(__builtin_fabsf(d0), __builtin_fabsf(d1)));
            l0[e] = (bs * kv[e]) * zoo_exp(d0);
            l1[e] = (bs * kv[4 + e]) * zoo_exp(d1);
            h0[e] = (bh * kv[e]) * zoo_exp(-d0);
            h1[e] = (bh * kv[4 + e]) * zoo_exp(-d1);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            l0[e] = bs * kv[e];
            l1[e] = bs * kv[4 + e];
            h0[e] = bh * kv[e];
            h1[e] = bh * kv[4 + e];
          }
        }
        *(lq_v4f*)(Lg_s + r * kOP + 8 * c8) = l0;
        *(lq_v4f*)(Lg_s + r * kOP + 8 * c8 + 4) = l1;
        *(lq_v4f*)(Hg_s + r * kOP + 8 * c8) = h0;
        *(lq_v4f*)(Hg_s + r * kOP + 8 * c8 + 4) = h1;
        if constexpr (CODES) {
          // Hw = beta^((1-sigma) tau) k rounded to the activation dtype, stored; its write codes
          // q8(Hw * fk, 1 / skw), fk = 1 | exp((1-eta)(g_last - g_t)) | exp(gk_last - gk_t - eta * le_t), go out
          // channel-major: the four lanes that hold tokens 4Q .. 4Q+3 of these eight channels (eight lanes apart)
          // exchange codes so that lane j of them owns channels 2j, 2j+1 of all four tokens, one dword each
          const float bw = bw_s[r], el = el_s[r];
          lq_v4i o;
#pragma unroll
          for (int d = 0; d < 4; ++d) o[d] = (int)zoo_enc2(bw * kv[2 * d], bw * kv[2 * d + 1], bf);
          *(lq_v4i*)(p.Hw + off) = o;
          const int n8 = 64 * ps + 8 * c8;
          const lq_v4f is0 = *(const lq_v4f*)(iskw_s + n8), is1 = *(const lq_v4f*)(iskw_s + n8 + 4);
          lq_v4f gl0 = {0.f, 0.f, 0.f, 0.f}, gl1 = gl0;
          if (DECAY == LQ_DECAY_DIAGONAL) gl0 = *(const lq_v4f*)(glast_s + n8), gl1 = *(const lq_v4f*)(glast_s + n8 + 4);
          int kc8[8];
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            float x0, x1;
            zoo_dec2((uint32_t)o[d], bf, x0, x1);
            if (DECAY == LQ_DECAY_SCALAR) x0 = x0 * el, x1 = x1 * el;
            if (DECAY == LQ_DECAY_DIAGONAL) {
              const float ga = d < 2 ? g0[(2 * d) & 3] : g1[(2 * d) & 3], gb = d < 2 ? g0[(2 * d + 1) & 3] : g1[(2 * d + 1) & 3];
              const float la = d < 2 ? gl0[(2 * d) & 3] : gl1[(2 * d) & 3], lb = d < 2 ? gl0[(2 * d + 1) & 3] : gl1[(2 * d + 1) & 3];
              x0 = x0 * zoo_exp(la - ga - el);
              x1 = x1 * zoo_exp(lb - gb - el);
            }
            const float ia = d < 2 ? is0[(2 * d) & 3] : is1[(2 * d) & 3], ib = d < 2 ? is0[(2 * d + 1) & 3] : is1[(2 * d + 1) & 3];
            kc8[2 * d] = zoo_q8(x0, ia, p.qmax), kc8[2 * d + 1] = zoo_q8(x1, ib, p.qmax);
          }
          c03[q] = zoo_pack_codes(kc8[0], kc8[1], kc8[2], kc8[3]), c47[q] = zoo_pack_codes(kc8[4], kc8[5], kc8[6], kc8[7]);
        }
      }
      if constexpr (CODES) {
        // the thread eight lanes away holds the other token pair of the quad (same channels): the even pair assembles
        // channels 0..3, the odd pair channels 4..7; four tokens x four channels are transposed bytewise in registers
        const int rr = tid >> 3, c8 = tid & 7;
        const bool odd = rr & 1;
        const uint32_t m0 = odd ? c47[0] : c03[0], m1 = odd ? c47[1] : c03[1];
        const uint32_t r0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(odd ? c03[0] : c47[0]), 0x128, 0xf, 0xf, false);  // row_ror:8
        const uint32_t r1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(odd ? c03[1] : c47[1]), 0x128, 0xf, 0xf, false);
        const uint32_t t0_ = odd ? r0 : m0, t1_ = odd ? r1 : m1, t2_ = odd ? m0 : r0, t3_ = odd ? m1 : r1;
        const uint32_t a01 = __builtin_amdgcn_perm(t1_, t0_, 0x05010400u), b01 = __builtin_amdgcn_perm(t3_, t2_, 0x05010400u);
        const uint32_t a23 = __builtin_amdgcn_perm(t1_, t0_, 0x07030602u), b23 = __builtin_amdgcn_perm(t3_, t2_, 0x07030602u);
        uint32_t ch[4];
        ch[0] = __builtin_amdgcn_perm(b01, a01, 0x05040100u), ch[1] = __builtin_amdgcn_perm(b01, a01, 0x07060302u);
        ch[2] = __builtin_amdgcn_perm(b23, a23, 0x05040100u), ch[3] = __builtin_amdgcn_perm(b23, a23, 0x07060302u);
        int8_t* kq = p.kqT + ((((int64_t)b * p.NT + ct) * H + h) * K + 64 * ps + 8 * c8 + 4 * (rr & 1)) * 64 + 4 * (rr >> 1);
#pragma unroll
        for (int e = 0; e < 4; ++e) *(uint32_t*)(kq + 64 * e) = ch[e];
      }
      __syncthreads();
#pragma unroll
      for (int q = 0; q < 3; ++q) {
        if (q >= nb) continue;
        const float* lp = Lg_s + (16 * blk_i(q) + rl) * kOP + 4 * kg;
        const float* hp = Hg_s + (16 * blk_j(q) + rl) * kOP + 4 * kg;
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
          const lq_v4f la = *(const lq_v4f*)(lp + 16 * s4), hb = *(const lq_v4f*)(hp + 16 * s4);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[q] = mfma_f32(la[e], hb[e], acc[q]);
        }
      }
    }
    bool one_anchor = true;
    if (DECAY == LQ_DECAY_DIAGONAL) one_anchor = __syncthreads_or(spread > 40.0f) == 0;
    else __syncthreads();
    // the operand buffers are dead: G overlays them
    if (one_anchor) {
      // lane holds column j = rl of block J, rows i = 4kg + r of block I
#pragma unroll
      for (int q = 0; q < 3; ++q) {
        if (q >= nb) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = 16 * blk_i(q) + 4 * kg + r, j = 16 * blk_j(q) + rl;
          float v = 0.0f;
          if (i > j) {
            v = acc[q][r];
            if (DECAY == LQ_DECAY_SCALAR) v = v * zoo_exp(gs_s[i] - gs_s[j]);
          }
          G_s[i * kGS + j] = v;
        }
      }
    } else {
      gram_rowblock<DECAY, K, BF, DK>(p, G_s, bs_s, bh_s, gs_s, wave, rl, kg, t0, h, dk_s);
    }
  }
  __syncthreads();

  // ---- T = (I + G)^-1: diagonal blocks by forward substitution (wave w, lane c < 16 holds column c of block w)
  if (lane < 16) {
    const int o = 16 * wave;
    float tc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float a = (i == lane) ? 1.0f : 0.0f;
#pragma unroll
      for (int j = 0; j < i; ++j) a = fmaf(-G_s[(o + i) * kGS + o + j], tc[j], a);
      tc[i] = a;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) T_s[(o + i) * kGS + o + lane] = tc[i];
  }
  __syncthreads();
  // block rows 1..3: wave J < I computes T_IJ = -T_II . sum_{J <= M < I} G_IM . T_MJ
  for (int I = 1; I < 4; ++I) {
    if (wave < I) {
      const int J = wave;
      lq_v4f sacc = {0.f, 0.f, 0.f, 0.f};
      for (int M = J; M < I; ++M)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const int m = 16 * M + 4 * s + kg;
          sacc = mfma_f32(G_s[(16 * I + rl) * kGS + m], T_s[m * kGS + 16 * J + rl], sacc);
        }
      // sacc: lane (rl = column, kg) holds rows 4kg + r, which is contraction index 4kg + s of the next product
      lq_v4f tacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) tacc = mfma_f32(T_s[(16 * I + rl) * kGS + 16 * I + 4 * kg + s], sacc[s], tacc);
#pragma unroll
      for (int r = 0; r < 4; ++r) T_s[(16 * I + 4 * kg + r) * kGS + 16 * J + rl] = -tacc[r];
    }
    __syncthreads();
  }

  // ---- T operands of this wave's two row blocks (w for the first half of the column tiles, 3 - w for the second:
  // equal work), split once and kept in registers
  lq_v4i th[2][2], tm[2][2], tl[2][2];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int st = 0; st < 2; ++st) t_operand(T_s, u ? 3 - wave : wave, st, rl, kg, th[u][st], tm[u][st], tl[u][st]);
  __syncthreads();  // T is dead from here on: the X tiles overlay it

  // each thread stages two adjacent tokens x 8 columns of a 64-column tile: a dword of the transposed tile is a token pair
  const int rp = tid >> 3, c8 = tid & 7;
  const int64_t tok0 = t0 + 2 * rp;
  auto stage = [&](const float (&xa)[8], const float (&xb)[8]) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      uint32_t hi, mid, lo;
      split3(xa[e], xb[e], hi, mid, lo);
      const int at = xt_index(8 * c8 + e, rp);
      Xt[at] = hi, Xt[kXT + at] = mid, Xt[2 * kXT + at] = lo;
    }
  };

  // ---- W and U passes, 64 columns at a time through the X tiles.  The global operands of a pass are requested while the
  // products of the pass before it run (requested at their point of use, each pass exposed a memory round trip between
  // two barriers).
  lq_v4i kraw[2], vraw[2];
  lq_v4f graw[2][2];
  float btr[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) btr[u] = p.beta[(tok0 + u) * H + h];
  auto request_k = [&](int kc) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int64_t off = ((tok0 + u) * H + h) * K + kc + 8 * c8;
      kraw[u] = *(const lq_v4i*)(p.k + off);
      if (DECAY == LQ_DECAY_DIAGONAL) graw[u][0] = *(const lq_v4f*)(p.g + off), graw[u][1] = *(const lq_v4f*)(p.g + off + 4);
    }
  };
  auto request_v = [&](int vc) {
#pragma unroll
    for (int u = 0; u < 2; ++u) vraw[u] = *(const lq_v4i*)(p.v + ((tok0 + u) * H + h) * V + vc + 8 * c8);
  };
  // (per-channel decay: its kernel sits at the register limit of four waves per SIMD, and holding a pass of k and g
  // across the products spilled: 272 -> 316 us; it requests at the point of use)
  constexpr bool kAhead = DECAY != LQ_DECAY_DIAGONAL;
  if (kAhead) request_k(0);
  float inv_sw = 0.0f;
  if constexpr (CODES) inv_sw = 1.0f / p.sw[h];

  // Hw is written straight out; X = beta^sigma k exp(g) is staged (over the dead Gram tile)
#pragma unroll
  for (int kc = 0; kc < K; kc += 64) {
    if (kc > 0) __syncthreads();
    if (!kAhead) request_k(kc);
    if constexpr (CODES) {
      // Hw and its codes were written while the Gram operands were staged: only X is formed here, two channels at a time
      // for both tokens of the thread (a token pair is one dword of the transposed tile), so that few values are live
      float bl[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        bl[u] = bs_s[2 * rp + u];
        if (DECAY == LQ_DECAY_SCALAR) bl[u] = bl[u] * zoo_exp(gs_s[2 * rp + u]);
      }
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        float x[2][2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          float k0, k1;
          zoo_dec2((uint32_t)kraw[u][d], bf, k0, k1);
          if constexpr (DK) {
            const int n = kc + 8 * c8 + 2 * d;
            const wy_v2f dd = *(const wy_v2f*)(dk_s + n), rr = *(const wy_v2f*)(dk_s + 128 + n);
            k0 = zoo_round_act(zoo_div_rn(k0, dd[0], rr[0]), BF);
            k1 = zoo_round_act(zoo_div_rn(k1, dd[1], rr[1]), BF);
          }
          float x0 = bl[u] * k0, x1 = bl[u] * k1;
          if (DECAY == LQ_DECAY_DIAGONAL) {
            x0 = x0 * zoo_exp(graw[u][d >> 1][(2 * d) & 3]);
            x1 = x1 * zoo_exp(graw[u][d >> 1][(2 * d + 1) & 3]);
          }
          x[u][0] = x0, x[u][1] = x1;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          uint32_t hi, mid, lo;
          split3(x[0][j], x[1][j], hi, mid, lo);
          const int at = xt_index(8 * c8 + 2 * d + j, rp);
          Xt[at] = hi, Xt[kXT + at] = mid, Xt[2 * kXT + at] = lo;
        }
      }
    } else
    {
      float xr[2][8];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int64_t off = ((tok0 + u) * H + h) * K + kc + 8 * c8;
        const float bw = powb(btr[u], (1.0f - sigma) * tau);
        float bl = bs_s[2 * rp + u];
        if (DECAY == LQ_DECAY_SCALAR) bl = bl * zoo_exp(gs_s[2 * rp + u]);
        float hw[8], kk[8];
#pragma unroll
        for (int d = 0; d < 4; ++d) zoo_dec2((uint32_t)kraw[u][d], bf, kk[2 * d], kk[2 * d + 1]);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const float k0 = kk[2 * d], k1 = kk[2 * d + 1];
          float x0 = bl * k0, x1 = bl * k1;
          if (DECAY == LQ_DECAY_DIAGONAL) {
            x0 = x0 * zoo_exp(graw[u][d >> 1][(2 * d) & 3]);
            x1 = x1 * zoo_exp(graw[u][d >> 1][(2 * d + 1) & 3]);
          }
          xr[u][2 * d] = x0, xr[u][2 * d + 1] = x1;
          hw[2 * d] = bw * k0, hw[2 * d + 1] = bw * k1;
        }
        lq_v4i o;
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = (int)zoo_enc2(hw[2 * d], hw[2 * d + 1], bf);
        *(lq_v4i*)(p.Hw + off) = o;
      }
      stage(xr[0], xr[1]);
    }
    __syncthreads();
    if (kc + 64 < K) {
      if (kAhead) request_k(kc + 64);
    } else if (kAhead) {
      request_v(0);
    }
    // W = T . X for these 64 columns
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int u = nt < 2 ? 0 : 1;
      const int I = u ? 3 - wave : wave;
      const lq_v4f a = tx_tile(Xt, th[u], tm[u], tl[u], I, nt, rl, kg);
      lq_v2i o;
      o[0] = (int)zoo_enc2(a[0], a[1], bf);
      o[1] = (int)zoo_enc2(a[2], a[3], bf);
      const int64_t woff = ((t0 + 16 * I + rl) * H + h) * K + kc + 16 * nt + 4 * kg;
      if (!CODES || p.W) *(lq_v2i*)(p.W + woff) = o;
      if constexpr (CODES) {  // state-read codes of the rounded W
        float w0, w1, w2, w3;
        zoo_dec2((uint32_t)o[0], bf, w0, w1);
        zoo_dec2((uint32_t)o[1], bf, w2, w3);
        *(uint32_t*)(p.wq + woff) = zoo_pack_codes(zoo_q8(w0, inv_sw, p.qmax), zoo_q8(w1, inv_sw, p.qmax),
                                                    zoo_q8(w2, inv_sw, p.qmax), zoo_q8(w3, inv_sw, p.qmax));
      }
    }
  }

  // ---- U = T . (beta^sigma v)
  for (int vc = 0; vc < V; vc += 64) {
    __syncthreads();
    if (!kAhead) request_v(vc);
    {
      float xr[2][8];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float bsr = bs_s[2 * rp + u];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          float v0, v1;
          zoo_dec2((uint32_t)vraw[u][d], bf, v0, v1);
          xr[u][2 * d] = bsr * v0, xr[u][2 * d + 1] = bsr * v1;
        }
      }
      stage(xr[0], xr[1]);
    }
    __syncthreads();
    if (kAhead) request_v(min(vc + 64, V - 64));  // unconditional: the last pass requests its own columns once more
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int u = nt < 2 ? 0 : 1;
      const int I = u ? 3 - wave : wave;
      const lq_v4f a = tx_tile(Xt, th[u], tm[u], tl[u], I, nt, rl, kg);
      lq_v2i o;
      o[0] = (int)zoo_enc2(a[0], a[1], bf);
      o[1] = (int)zoo_enc2(a[2], a[3], bf);
      *(lq_v2i*)(p.U + ((t0 + 16 * I + rl) * H + h) * V + vc + 16 * nt + 4 * kg) = o;
    }
  }
}

// ---- 128-token chunks: the same transform over a 128 x 128 Gram matrix (gated_delta_rule.py:20-47, kda.py:22-53 with
// chunk_size = 128), written for reach, not for speed: one workgroup per (chunk, batch*head) with the G tile in 67 KB of LDS
// (two workgroups per compute unit), inverted in place, everything on the fp32 MFMA.
//   Gram: wave w takes row blocks w and 7 - w (equal numbers of 16 x 16 blocks), per-channel decay anchored at the row
//     block's first row (both factors <= 1), operands straight from global memory (gram_rowblock).
//   Inverse, in place (row I of the tile holds G until block row I is done, T after): the eight diagonal blocks by forward
//     substitution, then block rows 1..7, every block of a row formed in registers before the row is overwritten.
//   W, U: T . X with X staged as fp32 in LDS 16 columns at a time.
// No write codes (lq_zoo_write_codes makes them from the stored Hw and W), no D_QK at load.
constexpr int kGS2 = 130;  // floats per row of the 128-row G / T tile (2 mod 4, as kGS)
constexpr int kXS2 = 20;   // floats per token row of the X slab (16 columns + pad); with the tile and the tables 77 KB

template <int DECAY, int K, bool BF>
__global__ __launch_bounds__(256, 2) void zoo_wy_prep128_kernel(WyParams p) {
  __shared__ __align__(16) float G_s[128 * kGS2];
  __shared__ __align__(16) float X_s[128 * kXS2];
  __shared__ float gs_s[128], bs_s[128], bh_s[128], bw_s[128];
  float* T_s = G_s;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rl = lane & 15, kg = lane >> 4;
  const int H = p.H, V = p.V;
  const int h = blockIdx.x % H;
  const int64_t grp = blockIdx.x / H;  // b * (T / 128) + chunk
  const int64_t t0 = grp * 128;        // (b * T + chunk * 128: T is a multiple of 128)
  const float sigma = p.sigma, tau = p.tau;
  constexpr bool bf = BF;

  if (tid < 128) {
    const float bt = p.beta[(t0 + tid) * H + h];
    bs_s[tid] = powb(bt, sigma);
    bh_s[tid] = powb(bt, 1.0f - sigma);
    bw_s[tid] = powb(bt, (1.0f - sigma) * tau);
    p.fw[(t0 + tid) * H + h] = powb(bt, (1.0f - sigma) * (1.0f - tau));
    gs_s[tid] = DECAY == LQ_DECAY_SCALAR ? p.g[(t0 + tid) * H + h] : 0.0f;
  }
  __syncthreads();

  // ---- Gram
#pragma unroll 1
  for (int u = 0; u < 2; ++u)
    gram_rowblock<DECAY, K, BF, false, 8, kGS2>(p, G_s, bs_s, bh_s, gs_s, u ? 7 - wave : wave, rl, kg, t0, h, nullptr);
  __syncthreads();

  // ---- T = (I + G)^-1: diagonal blocks (wave w: blocks w and w + 4; lane c < 16 holds column c)
  if (lane < 16) {
#pragma unroll 1
    for (int u = 0; u < 2; ++u) {
      const int o = 16 * (wave + 4 * u);
      float tc[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float a = (i == lane) ? 1.0f : 0.0f;
#pragma unroll
        for (int j = 0; j < i; ++j) a = fmaf(-G_s[(o + i) * kGS2 + o + j], tc[j], a);
        tc[i] = a;
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) T_s[(o + i) * kGS2 + o + lane] = tc[i];
    }
  }
  __syncthreads();
  // block rows 1..7: T_IJ = -T_II . sum_{J <= M < I} G_IM . T_MJ, the J of a row dealt to the waves
#pragma unroll 1
  for (int I = 1; I < 8; ++I) {
    lq_v4f tnew[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) tnew[u] = lq_v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int J = wave + 4 * u;
      if (J >= I) continue;
      lq_v4f sacc = {0.f, 0.f, 0.f, 0.f};
      for (int M = J; M < I; ++M)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const int m = 16 * M + 4 * s + kg;
          sacc = mfma_f32(G_s[(16 * I + rl) * kGS2 + m], T_s[m * kGS2 + 16 * J + rl], sacc);
        }
      // sacc: lane (rl = column, kg) holds rows 4kg + r, which is contraction index 4kg + s of the next product
      lq_v4f tacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) tacc = mfma_f32(T_s[(16 * I + rl) * kGS2 + 16 * I + 4 * kg + s], sacc[s], tacc);
      tnew[u] = tacc;
    }
    __syncthreads();  // every wave has read what it needs of row I's G blocks
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int J = wave + 4 * u;
      if (J < I) {
#pragma unroll
        for (int r = 0; r < 4; ++r) T_s[(16 * I + 4 * kg + r) * kGS2 + 16 * J + rl] = -tnew[u][r];
      }
    }
    __syncthreads();
  }

  // ---- W = T . X (X = beta^sigma k exp(g)) and U = T . (beta^sigma v), 16 columns at a time; Hw goes straight out.
  // Staging: thread (token = tid / 2, half = tid % 2) forms 8 columns of its token.
  const int tok = tid >> 1, hf = tid & 1;
  const int nslab = (K + V) / 16;
#pragma unroll 1
  for (int sl = 0; sl < nslab; ++sl) {
    const bool isk = sl < K / 16;
    const int cc = isk ? 16 * sl : 16 * sl - K;  // first column of the slab in k (or v)
    const int c0 = cc + 8 * hf;                  // first column of this thread
    __syncthreads();  // the slab is no longer read
    {
      float x[8];
      if (isk) {
        const int64_t off = ((t0 + tok) * H + h) * K + c0;
        float kk[8];
        zoo_ld8(p.k + off, bf, kk);
        float bl = bs_s[tok];
        if (DECAY == LQ_DECAY_SCALAR) bl = bl * zoo_exp(gs_s[tok]);
        const float bw = bw_s[tok];
        float hw[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          x[e] = bl * kk[e];
          hw[e] = bw * kk[e];
        }
        if (DECAY == LQ_DECAY_DIAGONAL) {
          const lq_v4f g0 = *(const lq_v4f*)(p.g + off), g1 = *(const lq_v4f*)(p.g + off + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) x[e] = x[e] * zoo_exp(g0[e]), x[4 + e] = x[4 + e] * zoo_exp(g1[e]);
        }
        lq_v4i o;
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = (int)zoo_enc2(hw[2 * d], hw[2 * d + 1], bf);
        *(lq_v4i*)(p.Hw + off) = o;
      } else {
        float vv[8];
        zoo_ld8(p.v + ((t0 + tok) * H + h) * V + c0, bf, vv);
        const float bsr = bs_s[tok];
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = bsr * vv[e];
      }
      *(lq_v4f*)(X_s + tok * kXS2 + 8 * hf) = lq_v4f{x[0], x[1], x[2], x[3]};
      *(lq_v4f*)(X_s + tok * kXS2 + 8 * hf + 4) = lq_v4f{x[4], x[5], x[6], x[7]};
    }
    __syncthreads();
    _Float16* dst = isk ? p.W : p.U;
    const int C = isk ? K : V;
#pragma unroll 1
    for (int u = 0; u < 2; ++u) {
      const int I = u ? 7 - wave : wave;
      lq_v4f acc = {0.f, 0.f, 0.f, 0.f};
      for (int s = 0; s < 4 * (I + 1); ++s)
        acc = mfma_f32(T_s[(16 * I + rl) * kGS2 + 4 * s + kg], X_s[(4 * s + kg) * kXS2 + rl], acc);
      // lane holds column rl of the slab, rows 16I + 4kg + r
#pragma unroll
      for (int r = 0; r < 4; ++r)
        *(uint16_t*)(dst + ((t0 + 16 * I + 4 * kg + r) * H + h) * C + cc + rl) = (uint16_t)zoo_enc1(acc[r], bf);
    }
  }
}

template <int DECAY, int K>
int launch128(const WyParams& p, hipStream_t stream) {
  const dim3 grid((uint32_t)((int64_t)(p.T / 128) * p.B * p.H));
  if (p.bf)
    hipLaunchKernelGGL((zoo_wy_prep128_kernel<DECAY, K, true>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_wy_prep128_kernel<DECAY, K, false>), grid, dim3(256), 0, stream, p);
  return lq_check_launch();
}

template <int K>
int launch128_decay(const WyParams& p, int decay, hipStream_t stream) {
  switch (decay) {
    case LQ_DECAY_NONE: return launch128<LQ_DECAY_NONE, K>(p, stream);
    case LQ_DECAY_SCALAR: return launch128<LQ_DECAY_SCALAR, K>(p, stream);
    case LQ_DECAY_DIAGONAL: return launch128<LQ_DECAY_DIAGONAL, K>(p, stream);
  }
  return LQ_ERR_SHAPE;
}

template <int DECAY, int K, bool CODES, bool DK>
int launch_c(const WyParams& p, dim3 grid, hipStream_t stream) {
  if (p.bf)
    hipLaunchKernelGGL((zoo_wy_prep_kernel<DECAY, K, true, CODES, DK>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((zoo_wy_prep_kernel<DECAY, K, false, CODES, DK>), grid, dim3(256), 0, stream, p);
  return lq_check_launch();
}

template <int DECAY, int K>
int launch(const WyParams& p, dim3 grid, hipStream_t stream) {
  if (p.dk_div) return launch_c<DECAY, K, true, true>(p, grid, stream);  // the rescaling comes with the codes (checked)
  return p.kqT ? launch_c<DECAY, K, true, false>(p, grid, stream) : launch_c<DECAY, K, false, false>(p, grid, stream);
}

template <int K>
int launch_decay(const WyParams& p, int decay, dim3 grid, hipStream_t stream) {
  switch (decay) {
    case LQ_DECAY_NONE: return launch<LQ_DECAY_NONE, K>(p, grid, stream);
    case LQ_DECAY_SCALAR: return launch<LQ_DECAY_SCALAR, K>(p, grid, stream);
    case LQ_DECAY_DIAGONAL: return launch<LQ_DECAY_DIAGONAL, K>(p, grid, stream);
  }
  return LQ_ERR_SHAPE;
}

}  // namespace

extern "C" int lq_zoo_wy_prep(const lq_zoo_wy_prep_args* a, hipStream_t stream) {
  if (!a || !a->k || !a->v || !a->beta || !a->Hw || !a->U || !a->fw) return LQ_ERR_NULL;
  if (a->decay != LQ_DECAY_NONE && !a->g) return LQ_ERR_NULL;
  const bool codes = a->kqT != nullptr;
  if (!codes && !a->W) return LQ_ERR_NULL;
  if (codes && (!a->wq || !a->ev || !a->gam || !a->skw || !a->sw)) return LQ_ERR_NULL;
  if (codes && a->decay == LQ_DECAY_DIAGONAL && !a->logenv) return LQ_ERR_NULL;
  if (codes && (a->qmax < 1 || a->qmax > 127)) return LQ_ERR_SHAPE;
  if (codes && (!zoo_al(a->kqT, 16) || !zoo_al(a->wq, 4) || !zoo_al(a->skw, 16))) return LQ_ERR_SHAPE;
  if ((a->dk_div != nullptr) != (a->dk_rcp != nullptr)) return LQ_ERR_NULL;
  if (a->pack && (!codes || !zoo_al(a->pack, 16))) return LQ_ERR_SHAPE;
  if (a->dk_div && !codes) return LQ_ERR_SHAPE;  // built for the launch that also makes the write operands
  if (a->dk_div && (!zoo_al(a->dk_div, 16) || !zoo_al(a->dk_rcp, 16))) return LQ_ERR_SHAPE;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  // 128-token chunks: a kernel of their own, without the write codes and without D_QK at load
  const bool big = a->chunk_size == 128;
  if (big && (codes || a->dk_div || !a->W)) return LQ_ERR_SHAPE;
  if ((a->chunk_size != 64 && !big) || a->seqlen % a->chunk_size != 0) return LQ_ERR_SHAPE;
  if ((a->kdim != 64 && a->kdim != 128) || a->vdim % 64 != 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  if (a->act_dtype != LQ_DT_F16 && a->act_dtype != LQ_DT_BF16) return LQ_ERR_SHAPE;
  if (!zoo_al(a->k, 16) || !zoo_al(a->v, 16) || !zoo_al(a->Hw, 16)) return LQ_ERR_SHAPE;
  if (a->decay == LQ_DECAY_DIAGONAL && !zoo_al(a->g, 16)) return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  WyParams p = {};
  p.k = (const _Float16*)a->k, p.v = (const _Float16*)a->v, p.beta = a->beta, p.g = a->g;
  p.Hw = (_Float16*)a->Hw, p.W = (_Float16*)a->W, p.U = (_Float16*)a->U, p.fw = a->fw;
  p.sigma = a->sigma, p.tau = a->tau, p.bf = a->act_dtype == LQ_DT_BF16;
  p.B = a->batch, p.T = a->seqlen, p.H = a->nheads, p.V = a->vdim;
  p.kqT = a->kqT, p.wq = a->wq, p.ev = a->ev, p.gam = a->gam, p.logenv = a->logenv, p.skw = a->skw, p.sw = a->sw;
  p.eta = a->eta, p.qmax = a->qmax, p.NT = a->seqlen / 64;
  p.dk_div = a->dk_div, p.dk_rcp = a->dk_rcp;
  p.pack = a->pack;
  if ((int64_t)(a->seqlen / 64) * a->batch * a->nheads > 0x7fffffff) return LQ_ERR_SHAPE;
  if (big) return a->kdim == 128 ? launch128_decay<128>(p, a->decay, stream) : launch128_decay<64>(p, a->decay, stream);
  dim3 grid((uint32_t)((a->seqlen / 64) * a->batch * a->nheads));
  return a->kdim == 128 ? launch_decay<128>(p, a->decay, grid, stream) : launch_decay<64>(p, a->decay, grid, stream);
}
