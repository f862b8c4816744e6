// WY / UT transform of the delta family, per chunk, in fp32.
// Replaces the torch prep linquant/kernels/zoo/gated_delta_rule.py:20-47 (no / scalar decay) and
// linquant/kernels/zoo/kda.py:22-53 (per-channel decay); the reference's default route through fla-core's
// prep kernels for sigma = tau = 1 is served by the same native prep.
//   L = beta^sigma k,  Hg = beta^(1-sigma) k
//   G[i][j] = sum_n L[i][n] Hg[j][n] * decay(i,j,n)  for i > j, decay = 1 | exp(g_i - g_j) | exp(g_in - g_jn)
//   T = (I + G)^-1  (unit lower triangular, forward substitution)
//   W = T (L * exp(g)),  U = T (beta^sigma v),  Hw = beta^((1-sigma) tau) k,  fw = beta^((1-sigma)(1-tau))
// Every decay exponent is <= 0 (i > j and g is non-increasing inside a chunk), so the per-channel Gram needs
// no anchoring when evaluated element by element.
//
// One 4-wave workgroup per (chunk, batch*head).  Tiles live in LDS as fp32; the Gram and the two products
// are register-tiled 4x4 per thread; the triangular inverse is done by one wavefront, lane c carrying
// column c of T in registers and reading G rows as LDS broadcasts.
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
  int B, T, H, V;
};

LQ_DEV float powb(float b, float e) {
  if (e == 0.0f) return 1.0f;
  if (e == 1.0f) return b;
  return __builtin_amdgcn_exp2f(e * __builtin_amdgcn_logf(b));
}

template <int DECAY, int K>
__global__ __launch_bounds__(256) void zoo_wy_prep_kernel(WyParams p) {
  constexpr int LS = K + 1;
  extern __shared__ __align__(16) float lds[];
  float* L_s = lds;                    // [64][LS]   L, later L * exp(g)
  float* H_s = L_s + 64 * LS;          // [64][LS]   Hg, later the value tile (64 columns at a time)
  float* G_s = H_s + 64 * LS;          // [64][65]   G, then T in place
  float* gd_s = G_s + 64 * 65;         // [64][LS]   per-channel cumulative decay (diagonal only)
  float* gs_s = (DECAY == LQ_DECAY_DIAGONAL) ? gd_s + 64 * LS : gd_s;  // [64] scalar cumulative decay
  float* bs_s = gs_s + 64;             // [64] beta^sigma

  const int tid = threadIdx.x;
  const int ct = blockIdx.x;
  const int b = blockIdx.y / p.H, h = blockIdx.y % p.H;
  const int H = p.H, V = p.V;
  const int64_t t0 = (int64_t)b * p.T + (int64_t)ct * 64;
  const float sigma = p.sigma, tau = p.tau;

  // ---- load: L, Hg, decay rows; Hw and fw are written straight out
  if (tid < 64) {
    const float bt = p.beta[(t0 + tid) * H + h];
    bs_s[tid] = powb(bt, sigma);
    p.fw[(t0 + tid) * H + h] = powb(bt, (1.0f - sigma) * (1.0f - tau));
    if (DECAY == LQ_DECAY_SCALAR) gs_s[tid] = p.g[(t0 + tid) * H + h];
  }
  for (int it = tid; it < 64 * (K / 8); it += 256) {
    const int r = it / (K / 8), c8 = it % (K / 8);
    const int64_t off = ((t0 + r) * H + h) * K + 8 * c8;
    const lq_v8h kv = *(const lq_v8h*)(p.k + off);
    const float bt = p.beta[(t0 + r) * H + h];
    const float bl = powb(bt, sigma), bh = powb(bt, 1.0f - sigma), bw = powb(bt, (1.0f - sigma) * tau);
    lq_v8h hw;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float kf = (float)kv[e];
      L_s[r * LS + 8 * c8 + e] = bl * kf;
      H_s[r * LS + 8 * c8 + e] = bh * kf;
      hw[e] = (_Float16)(bw * kf);
    }
    *(lq_v8h*)(p.Hw + off) = hw;
    if (DECAY == LQ_DECAY_DIAGONAL) {
      const lq_v4f g0 = *(const lq_v4f*)(p.g + off), g1 = *(const lq_v4f*)(p.g + off + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) gd_s[r * LS + 8 * c8 + e] = e < 4 ? g0[e & 3] : g1[e & 3];
    }
  }
  __syncthreads();

  // ---- Gram, strictly lower part: thread (ti, tj) owns rows 4ti..4ti+3, cols 4tj..4tj+3
  {
    const int ti = tid >> 4, tj = tid & 15;
    float a[4][4];
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int y = 0; y < 4; ++y) a[x][y] = 0.0f;
    if (tj <= ti) {
      for (int n = 0; n < K; ++n) {
        float lv[4], hv[4], gi[4], gj[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          lv[x] = L_s[(4 * ti + x) * LS + n];
          hv[x] = H_s[(4 * tj + x) * LS + n];
          if (DECAY == LQ_DECAY_DIAGONAL) {
            gi[x] = gd_s[(4 * ti + x) * LS + n];
            gj[x] = gd_s[(4 * tj + x) * LS + n];
          }
        }
#pragma unroll
        for (int x = 0; x < 4; ++x)
#pragma unroll
          for (int y = 0; y < 4; ++y) {
            if (DECAY == LQ_DECAY_DIAGONAL) {
              const float w = (4 * ti + x > 4 * tj + y) ? __expf(gi[x] - gj[y]) : 0.0f;
              a[x][y] = fmaf(lv[x] * hv[y], w, a[x][y]);
            } else {
              a[x][y] = fmaf(lv[x], hv[y], a[x][y]);
            }
          }
      }
    }
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int y = 0; y < 4; ++y) {
        const int i = 4 * ti + x, j = 4 * tj + y;
        float v = 0.0f;
        if (i > j) {
          v = a[x][y];
          if (DECAY == LQ_DECAY_SCALAR) v = v * __expf(gs_s[i] - gs_s[j]);
        }
        G_s[i * 65 + j] = v;
      }
  }
  __syncthreads();

  // ---- T = (I + G)^-1 by forward substitution (wave 0; lane c holds column c), stored over G
  if (tid < 64) {
    float tc[64];
#pragma unroll
    for (int i = 0; i < 64; ++i) {
      float acc = (i == tid) ? 1.0f : 0.0f;
#pragma unroll
      for (int j = 0; j < i; ++j) acc = fmaf(-G_s[i * 65 + j], tc[j], acc);
      tc[i] = acc;
    }
#pragma unroll
    for (int i = 0; i < 64; ++i) G_s[i * 65 + tid] = tc[i];
  }
  // meanwhile: L <- L * exp(g) (read-side decay of W's right-hand side)
  if (DECAY != LQ_DECAY_NONE && tid >= 64) {
    for (int it = tid - 64; it < 64 * K; it += 192) {
      const int r = it / K, n = it % K;
      const float gg = (DECAY == LQ_DECAY_SCALAR) ? gs_s[r] : gd_s[r * LS + n];
      L_s[r * LS + n] = L_s[r * LS + n] * __expf(gg);
    }
  }
  __syncthreads();

  // ---- W = T . L'  (64 x K): thread owns rows 4ti..+3, cols {tj + 16c}
  {
    const int ti = tid >> 4, tj = tid & 15;
    constexpr int NC = K / 16;
    float a[4][NC];
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int c = 0; c < NC; ++c) a[x][c] = 0.0f;
    for (int j = 0; j < 4 * ti + 4; ++j) {
      float tv[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) tv[x] = G_s[(4 * ti + x) * 65 + j];
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const float r = L_s[j * LS + tj + 16 * c];
#pragma unroll
        for (int x = 0; x < 4; ++x) a[x][c] = fmaf(tv[x], r, a[x][c]);
      }
    }
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int c = 0; c < NC; ++c) p.W[((t0 + 4 * ti + x) * H + h) * K + tj + 16 * c] = (_Float16)a[x][c];
  }

  // ---- U = T . (beta^sigma v), 64 value columns at a time through the Hg buffer
  for (int vc = 0; vc < V; vc += 64) {
    __syncthreads();
    for (int it = tid; it < 64 * 8; it += 256) {
      const int r = it >> 3, c8 = it & 7;
      const lq_v8h vv = *(const lq_v8h*)(p.v + ((t0 + r) * H + h) * V + vc + 8 * c8);
      const float bsr = bs_s[r];
#pragma unroll
      for (int e = 0; e < 8; ++e) H_s[r * LS + 8 * c8 + e] = bsr * (float)vv[e];
    }
    __syncthreads();
    const int ti = tid >> 4, tj = tid & 15;
    float a[4][4];
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int c = 0; c < 4; ++c) a[x][c] = 0.0f;
    for (int j = 0; j < 4 * ti + 4; ++j) {
      float tv[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) tv[x] = G_s[(4 * ti + x) * 65 + j];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float r = H_s[j * LS + tj + 16 * c];
#pragma unroll
        for (int x = 0; x < 4; ++x) a[x][c] = fmaf(tv[x], r, a[x][c]);
      }
    }
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int c = 0; c < 4; ++c) p.U[((t0 + 4 * ti + x) * H + h) * V + vc + tj + 16 * c] = (_Float16)a[x][c];
  }
}

template <int DECAY, int K>
int launch(const WyParams& p, dim3 grid, hipStream_t stream) {
  constexpr int LS = K + 1;
  const size_t lds = sizeof(float) * (2 * 64 * LS + 64 * 65 + (DECAY == LQ_DECAY_DIAGONAL ? 64 * LS : 0) + 128);
  if (lds > 65536 && hipFuncSetAttribute(reinterpret_cast<const void*>(&zoo_wy_prep_kernel<DECAY, K>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return LQ_ERR_LAUNCH;
  hipLaunchKernelGGL((zoo_wy_prep_kernel<DECAY, K>), grid, dim3(256), lds, stream, p);
  return lq_check_launch();
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
  if (!a || !a->k || !a->v || !a->beta || !a->Hw || !a->W || !a->U || !a->fw) return LQ_ERR_NULL;
  if (a->decay != LQ_DECAY_NONE && !a->g) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0) return LQ_ERR_SHAPE;
  if (a->chunk_size != 64 || a->seqlen % 64 != 0) return LQ_ERR_SHAPE;
  if ((a->kdim != 64 && a->kdim != 128) || a->vdim % 64 != 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  if (!zoo_al(a->k, 16) || !zoo_al(a->v, 16) || !zoo_al(a->Hw, 16)) return LQ_ERR_SHAPE;
  if ((int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  WyParams p = {};
  p.k = (const _Float16*)a->k, p.v = (const _Float16*)a->v, p.beta = a->beta, p.g = a->g;
  p.Hw = (_Float16*)a->Hw, p.W = (_Float16*)a->W, p.U = (_Float16*)a->U, p.fw = a->fw;
  p.sigma = a->sigma, p.tau = a->tau;
  p.B = a->batch, p.T = a->seqlen, p.H = a->nheads, p.V = a->vdim;
  dim3 grid(a->seqlen / 64, a->batch * a->nheads);
  return a->kdim == 128 ? launch_decay<128>(p, a->decay, grid, stream) : launch_decay<64>(p, a->decay, grid, stream);
}
