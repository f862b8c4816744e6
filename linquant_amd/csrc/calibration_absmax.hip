// Calibration collector: running absolute maximum of an activation tensor per (head, channel), per head or per tensor.
// Replaces the calibrating branch of Quantizer.__call__ (linquant/invariances.py:77-81) and the amax reductions of the
// SSD observers in scripts/nemotron_h_calibration.py (:327 x * scale_lut per (H, P); :536 gated B per (H, N); :583 x per
// (H, P)).  Pure HBM streaming: a workgroup owns a slab of rows and all H * D channels, a lane 8 adjacent channels (16
// bytes of fp16 / bf16, 32 of fp32); maxima live in registers and leave through one atomic maximum per lane and slab.
// |v| is never negative, so the fp32 bit pattern orders like an unsigned integer and atomicMax on the bits is exact.
// The two observers that reduce a product rather than a tensor (the chunk states of scripts/nemotron_h_calibration.py:
// 602-651 and C.B^T of scripts/nemotron_h_w4a8.py:126-169) form the product in fp32 on the vector ALU, tile by tile in
// registers, and keep only its running maximum: calibration-time code, a few GFLOP per batch, nothing is stored.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int kRowsPerBlock = 128;

LQ_DEV void load8(const void* x, int dtype, int64_t off, float (&v)[8]) {
  if (dtype == LQ_DT_F32) {
    const lq_v4f a = *(const lq_v4f*)((const float*)x + off), b = *(const lq_v4f*)((const float*)x + off + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = a[e], v[e + 4] = b[e];
  } else {
    const lq_v4i raw = *(const lq_v4i*)((const uint16_t*)x + off);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t w = (uint32_t)raw[d];
      if (dtype == LQ_DT_BF16) {
        v[2 * d] = __uint_as_float(w << 16);
        v[2 * d + 1] = __uint_as_float(w & 0xffff0000u);
      } else {
        const lq_v2h h = __builtin_bit_cast(lq_v2h, w);
        v[2 * d] = (float)h[0];
        v[2 * d + 1] = (float)h[1];
      }
    }
  }
}

__global__ __launch_bounds__(256) void absmax_kernel(lq_absmax_args a) {
  const int c8n = (a.nheads * a.dim) >> 3;  // 8-channel pieces per row
  const int b = blockIdx.z;
  const int r0 = blockIdx.y * kRowsPerBlock, r1 = min(a.rows, r0 + kRowsPerBlock);
  for (int piece = blockIdx.x * 256 + threadIdx.x; piece < c8n; piece += gridDim.x * 256) {
    const int h = (piece * 8) / a.dim, d = (piece * 8) % a.dim;
    const int64_t xo = (int64_t)b * a.x_stride_b + (int64_t)(h / a.heads_per_group) * a.x_stride_h + d;
    const int64_t go = (int64_t)b * a.gate_stride_b + (int64_t)h * a.gate_stride_h;
    float m[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int r = r0; r < r1; ++r) {
      float v[8];
      load8(a.x, a.x_dtype, xo + (int64_t)r * a.x_stride_t, v);
      const float gt = a.gate ? a.gate[go + (int64_t)r * a.gate_stride_t] : 1.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float y = a.gate ? v[e] * gt : v[e];
        const float ay = __builtin_fabsf(y);
        m[e] = (ay > m[e] || ay != ay) ? ay : m[e];  // a NaN sticks
      }
    }
    uint32_t* out = (uint32_t*)a.out;
    if (a.mode == 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) atomicMax(out + (int64_t)h * a.dim + d + e, __float_as_uint(m[e]));
    } else {
      float mm = m[0];
#pragma unroll
      for (int e = 1; e < 8; ++e) mm = (m[e] > mm || m[e] != m[e]) ? m[e] : mm;
      atomicMax(out + (a.mode == 1 ? h : 0), __float_as_uint(mm));
    }
  }
}

bool al(const void* q, int n) { return ((uintptr_t)q % n) == 0; }

LQ_DEV float load1(const void* x, int dtype, int64_t off) {
  if (dtype == LQ_DT_F32) return ((const float*)x)[off];
  const uint32_t w = ((const uint16_t*)x)[off];
  return dtype == LQ_DT_BF16 ? __uint_as_float(w << 16) : (float)__builtin_bit_cast(_Float16, (uint16_t)w);
}

LQ_DEV float nanmax(float m, float a) { return (a > m || a != a) ? a : m; }

// Chunk-state observer: one workgroup per (64 value channels, chunk, head, batch).  Thread (p = tid & 63, quarter =
// tid >> 6) keeps the N / 4 sums of its channel against one quarter of the state columns; a token's B row is the same
// for every lane of a wavefront (one broadcast request), its gated x value differs per lane (128 contiguous bytes).
// fp32 products and sums in token order: what an fp32 einsum of the same operands computes, in a fixed order.
template <int NPT>
__global__ __launch_bounds__(256) void chunk_state_absmax_kernel(lq_absmax_chunk_state_args a) {
  const int tid = threadIdx.x, p = (int)blockIdx.x * 64 + (tid & 63), quarter = tid >> 6;
  const int c = blockIdx.y;
  const int h = (int)blockIdx.z % a.nheads, b = (int)blockIdx.z / a.nheads;
  const int g = h / (a.nheads / a.ngroups);
  const int k0 = c * a.chunk_size, k1 = min(a.seqlen, k0 + a.chunk_size);
  float acc[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) acc[i] = 0.0f;
  const int64_t xb = (int64_t)b * a.x_stride_b + (int64_t)h * a.x_stride_h + p;
  const int64_t bb = (int64_t)b * a.B_stride_b + (int64_t)g * a.B_stride_g + quarter * NPT;
  const int64_t gb = (int64_t)b * a.gate_stride_b + (int64_t)h * a.gate_stride_h;
  for (int k = k0; k < k1; ++k) {
    const float xg = load1(a.x, a.x_dtype, xb + (int64_t)k * a.x_stride_l) * a.gate[gb + (int64_t)k * a.gate_stride_l];
#pragma unroll
    for (int i8 = 0; i8 < NPT; i8 += 8) {
      float bv[8];
      load8(a.B, a.B_dtype, bb + (int64_t)k * a.B_stride_l + i8, bv);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[i8 + e] = acc[i8 + e] + xg * bv[e];
    }
  }
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < NPT; ++i) m = nanmax(m, __builtin_fabsf(acc[i]));
  atomicMax((uint32_t*)a.out + (int64_t)h * a.headdim + p, __float_as_uint(m));
}

// C.B^T observer: one workgroup per (64 rows m, chunk, group, batch); thread (m = tid & 63, quarter = tid >> 6) meets
// its C row with the tokens k of one quarter of the chunk, sixteen at a time; B rows are broadcast
// requests, the C row piece is re-read per block of sixteen tokens (it stays in the first-level cache).
__global__ __launch_bounds__(256) void cb_absmax_kernel(lq_absmax_cb_args a) {
  const int tid = threadIdx.x, quarter = tid >> 6;
  const int Q = a.chunk_size;
  const int mtiles = (Q + 63) / 64;
  const int c = (int)blockIdx.x / mtiles, m = ((int)blockIdx.x % mtiles) * 64 + (tid & 63);
  const int g = blockIdx.y, b = blockIdx.z;
  const int t0 = c * Q, limit = min(Q, a.seqlen - t0);
  const int kq = (Q + 3) / 4;  // tokens per quarter
  const int kbeg = quarter * kq, kend = min(limit, kbeg + kq);
  const int mrow = min(m, limit - 1);  // rows past the end repeat the last one (a maximum does not mind)
  const int64_t cbase = (int64_t)b * a.C_stride_b + (int64_t)(t0 + mrow) * a.C_stride_l + (int64_t)g * a.C_stride_g;
  const int64_t bbase = (int64_t)b * a.B_stride_b + (int64_t)t0 * a.B_stride_l + (int64_t)g * a.B_stride_g;
  float best = 0.0f;
  for (int kb = kbeg; kb < kend; kb += 16) {
    float acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0.0f;
    for (int n = 0; n < a.dstate; n += 8) {
      float cv[8];
      load8(a.C, a.C_dtype, cbase + n, cv);
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int k = min(kb + j, limit - 1);
        float bv[8];
        load8(a.B, a.B_dtype, bbase + (int64_t)k * a.B_stride_l + n, bv);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j] = acc[j] + cv[e] * bv[e];
      }
    }
#pragma unroll
    for (int j = 0; j < 16; ++j)
      if (kb + j < kend) best = nanmax(best, __builtin_fabsf(acc[j]));
  }
  atomicMax((uint32_t*)a.out + g, __float_as_uint(best));
}

bool dtype_ok(int d) { return d == LQ_DT_F16 || d == LQ_DT_BF16 || d == LQ_DT_F32; }

// rows read as 16-byte (two-byte types) or 2 x 16-byte (fp32) pieces of eight elements
bool rows_ok(const void* p, int dtype, int64_t s0, int64_t s1, int64_t s2) {
  const int esz = dtype == LQ_DT_F32 ? 4 : 2;
  return al(p, 16) && (s0 * esz) % 16 == 0 && (s1 * esz) % 16 == 0 && (s2 * esz) % 16 == 0;
}

}  // namespace

extern "C" int lq_absmax_chunk_state(const lq_absmax_chunk_state_args* a, hipStream_t stream) {
  if (!a || !a->x || !a->B || !a->gate || !a->out) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0 || a->ngroups <= 0 || a->nheads % a->ngroups != 0) return LQ_ERR_SHAPE;
  if (a->headdim <= 0 || a->headdim % 64 != 0 || a->chunk_size <= 0) return LQ_ERR_SHAPE;
  if (a->dstate != 64 && a->dstate != 128 && a->dstate != 256) return LQ_ERR_SHAPE;
  if (!dtype_ok(a->x_dtype) || !dtype_ok(a->B_dtype)) return LQ_ERR_SHAPE;
  if (!rows_ok(a->B, a->B_dtype, a->B_stride_b, a->B_stride_l, a->B_stride_g)) return LQ_ERR_SHAPE;
  const int64_t nchunks = ((int64_t)a->seqlen + a->chunk_size - 1) / a->chunk_size;
  if (nchunks > 65535 || (int64_t)a->batch * a->nheads > 65535) return LQ_ERR_SHAPE;
  dim3 grid((unsigned)(a->headdim / 64), (unsigned)nchunks, (unsigned)(a->batch * a->nheads));
  if (a->dstate == 64)
    hipLaunchKernelGGL(chunk_state_absmax_kernel<16>, grid, dim3(256), 0, stream, *a);
  else if (a->dstate == 128)
    hipLaunchKernelGGL(chunk_state_absmax_kernel<32>, grid, dim3(256), 0, stream, *a);
  else
    hipLaunchKernelGGL(chunk_state_absmax_kernel<64>, grid, dim3(256), 0, stream, *a);
  return lq_check_launch();
}

extern "C" int lq_absmax_cb(const lq_absmax_cb_args* a, hipStream_t stream) {
  if (!a || !a->C || !a->B || !a->out) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->ngroups <= 0 || a->chunk_size <= 0) return LQ_ERR_SHAPE;
  if (a->dstate <= 0 || a->dstate % 8 != 0) return LQ_ERR_SHAPE;
  if (!dtype_ok(a->C_dtype) || !dtype_ok(a->B_dtype)) return LQ_ERR_SHAPE;
  if (!rows_ok(a->C, a->C_dtype, a->C_stride_b, a->C_stride_l, a->C_stride_g) ||
      !rows_ok(a->B, a->B_dtype, a->B_stride_b, a->B_stride_l, a->B_stride_g))
    return LQ_ERR_SHAPE;
  const int64_t nchunks = ((int64_t)a->seqlen + a->chunk_size - 1) / a->chunk_size;
  const int64_t mtiles = ((int64_t)a->chunk_size + 63) / 64;
  if (nchunks * mtiles >= (1ll << 31) || a->ngroups > 65535 || a->batch > 65535) return LQ_ERR_SHAPE;
  dim3 grid((unsigned)(nchunks * mtiles), (unsigned)a->ngroups, (unsigned)a->batch);
  hipLaunchKernelGGL(cb_absmax_kernel, grid, dim3(256), 0, stream, *a);
  return lq_check_launch();
}

extern "C" int lq_absmax(const lq_absmax_args* a, hipStream_t stream) {
  if (!a || !a->x || !a->out) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->rows <= 0 || a->nheads <= 0 || a->dim <= 0 || a->dim % 8 != 0) return LQ_ERR_SHAPE;
  if (a->heads_per_group <= 0 || a->nheads % a->heads_per_group != 0) return LQ_ERR_SHAPE;
  if (a->mode < 0 || a->mode > 2) return LQ_ERR_SHAPE;
  if (a->x_dtype != LQ_DT_F16 && a->x_dtype != LQ_DT_BF16 && a->x_dtype != LQ_DT_F32) return LQ_ERR_SHAPE;
  const int esz = a->x_dtype == LQ_DT_F32 ? 4 : 2;
  if (!al(a->x, 16) || (a->x_stride_b * esz) % 16 || (a->x_stride_t * esz) % 16 || (a->x_stride_h * esz) % 16)
    return LQ_ERR_SHAPE;
  if (a->batch > 65535) return LQ_ERR_SHAPE;
  const int c8n = (a->nheads * a->dim) / 8;
  const int slabs = (a->rows + kRowsPerBlock - 1) / kRowsPerBlock;
  if (slabs > 65535) return LQ_ERR_SHAPE;
  dim3 grid((unsigned)((c8n + 255) / 256), (unsigned)slabs, (unsigned)a->batch);
  hipLaunchKernelGGL(absmax_kernel, grid, dim3(256), 0, stream, *a);
  return lq_check_launch();
}
