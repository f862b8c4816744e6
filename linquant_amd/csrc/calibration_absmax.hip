// Calibration collector: running absolute maximum of an activation tensor per (head, channel), per head or per tensor.
// Replaces the calibrating branch of Quantizer.__call__ (linquant/invariances.py:77-81) and the amax reductions of the
// SSD observers in scripts/nemotron_h_calibration.py (:327 x * scale_lut per (H, P); :536 gated B per (H, N); :583 x per
// (H, P)).  Pure HBM streaming: a workgroup owns a slab of rows and all H * D channels, a lane 8 adjacent channels (16
// bytes of fp16 / bf16, 32 of fp32); maxima live in registers and leave through one atomic maximum per lane and slab.
// |v| is never negative, so the fp32 bit pattern orders like an unsigned integer and atomicMax on the bits is exact.
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

}  // namespace

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
