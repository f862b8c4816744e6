// Measurement aid: a matrix-core-only kernel that gives the INT8 / fp16 MFMA issue peak of the machine it runs on, the
// denominator of the "fraction of MFMA peak" the benchmark reports for the contraction kernels.  Every wave keeps eight
// independent accumulator tiles in flight, so the matrix pipeline never waits for a result; operands stay in registers.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

typedef int lq_v8i __attribute__((ext_vector_type(8)));

template <int KIND>
__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters, int* sink) {
  const int lane = threadIdx.x;
  if (KIND == 0) {  // v_mfma_i32_16x16x64_i8
    lq_v4i a = {lane, lane + 1, lane + 2, lane + 3}, b = {lane * 3, lane * 5, lane * 7, lane * 11};
    lq_v4i acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = lq_v4i{j, 0, 0, 0};
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[j], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
    if (s == 0x7fffffff) *sink = s;  // keeps the loop alive without a store on the timed path
  } else if (KIND == 1) {  // v_mfma_f32_16x16x32_f16
    lq_v8h a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] = (_Float16)(0.001f * (lane + e)), b[e] = (_Float16)(0.002f * (lane - e));
    lq_v4f acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = lq_v4f{(float)j, 0.f, 0.f, 0.f};
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
    if (s == 123456.789f) *sink = (int)s;
  } else {  // v_mfma_i32_32x32x32_i8
    lq_v4i a = {lane, lane + 1, lane + 2, lane + 3}, b = {lane * 3, lane * 5, lane * 7, lane * 11};
    lq_v16i acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[j][e] = j + e;
    for (int i = 0; i < iters; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[j], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) s += acc[j][e];
    if (s == 0x7fffffff) *sink = s;
  }
}

}  // namespace

extern "C" int lq_probe_mfma(const lq_probe_mfma_args* a, hipStream_t stream) {
  if (!a || !a->sink) return LQ_ERR_NULL;
  if (a->iters <= 0 || a->blocks <= 0 || a->kind < 0 || a->kind > 2) return LQ_ERR_SHAPE;
  const dim3 grid(a->blocks), block(256);
  if (a->kind == 0)
    hipLaunchKernelGGL((mfma_probe_kernel<0>), grid, block, 0, stream, a->iters, a->sink);
  else if (a->kind == 1)
    hipLaunchKernelGGL((mfma_probe_kernel<1>), grid, block, 0, stream, a->iters, a->sink);
  else
    hipLaunchKernelGGL((mfma_probe_kernel<2>), grid, block, 0, stream, a->iters, a->sink);
  return lq_check_launch();
}
