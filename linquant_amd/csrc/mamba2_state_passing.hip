// Mamba-2 SSD stage 3: all-integer Q0.S fixed-point inter-chunk state recurrence.
// Replaces linquant/kernels/mamba2/state_passing.py:25-93 (launcher :96-121):
//   gate_q = clamp(rha(exp(dA_last[c]) * 2^S), -127, 127)
//   s32    = ((s32 * gate_q + 2^(S-1)) >> S) + new_i8[c]        (s32 never clamped in between)
//   out[c+1] = clamp(s32, -127, 127)  (c < nchunks-1),  final = clamp(s32) after the last chunk,
//   out[0] = 0.
//
// Pure HBM streaming: every thread owns VEC consecutive bytes of the flattened (P*N) state of one
// (batch, head) and walks the chunks.  Loads do not depend on the recurrence, so DEPTH chunks are
// kept in flight per thread.  |s32| <= 128 * 128 and |gate_q| <= 127, so the 24-bit multiplier is exact.
#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

template <int VEC>
struct Vec;
template <>
struct Vec<16> {
  typedef lq_v4i T;
};
template <>
struct Vec<8> {
  typedef lq_v2i T;
};
template <>
struct Vec<4> {
  typedef int T;
};

LQ_DEV uint32_t step_word(uint32_t w, int* s, int gate_q, int shift, int half) {
  uint32_t o = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int v = ((__mul24(s[i], gate_q) + half) >> shift) + lq_sbyte(w, i);
    s[i] = v;
    o |= (uint32_t)(lq_clampi(v, -127, 127) & 0xff) << (8 * i);
  }
  return o;
}

// INPLACE: `states` and `out` are one buffer of nchunks + 1 slots (out = slot 0, states = slot 1): slot c + 1 is read as
// the local state of chunk c and then overwritten, by the same thread, with the state entering chunk c + 1, so the two
// pointers alias and carry no __restrict__.  A (batch, head) whose gates all quantize to zero is finished before it
// starts: the state entering chunk c + 1 is then the local state of chunk c, which already sits in slot c + 1; only the
// zero slot and the final state are written.  (Its states are requested after the gates are known, not before.)
template <int VEC, int DEPTH, bool INPLACE>
__global__ __launch_bounds__(256) void state_passing_kernel(
    const int8_t* states, int64_t ss_b, int64_t ss_c, int64_t ss_h, int8_t* out,
    int64_t so_b, int64_t so_c, int64_t so_h, int8_t* __restrict__ fin, int64_t sf_b, int64_t sf_h,
    const float* __restrict__ dA, int64_t sd_b, int64_t sd_h, int64_t sd_c, int dim, int nchunks, int shift) {
  typedef typename Vec<VEC>::T V;
  constexpr int W = VEC / 4;
  extern __shared__ int gate_lds[];
  const int b = blockIdx.z, h = blockIdx.y;
  const float fs = (float)(1 << shift);
  // (a surplus lane keeps working on a clamped, in-range slice and stores nothing: no early exit before the barrier, and
  // the first states are requested before the gates are computed, so the two round trips overlap)
  const int64_t d_raw = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  const bool live = d_raw < dim;
  const int64_t d0 = live ? d_raw : 0;
  const int8_t* sp = states + (int64_t)b * ss_b + (int64_t)h * ss_h + d0;
  int8_t* op = out + (int64_t)b * so_b + (int64_t)h * so_h + d0;
  int8_t* fp = fin ? fin + (int64_t)b * sf_b + (int64_t)h * sf_h + d0 : nullptr;
  const int half = (1 << shift) >> 1;
  const bool even = nchunks % DEPTH == 0;  // uniform: the branch-free loop below needs whole groups of DEPTH chunks

  // the gate's request goes first: memory operations retire in issue order, so waiting for it then does not wait for the
  // states requested behind it
  const int cg = min((int)threadIdx.x, nchunks - 1);
  const float dA0 = dA[(int64_t)b * sd_b + (int64_t)h * sd_h + (int64_t)cg * sd_c];
  V buf[DEPTH];
  if (!INPLACE) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) buf[j] = __builtin_nontemporal_load((const V*)(sp + (int64_t)min(j, nchunks - 1) * ss_c));
  }

  const int gq0 = lq_q_rha(lq_expf(dA0) * fs, 127);
  gate_lds[cg] = gq0;  // surplus threads rewrite the last gate with the same value
  bool any_gate = gq0 != 0;
  for (int c = threadIdx.x + blockDim.x; c < nchunks; c += blockDim.x) {
    const float g = lq_expf(dA[(int64_t)b * sd_b + (int64_t)h * sd_h + (int64_t)c * sd_c]) * fs;
    const int gq = lq_q_rha(g, 127);
    gate_lds[c] = gq;
    any_gate = any_gate || gq != 0;
  }
  const int some = __syncthreads_or((int)any_gate);  // also makes the gate table visible
  if (!live) return;
  if (INPLACE) {
    if (!some) {
      V zero = {};
      __builtin_nontemporal_store(zero, (V*)op);
      if (fp) *(V*)fp = *(const V*)(sp + (int64_t)(nchunks - 1) * ss_c);  // codes of a chunk state lie within +-127 already
      return;
    }
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) buf[j] = __builtin_nontemporal_load((const V*)(sp + (int64_t)min(j, nchunks - 1) * ss_c));
  }

  int s[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) s[i] = 0;
  V zero = {};
  __builtin_nontemporal_store(zero, (V*)op);

  auto step = [&](const V& cur, int c) {
    const int gq = gate_lds[c];
    V res;
    const uint32_t* cw = (const uint32_t*)&cur;
    uint32_t* rw = (uint32_t*)&res;
#pragma unroll
    for (int w = 0; w < W; ++w) rw[w] = step_word(cw[w], s + 4 * w, gq, shift, half);
    return res;
  };

  if (even) {
    // whole groups: every request and every store of the steady state is unconditional, which keeps the compiler's
    // count of outstanding operations exact (with guards around them it drained the whole ring once per group)
    for (int c0 = 0; c0 + DEPTH < nchunks; c0 += DEPTH) {
#pragma unroll
      for (int j = 0; j < DEPTH; ++j) {
        const int c = c0 + j;
        const V cur = buf[j];
        buf[j] = __builtin_nontemporal_load((const V*)(sp + (int64_t)(c + DEPTH) * ss_c));
        *(V*)(op + (int64_t)(c + 1) * so_c) = step(cur, c);  // cached store: the chunk scan reads it two launches later
      }
    }
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {  // last group: nothing left to request
      const int c = nchunks - DEPTH + j;
      const V res = step(buf[j], c);
      if (j < DEPTH - 1) {
        *(V*)(op + (int64_t)(c + 1) * so_c) = res;
      } else if (fp) {
        __builtin_nontemporal_store(res, (V*)fp);
      }
    }
    return;
  }

  for (int c0 = 0; c0 < nchunks; c0 += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      const int c = c0 + j;
      if (c < nchunks) {
        V cur = buf[j];
        if (c + DEPTH < nchunks) buf[j] = __builtin_nontemporal_load((const V*)(sp + (int64_t)(c + DEPTH) * ss_c));
        const V res = step(cur, c);
        if (c < nchunks - 1) {
          *(V*)(op + (int64_t)(c + 1) * so_c) = res;
        } else if (fp) {
          __builtin_nontemporal_store(res, (V*)fp);
        }
      }
    }
  }
}

// Any strides / sizes: one element per thread.
__global__ __launch_bounds__(256) void state_passing_generic_kernel(
    const int8_t* __restrict__ states, int64_t ss_b, int64_t ss_c, int64_t ss_h, int64_t ss_d,
    int8_t* __restrict__ out, int64_t so_b, int64_t so_c, int64_t so_h, int64_t so_d, int8_t* __restrict__ fin,
    int64_t sf_b, int64_t sf_h, int64_t sf_d, const float* __restrict__ dA, int64_t sd_b, int64_t sd_h,
    int64_t sd_c, int dim, int nchunks, int shift) {
  const int b = blockIdx.z, h = blockIdx.y;
  const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (d >= dim) return;
  const float fs = (float)(1 << shift);
  const int half = (1 << shift) >> 1;
  int s = 0;
  out[(int64_t)b * so_b + (int64_t)h * so_h + d * so_d] = 0;
  for (int c = 0; c < nchunks; ++c) {
    const int gq = lq_q_rha(lq_expf(dA[(int64_t)b * sd_b + (int64_t)h * sd_h + (int64_t)c * sd_c]) * fs, 127);
    s = ((__mul24(s, gq) + half) >> shift) + (int)states[(int64_t)b * ss_b + (int64_t)c * ss_c + (int64_t)h * ss_h + d * ss_d];
    const int8_t q = (int8_t)lq_clampi(s, -127, 127);
    if (c < nchunks - 1)
      out[(int64_t)b * so_b + (int64_t)(c + 1) * so_c + (int64_t)h * so_h + d * so_d] = q;
    else if (fin)
      fin[(int64_t)b * sf_b + (int64_t)h * sf_h + d * sf_d] = q;
  }
}

template <int VEC, int DEPTH, bool INPLACE>
void launch_vec(const lq_state_passing_args* a, hipStream_t stream) {
  // one wave per workgroup: the (batch, head, slice) count then divides evenly over the compute units (measured
  // 9 % faster than 256-thread groups at B4 H80 dim 8192, where 640 groups left some units with 3 and some with 2)
  const int threads = 64;
  const int per_block = threads * VEC;
  dim3 grid((a->dim + per_block - 1) / per_block, a->nheads, a->batch);
  hipLaunchKernelGGL((state_passing_kernel<VEC, DEPTH, INPLACE>), grid, dim3(threads), (size_t)a->nchunks * sizeof(int), stream,
                     a->states, a->states_stride_b, a->states_stride_c, a->states_stride_h, a->out, a->out_stride_b,
                     a->out_stride_c, a->out_stride_h, a->final_states, a->final_stride_b, a->final_stride_h,
                     a->dA_chunk_cumsum, a->dA_stride_b, a->dA_stride_h, a->dA_stride_c, a->dim, a->nchunks,
                     a->gate_shift);
}

bool aligned(const void* p, int64_t n) { return ((uintptr_t)p % n) == 0; }

}  // namespace

extern "C" int lq_state_passing(const lq_state_passing_args* a, hipStream_t stream) {
  if (!a || !a->states || !a->out || !a->dA_chunk_cumsum) return LQ_ERR_NULL;
  if (a->batch <= 0 || a->nheads <= 0 || a->nchunks <= 0 || a->dim <= 0) return LQ_ERR_SHAPE;
  if (a->batch > 65535 || a->nheads > 65535) return LQ_ERR_SHAPE;
  if (a->gate_shift < 0 || a->gate_shift > 15) return LQ_ERR_SHAPE;
  // the running INT32 state is multiplied as a 24-bit quantity: with a gate of 127/128 or less (shift >= 7) it stays
  // below 127 * 128; with fewer fractional bits the gate can be exactly 1 and the state grows by up to 127 per chunk
  if (a->gate_shift < 7 && a->nchunks > 65536) return LQ_ERR_SHAPE;
  if (a->nchunks > 12288) return LQ_ERR_SHAPE;                      // gate table lives in LDS

  int vec = a->vec_hint;
  if (vec != 4 && vec != 8 && vec != 16) vec = 16;
  auto ok = [&](int v) {
    const bool dense = a->states_stride_d == 1 && a->out_stride_d == 1 && (!a->final_states || a->final_stride_d == 1);
    const bool strides = a->states_stride_b % v == 0 && a->states_stride_c % v == 0 && a->states_stride_h % v == 0 &&
                         a->out_stride_b % v == 0 && a->out_stride_c % v == 0 && a->out_stride_h % v == 0 &&
                         (!a->final_states || (a->final_stride_b % v == 0 && a->final_stride_h % v == 0));
    return dense && strides && a->dim % v == 0 && aligned(a->states, v) && aligned(a->out, v) &&
           (!a->final_states || aligned(a->final_states, v));
  };
  while (vec >= 4 && !ok(vec)) vec >>= 1;
  if (a->in_place) {
    // one buffer of nchunks + 1 slots: out = slot 0, states = slot 1, same strides, 16-byte vectors only
    if (a->in_place != 1 || vec != 16 || a->out_stride_b != a->states_stride_b || a->out_stride_c != a->states_stride_c ||
        a->out_stride_h != a->states_stride_h || a->states != a->out + a->out_stride_c)
      return LQ_ERR_SHAPE;
    launch_vec<16, 8, true>(a, stream);
  } else if (vec == 16) {
    launch_vec<16, 8, false>(a, stream);
  } else if (vec == 8) {
    launch_vec<8, 8, false>(a, stream);
  } else if (vec == 4) {
    launch_vec<4, 8, false>(a, stream);
  } else {
    dim3 grid((a->dim + 255) / 256, a->nheads, a->batch);
    hipLaunchKernelGGL(state_passing_generic_kernel, grid, dim3(256), 0, stream, a->states, a->states_stride_b,
                       a->states_stride_c, a->states_stride_h, a->states_stride_d, a->out, a->out_stride_b,
                       a->out_stride_c, a->out_stride_h, a->out_stride_d, a->final_states, a->final_stride_b,
                       a->final_stride_h, a->final_stride_d, a->dA_chunk_cumsum, a->dA_stride_b, a->dA_stride_h,
                       a->dA_stride_c, a->dim, a->nchunks, a->gate_shift);
  }
  return lq_check_launch();
}
