// The Mamba-2 INT8 SSD forward as one C call: cumsum -> chunk state -> state passing -> C.B^T -> chunk scan launched
// back to back on the caller's stream.  Replaces the orchestration of linquant/kernels/mamba2/ssd_combined.py:58-131;
// the intermediates that function allocates per call live in one workspace: caller-supplied (lq_ssd_combined) or a
// device array that is part of the library image (lq_ssd_combined_static, for callers that cannot allocate).
#include <mutex>

#include "lq_common.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int64_t kAlign = 256;
int64_t up(int64_t n) { return (n + kAlign - 1) / kAlign * kAlign; }

struct Layout {
  int64_t dt, dA, slots, cb, rowmax, total;  // slots: (B, nchunks + 1, H, P*N), slot c = state entering chunk c
  int nchunks;
};

int plan(const lq_ssd_combined_args* a, Layout* l) {
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0 || a->headdim <= 0 || a->ngroups <= 0 || a->dstate <= 0 ||
      a->chunk_size <= 0)
    return LQ_ERR_SHAPE;
  const int64_t Q = a->chunk_size, nc = (a->seqlen + Q - 1) / Q;
  const int64_t fl = (int64_t)a->batch * a->nheads * nc * Q * 4;
  const int64_t st = (int64_t)a->batch * nc * a->nheads * a->headdim * a->dstate;
  const int64_t cb = (int64_t)a->batch * nc * a->ngroups * Q * Q;
  l->nchunks = (int)nc;
  l->dt = 0;
  l->dA = l->dt + up(fl);
  l->slots = l->dA + up(fl);
  l->cb = l->slots + up(st + (int64_t)a->batch * a->nheads * a->headdim * a->dstate);
  l->rowmax = l->cb + up(cb);
  l->total = l->rowmax + up((int64_t)a->batch * a->seqlen * a->ngroups * 4);
  return LQ_OK;
}

int run(const lq_ssd_combined_args* a, char* ws, const Layout& l, hipStream_t stream) {
  float* dt = (float*)(ws + l.dt);
  float* dA = (float*)(ws + l.dA);
  // chunk states and passed states share one buffer of nchunks + 1 slots per batch row: the chunk state kernel writes the
  // local state of chunk c into slot c + 1, state passing turns it in place into the state entering chunk c + 1 (nothing
  // to do where the gate quantizes to zero), the chunk scan reads slot c
  const int64_t slot = (int64_t)a->nheads * a->headdim * a->dstate;
  const int64_t slots_b = (int64_t)(l.nchunks + 1) * slot;
  int8_t* passed = (int8_t*)(ws + l.slots);
  int8_t* states = passed + slot;
  int8_t* cb = (int8_t*)(ws + l.cb);
  const int Q = a->chunk_size, nc = l.nchunks;
  int rc;

  lq_chunk_cumsum_args cs = {};
  cs.dt = a->dt, cs.dt_dtype = a->dt_dtype;
  cs.dt_stride_b = a->dt_stride_b, cs.dt_stride_l = a->dt_stride_l, cs.dt_stride_h = a->dt_stride_h;
  cs.dt_scale = a->dt_scale, cs.A_log = a->A_log, cs.A_log_stride_h = a->A_log_stride_h, cs.A_log_scale = a->A_log_scale;
  cs.dt_bias = a->dt_bias, cs.dt_bias_stride_h = a->dt_bias_stride_h;
  cs.dt_out = dt, cs.dA_cumsum = dA;
  cs.batch = a->batch, cs.seqlen = a->seqlen, cs.nheads = a->nheads, cs.chunk_size = Q;
  cs.dt_softplus = a->dt_softplus, cs.dt_min = a->dt_min, cs.dt_max = a->dt_max;
  if ((rc = lq_chunk_cumsum(&cs, stream)) != LQ_OK) return rc;

  if (a->keyside) {
    lq_chunk_state_key_args k = {};
    k.x = a->x, k.x_stride_b = a->x_stride_b, k.x_stride_l = a->x_stride_l, k.x_stride_h = a->x_stride_h;
    k.B = a->b_fp, k.B_stride_b = a->bfp_stride_b, k.B_stride_l = a->bfp_stride_l, k.B_stride_g = a->bfp_stride_g;
    k.dt = dt, k.dA_cumsum = dA;
    k.x_scale_hp = a->x_scale_hp, k.xs_stride_h = a->xs_stride_h, k.xs_stride_p = a->xs_stride_p;
    k.out_qscale = a->state_scale, k.oqs_stride_h = a->ss_stride_h, k.oqs_stride_p = a->ss_stride_p;
    k.b_gate_scale = a->b_gate_scale;
    k.bgs_stride_b = a->bgs_stride_b, k.bgs_stride_c = a->bgs_stride_c, k.bgs_stride_h = a->bgs_stride_h,
    k.bgs_stride_n = a->bgs_stride_n;
    k.states = states, k.states_stride_b = slots_b;
    // the table of per-token max |B| for the zero-slab test: the caller's (the prologue writes it beside b_fp) or this
    // call's own pre-pass into the workspace
    k.b_rowmax = a->b_rowmax ? const_cast<float*>(a->b_rowmax) : (float*)(ws + l.rowmax);
    k.b_rowmax_ready = a->b_rowmax ? 1 : 0;
    k.batch = a->batch, k.seqlen = a->seqlen, k.nheads = a->nheads, k.headdim = a->headdim, k.ngroups = a->ngroups;
    k.dstate = a->dstate, k.chunk_size = Q;
    if ((rc = lq_chunk_state_key(&k, stream)) != LQ_OK) return rc;
  } else {
    lq_chunk_state_value_args v = {};
    v.x = a->x, v.x_stride_b = a->x_stride_b, v.x_stride_l = a->x_stride_l, v.x_stride_h = a->x_stride_h;
    v.B = a->qB, v.B_stride_b = a->qB_stride_b, v.B_stride_l = a->qB_stride_l, v.B_stride_g = a->qB_stride_g;
    v.dt = dt, v.dA_cumsum = dA;
    v.alpha_hp = a->alpha_hp, v.alpha_stride_h = a->alpha_stride_h, v.alpha_stride_p = a->alpha_stride_p;
    v.bscale_g = a->bscale_g, v.bscale_stride_g = a->bscale_stride_g;
    v.out_qscale = a->state_scale, v.oqs_stride_h = a->ss_stride_h, v.oqs_stride_p = a->ss_stride_p;
    v.states = states, v.states_stride_b = slots_b;
    v.batch = a->batch, v.seqlen = a->seqlen, v.nheads = a->nheads, v.headdim = a->headdim, v.ngroups = a->ngroups;
    v.dstate = a->dstate, v.chunk_size = Q;
    if ((rc = lq_chunk_state_value(&v, stream)) != LQ_OK) return rc;
  }

  const int64_t dim = (int64_t)a->headdim * a->dstate;
  lq_state_passing_args sp = {};
  sp.states = states;
  sp.states_stride_b = slots_b, sp.states_stride_c = (int64_t)a->nheads * dim, sp.states_stride_h = dim,
  sp.states_stride_d = 1;
  sp.dA_chunk_cumsum = dA + (Q - 1);  // last cumsum entry of every chunk: a (B,H,nc) view of (B,H,nc,Q)
  sp.dA_stride_b = (int64_t)a->nheads * nc * Q, sp.dA_stride_h = (int64_t)nc * Q, sp.dA_stride_c = Q;
  sp.out = passed;
  sp.out_stride_b = sp.states_stride_b, sp.out_stride_c = sp.states_stride_c, sp.out_stride_h = dim, sp.out_stride_d = 1;
  sp.final_states = a->final_states;
  sp.final_stride_b = (int64_t)a->nheads * dim, sp.final_stride_h = dim, sp.final_stride_d = 1;
  sp.batch = a->batch, sp.nchunks = nc, sp.nheads = a->nheads, sp.dim = (int32_t)dim;
  sp.gate_shift = a->gate_shift, sp.vec_hint = 0, sp.in_place = 1;
  if (dim > 0x7fffffffLL) return LQ_ERR_SHAPE;
  if ((rc = lq_state_passing(&sp, stream)) != LQ_OK) return rc;

  lq_bmm_chunk_args bm = {};
  bm.a = a->qC, bm.a_stride_b = a->qC_stride_b, bm.a_stride_l = a->qC_stride_l, bm.a_stride_g = a->qC_stride_g;
  if (a->keyside) {
    bm.b = a->b_fp, bm.b_stride_b = a->bfp_stride_b, bm.b_stride_l = a->bfp_stride_l, bm.b_stride_g = a->bfp_stride_g;
  } else {
    bm.b = a->qB, bm.b_stride_b = a->qB_stride_b, bm.b_stride_l = a->qB_stride_l, bm.b_stride_g = a->qB_stride_g;
  }
  bm.a_scale = a->C_scale, bm.b_scale = a->B_scale, bm.cb_scale = a->cb_scale;
  bm.out = cb;
  bm.batch = a->batch, bm.seqlen = a->seqlen, bm.ngroups = a->ngroups, bm.dstate = a->dstate, bm.chunk_size = Q;
  bm.b_is_fp = a->keyside ? 1 : 0;
  if ((rc = lq_bmm_chunk(&bm, stream)) != LQ_OK) return rc;

  lq_chunk_scan_args sc = {};
  sc.cb = cb;
  sc.x = a->x, sc.x_stride_b = a->x_stride_b, sc.x_stride_l = a->x_stride_l, sc.x_stride_h = a->x_stride_h;
  sc.dt = dt, sc.dA_cumsum = dA;
  sc.C = a->qC, sc.C_stride_b = a->qC_stride_b, sc.C_stride_l = a->qC_stride_l, sc.C_stride_g = a->qC_stride_g;
  sc.C_scale = a->C_scale;
  sc.states = passed, sc.states_stride_b = slots_b;
  sc.states_scale = a->state_scale, sc.ss_stride_h = a->ss_stride_h, sc.ss_stride_p = a->ss_stride_p;
  sc.D = a->D, sc.D_stride_h = a->D_stride_h, sc.D_has_hdim = a->D_has_hdim, sc.D_scale = a->D_scale;
  sc.cb_scale = a->cb_scale;
  sc.out = a->out;
  sc.batch = a->batch, sc.seqlen = a->seqlen, sc.nheads = a->nheads, sc.headdim = a->headdim, sc.ngroups = a->ngroups;
  sc.dstate = a->dstate, sc.chunk_size = Q;
  return lq_chunk_scan(&sc, stream);
}

// Everything the five stages would reject, checked before the first launch (the intersection of their limits), so that a
// bad call returns without having queued a kernel or written into the workspace.
int check(const lq_ssd_combined_args* a) {
  if (!a || !a->x || !a->dt || !a->qC || !a->out) return LQ_ERR_NULL;
  if (!a->dt_scale || !a->A_log || !a->A_log_scale) return LQ_ERR_NULL;
  if (!a->state_scale || !a->cb_scale || !a->C_scale || !a->B_scale) return LQ_ERR_NULL;
  if (a->D && !a->D_scale) return LQ_ERR_NULL;
  if (a->keyside ? (!a->b_fp || !a->x_scale_hp || !a->b_gate_scale) : (!a->qB || !a->alpha_hp || !a->bscale_g))
    return LQ_ERR_NULL;
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0 || a->headdim <= 0 || a->ngroups <= 0 || a->dstate <= 0 ||
      a->chunk_size <= 0)
    return LQ_ERR_SHAPE;
  const int Q = a->chunk_size;
  if (Q != 64 && Q != 128 && Q != 256 && Q != 512) return LQ_ERR_SHAPE;  // the chunk scan's sizes
  if (a->dstate % 64 != 0 || a->dstate > 256 || a->headdim % 64 != 0) return LQ_ERR_SHAPE;
  if (a->nheads % a->ngroups != 0) return LQ_ERR_SHAPE;
  if ((int64_t)a->headdim * a->dstate > 0x7fffffffLL) return LQ_ERR_SHAPE;
  if (a->gate_shift < 0 || a->gate_shift > 15) return LQ_ERR_SHAPE;
  return LQ_OK;
}

}  // namespace

// Scratch of the allocation-free entry point: one copy per GPU, inside the library's code object.  Its name is a
// host-side stand-in, not a device address: the address on each device comes from hipGetSymbolAddress, once per device,
// and only that address is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[LQ_SSD_STATIC_WORKSPACE_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
char* scratch_ptr[kMaxDevices];  // by device ordinal; nullptr until resolved

// Address of the current device's copy of `scratch`.  The look-up (which may load the code object) runs once per
// device and never while `stream` is being captured into a graph: a call under capture on a device whose address is not
// known yet is refused, so set-up work cannot land inside a capture (lq_ssd_static_init or one eager call comes first).
int static_workspace(char** out, hipStream_t stream, bool may_be_capturing) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return LQ_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    if (may_be_capturing) {
      hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
      if (hipStreamIsCapturing(stream, &st) != hipSuccess) return LQ_ERR_LAUNCH;
      if (st != hipStreamCaptureStatusNone) return LQ_ERR_STATE;
    }
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return LQ_ERR_LAUNCH;
    scratch_ptr[dev] = (char*)p;
  }
  *out = scratch_ptr[dev];
  return LQ_OK;
}

}  // namespace

extern "C" int lq_ssd_combined_workspace_bytes(const lq_ssd_combined_args* a, int64_t* bytes) {
  if (!a || !bytes) return LQ_ERR_NULL;
  Layout l;
  const int rc = plan(a, &l);
  if (rc != LQ_OK) return rc;
  *bytes = l.total;
  return LQ_OK;
}

extern "C" int lq_ssd_combined(const lq_ssd_combined_args* a, hipStream_t stream) {
  int rc = check(a);
  if (rc != LQ_OK) return rc;
  if (!a->workspace) return LQ_ERR_NULL;
  Layout l;
  if ((rc = plan(a, &l)) != LQ_OK) return rc;
  if (a->workspace_bytes < l.total || ((uintptr_t)a->workspace % kAlign) != 0) return LQ_ERR_SHAPE;
  return run(a, (char*)a->workspace, l, stream);
}

extern "C" int lq_ssd_combined_static(const lq_ssd_combined_args* a, hipStream_t stream) {
  int rc = check(a);
  if (rc != LQ_OK) return rc;
  Layout l;
  if ((rc = plan(a, &l)) != LQ_OK) return rc;
  if (l.total > LQ_SSD_STATIC_WORKSPACE_BYTES) return LQ_ERR_SHAPE;  // larger than the built-in scratch: use lq_ssd_combined
  char* ws = nullptr;
  if ((rc = static_workspace(&ws, stream, true)) != LQ_OK) return rc;
  return run(a, ws, l, stream);
}

extern "C" int lq_ssd_static_init(void) {
  char* ws = nullptr;
  return static_workspace(&ws, nullptr, false);
}
