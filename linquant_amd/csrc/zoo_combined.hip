// One call for the whole no / scalar decay chunk forward: chunk_simple_gla_int8 (linquant/kernels/zoo/simple_gla.py:175-212)
// as one C entry.  The four stages -- cumsum (scalar decay only), write-operand pre-pass, state recurrence, output -- are
// the stand-alone entry points, launched back to back on the caller's stream over one caller-supplied workspace that holds
// what the Python wrapper would otherwise allocate per call (cumulative decay, write codes, per-token factors, stored
// states).  Same kernels, same arguments, same bits; what it saves is the host: one foreign call and one allocation per
// forward instead of four calls and nine allocations, which is what bounds small shapes (B1 T2048 H8: the kernels take
// 30 us, issuing them from Python 50).
#include "zoo_common.h"
#include "../../include/linquant_hip.h"

namespace {

constexpr int64_t kAlign = 256;
int64_t up(int64_t n) { return (n + kAlign - 1) / kAlign * kAlign; }

struct Layout {
  int64_t gc, kqT, vqT, ev, gam, h_i8, cross, total;
};

// Offsets of the intermediates for the dims in `a` (64-token chunks; chunk sizes above 64 keep the 64-token layouts)
int plan(const lq_zoo_simple_gla_args* a, Layout* l) {
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0 || a->kdim <= 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  const int cs = a->chunk_size;
  if (cs != 64 && cs != 128 && cs != 192 && cs != 256) return LQ_ERR_SHAPE;
  if (a->seqlen % cs != 0) return LQ_ERR_SHAPE;
  const int64_t B = a->batch, T = a->seqlen, H = a->nheads, K = a->kdim, V = a->vdim, NT = T / 64;
  int64_t off = 0;
  l->gc = off, off += up(B * T * H * 4);
  l->kqT = off, off += up(B * NT * H * K * 64);
  l->vqT = off, off += up(B * NT * H * V * 64);
  l->ev = off, off += up(B * T * H * 4);
  l->gam = off, off += up(B * NT * H * K * 4);
  l->h_i8 = off, off += up(B * (T / cs) * H * V * K);
  l->cross = off, off += cs == 64 ? 0 : up(B * T * H * V * 4);
  l->total = off;
  return LQ_OK;
}

}  // namespace

extern "C" int lq_zoo_simple_gla_workspace_bytes(const lq_zoo_simple_gla_args* a, int64_t* bytes) {
  if (!a || !bytes) return LQ_ERR_NULL;
  Layout l;
  const int rc = plan(a, &l);
  if (rc != LQ_OK) return rc;
  *bytes = l.total;
  return LQ_OK;
}

extern "C" int lq_zoo_simple_gla(const lq_zoo_simple_gla_args* a, hipStream_t stream) {
  if (!a || !a->q || !a->k || !a->v || !a->o || !a->workspace) return LQ_ERR_NULL;
  if (!a->sq || !a->sk || !a->skw || !a->svw || !a->svl || !a->ss) return LQ_ERR_NULL;
  Layout l;
  int rc = plan(a, &l);
  if (rc != LQ_OK) return rc;
  if (a->workspace_bytes < l.total || ((uintptr_t)a->workspace % kAlign) != 0) return LQ_ERR_SHAPE;
  char* ws = (char*)a->workspace;
  const int decay = a->g ? LQ_DECAY_SCALAR : LQ_DECAY_NONE;
  float* gc = a->g ? (float*)(ws + l.gc) : nullptr;

  // every stage validates its own arguments before it launches; the stages share the dims, so what the first accepts the
  // later ones accept as well, except for pointer alignment, which each checks on its own operands: a call refused by a
  // later stage has queued the earlier ones (they only write the workspace)
  if (a->g) {
    lq_zoo_cumsum_args c = {};
    c.g = a->g, c.gc = gc, c.batch = a->batch, c.seqlen = a->seqlen, c.nheads = a->nheads, c.kdim = 0, c.chunk_size = a->chunk_size;
    if ((rc = lq_zoo_cumsum(&c, stream)) != LQ_OK) return rc;
  }
  {
    lq_zoo_write_codes_args w = {};
    w.key = a->k, w.val = a->v, w.g = gc, w.kqT = (int8_t*)(ws + l.kqT), w.vqT = (int8_t*)(ws + l.vqT);
    w.ev = (float*)(ws + l.ev), w.gam = (float*)(ws + l.gam), w.skw = a->skw, w.svw = a->svw, w.eta = a->eta, w.qmax = a->qmax;
    w.batch = a->batch, w.seqlen = a->seqlen, w.nheads = a->nheads, w.kdim = a->kdim, w.vdim = a->vdim, w.chunk_size = a->chunk_size;
    w.decay = decay, w.act_dtype = a->act_dtype;
    if ((rc = lq_zoo_write_codes(&w, stream)) != LQ_OK) return rc;
  }
  {
    lq_zoo_state_args s = {};
    s.kqT = (const int8_t*)(ws + l.kqT), s.vqT = (const int8_t*)(ws + l.vqT), s.gam = (const float*)(ws + l.gam);
    s.h_i8 = (int8_t*)(ws + l.h_i8), s.ht = a->ht, s.skw = a->skw, s.svw = a->svw, s.ss = a->ss, s.qmax = a->qmax;
    s.batch = a->batch, s.seqlen = a->seqlen, s.nheads = a->nheads, s.kdim = a->kdim, s.vdim = a->vdim, s.chunk_size = a->chunk_size;
    s.family = LQ_FAMILY_LINEAR, s.vtile = 0, s.act_dtype = a->act_dtype;
    if ((rc = lq_zoo_state(&s, stream)) != LQ_OK) return rc;
  }
  {
    lq_zoo_output_args o = {};
    o.q = a->q, o.k = a->k, o.v = a->v, o.h_i8 = (const int8_t*)(ws + l.h_i8), o.g = gc, o.o = a->o, o.o_is_f32 = a->o_is_f32;
    o.sq = a->sq, o.sk = a->sk, o.svl = a->svl, o.ss = a->ss, o.scale = a->scale, o.qmax = a->qmax;
    o.batch = a->batch, o.seqlen = a->seqlen, o.nheads = a->nheads, o.kdim = a->kdim, o.vdim = a->vdim, o.chunk_size = a->chunk_size;
    o.decay = decay, o.act_dtype = a->act_dtype, o.cross = a->chunk_size == 64 ? nullptr : (float*)(ws + l.cross);
    if ((rc = lq_zoo_output(&o, stream)) != LQ_OK) return rc;
  }
  return LQ_OK;
}

// ---- the other cells: chunk_gla_int8 (linquant/kernels/zoo/gla.py:235-279), chunk_delta_int8
// (gated_delta_rule.py:159-203) and chunk_kda_int8 (kda.py:154-203) as one C entry each way round: the stage entry points in
// the order the Python wrappers issue them, over one workspace.  64-token chunks take the fused pre-passes (the cumsum / WY
// launch also makes the write codes), 128-token chunks the separate write-codes launch.
namespace {

struct FLayout {
  int64_t gc, logenv, kqT, vqT, wq, ev, gam, pack, A, Ax, qg, Hw, W, U, fw, e_out, h_i8, cross, total;
};

int fplan(const lq_zoo_chunk_forward_args* a, FLayout* l) {
  if (a->batch <= 0 || a->seqlen <= 0 || a->nheads <= 0 || a->kdim <= 0 || a->vdim <= 0) return LQ_ERR_SHAPE;
  const int cs = a->chunk_size;
  if ((cs != 64 && cs != 128) || a->seqlen % cs != 0) return LQ_ERR_SHAPE;
  if (a->family != LQ_FAMILY_LINEAR && a->family != LQ_FAMILY_DELTA) return LQ_ERR_SHAPE;
  if (a->decay < LQ_DECAY_NONE || a->decay > LQ_DECAY_DIAGONAL) return LQ_ERR_SHAPE;
  if (a->family == LQ_FAMILY_LINEAR && a->decay != LQ_DECAY_DIAGONAL) return LQ_ERR_SHAPE;  // lq_zoo_simple_gla serves those
  const bool delta = a->family == LQ_FAMILY_DELTA, diag = a->decay == LQ_DECAY_DIAGONAL, big = cs == 128;
  const int64_t B = a->batch, T = a->seqlen, H = a->nheads, K = a->kdim, V = a->vdim, NT = T / 64;
  int64_t off = 0;
  auto take = [&](int64_t& slot, int64_t n) { slot = off, off += up(n); };
  take(l->gc, a->decay == LQ_DECAY_NONE ? 0 : B * T * H * (diag ? K : 1) * 4);
  take(l->logenv, diag ? B * T * H * 4 : 0);
  take(l->kqT, B * NT * H * K * 64);
  take(l->vqT, delta ? 0 : B * NT * H * V * 64);
  take(l->wq, delta ? B * T * H * K : 0);
  take(l->ev, B * T * H * 4);
  take(l->gam, B * NT * H * K * 4);
  take(l->pack, delta && !big ? B * NT * H * (128 + K) * 4 : 0);
  take(l->A, diag ? B * T * H * 64 * 2 : 0);
  take(l->Ax, diag && big ? B * T * H * 64 * 2 : 0);
  take(l->qg, diag ? B * T * H * K : 0);
  take(l->Hw, delta ? B * T * H * K * 2 : 0);
  take(l->W, delta && big ? B * T * H * K * 2 : 0);
  take(l->U, delta ? B * T * H * V * 2 : 0);
  take(l->fw, delta ? B * T * H * 4 : 0);
  take(l->e_out, delta ? B * T * H * V * 2 : 0);
  take(l->h_i8, B * (T / cs) * H * V * K);
  take(l->cross, big ? B * T * H * V * 4 : 0);
  l->total = off;
  return LQ_OK;
}

}  // namespace

extern "C" int lq_zoo_chunk_forward_workspace_bytes(const lq_zoo_chunk_forward_args* a, int64_t* bytes) {
  if (!a || !bytes) return LQ_ERR_NULL;
  FLayout l;
  const int rc = fplan(a, &l);
  if (rc != LQ_OK) return rc;
  *bytes = l.total;
  return LQ_OK;
}

extern "C" int lq_zoo_chunk_forward(const lq_zoo_chunk_forward_args* a, hipStream_t stream) {
  if (!a || !a->q || !a->k || !a->v || !a->o || !a->workspace) return LQ_ERR_NULL;
  if (!a->sq || !a->skw || !a->svw || !a->svl || !a->ss) return LQ_ERR_NULL;
  FLayout l;
  int rc = fplan(a, &l);
  if (rc != LQ_OK) return rc;
  const bool delta = a->family == LQ_FAMILY_DELTA, diag = a->decay == LQ_DECAY_DIAGONAL, big = a->chunk_size == 128;
  if (a->decay != LQ_DECAY_NONE && !a->g) return LQ_ERR_NULL;
  if (delta && (!a->beta || !a->sw)) return LQ_ERR_NULL;
  if (!a->sk) return LQ_ERR_NULL;
  if ((a->dq != nullptr) != (a->dq_rcp != nullptr)) return LQ_ERR_NULL;
  if (a->dq && (!delta || !diag || big)) return LQ_ERR_SHAPE;  // D_QK at load: KDA, 64-token chunks
  if (a->rot && !diag) return LQ_ERR_SHAPE;
  if (a->workspace_bytes < l.total || ((uintptr_t)a->workspace % kAlign) != 0) return LQ_ERR_SHAPE;
  char* ws = (char*)a->workspace;
  float* gc = a->decay == LQ_DECAY_NONE ? nullptr : (float*)(ws + l.gc);
  float* logenv = diag ? (float*)(ws + l.logenv) : nullptr;
  int8_t* kqT = (int8_t*)(ws + l.kqT);
  int8_t* vqT = delta ? nullptr : (int8_t*)(ws + l.vqT);
  int8_t* wq = delta ? (int8_t*)(ws + l.wq) : nullptr;
  float* ev = (float*)(ws + l.ev);
  float* gam = (float*)(ws + l.gam);
  float* pack = delta && !big ? (float*)(ws + l.pack) : nullptr;
  void* Hw = delta ? ws + l.Hw : nullptr;
  void* W = delta && big ? ws + l.W : nullptr;
  void* U = delta ? ws + l.U : nullptr;
  float* fw = delta ? (float*)(ws + l.fw) : nullptr;
  void* e_out = delta ? ws + l.e_out : nullptr;
  int8_t* h_i8 = (int8_t*)(ws + l.h_i8);
  void* A = diag ? ws + l.A : nullptr;
  void* Ax = diag && big ? ws + l.Ax : nullptr;
  int8_t* qg = diag ? (int8_t*)(ws + l.qg) : nullptr;
  float* cross = big ? (float*)(ws + l.cross) : nullptr;

  // (every stage validates its own arguments before it launches: see lq_zoo_simple_gla)
  if (a->decay != LQ_DECAY_NONE) {
    lq_zoo_cumsum_args c = {};
    c.g = a->g, c.gc = gc, c.logenv = logenv, c.batch = a->batch, c.seqlen = a->seqlen, c.nheads = a->nheads;
    c.kdim = diag ? a->kdim : 0, c.chunk_size = a->chunk_size;
    if (!delta && !big) {  // GLA, 64-token chunks: the write operands come with the cumsum
      c.k = a->k, c.v = a->v, c.kqT = kqT, c.vqT = vqT, c.ev = ev, c.gam = gam, c.skw = a->skw, c.svw = a->svw;
      c.eta = a->eta, c.qmax = a->qmax, c.vdim = a->vdim, c.act_dtype = a->act_dtype;
    }
    if ((rc = lq_zoo_cumsum(&c, stream)) != LQ_OK) return rc;
  }
  if (delta) {
    lq_zoo_wy_prep_args w = {};
    w.k = a->k, w.v = a->v, w.beta = a->beta, w.g = gc, w.Hw = Hw, w.W = W, w.U = U, w.fw = fw, w.sigma = a->sigma, w.tau = a->tau;
    w.batch = a->batch, w.seqlen = a->seqlen, w.nheads = a->nheads, w.kdim = a->kdim, w.vdim = a->vdim, w.chunk_size = a->chunk_size;
    w.decay = a->decay, w.act_dtype = a->act_dtype;
    if (!big) {  // the write operands come with the transform
      w.kqT = kqT, w.wq = wq, w.ev = ev, w.gam = gam, w.logenv = logenv, w.skw = a->skw, w.sw = a->sw, w.eta = a->eta, w.qmax = a->qmax;
      w.dk_div = a->dq, w.dk_rcp = a->dq_rcp, w.pack = pack;
    }
    if ((rc = lq_zoo_wy_prep(&w, stream)) != LQ_OK) return rc;
  }
  if (big) {
    lq_zoo_write_codes_args w = {};
    w.key = delta ? Hw : a->k, w.val = delta ? nullptr : a->v, w.w = W, w.g = gc, w.logenv = logenv, w.kqT = kqT, w.vqT = vqT, w.wq = wq;
    w.ev = ev, w.gam = gam, w.skw = a->skw, w.svw = delta ? nullptr : a->svw, w.sw = a->sw, w.eta = a->eta, w.qmax = a->qmax;
    w.batch = a->batch, w.seqlen = a->seqlen, w.nheads = a->nheads, w.kdim = a->kdim, w.vdim = a->vdim, w.chunk_size = a->chunk_size;
    w.decay = a->decay, w.act_dtype = a->act_dtype;
    if ((rc = lq_zoo_write_codes(&w, stream)) != LQ_OK) return rc;
  }
  if (diag) {
    lq_zoo_gla_A_args g = {};
    g.q = a->q, g.k = delta ? Hw : a->k, g.g = gc, g.A = A, g.qg = qg, g.rot = a->rot, g.sq = a->sq, g.sk = a->sk, g.scale = a->scale;
    g.qmax = a->qmax, g.batch = a->batch, g.seqlen = a->seqlen, g.nheads = a->nheads, g.kdim = a->kdim, g.chunk_size = a->chunk_size;
    g.act_dtype = a->act_dtype, g.dq = a->dq, g.A_cross = Ax;
    if ((rc = lq_zoo_gla_A(&g, stream)) != LQ_OK) return rc;
  }
  {
    lq_zoo_state_args s = {};
    s.kqT = kqT, s.vqT = vqT, s.wq = wq, s.u = U, s.fw = fw, s.ev = delta ? ev : nullptr, s.gam = gam, s.h_i8 = h_i8, s.e_out = e_out;
    s.ht = a->ht, s.skw = a->skw, s.svw = a->svw, s.sw = a->sw, s.ss = a->ss, s.qmax = a->qmax;
    s.batch = a->batch, s.seqlen = a->seqlen, s.nheads = a->nheads, s.kdim = a->kdim, s.vdim = a->vdim, s.chunk_size = a->chunk_size;
    s.family = a->family, s.vtile = 0, s.act_dtype = a->act_dtype, s.pack = pack;
    if ((rc = lq_zoo_state(&s, stream)) != LQ_OK) return rc;
  }
  {
    lq_zoo_output_args o = {};
    o.q = diag ? nullptr : a->q, o.qg = qg, o.k = diag ? nullptr : (delta ? Hw : a->k), o.v = delta ? e_out : a->v, o.h_i8 = h_i8;
    o.g = diag ? nullptr : gc, o.A = A, o.o = a->o, o.o_is_f32 = a->o_is_f32, o.sq = a->sq, o.sk = a->sk, o.svl = a->svl, o.ss = a->ss;
    o.scale = a->scale, o.qmax = a->qmax;
    o.batch = a->batch, o.seqlen = a->seqlen, o.nheads = a->nheads, o.kdim = a->kdim, o.vdim = a->vdim, o.chunk_size = a->chunk_size;
    o.decay = a->decay, o.act_dtype = a->act_dtype, o.cross = cross, o.A_cross = Ax;
    if ((rc = lq_zoo_output(&o, stream)) != LQ_OK) return rc;
  }
  return LQ_OK;
}
