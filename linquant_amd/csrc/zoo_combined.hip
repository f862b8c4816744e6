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
