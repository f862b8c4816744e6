"""INT8 chunk_kda (delta rule with diagonal, per-channel decay) on HIP.

Call surface of linquant/kernels/zoo/kda.py:154-203: fp32 WY prep with per-channel gates, the GLA A kernel on
(q, Hw), a state kernel with E = (U - W.S) * fw formed in-loop and per-channel write gates under the scalar
eta envelope, and the GLA output kernel on (q, E, A).  ``fla_prep`` is accepted and ignored."""

from __future__ import annotations

import torch

from . import _common as C
from .gla import BC


def chunk_kda_int8(q, k, v, g, beta, scales, *, sigma=1.0, tau=1.0, eta=0.0, scale=None, chunk_size=64,
                   output_final_state=False, unrot=None, rot=None, fla_prep=True, bits=8, out_dtype=None, dqk=None,
                   _debug=None, _staged=False):
    """q,k [B,T,H,K], v [B,T,H,V] fp16, g [B,T,H,K] fp32 per-channel log decay, beta [B,T,H].
    scales: 'q','k','w' (H,), 'kw' (H,K), 'el','ew','state' (H,V). Returns (o, final fp32 state or None).
    ``dqk`` (H,K) fp32, not in the reference's signature: the diagonal rescaling D_QK of linquant/harness.py:68-88
    (q' = q D, k' = k / D, rounded to the activation dtype) applied inside the kernels as they load q and k, with the
    result of calling ``rotate_qkv(q, k, None, dqk=dqk)`` first, bit for bit, and without that launch.
    ``chunk_size``: a multiple of 16 up to 64, or up to 128 (as ``chunk_delta_int8``)."""
    assert g.shape == q.shape
    span = C.chunk_span(chunk_size)
    if dqk is not None and q.shape[-1] in (64, 128) and span != C.CHUNK:
        from .prologue import rotate_qkv  # (the 128-token WY kernel does not rescale at load: one launch up front)

        q, k, _ = rotate_qkv(q.contiguous(), k.contiguous(), None, dqk=dqk)
        dqk = None
    if dqk is not None and q.shape[-1] not in (64, 128):
        # widths the kernels widen with zero channels: rescale up front (same roundings: one fp32 product, one quotient)
        d = dqk.to(q.device)
        q, k = (q.float() * d.float()).to(q.dtype), (k.double() / d.double()).float().to(k.dtype)
        dqk = None
    q, k, v, g, beta, restore = C.pad_chunks(chunk_size, q, k, v, g, beta, span=span)
    q, k, g, scales, rot, K0 = C.pad_keys(q, k, g, scales, rot)
    v, scales, V0 = C.pad_values(v, scales, unrot)
    q, k, v, beta = q.contiguous(), k.contiguous(), v.contiguous(), beta.contiguous()
    dims = C.check_shapes(q, k, v, C.CHUNK)
    B, T, H, K, V = dims
    assert chunk_size % BC == 0 and beta.shape == (B, T, H)
    Ru = C.unrot_matrix(unrot, V)
    R = None if rot is None else rot.to(torch.float16).contiguous()
    scale = K0 ** -0.5 if scale is None else scale
    qmax = 2 ** (bits - 1) - 1
    sc = {n: C.f32(scales[n]) for n in ("q", "k", "w", "kw", "el", "ew", "state")}
    dq, dq_rcp = C.dqk_tables(dqk, H, K)
    if unrot is None and _debug is None and not _staged:
        # the whole forward as one C call over one workspace (same kernels and bits as the stage-by-stage route below)
        o, ht = C.one_call_forward(C.FAMILY_DELTA, C.DECAY_DIAGONAL, q, k, v, C.f32(g), C.f32(beta), sc, dims, span, sigma=sigma,
                                   tau=tau, eta=eta, scale=scale, qmax=qmax, final_state=output_final_state, out_dtype=out_dtype,
                                   rot=R, dq=dq, dq_rcp=dq_rcp)
        return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
    gc, logenv = C.cumsum(g, B, T, H, K, span=span)
    # one launch makes Hw, U, fw and the state kernel's write-operand codes; W leaves the chip only for a caller that asks
    if span == C.CHUNK:
        Hw, W, U, fw, codes = C.run_wy_prep(k, v, C.f32(beta), gc, sigma, tau, dims, C.DECAY_DIAGONAL,
                                            write=dict(logenv=logenv, skw=sc["kw"], sw=sc["w"], eta=eta, qmax=qmax),
                                            keep_W=_debug is not None, dk=(dq, dq_rcp))
    else:  # (D_QK was applied up front; the write-operand codes come from the pre-pass launch)
        Hw, W, U, fw, codes = C.run_wy_prep(k, v, C.f32(beta), gc, sigma, tau, dims, C.DECAY_DIAGONAL, span=span)
    A, qg = C.run_gla_A(q, Hw, gc, sc["q"], sc["k"], scale, qmax, dims, rot=R, dq=dq, span=span)
    NT = T // span
    h_i8 = torch.empty(B, NT, H, V, K, dtype=torch.int8, device=q.device)
    e_out = torch.empty_like(v)
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
    o = C.out_buffer(v, out_dtype)
    codes = C.run_state(Hw, U, gc, logenv, h_i8, ht, sc["kw"], sc["ew"], sc["state"], eta, qmax, dims, C.FAMILY_DELTA,
                        C.DECAY_DIAGONAL, w=W, fw=fw, e_out=e_out, sw=sc["w"], unrot=Ru, codes=codes, span=span)
    C.run_output(None, None, e_out, h_i8, None, A, o, sc["q"], None, sc["el"], sc["state"], scale, qmax, dims, C.DECAY_DIAGONAL,
                 unrot=Ru, qg=qg, span=span)
    C.export_debug(_debug, h_i8, codes, A=A, qg=qg, Hw=Hw, W=W, U=U, fw=fw, e_out=e_out)
    return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
