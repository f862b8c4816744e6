"""INT8 chunk_gla (linear attention with diagonal, per-channel decay) on HIP.

Call surface of linquant/kernels/zoo/gla.py:235-279: intra-chunk product A over 16-token sub-blocks (INT8 dots
on anchor-rescaled operands off the diagonal, fp32 reduction on the diagonal blocks), state kernel with
per-channel write gates under the scalar eta envelope, output o = q8(q*exp(g)*scale).h + A.q8(v)."""

from __future__ import annotations

import torch

from . import _common as C

BC = 16  # secondary chunk


def chunk_gla_int8(q, k, v, g, scales, *, eta=0.0, scale=None, chunk_size=64, output_final_state=False, unrot=None,
                   rot=None, bits=8, out_dtype=None, _debug=None, _staged=False):
    """q,k [B,T,H,K], v [B,T,H,V] fp16, g [B,T,H,K] fp32 per-channel log decay. scales as chunk_simple_gla_int8.
    Returns (o, final fp32 state or None).  ``chunk_size``: a multiple of 16 up to 64, or up to 128 (the
    kernels walk a chunk of more than 64 tokens as two 64-token halves, padded to 128 tokens; the sub-block anchoring over its eight sub-blocks is the reference's)."""
    assert g.shape == q.shape
    span = C.chunk_span(chunk_size)
    q, k, v, g, _, restore = C.pad_chunks(chunk_size, q, k, v, g, span=span)
    q, k, g, scales, rot, K0 = C.pad_keys(q, k, g, scales, rot)
    v, scales, V0 = C.pad_values(v, scales, unrot)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    dims = C.check_shapes(q, k, v, C.CHUNK)
    B, T, H, K, V = dims
    assert chunk_size % BC == 0
    Ru = C.unrot_matrix(unrot, V)
    R = None if rot is None else rot.to(torch.float16).contiguous()
    scale = K0 ** -0.5 if scale is None else scale
    qmax = 2 ** (bits - 1) - 1
    sc = {n: C.f32(scales[n]) for n in ("q", "k", "kw", "vw", "vl", "state")}
    if unrot is None and _debug is None and not _staged:
        # the whole forward as one C call over one workspace (same kernels and bits as the stage-by-stage route below)
        o, ht = C.one_call_forward(C.FAMILY_LINEAR, C.DECAY_DIAGONAL, q, k, v, C.f32(g), None, sc, dims, span, eta=eta, scale=scale,
                                   qmax=qmax, final_state=output_final_state, out_dtype=out_dtype, rot=R)
        return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
    # the cumsum launch also makes the state kernel's write operands (it holds the chunk's decay tile): no pre-pass
    if span == C.CHUNK:
        gc, logenv, codes = C.cumsum(g, B, T, H, K, write=dict(k=k, v=v, skw=sc["kw"], svw=sc["vw"], eta=eta, qmax=qmax))
    else:
        (gc, logenv), codes = C.cumsum(g, B, T, H, K, span=span), None
    A, qg = C.run_gla_A(q, k, gc, sc["q"], sc["k"], scale, qmax, dims, rot=R, span=span)
    NT = T // span
    h_i8 = torch.empty(B, NT, H, V, K, dtype=torch.int8, device=q.device)
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
    o = C.out_buffer(v, out_dtype)
    codes = C.run_state(k, v, gc, logenv, h_i8, ht, sc["kw"], sc["vw"], sc["state"], eta, qmax, dims, C.FAMILY_LINEAR,
                        C.DECAY_DIAGONAL, unrot=Ru, codes=codes, span=span)
    C.run_output(None, None, v, h_i8, None, A, o, sc["q"], None, sc["vl"], sc["state"], scale, qmax, dims, C.DECAY_DIAGONAL,
                 unrot=Ru, qg=qg, span=span)
    C.export_debug(_debug, h_i8, codes, A=A, qg=qg, g=gc, logenv=logenv)
    return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
