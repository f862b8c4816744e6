"""INT8 chunk_gated_delta_rule / chunk_delta_rule (delta family, no or scalar decay) on HIP.

Call surface of linquant/kernels/zoo/gated_delta_rule.py:159-203: WY prep (Gram, triangular inverse,
W = T.(beta^sigma k * exp(g)), U = T.(beta^sigma v)) -> state kernel with E = (U - W.S) * fw formed inside the
chunk loop -> the simple_gla output kernel on (q, Hw, E).  The prep is always the native fp32 HIP kernel
(``fla_prep`` is accepted for compatibility and ignored)."""

from __future__ import annotations

import torch

from . import _common as C


def chunk_delta_int8(q, k, v, g, beta, scales, *, sigma=1.0, tau=1.0, eta=1.0, scale=None, chunk_size=64,
                     output_final_state=False, unrot=None, fla_prep=True, bits=8, out_dtype=None, _debug=None, _staged=False):
    """q,k [B,T,H,K], v [B,T,H,V] fp16, g [B,T,H] fp32 log decay or None (DeltaNet), beta [B,T,H].
    scales: 'q','k','w' (H,), 'kw' (H,K), 'el','ew','state' (H,V). Returns (o, final fp32 state or None).
    ``chunk_size``: up to 64 (padded to 64 tokens), or up to 128 (padded to 128: the WY transform then
    runs over 128 x 128 Gram matrices in a kernel of its own, the state and output kernels walk a chunk as two halves)."""
    span = C.chunk_span(chunk_size)
    q, k, v, g, beta, restore = C.pad_chunks(chunk_size, q, k, v, g, beta, span=span)
    q, k, g, scales, _, K0 = C.pad_keys(q, k, g, scales)
    v, scales, V0 = C.pad_values(v, scales, unrot)
    q, k, v, beta = q.contiguous(), k.contiguous(), v.contiguous(), beta.contiguous()
    dims = C.check_shapes(q, k, v, C.CHUNK)
    B, T, H, K, V = dims
    assert beta.shape == (B, T, H)
    Ru = C.unrot_matrix(unrot, V)
    scale = K0 ** -0.5 if scale is None else scale
    qmax = 2 ** (bits - 1) - 1
    decay = C.DECAY_NONE if g is None else C.DECAY_SCALAR
    assert g is None or g.shape == (B, T, H)
    sc = {n: C.f32(scales[n]) for n in ("q", "k", "w", "kw", "el", "ew", "state")}
    if unrot is None and _debug is None and not _staged:
        # the whole forward as one C call over one workspace (same kernels and bits as the stage-by-stage route below)
        o, ht = C.one_call_forward(C.FAMILY_DELTA, decay, q, k, v, None if g is None else C.f32(g), C.f32(beta), sc, dims, span,
                                   sigma=sigma, tau=tau, eta=eta, scale=scale, qmax=qmax, final_state=output_final_state,
                                   out_dtype=out_dtype)
        return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
    gg = None
    if g is not None:
        gg, _ = C.cumsum(g, B, T, H, 0, span=span)
    # one launch makes Hw, U, fw and the state kernel's write-operand codes; W leaves the chip only for a caller that asks
    if span == C.CHUNK:
        Hw, W, U, fw, codes = C.run_wy_prep(k, v, C.f32(beta), gg, sigma, tau, dims, decay,
                                            write=dict(logenv=None, skw=sc["kw"], sw=sc["w"], eta=eta, qmax=qmax),
                                            keep_W=_debug is not None)
    else:  # the write-operand codes come from the pre-pass launch
        Hw, W, U, fw, codes = C.run_wy_prep(k, v, C.f32(beta), gg, sigma, tau, dims, decay, span=span)
    NT = T // span
    h_i8 = torch.empty(B, NT, H, V, K, dtype=torch.int8, device=q.device)
    e_out = torch.empty_like(v)
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
    o = C.out_buffer(v, out_dtype)
    codes = C.run_state(Hw, U, gg, None, h_i8, ht, sc["kw"], sc["ew"], sc["state"], eta, qmax, dims, C.FAMILY_DELTA, decay,
                        w=W, fw=fw, e_out=e_out, sw=sc["w"], unrot=Ru, codes=codes, span=span)
    C.run_output(q, Hw, e_out, h_i8, gg, None, o, sc["q"], sc["k"], sc["el"], sc["state"], scale, qmax, dims, decay, unrot=Ru,
                 span=span)
    C.export_debug(_debug, h_i8, codes, Hw=Hw, W=W, U=U, fw=fw, e_out=e_out)
    return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
