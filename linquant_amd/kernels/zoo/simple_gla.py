"""INT8 chunk_simple_gla (linear attention with no or scalar decay) on HIP.

Call surface of linquant/kernels/zoo/simple_gla.py:175-212; matches the reference oracle's chunk recurrence
with policy kernel_static / kernel_pt / kernel_ptk, INT8 state, fp32 carry, read_post, tied q roles,
round-half-away rounding.  eta splits the write decay between the key factor (Omega^(1-eta)) and the value
factor (Omega^eta)."""

from __future__ import annotations

import torch

from . import _common as C


def chunk_simple_gla_int8(q, k, v, g, scales, *, eta=1.0, scale=None, chunk_size=64, output_final_state=False,
                          unrot=None, bits=8, out_dtype=None, _debug=None):
    """q,k [B,T,H,K], v [B,T,H,V] fp16, g [B,T,H] fp32 log decay or None. scales: 'q','k' (H,), 'kw' (H,K),
    'vw','vl','state' (H,V) fp32. Returns (o [B,T,H,V] in v.dtype or out_dtype, final fp32 state [B,H,K,V] or None)."""
    q, k, g, scales, _, K0 = C.pad_keys(q, k, g, scales)
    v, scales, V0 = C.pad_values(v, scales, unrot)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    dims = C.check_shapes(q, k, v, chunk_size)
    B, T, H, K, V = dims
    Ru = C.unrot_matrix(unrot, V)
    scale = K0 ** -0.5 if scale is None else scale
    qmax = 2 ** (bits - 1) - 1
    decay = C.DECAY_NONE if g is None else C.DECAY_SCALAR
    gg = None
    if g is not None:
        assert g.shape == (B, T, H)
        gg, _ = C.cumsum(g, B, T, H, 0)
    NT = T // chunk_size
    h_i8 = torch.empty(B, NT, H, V, K, dtype=torch.int8, device=q.device)
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
    o = C.out_buffer(v, out_dtype)
    sc = {n: C.f32(scales[n]) for n in ("q", "k", "kw", "vw", "vl", "state")}
    codes = C.run_state(k, v, gg, None, h_i8, ht, sc["kw"], sc["vw"], sc["state"], eta, qmax, dims, C.FAMILY_LINEAR, decay, unrot=Ru)
    C.run_output(q, k, v, h_i8, gg, None, o, sc["q"], sc["k"], sc["vl"], sc["state"], scale, qmax, dims, decay, unrot=Ru)
    C.export_debug(_debug, h_i8, codes, g=gg)
    return C.cut_values(o, C.cut_keys(ht, K0), V0)
