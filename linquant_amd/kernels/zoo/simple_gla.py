"""INT8 chunk_simple_gla (linear attention with no or scalar decay) on HIP.

Call surface of linquant/kernels/zoo/simple_gla.py:175-212; matches the reference oracle's chunk recurrence
with policy kernel_static / kernel_pt / kernel_ptk, INT8 state, fp32 carry, read_post, tied q roles,
round-half-away rounding.  eta splits the write decay between the key factor (Omega^(1-eta)) and the value
factor (Omega^eta)."""

from __future__ import annotations

import torch

from . import _common as C


def chunk_simple_gla_int8(q, k, v, g, scales, *, eta=1.0, scale=None, chunk_size=64, output_final_state=False,
                          unrot=None, bits=8, out_dtype=None, prologue=None, _debug=None, _staged=False):
    """q,k [B,T,H,K], v [B,T,H,V] fp16, g [B,T,H] fp32 log decay or None. scales: 'q','k' (H,), 'kw' (H,K),
    'vw','vl','state' (H,V) fp32. Returns (o [B,T,H,V] in v.dtype or out_dtype, final fp32 state [B,H,K,V] or None).
    ``prologue`` (not in the reference's signature) = dict(signs_qk=, signs_v=, dqk=), each optional: q, k, v arrive as
    the model produced them, and the persistent rotations R_QK / R_V (``rotation_signs`` of a signed Hadamard matrix) and
    the D_QK rescaling are applied in the launch that also quantizes the operands: the result of calling
    ``rotate_qkv(q, k, v, ...)`` first and this function on its outputs, bit for bit, in one launch fewer and without the
    rotated activations ever reaching memory (K, V in {64, 128}, rotated storage).
    ``chunk_size``: up to 256 in rotated storage, up to 128 in canonical storage (padded to the next multiple of 64):
    above 64 the kernels walk every chunk as two to four 64-token pieces, with one stored state, one carry update (the INT8
    write product summed over the chunk's tokens) and one fp32 local accumulation per chunk."""
    span = C.chunk_span(chunk_size, pieces=2 if unrot is not None else 4)
    if prologue is not None and (q.shape[-1] not in (64, 128) or v.shape[-1] not in (64, 128) or unrot is not None or span != C.CHUNK):
        from .prologue import rotate_qkv  # shapes the fused launch is not built for: rotate up front

        K, V = q.shape[-1], v.shape[-1]
        assert (K in (64, 128) or not (prologue.get("signs_qk") is not None or prologue.get("dqk") is not None)) and \
            (V in (64, 128) or prologue.get("signs_v") is None), "rotations are built for row widths 64 and 128"
        do_qk, do_v = K in (64, 128), V in (64, 128)
        rq, rk, rv = rotate_qkv(q.contiguous() if do_qk else None, k.contiguous() if do_qk else None,
                                v.contiguous() if do_v else None, **prologue)
        if do_qk:
            q, k = rq, rk
        if do_v:
            v = rv
        prologue = None
    q, k, v, g, _, restore = C.pad_chunks(chunk_size, q, k, v, g, span=span)
    q, k, g, scales, _, K0 = C.pad_keys(q, k, g, scales)
    v, scales, V0 = C.pad_values(v, scales, unrot)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    dims = C.check_shapes(q, k, v, C.CHUNK)
    B, T, H, K, V = dims
    Ru = C.unrot_matrix(unrot, V)
    scale = K0 ** -0.5 if scale is None else scale
    qmax = 2 ** (bits - 1) - 1
    decay = C.DECAY_NONE if g is None else C.DECAY_SCALAR
    assert g is None or g.shape == (B, T, H)
    if prologue is None and unrot is None and _debug is None and not _staged:
        # the whole forward as one C call over one workspace (same kernels and bits as the stage-by-stage route below)
        o, ht = _one_call(q, k, v, g, scales, eta, scale, qmax, dims, span, output_final_state, out_dtype)
        return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
    gg = None
    if g is not None:
        gg, _ = C.cumsum(g, B, T, H, 0, span=span)
    NT = T // span
    h_i8 = torch.empty(B, NT, H, V, K, dtype=torch.int8, device=q.device)
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
    o = C.out_buffer(v, out_dtype)
    sc = {n: C.f32(scales[n]) for n in ("q", "k", "kw", "vw", "vl", "state")}
    if prologue is not None:
        # one launch: rotation / rescaling + every INT8 operand of the two kernels below
        codes, local, rotated = C.rotate_quant(q, k, v, gg, sc["q"], sc["k"], sc["vl"], sc["kw"], sc["vw"], eta, scale, qmax, dims,
                                               keep=_debug is not None, **prologue)
        C.state_kernel(codes, v, None, h_i8, None, ht, sc["kw"], sc["vw"], None, sc["state"], qmax, dims, C.FAMILY_LINEAR)
        C.run_output(None, None, None, h_i8, gg, None, o, sc["q"], sc["k"], sc["vl"], sc["state"], scale, qmax, dims, decay,
                     local=local, act=C.act_code(v))
        C.export_debug(_debug, h_i8, codes, g=gg, local=local, rotated=rotated)
        return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)
    codes = C.run_state(k, v, gg, None, h_i8, ht, sc["kw"], sc["vw"], sc["state"], eta, qmax, dims, C.FAMILY_LINEAR, decay, unrot=Ru,
                        span=span)
    C.run_output(q, k, v, h_i8, gg, None, o, sc["q"], sc["k"], sc["vl"], sc["state"], scale, qmax, dims, decay, unrot=Ru, span=span)
    C.export_debug(_debug, h_i8, codes, g=gg)
    return C.cut_values(restore(o), C.cut_keys(ht, K0), V0)


def _one_call(q, k, v, g, scales, eta, scale, qmax, dims, span, final_state, out_dtype):
    """lq_zoo_simple_gla: cumsum, write-operand pre-pass, state recurrence and output from one foreign call."""
    import ctypes

    from ... import _lib

    B, T, H, K, V = dims
    dev = q.device
    sc = {n: C.f32(scales[n]) for n in ("q", "k", "kw", "vw", "vl", "state")}
    svl, ss = _lib.aligned(sc["vl"]), _lib.aligned(sc["state"])
    gf = None if g is None else C.f32(g)
    key = (B, T, H, K, V, span)
    nbytes = _WS_BYTES.get(key)
    if nbytes is None:
        st = _lib.fill("lq_zoo_simple_gla_args", batch=B, seqlen=T, nheads=H, kdim=K, vdim=V, chunk_size=span)
        n = ctypes.c_int64(0)
        rc = _lib.load().lq_zoo_simple_gla_workspace_bytes(ctypes.byref(st), ctypes.byref(n))
        if rc != 0:
            raise _lib.LinQuantHipError(f"lq_zoo_simple_gla_workspace_bytes failed with code {rc}")
        nbytes = _WS_BYTES[key] = n.value
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    o = C.out_buffer(v, out_dtype)
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=dev) if final_state else None
    _lib.call("lq_zoo_simple_gla", dev, q=_lib.ptr(q), k=_lib.ptr(k), v=_lib.ptr(v), g=_lib.ptr(gf), o=_lib.ptr(o),
              o_is_f32=int(o.dtype == torch.float32), ht=_lib.ptr(ht), sq=_lib.ptr(sc["q"]), sk=_lib.ptr(sc["k"]),
              skw=_lib.ptr(sc["kw"]), svw=_lib.ptr(sc["vw"]), svl=_lib.ptr(svl), ss=_lib.ptr(ss), eta=float(eta), scale=float(scale),
              qmax=int(qmax), batch=B, seqlen=T, nheads=H, kdim=K, vdim=V, chunk_size=span, act_dtype=C.act_code(v),
              workspace=_lib.ptr(ws), workspace_bytes=nbytes)
    return o, ht


_WS_BYTES = {}
