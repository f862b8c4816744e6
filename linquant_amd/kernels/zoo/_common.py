"""Shared launch helpers of the zoo wrappers (thin ctypes calls into liblinquant_hip.so)."""

from __future__ import annotations

import torch

from linquant_amd import _lib

FAMILY_LINEAR, FAMILY_DELTA = 0, 1
DECAY_NONE, DECAY_SCALAR, DECAY_DIAGONAL = 0, 1, 2
CHUNK = 64


def pad_keys(q, k, g, scales, rot=None):
    """Key widths other than 64 and 128 run as the next of the two (the reference pads to the next power of two inside its
    kernels, linquant/kernels/zoo/gla.py:253, kda.py:176, gated_delta_rule.py:182).  q and k gain zero channels: their
    codes are zero, so every dot product, the Gram matrix and the state rows of the real channels keep their values.  A
    per-channel decay repeats its first channel there (the envelope, a maximum over channels, is unchanged; a zero decay
    would raise it to one), the per-channel key scale is one and a local rotation is extended by the identity.
    Returns (q, k, g, scales, rot, K) with K the caller's key width (final states are cut back to it)."""
    K = q.shape[-1]
    assert 1 <= K <= 128, f"K={K}: the state kernels hold the whole key axis (K <= 128)"
    Kp = 64 if K <= 64 else 128
    if K == Kp:
        return q, k, g, scales, rot, K
    pad = Kp - K
    q, k = torch.nn.functional.pad(q, (0, pad)), torch.nn.functional.pad(k, (0, pad))
    if g is not None and g.dim() == 4:
        g = torch.cat([g, g[..., :1].expand(*g.shape[:3], pad)], dim=-1)
    scales = dict(scales)
    kw = f32(scales["kw"])
    assert kw.shape[-1] == K, f"scales['kw']: (H, {K}) per key channel"
    scales["kw"] = torch.nn.functional.pad(kw, (0, pad), value=1.0)
    if rot is not None:
        assert tuple(rot.shape) == (K, K), "rot: (K, K) R_QK"
        ext = torch.eye(Kp, dtype=rot.dtype, device=rot.device)
        ext[:K, :K] = rot
        rot = ext
    return q, k, g, scales, rot, K


def chunk_span(chunk_size, pieces=2):
    """Tokens per chunk as the kernels run it: the next multiple of 64 (pad_chunks fills up), at most ``pieces`` x 64."""
    assert 1 <= chunk_size <= pieces * CHUNK, f"chunk_size={chunk_size}: the HIP kernels hold chunks of at most {pieces * CHUNK} tokens"
    return -(-chunk_size // CHUNK) * CHUNK


def pad_chunks(chunk_size, q, k, v, g=None, beta=None, span=CHUNK):
    """Chunk sizes below ``span`` (64; 128 where the kernels walk a chunk as two halves) run on the ``span``-token kernels:
    every chunk of C tokens is followed by span - C padding tokens with
    q = k = v = 0, log decay 0 and beta = 1.  Padding tokens add nothing to any product (their codes are zero), leave the
    decay accumulated over the chunk and hence the carried state unchanged, their Gram rows and columns are zero (the
    triangular inverse is the identity there), and the sub-block anchoring of the per-channel decay (16-token sub-blocks
    from the start of the chunk) is the reference's own for C a multiple of 16; the state is quantized at every chunk
    boundary as before, i.e. every C real tokens.  Returns (q, k, v, g, beta, restore) with ``restore`` cutting an
    output back to the caller's tokens.  (128-token chunks: the no / scalar decay wrapper runs them as pairs of halves.)"""
    T = q.shape[1]
    assert T % chunk_size == 0, f"T={T} must be a multiple of the chunk size {chunk_size}"
    assert 1 <= chunk_size <= span, f"chunk_size={chunk_size}: the HIP kernels hold chunks of at most {span} tokens"
    if chunk_size == span:
        return q, k, v, g, beta, lambda o: o
    NT, pad = T // chunk_size, span - chunk_size

    def widen(t, value=0.0):
        if t is None:
            return None
        x = t.reshape(t.shape[0], NT, chunk_size, *t.shape[2:])
        x = torch.nn.functional.pad(x, (0, 0) * (x.dim() - 3) + (0, pad), value=value)
        return x.reshape(t.shape[0], NT * span, *t.shape[2:])

    def restore(o):
        x = o.reshape(o.shape[0], NT, span, *o.shape[2:])[:, :, :chunk_size]
        return x.reshape(o.shape[0], T, *o.shape[2:]).contiguous()

    return widen(q), widen(k), widen(v), widen(g), widen(beta, 1.0), restore


_VALUE_SCALES = ("vw", "vl", "state", "el", "ew")


def pad_values(v, scales, unrot=None):
    """Value widths that are not a multiple of 64 run as the next one (the reference masks the surplus channels of its
    64- or 128-wide tiles, linquant/kernels/zoo/simple_gla.py:40-55): v gains zero channels, whose codes, pseudo-values,
    state columns and outputs stay zero; the per-channel value / state scales there are one.  Canonical storage keeps
    the reference's own restriction to V = 64 or 128.  Returns (v, scales, V) with V the caller's value width."""
    V = v.shape[-1]
    Vp = (V + 63) // 64 * 64
    if V == Vp or unrot is not None:
        return v, scales, V
    pad = Vp - V
    v = torch.nn.functional.pad(v, (0, pad))
    scales = dict(scales)
    for name in _VALUE_SCALES:
        if name in scales:
            s = f32(scales[name])
            assert s.shape[-1] == V, f"scales['{name}']: (H, {V}) per value channel"
            scales[name] = torch.nn.functional.pad(s, (0, pad), value=1.0)
    return v, scales, V


def cut_values(o, ht, V):
    """Outputs and final state of the caller's value channels."""
    if o.shape[-1] != V:
        o = o[..., :V].contiguous()
        ht = None if ht is None else ht[..., :V].contiguous()
    return o, ht


def cut_keys(ht, K):
    """Final state of the caller's key channels (the padded rows hold zeros)."""
    return ht if ht is None or ht.shape[2] == K else ht[:, :, :K].contiguous()


def check_shapes(q, k, v, chunk_size):
    B, T, H, K = q.shape
    V = v.shape[-1]
    assert T % chunk_size == 0, f"T={T} must be a multiple of the chunk size {chunk_size}"
    assert chunk_size == CHUNK, f"chunk_size={chunk_size}: the HIP kernels are built for 64-token chunks (pad_chunks widens smaller ones)"
    assert K in (64, 128), f"K={K}: the kernels take 64 or 128 key channels (pad_keys widens anything else)"
    assert V % 64 == 0, f"V={V}: value dim must be a multiple of 64"
    assert q.dtype in (torch.float16, torch.bfloat16) and k.dtype == q.dtype and v.dtype == q.dtype, \
        "q, k, v: one 16-bit activation dtype (fp16 or bf16)"
    assert k.shape == q.shape and v.shape[:3] == q.shape[:3]
    return B, T, H, K, V


def act_code(t):
    return _lib.LQ_DT_BF16 if t.dtype == torch.bfloat16 else _lib.LQ_DT_F16


def f32(t):
    return t if (t.dtype == torch.float32 and t.is_contiguous()) else t.float().contiguous()


def unrot_matrix(unrot, V):
    """(V,V) fp16 R_V^T of canonical storage (v arrives rotated, the state and the output come out canonical)."""
    if unrot is None:
        return None
    assert V in (64, 128), "canonical storage needs one V-tile spanning all value channels"
    assert tuple(unrot.shape) == (V, V)
    return unrot.to(torch.float16).contiguous()


def cumsum(g, B, T, H, kdim, write=None, span=CHUNK):
    """Chunk-local cumulative log decay (fp32) over chunks of ``span`` tokens and, for per-channel decay, the log envelope.  ``write`` = dict(k, v, skw,
    svw, eta, qmax) (per-channel decay, linear family): the launch also makes the state kernel's write operands while
    the chunk's decay tile is on chip (what ``write_codes`` would make, same bits) and returns them as a third value."""
    g = f32(g)
    gc = torch.empty_like(g)
    dev = g.device
    logenv = torch.empty(B, T, H, dtype=torch.float32, device=dev) if kdim else None
    if write is None:
        _lib.call("lq_zoo_cumsum", dev, g=_lib.ptr(g), gc=_lib.ptr(gc), logenv=_lib.ptr(logenv), batch=B, seqlen=T,
                  nheads=H, kdim=kdim, chunk_size=span)
        return gc, logenv
    assert span == CHUNK
    k, v = write["k"], write["v"]
    NT, V = T // CHUNK, v.shape[-1]
    c = {"kqT": torch.empty(B, NT, H, kdim, CHUNK, dtype=torch.int8, device=dev),
         "vqT": torch.empty(B, NT, H, V, CHUNK, dtype=torch.int8, device=dev), "wq": None,
         "ev": torch.empty(B, T, H, dtype=torch.float32, device=dev),
         "gam": torch.empty(B, NT, H, kdim, dtype=torch.float32, device=dev)}
    _lib.call("lq_zoo_cumsum", dev, g=_lib.ptr(g), gc=_lib.ptr(gc), logenv=_lib.ptr(logenv), batch=B, seqlen=T,
              nheads=H, kdim=kdim, chunk_size=CHUNK, k=_lib.ptr(k), v=_lib.ptr(v), kqT=_lib.ptr(c["kqT"]),
              vqT=_lib.ptr(c["vqT"]), ev=_lib.ptr(c["ev"]), gam=_lib.ptr(c["gam"]), skw=_lib.ptr(write["skw"]),
              svw=_lib.ptr(write["svw"]), eta=float(write["eta"]), qmax=int(write["qmax"]), vdim=V, act_dtype=act_code(k))
    return gc, logenv, c


def write_codes(key, value, w, g, logenv, skw, svw, sw, eta, qmax, dims, family, decay, span=CHUNK):
    """Write-operand pre-pass: INT8 codes (and decay factors) of everything that does not depend on the carry.
    ``span`` = tokens per chunk (64, or 128 for the linear family: same buffers, decays to the end of the 128-token chunk)."""
    B, T, H, K, V = dims
    dev, NT = key.device, T // CHUNK
    delta = family == FAMILY_DELTA
    c = {"kqT": torch.empty(B, NT, H, K, CHUNK, dtype=torch.int8, device=dev),
         "vqT": None if delta else torch.empty(B, NT, H, V, CHUNK, dtype=torch.int8, device=dev),
         "wq": torch.empty(B, T, H, K, dtype=torch.int8, device=dev) if delta else None,
         "ev": torch.empty(B, T, H, dtype=torch.float32, device=dev),
         "gam": torch.empty(B, NT, H, K, dtype=torch.float32, device=dev)}
    _lib.call("lq_zoo_write_codes", dev, key=_lib.ptr(key), val=None if delta else _lib.ptr(value), w=_lib.ptr(w),
              g=_lib.ptr(g), logenv=_lib.ptr(logenv), kqT=_lib.ptr(c["kqT"]), vqT=_lib.ptr(c["vqT"]), wq=_lib.ptr(c["wq"]),
              ev=_lib.ptr(c["ev"]), gam=_lib.ptr(c["gam"]), skw=_lib.ptr(skw), svw=None if delta else _lib.ptr(svw),
              sw=_lib.ptr(sw), eta=float(eta), qmax=int(qmax), batch=B, seqlen=T, nheads=H, kdim=K, vdim=V,
              chunk_size=span, decay=decay, act_dtype=act_code(key))
    return c


def state_kernel(c, value, fw, h_i8, e_out, ht, skw, svw, sw, ss, qmax, dims, family, vtile=0, unrot=None, span=CHUNK):
    """Sequential chunk recurrence over the pre-quantized operands ``c`` (see write_codes)."""
    B, T, H, K, V = dims
    delta = family == FAMILY_DELTA
    _lib.call("lq_zoo_state", h_i8.device, kqT=_lib.ptr(c["kqT"]), vqT=_lib.ptr(c["vqT"]), wq=_lib.ptr(c["wq"]),
              u=_lib.ptr(value) if delta else None, fw=_lib.ptr(fw), ev=_lib.ptr(c["ev"]) if delta else None,
              gam=_lib.ptr(c["gam"]), h_i8=_lib.ptr(h_i8), e_out=_lib.ptr(e_out), ht=_lib.ptr(ht), skw=_lib.ptr(skw),
              svw=_lib.ptr(svw), sw=_lib.ptr(sw), ss=_lib.ptr(ss), unrot=_lib.ptr(unrot), qmax=int(qmax), batch=B, seqlen=T, nheads=H,
              kdim=K, vdim=V, chunk_size=span, family=family, vtile=int(vtile),
              act_dtype=act_code(value), pack=_lib.ptr(c.get("pack")) if delta else None)


def run_state(key, value, g, logenv, h_i8, ht, skw, svw, ss, eta, qmax, dims, family, decay, w=None, fw=None, e_out=None,
              sw=None, vtile=0, unrot=None, codes=None, span=CHUNK):
    """``value`` is v (linear family) or U (delta family); ``codes``: write-operand codes that ``run_wy_prep`` already made
    (no pre-pass then)."""
    c = codes if codes is not None else write_codes(key, value, w, g, logenv, skw, svw, sw, eta, qmax, dims, family, decay, span)
    state_kernel(c, value, fw, h_i8, e_out, ht, skw, svw, sw, ss, qmax, dims, family, vtile, unrot, span)
    return c


def run_output(q, key, value, h_i8, g, A, o, sq, sk, svl, ss, scale, qmax, dims, decay, unrot=None, qg=None, local=None,
               act=None, span=CHUNK):
    """``A`` (fp16) and ``qg`` (INT8 codes of the decayed query) come from run_gla_A under per-channel decay; q and key
    are only read under no / scalar decay.  ``local`` = (qc, kc, vc): ready-made local codes from ``rotate_quant`` (q,
    key and value are then not read; ``act`` names the activation dtype code)."""
    B, T, H, K, V = dims
    svl, ss = _lib.aligned(svl), _lib.aligned(ss)
    qc, kc, vc = local if local is not None else (None, None, None)
    A, Ax = A if isinstance(A, tuple) else (A, None)
    # 128-token chunks: workspace for the second halves' products with the first halves' tokens
    cross = torch.empty(B, T, H, V, dtype=torch.float32, device=h_i8.device) if span != CHUNK else None
    _lib.call("lq_zoo_output", h_i8.device, q=_lib.ptr(q), qg=_lib.ptr(qg), k=_lib.ptr(key), v=_lib.ptr(value), h_i8=_lib.ptr(h_i8),
              g=_lib.ptr(g), A=_lib.ptr(A), o=_lib.ptr(o), o_is_f32=int(o.dtype == torch.float32), sq=_lib.ptr(sq),
              sk=_lib.ptr(sk), svl=_lib.ptr(svl), ss=_lib.ptr(ss), unrot=_lib.ptr(unrot), scale=float(scale), qmax=int(qmax),
              batch=B, seqlen=T, nheads=H, kdim=K, vdim=V, chunk_size=span, decay=decay,
              act_dtype=act if act is not None else act_code(value), qc=_lib.ptr(qc), kc=_lib.ptr(kc), vc=_lib.ptr(vc),
              cross=_lib.ptr(cross), A_cross=_lib.ptr(Ax))


def rotate_quant(q, k, v, g, sq, sk, svl, skw, svw, eta, scale, qmax, dims, signs_qk=None, signs_v=None, dqk=None,
                 keep=False):
    """The fused operand prologue of the linear family (no / scalar decay): one launch rotates / rescales q, k, v and
    emits every INT8 operand of the state and output kernels.  Returns (codes for ``state_kernel``, (qc, kc, vc) for
    ``run_output``, (q', k', v') or None): the rotated activations are stored only when ``keep``."""
    B, T, H, K, V = dims
    dev, NT = q.device, T // CHUNK
    i8 = lambda *shape: torch.empty(*shape, dtype=torch.int8, device=dev)  # noqa: E731
    c = {"kqT": i8(B, NT, H, K, CHUNK), "vqT": i8(B, NT, H, V, CHUNK), "wq": None,
         "ev": torch.empty(B, T, H, dtype=torch.float32, device=dev),
         "gam": torch.empty(B, NT, H, K, dtype=torch.float32, device=dev)}
    local = (i8(B, T, H, K), i8(B, T, H, K), i8(B, T, H, V))
    outs = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)) if keep else (None, None, None)
    dq, dk = dqk_tables(dqk, H, K)
    al = _lib.aligned
    sg = lambda t, n: None if t is None else al(f32(t).reshape(n))  # noqa: E731
    svl, skw, svw = al(svl), al(skw), al(svw)
    _lib.call("lq_zoo_rotate_quant", dev, q=_lib.ptr(q), k=_lib.ptr(k), v=_lib.ptr(v), q_out=_lib.ptr(outs[0]),
              k_out=_lib.ptr(outs[1]), v_out=_lib.ptr(outs[2]), qc=_lib.ptr(local[0]), kc=_lib.ptr(local[1]),
              vc=_lib.ptr(local[2]), kqT=_lib.ptr(c["kqT"]), vqT=_lib.ptr(c["vqT"]), ev=_lib.ptr(c["ev"]), gam=_lib.ptr(c["gam"]),
              dq=_lib.ptr(dq), dk=_lib.ptr(dk), signs_qk=_lib.ptr(sg(signs_qk, K)), signs_v=_lib.ptr(sg(signs_v, V)),
              g=_lib.ptr(g), sq=_lib.ptr(sq), sk=_lib.ptr(sk), svl=_lib.ptr(svl), skw=_lib.ptr(skw), svw=_lib.ptr(svw),
              eta=float(eta), scale=float(scale), qmax=int(qmax), batch=B, seqlen=T, nheads=H, kdim=K, vdim=V,
              chunk_size=CHUNK, act_dtype=act_code(q))
    return c, local, (outs if keep else None)


def dqk_tables(dqk, H, K):
    """(D, RN(1 / D)) as aligned fp32 (H,K) tables for the kernels that apply D_QK while they load q / k (None, None
    without one)."""
    if dqk is None:
        return None, None
    d = _lib.aligned(f32(dqk))
    assert tuple(d.shape) == (H, K), f"dqk: (H, K) = ({H}, {K}) positive factors"
    return d, _lib.aligned((1.0 / d).contiguous())


def run_gla_A(q, key, gc, sq, sk, scale, qmax, dims, rot=None, dq=None, span=CHUNK):
    """Returns (A fp16 (B,T,H,64), qg int8 (B,T,H,K)): the intra-chunk product and the codes of q*exp(g)*scale.
    ``dq`` (H,K): q is multiplied by it (and rounded to the activation dtype) as it is loaded.  ``span`` = 128: A is a pair
    (A, A_cross), the blocks inside the 64-token halves and the second halves' blocks with the first halves' tokens."""
    B, T, H, K, _ = dims
    A = torch.empty(B, T, H, CHUNK, dtype=torch.float16, device=q.device)
    Ax = torch.empty(B, T, H, CHUNK, dtype=torch.float16, device=q.device) if span != CHUNK else None
    qg = torch.empty(B, T, H, K, dtype=torch.int8, device=q.device)
    assert rot is None or tuple(rot.shape) == (K, K), "rot: (K, K) R_QK"
    _lib.call("lq_zoo_gla_A", q.device, q=_lib.ptr(q), k=_lib.ptr(key), g=_lib.ptr(gc), A=_lib.ptr(A), qg=_lib.ptr(qg), rot=_lib.ptr(rot),
              sq=_lib.ptr(sq), sk=_lib.ptr(sk), scale=float(scale), qmax=int(qmax), batch=B, seqlen=T, nheads=H, kdim=K,
              chunk_size=span, act_dtype=act_code(q), dq=_lib.ptr(dq), A_cross=_lib.ptr(Ax))
    return (A if Ax is None else (A, Ax)), qg


def run_wy_prep(k, v, beta, gc, sigma, tau, dims, decay, write=None, keep_W=True, dk=(None, None), span=CHUNK):
    """Returns (Hw, W, U, fw, codes): operands of the delta state kernel in the activation dtype and the value-side share
    of beta.  ``write`` = dict(logenv, skw, sw, eta, qmax): the launch also makes the state kernel's write-operand codes
    (what ``write_codes`` would make from the stored Hw and W, same bits) and returns them as ``codes``; W itself is
    then stored only when ``keep_W``.  ``dk`` = (D, 1 / D) from ``dqk_tables``: k is divided by D (and rounded to the
    activation dtype) as it is loaded; needs ``write``.  ``span`` = 128: the transform over 128-token chunks (a kernel of
    its own; neither ``write`` nor ``dk``)."""
    assert span == CHUNK or (write is None and dk[0] is None)
    B, T, H, K, V = dims
    dev, NT = k.device, T // CHUNK
    Hw = torch.empty_like(k)
    W = torch.empty_like(k) if (keep_W or write is None) else None
    U = torch.empty_like(v)
    fw = torch.empty(B, T, H, dtype=torch.float32, device=dev)
    extra, c = {}, None
    if write is not None:
        c = {"kqT": torch.empty(B, NT, H, K, CHUNK, dtype=torch.int8, device=dev), "vqT": None,
             "wq": torch.empty(B, T, H, K, dtype=torch.int8, device=dev),
             "ev": torch.empty(B, T, H, dtype=torch.float32, device=dev),
             "gam": torch.empty(B, NT, H, K, dtype=torch.float32, device=dev),
             # fw | ev | gam once more, contiguous per (batch, chunk, head): what the state kernel fetches them from
             "pack": torch.empty(B, NT, H, 128 + K, dtype=torch.float32, device=dev)}
        skw = _lib.aligned(write["skw"])
        extra = dict(kqT=_lib.ptr(c["kqT"]), wq=_lib.ptr(c["wq"]), ev=_lib.ptr(c["ev"]), gam=_lib.ptr(c["gam"]), pack=_lib.ptr(c["pack"]),
                     logenv=_lib.ptr(write["logenv"]), skw=_lib.ptr(skw), sw=_lib.ptr(write["sw"]), eta=float(write["eta"]),
                     qmax=int(write["qmax"]))
    _lib.call("lq_zoo_wy_prep", dev, k=_lib.ptr(k), v=_lib.ptr(v), beta=_lib.ptr(beta), g=_lib.ptr(gc),
              Hw=_lib.ptr(Hw), W=_lib.ptr(W), U=_lib.ptr(U), fw=_lib.ptr(fw), sigma=float(sigma), tau=float(tau),
              batch=B, seqlen=T, nheads=H, kdim=K, vdim=V, chunk_size=span, decay=decay, act_dtype=act_code(k),
              dk_div=_lib.ptr(dk[0]), dk_rcp=_lib.ptr(dk[1]), **extra)
    return Hw, W, U, fw, c


def out_buffer(v, out_dtype):
    dt = out_dtype or v.dtype
    assert dt in (v.dtype, torch.float32), f"output dtype {dt}: the activation dtype {v.dtype} or fp32"
    return torch.empty(v.shape, dtype=dt, device=v.device)


def export_debug(debug, h_i8, codes=None, **extra):
    """Optional hook for tests: the stored INT8 state in the reference's (B,NT,H,K,V) orientation and the INT8
    operand codes of the pre-pass in token-major orientation (kq (B,T,H,K), vq (B,T,H,V), wq (B,T,H,K))."""
    if debug is not None:
        debug["h_i8"] = h_i8.transpose(-1, -2)
        if codes is not None:
            B, NT, H = codes["kqT"].shape[:3]
            tok = lambda t: None if t is None else t.permute(0, 1, 4, 2, 3).reshape(B, NT * CHUNK, H, t.shape[3])  # noqa: E731
            debug.update(kq=tok(codes["kqT"]), vq=tok(codes["vqT"]), wq=codes["wq"])
        debug.update(extra)


_FORWARD_WS = {}


def one_call_forward(family, decay, q, k, v, g, beta, sc, dims, span, *, sigma=1.0, tau=1.0, eta, scale, qmax, final_state,
                     out_dtype, rot=None, dq=None, dq_rcp=None):
    """lq_zoo_chunk_forward: every stage of a chunk forward (GLA, DeltaNet, Gated DeltaNet, KDA; rotated storage) from one
    foreign call over one workspace.  ``sc``: fp32 scales by role ('q','k','w','kw', value write 'vw' / 'ew', value local
    'vl' / 'el', 'state').  Returns (o, final fp32 state or None)."""
    import ctypes

    B, T, H, K, V = dims
    dev = q.device
    delta = family == FAMILY_DELTA
    svw, svl = (sc["ew"], sc["el"]) if delta else (sc["vw"], sc["vl"])
    svl, ss, skw = _lib.aligned(svl), _lib.aligned(sc["state"]), _lib.aligned(sc["kw"])
    key = (family, decay, B, T, H, K, V, span)
    nbytes = _FORWARD_WS.get(key)
    if nbytes is None:
        st = _lib.fill("lq_zoo_chunk_forward_args", family=family, decay=decay, batch=B, seqlen=T, nheads=H, kdim=K, vdim=V,
                       chunk_size=span)
        n = ctypes.c_int64(0)
        rc = _lib.load().lq_zoo_chunk_forward_workspace_bytes(ctypes.byref(st), ctypes.byref(n))
        if rc != 0:
            raise _lib.LinQuantHipError(f"lq_zoo_chunk_forward_workspace_bytes failed with code {rc}")
        nbytes = _FORWARD_WS[key] = n.value
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    o = out_buffer(v, out_dtype)
    ht = torch.empty(B, H, K, V, dtype=torch.float32, device=dev) if final_state else None
    _lib.call("lq_zoo_chunk_forward", dev, q=_lib.ptr(q), k=_lib.ptr(k), v=_lib.ptr(v), g=_lib.ptr(g), beta=_lib.ptr(beta),
              o=_lib.ptr(o), o_is_f32=int(o.dtype == torch.float32), ht=_lib.ptr(ht), sq=_lib.ptr(sc["q"]), sk=_lib.ptr(sc["k"]),
              sw=_lib.ptr(sc.get("w")), skw=_lib.ptr(skw), svw=_lib.ptr(svw), svl=_lib.ptr(svl), ss=_lib.ptr(ss), rot=_lib.ptr(rot),
              dq=_lib.ptr(dq), dq_rcp=_lib.ptr(dq_rcp), sigma=float(sigma), tau=float(tau), eta=float(eta), scale=float(scale),
              qmax=int(qmax), family=family, decay=decay, batch=B, seqlen=T, nheads=H, kdim=K, vdim=V, chunk_size=span,
              act_dtype=act_code(v), workspace=_lib.ptr(ws), workspace_bytes=nbytes)
    return o, ht
