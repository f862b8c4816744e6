"""TEST INFRASTRUCTURE ONLY (CPU checker; never imported by the product package).

float64 restatement of the reference's chunkwise recurrence for the six (family x decay) cells and of its
per-role fake quantizer, including the "kernel arithmetic" casts that make it an emulation of the INT8 zoo
kernels (fp32 operand * fp32 reciprocal scale, fp32 chunk-local cumsum, fp32 carry with an INT8 stored copy,
fp16-rounded local product, activation-dtype materialisation of rotated / prepared operands).

Follows (reference file:line):
  ZooQuantizer            linquant/invariances.py:7-25 (schemes, roles, policies), :36-57, :59-100 (call, round),
                          :102-135 (kernel_scales, state_scale, finalize)
  chunk_forward           linquant/reference.py:24-73   (chunk_core)
  _carry_update           linquant/reference.py:77-103  (_state_update)
  _decay                  linquant/reference.py:107-122 (_decay_terms)
  _intra_product          linquant/reference.py:125-152 (_local_prod, BC = 16 sub-blocks for diagonal decay)
  _write_split            linquant/reference.py:155-163 (_write_weights)
  _state_read/_basis/_av  linquant/reference.py:167-187 (_read, _un, _local_value_product)
  _linear_chunk           linquant/reference.py:190-199
  _delta_chunk            linquant/reference.py:202-229
  signed_hadamard         linquant/reference.py:232-239 (sign stream from torch's CPU generator)
  rotate_operands         linquant/reference.py:40-46 (entry rotations), linquant/harness.py:84-87 (D_QK)

Pinned by tests/test_oracle_zoo.py: golden vectors written by the reference itself (tests/golden/zoo_golden.npz,
generator tests/golden/make_zoo_golden.py) for every cell x policy incl. calibrated scales, rotations, canonical
storage and per-chunk INT8 state codes; brute-force token-by-token recurrences; the reference's own invariance
suite (tests/test_reference.py:74-228) and its closed-form state-pass known answer (:204-217).
"""

from __future__ import annotations

import torch

SUB = 16  # secondary chunk for diagonal decay

SCHEMES = ("none", "pt_static", "ph_static", "pc_static", "row_dyn")
ROLES = ("q_read", "q_local", "k_local", "w_read", "v_local", "e_local", "k_write", "v_write", "e_write", "state")
_PER_HEAD = ("q_read", "q_local", "k_local", "w_read")
_PER_CHANNEL = ("v_local", "e_local", "k_write", "v_write", "e_write", "state")
POLICIES = {"kernel_static": {**{r: "ph_static" for r in _PER_HEAD}, **{r: "pc_static" for r in _PER_CHANNEL}}}
POLICIES["kernel_pt"] = {r: ("pc_static" if r == "state" else "pt_static") for r in POLICIES["kernel_static"]}
POLICIES["kernel_ptk"] = {**POLICIES["kernel_static"],
                          **{r: "pt_static" for r in ("q_read", "q_local", "k_local", "k_write", "w_read")}}
CELLS = {"linear_none": ("linear", "none"), "mamba2": ("linear", "scalar"), "gla": ("linear", "diagonal"),
         "deltanet": ("delta", "none"), "gated_deltanet": ("delta", "scalar"), "kda": ("delta", "diagonal")}


class ZooQuantizer:
    """qz(role, x) with x [B,H,rows,D] float64: static absmax scales per role, fake quantization on the grid."""

    ALIAS = {"q_local": "q_read"}  # one INT8 q tile serves the state read and the local product

    def __init__(self, scheme="none", bits=8, roles=("ALL",), scheme_by_role=None, state_bits=None, round_away=False):
        assert scheme in SCHEMES
        self.scheme, self.bits, self.roles = scheme, bits, set(roles)
        self.scheme_by_role = dict(scheme_by_role or {})
        self.state_bits, self.round_away = state_bits, round_away
        self.tie_roles = self.local_fp16 = self.kernel_arith = False
        self.qmax = 2 ** (bits - 1) - 1
        self.calibrating, self.layer, self.disabled = False, 0, False
        self.absmax, self.scales = {}, {}
        self.trace = None  # optional list collecting the stored INT8 state codes of every chunk
        self.code_trace = None  # optional dict role -> list of the INT8 operand codes of every call (one per chunk)

    @classmethod
    def kernel_profile(cls, policy="kernel_static", bits=8):
        """The profile the zoo kernels implement: per-role static scales, INT8 state, half-away rounding, tied q
        roles, fp16 local product, kernel arithmetic (tests/test_kernel_gla.py:22-26)."""
        q = cls("none", bits, ["ALL"], dict(POLICIES[policy]), state_bits=8, round_away=True)
        q.tie_roles = q.local_fp16 = q.kernel_arith = True
        return q

    def _key(self, role, layer=None):
        role = self.ALIAS.get(role, role) if self.tie_roles else role
        return (self.layer if layer is None else layer, role)

    def scheme_for(self, role):
        if role == "state":
            return self.scheme_by_role.get("state", "pc_static") if self.state_bits else "none"
        if role in self.scheme_by_role:
            return self.scheme_by_role[role]
        return self.scheme if ("ALL" in self.roles or role in self.roles) else "none"

    def round(self, x):
        if self.round_away:
            return torch.where(x >= 0, torch.floor(x + 0.5), torch.ceil(x - 0.5))
        return x.round()

    def __call__(self, role, x):
        if self.disabled:
            return x
        scheme = self.scheme_for(role)
        if scheme == "none":
            return x
        qmax = 2 ** (self.state_bits - 1) - 1 if role == "state" else self.qmax
        key = self._key(role)
        if self.calibrating:
            if scheme != "row_dyn":
                a = x.abs()
                a = a.amax(dim=(0, 2)) if scheme == "pc_static" else a.amax(dim=(0, 2, 3)) if scheme == "ph_static" else a.amax()
                self.absmax[key] = torch.maximum(self.absmax[key], a) if key in self.absmax else a
            return x
        if scheme == "row_dyn":
            scale = x.abs().amax(dim=-1, keepdim=True) / qmax
        elif scheme == "pc_static":
            scale = self.scales[key][None, :, None, :]
        elif scheme == "ph_static":
            scale = self.scales[key].view(1, -1, 1, 1)
        else:
            scale = self.scales[key]
        scale = scale.clamp_min(1e-12)
        if self.kernel_arith:
            codes = self.round((x.float() * (1.0 / scale.float())).double())
        else:
            codes = self.round(x / scale)
        if self.code_trace is not None:
            self.code_trace.setdefault(role, []).append(codes.clamp(-qmax, qmax).to(torch.int8))
        return codes.clamp(-qmax, qmax) * scale

    def finalize(self):
        sq = 2 ** (self.state_bits - 1) - 1 if self.state_bits else None
        self.scales = {k: a / (sq if k[1] == "state" else self.qmax) for k, a in self.absmax.items()}
        self.calibrating = False

    def state_scale(self, layer, like):
        if self.disabled or not self.state_bits or self.calibrating:
            return None
        scheme = self.scheme_for("state")
        assert scheme in ("pt_static", "ph_static", "pc_static")
        sc = self.scales[(layer, "state")].to(like.dtype).clamp_min(1e-12)
        if self.kernel_arith:
            sc = sc.float().to(like.dtype)
        if scheme == "pc_static":
            return sc[None, :, None, :]
        if scheme == "ph_static":
            return sc.view(1, -1, 1, 1)
        return sc

    def kernel_scales(self, layer, H, K, V, device="cpu", delta=False):
        """fp32 scale tensors in the shapes the kernels take: q,k,(w) (H,), kw (H,K), vw,vl,(el,ew),state (H,V)."""
        def get(role, shape):
            key = (layer, "state") if role == "state" else self._key(role, layer)
            sc = self.scales.get(key)
            if sc is None:
                return torch.ones(shape, dtype=torch.float32, device=device)
            sc = sc.float().clamp_min(1e-6)
            sc = sc.reshape(shape) if sc.numel() > 1 else sc.expand(shape).contiguous()
            return sc.to(device)

        out = {"q": get("q_read", (H,)), "k": get("k_local", (H,)), "kw": get("k_write", (H, K)),
               "vw": get("v_write", (H, V)), "vl": get("v_local", (H, V)), "state": get("state", (H, V))}
        if delta:
            out.update(w=get("w_read", (H,)), el=get("e_local", (H, V)), ew=get("e_write", (H, V)))
        return out


def signed_hadamard(n, seed, device=None):
    """Sylvester Hadamard / sqrt(n) with a seeded +-1 sign per column."""
    Hm = torch.ones(1, 1, dtype=torch.float64)
    while Hm.shape[0] < n:
        Hm = torch.cat([torch.cat([Hm, Hm], 1), torch.cat([Hm, -Hm], 1)], 0)
    gen = torch.Generator().manual_seed(seed)
    signs = torch.randint(0, 2, (n,), generator=gen).double() * 2 - 1
    return (Hm / n ** 0.5 * signs).to(device)


def rotate_operands(q, k, v, rot_qk=None, rot_v=None, dqk=None):
    """The operand prologue in front of a kernel call: q' = mat((q D) @ R_QK), k' = mat((k / D) @ R_QK),
    v' = mat(v @ R_V) with mat = float64 -> fp32 -> activation dtype (linquant/reference.py:40-46; D_QK as
    linquant/harness.py:84-87 applies it: a float64 product for q, a float64 division for k).  Any of rot_qk, rot_v,
    dqk (H,K) may be None.  Returns tensors in the inputs' dtype."""
    def mat(t, like):
        return t.float().to(like.dtype)

    qq, kk = q.double(), k.double()
    if dqk is not None:
        d = dqk.double()
        qq, kk = qq * d[None, None], kk / d[None, None]
    if rot_qk is not None:
        qq, kk = qq @ rot_qk.double(), kk @ rot_qk.double()
    vv = v.double() if rot_v is None else v.double() @ rot_v.double()
    return mat(qq, q), mat(kk, k), mat(vv, v)


# ----------------------------------------------------------------------------------------- pieces
def _karith(qz):
    return bool(getattr(qz, "kernel_arith", False))


def _basis(x, R, qz=None):
    """x @ R; kernel arithmetic rotates the fp32 product with an fp16 dot."""
    if R is None:
        return x
    if qz is not None and _karith(qz):
        h = lambda t: t.float().to(torch.float16).to(t.dtype)  # noqa: E731
        return (h(x) @ R.to(torch.float16).to(x.dtype)).float().to(x.dtype)
    return x @ R


def _carry_update(S, carry, gam, local, qz):
    """Returns (state the next chunk reads, fp32 carry or None)."""
    if not qz.state_bits:
        return gam * S + local, None
    nxt = gam * S + local if carry is None else gam * carry + local
    if qz.calibrating:
        qz("state", nxt)
        return nxt, nxt
    sc = qz.state_scale(qz.layer, S)
    if sc is None:
        return gam * S + local, None
    qmax = 2 ** (qz.state_bits - 1) - 1
    if _karith(qz):
        nxt = nxt.float().to(nxt.dtype)
        codes = qz.round((nxt.float() * (1.0 / sc.float())).double())
    else:
        codes = qz.round(nxt / sc)
    codes = codes.clamp(-qmax, qmax)
    if qz.trace is not None:
        qz.trace.append(codes.clone())
    return codes * sc, nxt


def _decay(gc, decay, C, like):
    """(read weights pq, terminal-write weights Om, state decay gam, causal decay mask lam)."""
    tril = torch.ones(C, C, dtype=torch.bool, device=like.device).tril()
    if gc is None:
        one = like.new_ones(1, 1, 1, 1)
        return one, one, one, tril.to(like.dtype)
    if decay == "scalar":
        last = gc[..., -1:]
        lam = (gc[..., :, None] - gc[..., None, :]).masked_fill(~tril, float("-inf")).exp()
        return gc.exp()[..., None], (last - gc).exp()[..., None], last.exp()[..., None], lam
    last = gc[..., -1:, :]
    return gc.exp(), (last - gc).exp(), gc[..., -1, :, None].exp(), None


def _intra_product(Xq, Xk, gc, lam, decay, qz, role_q, role_k, local_rot, strict):
    """A_ij = sum_n Xq_in Xk_jn exp(gc_in - gc_jn) for i > j (strict) or i >= j; a None role keeps fp."""
    fq = (lambda t: t) if role_q is None else (lambda t: qz(role_q, t))
    fk = (lambda t: t) if role_k is None else (lambda t: qz(role_k, t))
    if decay != "diagonal":
        A = (fq(Xq) @ fk(Xk).transpose(-1, -2)) * lam
        return A.tril(-1) if strict else A
    C = Xq.shape[-2]
    A = Xq.new_zeros(*Xq.shape[:-1], C)
    quantized = any(r is not None and qz.scheme_for(r) != "none" for r in (role_q, role_k))
    diag = -1 if strict else 0
    for s in range(0, C, SUB):
        blk = slice(s, s + SUB)
        if s > 0:
            anchor = gc[..., s:s + 1, :]
            Qa = Xq[..., blk, :] * (gc[..., blk, :] - anchor).exp()
            Ka = Xk[..., :s, :] * (anchor - gc[..., :s, :]).exp()
            if local_rot is not None and quantized:
                Qa, Ka = _basis(Qa, local_rot, qz), _basis(Ka, local_rot, qz)
            A[..., blk, :s] = fq(Qa) @ fk(Ka).transpose(-1, -2)
        gd = gc[..., blk, :]
        n = gd.shape[-2]
        keep = torch.ones(n, n, dtype=torch.bool, device=gd.device).tril(diag)[..., None]
        w = (gd[..., :, None, :] - gd[..., None, :, :]).masked_fill(~keep, float("-inf")).exp()
        Ad = torch.einsum("...in,...jn,...ijn->...ij", fq(Xq[..., blk, :]), fk(Xk[..., blk, :]), w)
        A[..., blk, blk] = Ad.tril(diag)
    return A


def _write_split(Om, decay, eta):
    """(key factor, value factor) of the terminal write under the eta split."""
    if decay != "diagonal":
        return Om ** (1 - eta), Om ** eta
    env = Om.amax(dim=-1, keepdim=True)
    kf = Om * env ** (-eta)
    if eta > 0:
        kf = torch.where(env > 0, kf, torch.zeros_like(kf))
    return kf, env ** eta


def _state_read(Q, pq, S, decay, qz, read_post):
    if read_post and decay != "diagonal":
        return (qz("q_read", Q) @ S) * pq
    return qz("q_read", Q * pq) @ S


def _av(A, Vq, qz):
    if getattr(qz, "local_fp16", False):
        A = A.float().to(torch.float16).to(A.dtype)
    return A @ Vq


def _linear_chunk(Q, Kx, Vx, gc, bt, S, carry, o):
    qz, decay = o["qz"], o["decay"]
    pq, Om, gam, lam = _decay(gc, decay, Q.shape[-2], Q)
    Y = _state_read(Q, pq, S, decay, qz, o["read_post"])
    A = _intra_product(Q, Kx, gc, lam, decay, qz, "q_local", "k_local", o["local_rot"], strict=False)
    Y = Y + _basis(_av(A, qz("v_local", Vx), qz), o["unrot"], qz)
    wk, wv = _write_split(Om, decay, o["eta"])
    local = _basis(qz("k_write", Kx * wk).transpose(-1, -2) @ qz("v_write", Vx * wv), o["unrot"], qz)
    S, carry = _carry_update(S, carry, gam, local, qz)
    return Y, S, carry


def _delta_chunk(Q, Kx, Vx, gc, bt, S, carry, o):
    qz, decay, mat, rho, tau, unrot = o["qz"], o["decay"], o["mat"], o["rho"], o["tau"], o["unrot"]
    C = Q.shape[-2]
    pq, Om, gam, lam = _decay(gc, decay, C, Q)
    L = bt ** rho * Kx
    Hg = bt ** (1 - rho) * Kx
    Hm = mat(bt ** ((1 - rho) * tau) * Kx)
    fw = bt ** ((1 - rho) * (1 - tau))
    G = _intra_product(L, Hg, gc, lam, decay, qz, None, None, o["local_rot"], strict=True)
    eye = torch.eye(C, dtype=Q.dtype, device=Q.device)
    Tm = torch.linalg.solve_triangular(eye + G, eye.expand(G.shape).clone(), upper=False, unitriangular=True)
    W = mat(Tm @ (L * pq))
    U = mat(Tm @ (bt ** rho * Vx))
    if unrot is not None:
        F = U - _basis(qz("w_read", W) @ S, unrot.T, qz)
    else:
        F = U - qz("w_read", W) @ S
    F = F * fw
    Y = _state_read(Q, pq, S, decay, qz, o["read_post"])
    A = _intra_product(Q, Hm, gc, lam, decay, qz, "q_local", "k_local", o["local_rot"], strict=False)
    Y = Y + _basis(_av(A, qz("e_local", mat(F)), qz), unrot, qz)
    wk, wv = _write_split(Om, decay, o["eta"])
    local = _basis(qz("k_write", Hm * wk).transpose(-1, -2) @ qz("e_write", F * wv), unrot, qz)
    S, carry = _carry_update(S, carry, gam, local, qz)
    return Y, S, carry


def chunk_forward(q, k, v, g, beta, *, family, decay, scale, qz, rot_qk=None, rot_v=None, eta=0.0, rho=1.0, C=64,
                  read_post=False, storage="rotated", tau=1.0, out_dtype=None, act_dtype=None):
    """Chunkwise forward of one (family, decay) cell; q,k [B,T,H,K], v [B,T,H,V], g [B,T,H] or [B,T,H,K] log
    decay, beta [B,T,H]. Returns o [B,T,H,V]."""
    B, T, H, K = q.shape
    assert T % C == 0, f"T={T} must be a multiple of the chunk size {C}"
    f64 = torch.float64
    adt = act_dtype or q.dtype
    mat = (lambda t: t.float().to(adt).to(f64)) if _karith(qz) else (lambda t: t)
    odt = out_dtype or q.dtype
    q, k, v = q.to(f64), k.to(f64), v.to(f64)
    if rot_qk is not None and decay != "diagonal":
        q, k = mat(q @ rot_qk), mat(k @ rot_qk)
    if rot_v is not None:
        v = mat(v @ rot_v)
    q = q * scale
    nc = T // C
    chunked = lambda t: t.reshape(B, nc, C, H, -1).permute(0, 3, 1, 2, 4)  # noqa: E731
    Qc, Kc, Vc = chunked(q), chunked(k), chunked(v)
    gcs = None
    if g is not None:
        gcs = g.to(f64).reshape(B, nc, C, H, *g.shape[3:]).movedim(3, 1)
        gcs = gcs.float().cumsum(dim=3).to(f64) if _karith(qz) else gcs.cumsum(dim=3)
    bts = beta.to(f64).reshape(B, nc, C, H).permute(0, 3, 1, 2).unsqueeze(-1) if beta is not None else None
    opts = dict(qz=qz, decay=decay, eta=eta, rho=rho, tau=tau, read_post=read_post, mat=mat,
                local_rot=rot_qk if (rot_qk is not None and decay == "diagonal") else None,
                unrot=rot_v.T if (rot_v is not None and storage == "canonical") else None)
    step = _linear_chunk if family == "linear" else _delta_chunk
    S = q.new_zeros(B, H, K, Vc.shape[-1])
    carry = None
    out = torch.empty_like(Vc)
    for c in range(nc):
        out[:, :, c], S, carry = step(Qc[:, :, c], Kc[:, :, c], Vc[:, :, c], None if gcs is None else gcs[:, :, c],
                                      None if bts is None else bts[:, :, c], S, carry, opts)
    o = out.permute(0, 2, 3, 1, 4).reshape(B, T, H, -1)
    if rot_v is not None and opts["unrot"] is None:
        o = o @ rot_v.T
    return o.to(odt)
