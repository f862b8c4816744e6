"""TEST INFRASTRUCTURE ONLY (CPU checker; never imported by the product package).

Restatement of the reference's Mamba-2 INT8 SSD pipeline (SSDi8 lineage) on the CPU, stage by stage, in the
evaluation order of the reference's Triton kernels; integer tensors are exact, fp32 steps are individually
rounded (oracle/kernel_arith.py), the fp16 output stage is evaluated in float64 from the same rounded
operands.  numpy arrays in, numpy arrays out.

Follows (reference file:line):
  chunk_cumsum        linquant/kernels/mamba2/chunk_cumsum.py:45-74
  chunk_state_value   linquant/kernels/mamba2/chunk_state.py:146-255
  chunk_state_key     linquant/kernels/mamba2/chunk_state_keyside.py:223-330
  state_passing       linquant/kernels/mamba2/state_passing.py:40-93
  bmm_chunk           linquant/kernels/mamba2/bmm_chunk.py:82-139
  chunk_scan          linquant/kernels/mamba2/chunk_scan_v2.py:120-256
  ssd_combined        linquant/kernels/mamba2/ssd_combined.py:58-131
  split_rotate_quant  linquant/kernels/mamba2/fused_split_rotate_xBC.py:73-227
  kron_hadamard       linquant/kernels/hadamard.py:46-103

Parity status: the reference holds no test, golden vector or fixture for any of these kernels and its
dependency SSDi8 (un-vendored submodule, no pinned revision) is absent, so agreement with the reference's
GPU bits is PARITY UNPINNED.  What is pinned (tests/test_oracle_mamba2.py): the integer formulas against brute-force
scalar loops; state passing against the fp32-arithmetic structural restatement the reference carries
(patches/ssdi8.patch:2515-2562) and a closed-form geometric series; the rotation against scipy's Hadamard
matrix and an exact float64 bf16 dot; the whole pipeline against the unquantized sequential SSD recurrence
h_t = exp(dt_t A) h_{t-1} + dt_t B_t x_t^T, y_t = C_t h_t + D x_t at quantization-noise tolerance.
The prefix-sum association order inside chunk_cumsum is the HIP kernel's (the reference's `tl.cumsum` order is
unspecified); it is pinned against a float64 cumsum at 1e-6.
"""

from __future__ import annotations

import math

import numpy as np

from .kernel_arith import F, bf16_round, f32, fp16_round, int_dot_exact, lq_expf, lq_logf, q_rha, q_rint


# ------------------------------------------------------------------------------------------ stage 1
def wave_cumsum(v):
    """Inclusive prefix sum over the last axis (length Q = 64*E) in the HIP kernel's association order:
    sequential inside each group of E consecutive elements, Hillis-Steele over the 64 group totals, then
    exclusive group prefix + local prefix."""
    v = f32(v)
    Q = v.shape[-1]
    assert Q % 64 == 0
    E = Q // 64
    g = v.reshape(*v.shape[:-1], 64, E)
    pre = np.empty_like(g)
    pre[..., 0] = g[..., 0]
    for i in range(1, E):
        pre[..., i] = pre[..., i - 1] + g[..., i]
    t = pre[..., E - 1].copy()
    off = 1
    while off < 64:
        nt = t.copy()
        nt[..., off:] = t[..., off:] + t[..., :-off]
        t = nt
        off *= 2
    ex = np.zeros_like(t)
    ex[..., 1:] = t[..., :-1]
    return (ex[..., None] + pre).reshape(v.shape).astype(np.float32)


def chunk_cumsum(dt_raw, dt_scale, A_log_i8, A_log_scale, chunk_size, dt_bias=None, dt_softplus=False,
                 dt_limit=(0.0, float("inf"))):
    """Returns (dA_cumsum, dt_out), both (B,H,nc,Q) fp32."""
    B, L, H = dt_raw.shape
    Q = chunk_size
    nc = math.ceil(L / Q)
    v = F(dt_scale) * f32(dt_raw.astype(np.float32))
    if dt_bias is not None:
        v = v + f32(dt_bias)[None, None, :]
    if dt_softplus:
        with np.errstate(all="ignore"):
            sp = lq_logf(F(1.0) + lq_expf(v))
        v = np.where(v > F(20.0), v, sp).astype(np.float32)
    v = np.minimum(np.maximum(v, F(dt_limit[0])), F(dt_limit[1])).astype(np.float32)
    pad = nc * Q - L
    if pad:
        v = np.concatenate([v, np.zeros((B, pad, H), np.float32)], axis=1)
    A = -lq_expf(F(A_log_scale) * A_log_i8.astype(np.float32))  # (H,)
    dt_out = np.ascontiguousarray(v.reshape(B, nc, Q, H).transpose(0, 3, 1, 2))
    dA = (dt_out * A[None, :, None, None]).astype(np.float32)
    return wave_cumsum(dA), dt_out


# ------------------------------------------------------------------------------------------ stage 2
def _gate(dt, dA):
    """exp(dA_last - dA_k) * dt_k, (B,H,nc,Q) fp32."""
    return (lq_expf(dA[..., -1:] - dA) * dt).astype(np.float32)


def _chunks(t, Q):
    """(B,L,...) -> (B,nc,Q,...) zero-padded."""
    B, L = t.shape[:2]
    nc = math.ceil(L / Q)
    pad = nc * Q - L
    if pad:
        t = np.concatenate([t, np.zeros((B, pad, *t.shape[2:]), t.dtype)], axis=1)
    return t.reshape(B, nc, Q, *t.shape[2:])


def _hp(scale, H, P):
    """Broadcast a (H,P) scale view (possibly with a broadcast P axis) to a dense (H,P) fp32 array."""
    return np.broadcast_to(f32(scale), (H, P)).astype(np.float32)


def chunk_state_value(x, B_i8, dt, dA, alpha_hp, bscale_g, out_qscale):
    """x (B,L,H,P) fp16, B_i8 (B,L,G,N) int8 -> INT8 chunk states (B,nc,H,P,N)."""
    Bsz, L, H, P = x.shape
    G, N = B_i8.shape[2:]
    Q = dt.shape[-1]
    alpha, sout = _hp(alpha_hp, H, P), _hp(out_qscale, H, P)
    inv_alpha = (F(1.0) / alpha).astype(np.float32)
    gate = _gate(dt, dA)  # (B,H,nc,Q)
    xc = _chunks(x.astype(np.float32), Q)  # (B,nc,Q,H,P)
    y = xc * inv_alpha[None, None, None]
    y = y * gate.transpose(0, 2, 3, 1)[..., None]
    xq = q_rha(y, 127)  # (B,nc,Q,H,P)
    Bc = _chunks(B_i8, Q)  # (B,nc,Q,G,N)
    Bh = np.repeat(Bc, H // G, axis=3)  # (B,nc,Q,H,N)
    acc = int_dot_exact(xq.transpose(0, 1, 3, 4, 2), Bh.transpose(0, 1, 3, 2, 4))  # (B,nc,H,P,N)
    bs = np.repeat(f32(bscale_g), H // G)  # (H,)
    req = ((alpha / sout) * bs[:, None]).astype(np.float32)  # (H,P)
    return q_rha(acc.astype(np.float32) * req[None, None, :, :, None], 127).astype(np.int8)


def chunk_state_key(x, x_scale_hp, b_fp, dt, dA, out_qscale, b_gate_scale):
    """x (B,L,H,P) fp16, b_fp (B,L,G,N) fp16, b_gate_scale broadcastable to (B,nc,H,N) -> INT8 states."""
    Bsz, L, H, P = x.shape
    G, N = b_fp.shape[2:]
    Q = dt.shape[-1]
    nc = dt.shape[2]
    xs, sout = _hp(x_scale_hp, H, P), _hp(out_qscale, H, P)
    x_inv = (F(1.0) / np.maximum(xs, F(1e-10))).astype(np.float32)
    gate = _gate(dt, dA)
    xc = _chunks(x.astype(np.float32), Q)
    xq = q_rint(xc * x_inv[None, None, None], -127, 127)  # (B,nc,Q,H,P)
    bgs = np.broadcast_to(f32(b_gate_scale), (Bsz, nc, H, N)).astype(np.float32)
    b_inv = (F(127.0) / bgs).astype(np.float32)
    bc = np.repeat(_chunks(b_fp.astype(np.float32), Q), H // G, axis=3)  # (B,nc,Q,H,N)
    gb = bc * gate.transpose(0, 2, 3, 1)[..., None]
    bq = q_rint(gb * b_inv[:, :, None], -127, 127)
    acc = int_dot_exact(xq.transpose(0, 1, 3, 4, 2), bq.transpose(0, 1, 3, 2, 4))  # (B,nc,H,P,N)
    af = acc.astype(np.float32) * (bgs / F(127.0))[:, :, :, None, :]
    af = af * (xs / sout)[None, None, :, :, None]
    return q_rint(af, -127, 127).astype(np.int8)


# ------------------------------------------------------------------------------------------ stage 3
def state_passing(states_i8, dA_chunk, gate_shift=7):
    """states (B,nc,H,dim) int8, dA_chunk (B,H,nc) -> (out (B,nc,H,dim) int8, final (B,H,dim) int8)."""
    Bsz, nc, H, dim = states_i8.shape
    S = 1 << gate_shift
    gq = q_rha(lq_expf(f32(dA_chunk)) * F(S), 127)  # (B,H,nc)
    out = np.empty_like(states_i8)
    s32 = np.zeros((Bsz, H, dim), np.int32)
    out[:, 0] = 0
    final = None
    for c in range(nc):
        s32 = ((s32 * gq[:, :, c, None] + (S >> 1)) >> gate_shift) + states_i8[:, c].astype(np.int32)
        q = np.clip(s32, -127, 127).astype(np.int8)
        if c < nc - 1:
            out[:, c + 1] = q
        else:
            final = q
    return out, final


# ------------------------------------------------------------------------------------------ stage 4
def bmm_chunk(C_i8, C_scale, b, B_scale, chunk_size, cb_scale, b_is_fp=False):
    """C (B,L,G,N) int8, b int8 or fp16 -> CB (B,nc,G,Q,Q) int8."""
    Q = chunk_size
    sC, sB, scb = f32(C_scale), f32(B_scale), f32(cb_scale)
    if b_is_fp:
        b_inv = (F(1.0) / sB).astype(np.float32)  # (G,)
        b = q_rint(b.astype(np.float32) * b_inv[None, None, :, None], -127, 127)
    Cc = _chunks(np.asarray(C_i8), Q).transpose(0, 1, 3, 2, 4)  # (B,nc,G,Q,N)
    Bc = _chunks(np.asarray(b), Q).transpose(0, 1, 3, 4, 2)  # (B,nc,G,N,Q)
    acc = int_dot_exact(Cc, Bc)
    inv = ((sC * sB) / scb).astype(np.float32)
    return q_rint(acc.astype(np.float32) * inv[None, None, :, None, None], -127, 127).astype(np.int8)


# ------------------------------------------------------------------------------------------ stage 5
def chunk_scan(cb_i8, x, dt, dA, C_i8, C_scale, states_i8, D_i8, D_scale, states_scale, cb_scale):
    """Returns the pre-rounding output (B,L,H,P) in float64 (the kernels store fp16)."""
    Bsz, L, H, P = x.shape
    G, N = C_i8.shape[2:]
    nc, Q = dt.shape[2:]
    rep = H // G
    ss = _hp(states_scale, H, P).astype(np.float64)
    Cc = _chunks(np.asarray(C_i8), Q)  # (B,nc,Q,G,N)
    Ch = np.repeat(Cc, rep, axis=3).transpose(0, 1, 3, 2, 4)  # (B,nc,H,Q,N)
    acc = int_dot_exact(Ch, np.asarray(states_i8).transpose(0, 1, 2, 4, 3)).astype(np.float64)  # (B,nc,H,Q,P)
    sCh = np.repeat(f32(C_scale), rep).astype(np.float64)
    dAc = dA.transpose(0, 2, 1, 3)  # (B,nc,H,Q)
    dtc = dt.transpose(0, 2, 1, 3)
    out = acc * sCh[None, None, :, None, None] * ss[None, None, :, None, :] * np.exp(dAc.astype(np.float64))[..., None]
    # causal path: fp16(CB * S_cb * exp(dA_m - dA_k) * dt_k) @ fp16 x, fp32 products in the reference's order
    scb_h = np.repeat(f32(cb_scale), rep)  # (H,)
    cbh = np.repeat(np.asarray(cb_i8), rep, axis=2).astype(np.float32)  # (B,nc,H,Q,Q)
    with np.errstate(all="ignore"):
        w = cbh * scb_h[None, None, :, None, None]
        w = w * np.exp((dAc[..., :, None] - dAc[..., None, :]).astype(np.float32))
        w = w * dtc[..., None, :]
    tril = np.tril(np.ones((Q, Q), bool))
    w = np.where(tril, w, F(0.0)).astype(np.float16).astype(np.float64)
    xc = _chunks(x.astype(np.float64), Q).transpose(0, 1, 3, 2, 4)  # (B,nc,H,Q,P)
    out = out + np.matmul(w, xc)
    if D_i8 is not None:
        Dv = (F(D_scale) * np.asarray(D_i8).astype(np.float32)).astype(np.float64)
        Dv = Dv[:, None] if Dv.ndim == 1 else Dv  # (H,1) or (H,P)
        out = out + xc * Dv[None, None, :, None, :]
    return out.transpose(0, 1, 3, 2, 4).reshape(Bsz, nc * Q, H, P)[:, :L]


# ------------------------------------------------------------------------------------------ prologue
def fwht(v):
    """Unnormalized Sylvester Walsh-Hadamard transform over the last axis, fp32 butterflies in stage order
    1,2,4,...  (pairs (i, i+h) -> (a+b, a-b))."""
    v = f32(v)
    n = v.shape[-1]
    lead = v.shape[:-1]
    h = 1
    while h < n:
        w = v.reshape(*lead, n // (2 * h), 2, h)
        a, b = w[..., 0, :], w[..., 1, :]
        v = np.stack([a + b, a - b], axis=-2).reshape(*lead, n).astype(np.float32)
        h *= 2
    return v


def kron_rotate(b, signs):
    """(b * signs) . (H2 (x) H_{N/2}) with bf16 operands as the reference defines it; b (...,N) fp32 holding
    fp16-representable values, signs broadcastable (...,N). Returns fp32 (before any fp16 rounding)."""
    N = b.shape[-1]
    BS = N // 2
    hb = bf16_round(F(1.0) / np.sqrt(F(BS)))
    kron = F(1.0 / math.sqrt(2.0))
    v = bf16_round(f32(b) * f32(signs))
    w0 = fwht(v[..., :BS]) * hb
    w1 = fwht(v[..., BS:]) * hb
    return np.concatenate([(w0 + w1) * kron, (w0 - w1) * kron], axis=-1).astype(np.float32)


def split_rotate_quant_xBC(xBC, r_signs, nheads, ngroups, d_state, headdim, B_inv_scale, C_inv_scale, dqk_b=None,
                           dqk_c=None):
    """xBC (B,T,d_ssm+2GN) fp16 -> (x view, q_B, q_C) with q (B,T,G,N) int8 clamped to [-128, 127]."""
    Bsz, T, _ = xBC.shape
    d_ssm, gn = nheads * headdim, ngroups * d_state
    x = xBC[..., :d_ssm].reshape(Bsz, T, nheads, headdim)
    outs = []
    for off, inv, dqk in ((d_ssm, B_inv_scale, dqk_b), (d_ssm + gn, C_inv_scale, dqk_c)):
        b = xBC[..., off:off + gn].astype(np.float32).reshape(Bsz, T, ngroups, d_state)
        if dqk is not None:
            d = fp16_round(np.asarray(dqk, np.float32).reshape(ngroups, d_state))
            b = fp16_round(b * d[None, None])
        if r_signs is not None:
            y = fp16_round(kron_rotate(b, np.asarray(r_signs, np.float32).reshape(ngroups, d_state)[None, None]))
        else:
            y = fp16_round(b)
        outs.append(q_rint(y * f32(inv)[None, None, :, None], -128, 127).astype(np.int8))
    return x, outs[0], outs[1]


def kron_hadamard(x, signs, bf16=False):
    """x (B,T,H,D) fp16, signs (H,D) -> rotated fp16 (linquant/kernels/hadamard.py:81-103: the fp32 result cast to the
    input dtype).  bf16=True: x is an fp32 array of bf16-representable values and so is the result."""
    y = kron_rotate(x.astype(np.float32), np.asarray(signs, np.float32)[None, None])
    return bf16_round(y) if bf16 else y.astype(np.float16)


# ------------------------------------------------------------------------------------------ pipeline
def ssd_combined(x, dt_raw, dt_scale, A_log_i8, A_log_scale, q_B, B_scale, q_C, C_scale, chunk_size, D_i8, D_scale,
                 dt_bias=None, dt_softplus=True, dt_limit=(0.0, float("inf")), static_state_scale=None,
                 static_cb_scale=None, alpha_hp=None, bscale_g=None, keyside=False, x_scale_hp=None, b_fp=None,
                 b_gate_scale=None):
    """Whole pipeline; returns a dict of every intermediate (dA_cumsum, dt, states, passed, final, cb, out)."""
    dA, dt = chunk_cumsum(dt_raw, dt_scale, A_log_i8, A_log_scale, chunk_size, dt_bias, dt_softplus, dt_limit)
    if keyside:
        states = chunk_state_key(x, x_scale_hp, b_fp, dt, dA, static_state_scale, b_gate_scale)
    else:
        states = chunk_state_value(x, q_B, dt, dA, alpha_hp, bscale_g, static_state_scale)
    Bsz, nc, H, P, N = states.shape
    passed, final = state_passing(states.reshape(Bsz, nc, H, P * N), dA[:, :, :, -1])
    passed = passed.reshape(Bsz, nc, H, P, N)
    cb = bmm_chunk(q_C, C_scale, b_fp if keyside else q_B, B_scale, chunk_size, static_cb_scale, b_is_fp=keyside)
    out = chunk_scan(cb, x, dt, dA, q_C, C_scale, passed, D_i8, D_scale, static_state_scale, static_cb_scale)
    return dict(dA_cumsum=dA, dt=dt, states=states, passed=passed, final=final, cb=cb, out=out)
