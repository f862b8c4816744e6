"""Synthetic inputs and absmax calibration of the static scales the INT8 SSD kernels take.

Plain torch reductions that run on whatever device the tensors live on (the GPU in the benchmark, the CPU in
tests).  Scale semantics follow the reference's calibration collectors:
  alpha_hp            amax |x * exp(dA_last - dA) * dt| / 127 per (H,P)   scripts/nemotron_h_calibration.py:293-343
  x_scale_hp          amax |x| / 127 per (H,P)                            scripts/nemotron_h_calibration.py:558-599
  B_scale / C_scale   amax of the rotated B / C per group / 127           scripts/nemotron_h_calibration.py:346-401
  bscale_g            max over N of amax |B_rot| / 127 per group          scripts/nemotron_h_calibration.py:404-459
  b_gate_scale        raw amax |gate * B_rot| per (H,N), shape (1,1,H,N)  scripts/nemotron_h_calibration.py:462-555
  static_state_scale  amax of the chunk-local fp states / 127 per (H,P)   scripts/nemotron_h_calibration.py:602-651
  static_cb_scale     amax |C_rot . B_rot^T| / 127 per group              scripts/nemotron_h_w4a8.py:126-169
  A_log_scale, D_scale  amax / 127 scalars                                scripts/nemotron_h_w4a8.py:474
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as Fn


@dataclass
class Mamba2Shape:
    batch: int
    seqlen: int
    nheads: int
    headdim: int
    dstate: int
    ngroups: int
    chunk: int

    @property
    def d_ssm(self):
        return self.nheads * self.headdim

    @property
    def xbc_dim(self):
        return self.d_ssm + 2 * self.ngroups * self.dstate


def hadamard(n: int, device=None, dtype=torch.float32) -> torch.Tensor:
    H = torch.ones(1, 1, dtype=dtype, device=device)
    while H.shape[0] < n:
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    return H / math.sqrt(n)


def mamba2_synthetic(shape: Mamba2Shape, seed: int, device="cpu", dt_mean: float = -2.0):
    """Seeded synthetic activations of one Mamba-2 SSD layer: xBC ~ N(0,1) fp16, raw dt ~ N(dt_mean, 0.5) fp16
    (softplus applied in-kernel), drawn on the CPU generator in this order then moved to ``device``.  The default
    dt_mean = -2 gives dt ~ 0.13; -4.5 gives the weak-decay regime dt ~ 0.011 of trained Mamba-2 layers."""
    g = torch.Generator().manual_seed(seed)
    xBC = torch.randn(shape.batch, shape.seqlen, shape.xbc_dim, generator=g).to(torch.float16)
    dt_raw = (torch.randn(shape.batch, shape.seqlen, shape.nheads, generator=g) * 0.5 + dt_mean).to(torch.float16)
    return xBC.to(device), dt_raw.to(device)


def mamba2_params(shape: Mamba2Shape, seed: int, device="cpu", a_max: float = 16.0):
    """Per-layer parameters: A = -exp(U(log 1, log a_max)) as INT8 A_log codes, D ~ N(0,1) as INT8 codes, zero
    dt_bias, +-1 rotation signs (G,N)."""
    g = torch.Generator().manual_seed(seed)
    a_log = torch.rand(shape.nheads, generator=g) * math.log(a_max)
    D = torch.randn(shape.nheads, generator=g)
    signs = (torch.randint(0, 2, (shape.ngroups, shape.dstate), generator=g) * 2 - 1).to(torch.float32)
    A_log_scale = (a_log.abs().amax() / 127.0).clamp_min(1e-8)
    D_scale = (D.abs().amax() / 127.0).clamp_min(1e-8)
    return dict(
        A_log=torch.round(a_log / A_log_scale).clamp(-127, 127).to(torch.int8).to(device),
        A_log_scale=A_log_scale.float().to(device),
        D=torch.round(D / D_scale).clamp(-127, 127).to(torch.int8).to(device),
        D_scale=D_scale.float().to(device),
        dt_bias=torch.zeros(shape.nheads, dtype=torch.float32, device=device),
        dt_scale=torch.ones((), dtype=torch.float32, device=device),
        r_signs=signs.to(device),
    )


@torch.no_grad()
def calibrate_mamba2(shape: Mamba2Shape, xBC, dt_raw, params, head_block: int = 8):
    """Static scales from one calibration batch (fp32 math on xBC's device)."""
    dev = xBC.device
    B, L, H, P, N, G, Q = shape.batch, shape.seqlen, shape.nheads, shape.headdim, shape.dstate, shape.ngroups, shape.chunk
    B = xBC.shape[0]
    nc = L // Q
    assert L % Q == 0
    d_ssm, gn = shape.d_ssm, G * N
    Hn = hadamard(N, dev)
    signs = params["r_signs"].to(dev).float()
    Brot = (xBC[..., d_ssm:d_ssm + gn].float().view(B, L, G, N) * signs) @ Hn
    Crot = (xBC[..., d_ssm + gn:].float().view(B, L, G, N) * signs) @ Hn
    B_scale = (Brot.abs().amax(dim=(0, 1, 3)) / 127.0).clamp_min(1e-8)
    C_scale = (Crot.abs().amax(dim=(0, 1, 3)) / 127.0).clamp_min(1e-8)
    dt = Fn.softplus(dt_raw.float() * params["dt_scale"] + params["dt_bias"])  # (B,L,H)
    A = -torch.exp(params["A_log_scale"] * params["A_log"].float())  # (H,)
    dA = (dt * A).view(B, nc, Q, H).cumsum(dim=2)
    gate = (torch.exp(dA[:, :, -1:, :] - dA) * dt.view(B, nc, Q, H))  # (B,nc,Q,H)
    # the device reductions cover the shapes the SSD kernels themselves take; any other shape (small debug sizes, N = 16
    # or 32, rows that are not 16-byte multiples) goes through the torch expressions below, which run on any device
    on_gpu = (xBC.is_cuda and N in (64, 128, 256) and P % 64 == 0 and (xBC.stride(1) * xBC.element_size()) % 16 == 0
              and (xBC.stride(0) * xBC.element_size()) % 16 == 0 and xBC.data_ptr() % 16 == 0 and B * H <= 65535)
    if on_gpu:  # the C.B^T observer as a device reduction: the products are never stored
        cb_amax = torch.zeros(G, device=dev)
        absmax_cb_update(cb_amax, Crot.contiguous(), Brot.contiguous(), Q)
        static_cb_scale = (cb_amax / 127.0).clamp_min(1e-8)
    else:
        cb = torch.einsum("bcqgn,bckgn->bcgqk", Crot.view(B, nc, Q, G, N), Brot.view(B, nc, Q, G, N))
        static_cb_scale = (cb.abs().amax(dim=(0, 1, 3, 4)) / 127.0).clamp_min(1e-8)
        del cb
    alpha = torch.empty(H, P, device=dev)
    x_scale = torch.empty(H, P, device=dev)
    b_gate = torch.empty(H, N, device=dev)
    state_scale = torch.empty(H, P, device=dev)
    rep = H // G
    if on_gpu:  # every observer as a device reduction straight from the fp16 view (no fp32 copy of x, no stored states)
        gate_blh = gate.reshape(B, L, H)
        xs_hp, x_hp, bg_hn, st_hp = (torch.zeros(n, device=dev) for n in (H * P, H * P, H * N, H * P))
        x_view = xBC[..., :d_ssm].view(B, L, H, P)
        Bc = Brot.contiguous()
        absmax_update(xs_hp, x_view, "pc_static", gate=gate_blh)
        absmax_update(x_hp, x_view, "pc_static")
        absmax_update(bg_hn, Bc, "pc_static", gate=gate_blh, heads_per_group=rep)
        absmax_chunk_state_update(st_hp, x_view, Bc, gate_blh, Q)
        state_scale = st_hp.view(H, P) / 127.0
        alpha, x_scale, b_gate = xs_hp.view(H, P) / 127.0, x_hp.view(H, P) / 127.0, bg_hn.view(H, N)
    else:  # the same observers as torch expressions (CPU tensors: the checker's side of the CPU tests)
        for h0 in range(0, H, head_block):
            h1 = min(H, h0 + head_block)
            xh = xBC[..., h0 * P:h1 * P].float().view(B, nc, Q, h1 - h0, P)
            gh = gate[..., h0:h1]
            xg = xh * gh[..., None]
            gidx = torch.arange(h0, h1, device=dev) // rep
            Bh = Brot.view(B, nc, Q, G, N)[:, :, :, gidx]  # (B,nc,Q,hb,N)
            alpha[h0:h1] = xg.abs().amax(dim=(0, 1, 2)) / 127.0
            x_scale[h0:h1] = xh.abs().amax(dim=(0, 1, 2)) / 127.0
            b_gate[h0:h1] = (Bh * gh[..., None]).abs().amax(dim=(0, 1, 2))
            st = torch.einsum("bcqhp,bcqhn->bchpn", xg, Bh)
            state_scale[h0:h1] = st.abs().amax(dim=(0, 1, 4)) / 127.0
    tiny = 1e-8
    return dict(
        B_scale=B_scale.float().contiguous(), C_scale=C_scale.float().contiguous(),
        B_inv_scale=(1.0 / B_scale).float().contiguous(), C_inv_scale=(1.0 / C_scale).float().contiguous(),
        bscale_g=B_scale.float().clone(), alpha_hp=alpha.clamp_min(tiny).contiguous(),
        x_scale_hp=x_scale.clamp_min(tiny).contiguous(), b_gate_scale=b_gate.clamp_min(tiny).view(1, 1, H, N).contiguous(),
        static_state_scale=state_scale.clamp_min(tiny).contiguous(), static_cb_scale=static_cb_scale.float().contiguous(),
    )


# ---------------------------------------------------------------------------------------------------------------
# Device-side absmax collectors (HIP): the calibrating half of the reference Quantizer and the amax SSD observers.
# ---------------------------------------------------------------------------------------------------------------
_ABSMAX_MODES = {"pc_static": 0, "ph_static": 1, "pt_static": 2}


def absmax_update(out: torch.Tensor, x: torch.Tensor, scheme: str, gate: torch.Tensor | None = None,
                  heads_per_group: int = 1) -> torch.Tensor:
    """``out = max(out, amax |x [* gate]|)`` on the device, in place, without an fp32 copy of ``x``.

    x: (B, T, Hx, D) view with unit stride along D (any other stride order), fp16 / bf16 / fp32; Hx = H // heads_per_group.
    gate: optional fp32 (B, T, H) view (the per-token factor of the SSD observers).
    scheme / out: "pc_static" -> (H, D), "ph_static" -> (H,), "pt_static" -> (1,), fp32; zero-filled by the caller before
    the first batch (linquant/invariances.py:77-81 keeps the same running maximum)."""
    from linquant_amd import _lib

    codes = {torch.float16: _lib.LQ_DT_F16, torch.bfloat16: _lib.LQ_DT_BF16, torch.float32: _lib.LQ_DT_F32}
    assert x.dim() == 4 and x.stride(3) == 1 and x.dtype in codes
    B, T, Hx, D = x.shape
    H = Hx * heads_per_group
    mode = _ABSMAX_MODES[scheme]
    assert out.dtype == torch.float32 and out.is_contiguous() and out.numel() == (H * D, H, 1)[mode]
    if gate is not None:
        assert gate.dtype == torch.float32 and gate.shape == (B, T, H)
    _lib.call("lq_absmax", x.device, x=_lib.ptr(x), x_dtype=codes[x.dtype], x_stride_b=x.stride(0), x_stride_t=x.stride(1),
              x_stride_h=x.stride(2), gate=_lib.ptr(gate), gate_stride_b=0 if gate is None else gate.stride(0),
              gate_stride_t=0 if gate is None else gate.stride(1), gate_stride_h=0 if gate is None else gate.stride(2),
              out=_lib.ptr(out), batch=B, rows=T, nheads=H, dim=D, heads_per_group=heads_per_group, mode=mode)
    return out


def _dt_code(t):
    from linquant_amd import _lib

    return {torch.float16: _lib.LQ_DT_F16, torch.bfloat16: _lib.LQ_DT_BF16, torch.float32: _lib.LQ_DT_F32}[t.dtype]


def absmax_chunk_state_update(out: torch.Tensor, x: torch.Tensor, B: torch.Tensor, gate: torch.Tensor, chunk_size: int) -> torch.Tensor:
    """``out[h, p] = max(out[h, p], max_{b, chunk, n} |sum_k x[b,k,h,p] gate[b,k,h] B[b,k,g,n]|)`` on the device, in place:
    the chunk-state observer of the reference's calibration script (scripts/nemotron_h_calibration.py:602-651) without
    materializing the fp32 states.  x (B,L,H,P) and B (B,L,G,N) views with unit last stride, gate (B,L,H) fp32, out (H,P)
    fp32 zero-filled before the first batch."""
    from linquant_amd import _lib

    Bn, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    assert x.stride(3) == 1 and B.stride(3) == 1 and B.shape[:2] == (Bn, L) and H % G == 0
    assert gate.dtype == torch.float32 and gate.shape == (Bn, L, H)
    assert out.dtype == torch.float32 and out.is_contiguous() and out.numel() == H * P
    _lib.call("lq_absmax_chunk_state", x.device, x=_lib.ptr(x), x_dtype=_dt_code(x), x_stride_b=x.stride(0),
              x_stride_l=x.stride(1), x_stride_h=x.stride(2), B=_lib.ptr(B), B_dtype=_dt_code(B), B_stride_b=B.stride(0),
              B_stride_l=B.stride(1), B_stride_g=B.stride(2), gate=_lib.ptr(gate), gate_stride_b=gate.stride(0),
              gate_stride_l=gate.stride(1), gate_stride_h=gate.stride(2), out=_lib.ptr(out), batch=Bn, seqlen=L, nheads=H,
              headdim=P, ngroups=G, dstate=N, chunk_size=chunk_size)
    return out


def absmax_cb_update(out: torch.Tensor, C: torch.Tensor, B: torch.Tensor, chunk_size: int) -> torch.Tensor:
    """``out[g] = max(out[g], max |C . B^T|)`` over every (m, k) pair of every chunk, on the device, in place: the C.B^T
    observer of scripts/nemotron_h_w4a8.py:126-169 without materializing the products.  C, B (B,L,G,N) views with unit last
    stride, out (G,) fp32 zero-filled before the first batch."""
    from linquant_amd import _lib

    Bn, L, G, N = C.shape
    assert B.shape == C.shape and C.stride(3) == 1 and B.stride(3) == 1
    assert out.dtype == torch.float32 and out.is_contiguous() and out.numel() == G
    _lib.call("lq_absmax_cb", C.device, C=_lib.ptr(C), C_dtype=_dt_code(C), C_stride_b=C.stride(0), C_stride_l=C.stride(1),
              C_stride_g=C.stride(2), B=_lib.ptr(B), B_dtype=_dt_code(B), B_stride_b=B.stride(0), B_stride_l=B.stride(1),
              B_stride_g=B.stride(2), out=_lib.ptr(out), batch=Bn, seqlen=L, ngroups=G, dstate=N, chunk_size=chunk_size)
    return out


class AbsmaxCollector:
    """Calibrating half of linquant.invariances.Quantizer on the device: ``collector(role, x)`` with x [B, H, rows, D]
    (the reference's operand layout; any view with unit D stride) keeps the running absolute maximum per role under the
    role's scheme ("pc_static": per (H, D); "ph_static": per H; "pt_static": one value), ``scales(qmax)`` turns them
    into static scales ``absmax / qmax`` clamped at 1e-12 like the reference."""

    def __init__(self, scheme: str = "pc_static", scheme_by_role: dict | None = None):
        self.scheme, self.scheme_by_role, self.absmax = scheme, dict(scheme_by_role or {}), {}

    def __call__(self, role: str, x: torch.Tensor) -> torch.Tensor:
        scheme = self.scheme_by_role.get(role, self.scheme)
        B, H, rows, D = x.shape
        if role not in self.absmax:
            n = (H * D, H, 1)[_ABSMAX_MODES[scheme]]
            self.absmax[role] = torch.zeros(n, dtype=torch.float32, device=x.device)
        absmax_update(self.absmax[role], x.permute(0, 2, 1, 3), scheme)
        return x

    def scales(self, qmax: int = 127) -> dict:
        out = {}
        for role, a in self.absmax.items():
            out[role] = (a / qmax).clamp_min(1e-12)
        return out


# ---------------------------------------------------------------------------------------------------------------
# Zoo cells: synthetic inputs of the benchmark configurations and the diagonal q/k rescaling D_QK.
# ---------------------------------------------------------------------------------------------------------------
ZOO_CELLS = {"linear_none": ("linear", "none"), "mamba2": ("linear", "scalar"), "gla": ("linear", "diagonal"),
             "deltanet": ("delta", "none"), "gated_deltanet": ("delta", "scalar"), "kda": ("delta", "diagonal")}


def zoo_synthetic(cell: str, B: int, T: int, H: int, K: int, V: int, seed: int):
    """Seeded fp32 CPU inputs (q, k, v, g, beta) of one zoo cell in the benchmark recipes: q, v ~ N(0,1); k ~ N(0,1),
    L2-normalized for the delta family; beta = sigmoid(N(0,1)); log decay g = logsigmoid(N(0,1)) / 16 per channel (GLA),
    logsigmoid(N(1,1)) per channel (KDA), logsigmoid(N(2,1)) per head (Gated DeltaNet), -softplus(N(-2,0.5)) * A with
    A = exp(U(0, log 16)) (the Mamba-2 cell).  Draw order: q, k, v, beta, g."""
    fam, dec = ZOO_CELLS[cell]
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *shape: torch.randn(*shape, generator=gen)  # noqa: E731
    q, k = rn(B, T, H, K), rn(B, T, H, K)
    if fam == "delta":
        k = Fn.normalize(k, dim=-1)
    v = rn(B, T, H, V)
    beta = torch.sigmoid(rn(B, T, H)) if fam == "delta" else None
    g = None
    if cell == "gla":
        g = Fn.logsigmoid(rn(B, T, H, K)) / 16
    elif cell == "kda":
        g = Fn.logsigmoid(rn(B, T, H, K) + 1.0)
    elif cell == "gated_deltanet":
        g = Fn.logsigmoid(rn(B, T, H) + 2.0)
    elif cell == "mamba2":
        g = -Fn.softplus(rn(B, T, H) * 0.5 - 2.0) * torch.exp(torch.rand(H, generator=gen) * 2.77)
    return q, k, v, (None if g is None else g.float()), beta


def dqk_from_absmax(q: torch.Tensor, k: torch.Tensor, alpha: float = 0.5) -> torch.Tensor:
    """Diagonal rescaling D_QK per (H, K) from a calibration batch: D = (max|k| / max|q|)^alpha with the maxima over
    batch and tokens, clamped at 1e-8; applied as q' = q * D, k' = k / D (linquant/harness.py:68-88)."""
    aq = q.detach().abs().amax(dim=(0, 1)).double().clamp_min(1e-8)
    ak = k.detach().abs().amax(dim=(0, 1)).double().clamp_min(1e-8)
    return ((ak / aq) ** alpha).float()
