"""Fused split + Kronecker-Hadamard rotation + INT8 quantization of the B and C lanes of xBC (HIP).

Call surface of linquant/kernels/mamba2/fused_split_rotate_xBC.py:230-329. x is returned as a view of xBC.
"""

from __future__ import annotations

import torch

from linquant_amd import _lib

_SIGN_CODES = {torch.float16: _lib.LQ_DT_F16, torch.float32: _lib.LQ_DT_F32, torch.int8: _lib.LQ_DT_I8}


def prepare_dqk(d: torch.Tensor) -> torch.Tensor:
    """Diagonal key scaling vector as the kernel wants it: fp16-rounded values in a contiguous fp32 tensor."""
    return d.reshape(-1).to(torch.float16).to(torch.float32).contiguous()


def _signs_arg(signs):
    if signs.dtype not in _SIGN_CODES:
        signs = signs.float()
    return signs.contiguous()


def fused_split_rotate_quant_xBC(xBC, r_signs, nheads, ngroups, d_state, headdim, B_inv_scale, C_inv_scale,
                                 dqk_b=None, dqk_c=None, return_b_fp=False, return_b_rowmax=False):
    """xBC (B,T,d_ssm+2*G*N) fp16; r_signs (G,N) +-1 or None (split + INT8 only); B/C_inv_scale (G,) fp32;
    dqk_b/dqk_c (G*N,) or (G,N) diagonal key scalings applied (fp16-rounded) before the rotation, or None.
    Returns (x view (B,T,H,P), q_B (B,T,G,N) int8, q_C (B,T,G,N) int8).  With ``return_b_fp`` (an extension of the
    reference signature) a fourth value follows: the rotated fp16 B that q_B is quantized from, identical to
    ``kronecker_hadamard_fwd`` of the [dqk-scaled] B lanes, so a key-side caller saves that second launch.  With
    ``return_b_rowmax`` as well a fifth: max_n |b_fp| per (batch, token, group), fp32, the table the key-side chunk state
    uses to leave out all-zero slabs (its ``b_rowmax``), which saves that stage's pre-pass over B."""
    batch, seq_len, xBC_dim = xBC.shape
    d_ssm = nheads * headdim
    g_n = ngroups * d_state
    assert xBC_dim == d_ssm + 2 * g_n, f"xBC_dim={xBC_dim} != {d_ssm + 2 * g_n}"
    assert xBC.dtype == torch.float16 and xBC.stride(2) == 1, "xBC must be fp16 with a dense last axis"
    assert d_state in (64, 128), f"d_state={d_state}: the two-half Kronecker rotation covers 64 and 128"
    x_out = xBC[..., :d_ssm].view(batch, seq_len, nheads, headdim)
    has_dqk = dqk_b is not None
    if has_dqk:
        dqk_b = dqk_b if dqk_b.dtype == torch.float32 and dqk_b.is_contiguous() else prepare_dqk(dqk_b)
        dqk_c = dqk_c if dqk_c.dtype == torch.float32 and dqk_c.is_contiguous() else prepare_dqk(dqk_c)
    signs = None if r_signs is None else _signs_arg(r_signs)
    if signs is not None:
        assert signs.numel() == g_n, f"r_signs must hold G*N={g_n} entries"
    q_B = torch.empty(batch, seq_len, ngroups, d_state, device=xBC.device, dtype=torch.int8)
    q_C = torch.empty(batch, seq_len, ngroups, d_state, device=xBC.device, dtype=torch.int8)
    b_fp = torch.empty(batch, seq_len, ngroups, d_state, device=xBC.device, dtype=torch.float16) if return_b_fp else None
    assert return_b_fp or not return_b_rowmax, "the row maxima are a by-product of b_fp"
    b_rowmax = torch.empty(batch, seq_len, ngroups, device=xBC.device, dtype=torch.float32) if return_b_rowmax else None
    _lib.call("lq_split_rotate_quant_xBC", xBC.device,
              xBC=_lib.ptr(xBC), xBC_stride_b=xBC.stride(0), xBC_stride_t=xBC.stride(1),
              qB=_lib.ptr(q_B), qC=_lib.ptr(q_C), b_fp=_lib.ptr(b_fp), signs=_lib.ptr(signs),
              signs_dtype=0 if signs is None else _SIGN_CODES[signs.dtype],
              B_inv_scale=_lib.ptr(_lib.f32(B_inv_scale)), C_inv_scale=_lib.ptr(_lib.f32(C_inv_scale)),
              dqk_b=_lib.ptr(dqk_b) if has_dqk else None, dqk_c=_lib.ptr(dqk_c) if has_dqk else None,
              batch=batch, seqlen=seq_len, d_ssm=d_ssm, ngroups=ngroups, dstate=d_state, b_rowmax=_lib.ptr(b_rowmax))
    if return_b_rowmax:
        return x_out, q_B, q_C, b_fp, b_rowmax
    if return_b_fp:
        return x_out, q_B, q_C, b_fp
    return x_out, q_B, q_C
