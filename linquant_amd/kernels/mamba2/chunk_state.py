"""Value-side INT8 chunk states (HIP). Call surface of linquant/kernels/mamba2/chunk_state.py:258-349."""

from __future__ import annotations

import torch

from linquant_amd import _lib


def _quant_chunk_state_fwd_xfp_static_int8(x_fp, q_B, dt, dA_cumsum, alpha_hp, bscale_g, out_qscale):
    """x_fp (B,L,H,P) fp16 (any batch/seq/head stride, unit P stride), q_B (B,L,G,N) int8, dt / dA_cumsum
    (B,H,nc,Q) fp32, alpha_hp and out_qscale (H,P) fp32 views (P stride 0 = one scalar per head), bscale_g (G,).
    Returns INT8 chunk states (B,nc,H,P,N)."""
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = q_B.shape
    batch, seqlen, nheads, headdim = x_fp.shape
    assert x_fp.dtype == torch.float16 and x_fp.stride(3) == 1, "x must be fp16 with unit headdim stride"
    assert q_B.dtype == torch.int8 and q_B.stride(3) == 1
    dt, dA_cumsum = _lib.f32(dt).contiguous(), _lib.f32(dA_cumsum).contiguous()
    alpha_hp, bscale_g, out_qscale = _lib.f32(alpha_hp), _lib.f32(bscale_g), _lib.f32(out_qscale)
    states = torch.empty((batch, nchunks, nheads, headdim, dstate), device=x_fp.device, dtype=torch.int8)
    _lib.call("lq_chunk_state_value", x_fp.device,
              x=_lib.ptr(x_fp), x_stride_b=x_fp.stride(0), x_stride_l=x_fp.stride(1), x_stride_h=x_fp.stride(2),
              B=_lib.ptr(q_B), B_stride_b=q_B.stride(0), B_stride_l=q_B.stride(1), B_stride_g=q_B.stride(2),
              dt=_lib.ptr(dt), dA_cumsum=_lib.ptr(dA_cumsum),
              alpha_hp=_lib.ptr(alpha_hp), alpha_stride_h=alpha_hp.stride(0), alpha_stride_p=alpha_hp.stride(1),
              bscale_g=_lib.ptr(bscale_g), bscale_stride_g=bscale_g.stride(0),
              out_qscale=_lib.ptr(out_qscale), oqs_stride_h=out_qscale.stride(0), oqs_stride_p=out_qscale.stride(1),
              states=_lib.ptr(states), batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim,
              ngroups=ngroups, dstate=dstate, chunk_size=chunk_size)
    return states
