"""Key-side INT8 chunk states (HIP). Call surface of linquant/kernels/mamba2/chunk_state_keyside.py:333-424."""

from __future__ import annotations

import torch

from linquant_amd import _lib


def _bgs_strides(t):
    """(batch, chunk, head, dstate) strides of b_gate_scale with size-1 dims zeroed so they broadcast."""
    assert t.dim() == 4, f"b_gate_scale must be 4D (B,C,H,N), got {t.dim()}D"
    return tuple(t.stride(i) if t.size(i) > 1 else 0 for i in range(4))


def _chunk_state_keyside_fwd(x_fp, x_scale_hp, b_fp, dt, dA_cumsum, out_qscale, b_gate_scale, elide_zero_slabs=True,
                             b_rowmax=None):
    """x_fp (B,L,H,P) fp16, x_scale_hp / out_qscale (H,P) fp32, b_fp (B,L,G,N) fp16, dt / dA_cumsum (B,H,nc,Q),
    b_gate_scale 4-D broadcastable (B,nc,H,N) raw amax of |gate*B|. Returns INT8 chunk states (B,nc,H,P,N).
    ``elide_zero_slabs``: leave out 64-token slabs whose gated key codes are provably all zero (same codes, bit for bit).
    ``b_rowmax`` (B,L,G) fp32, optional: max_n |b_fp| per token row as the prologue returns it beside ``b_fp``; without it
    the call computes the table itself."""
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = b_fp.shape
    batch, seqlen, nheads, headdim = x_fp.shape
    assert x_fp.dtype == torch.float16 and x_fp.stride(3) == 1, "x must be fp16 with unit headdim stride"
    assert b_fp.dtype == torch.float16 and b_fp.stride(3) == 1, "b_fp must be fp16 with unit dstate stride"
    x_scale_hp, out_qscale, b_gate_scale = _lib.f32(x_scale_hp), _lib.f32(out_qscale), _lib.f32(b_gate_scale)
    bgs = _bgs_strides(b_gate_scale)
    dt, dA_cumsum = _lib.f32(dt).contiguous(), _lib.f32(dA_cumsum).contiguous()
    states = torch.empty((batch, nchunks, nheads, headdim, dstate), device=x_fp.device, dtype=torch.int8)
    ready = 0
    if b_rowmax is not None and elide_zero_slabs:
        assert b_rowmax.dtype == torch.float32 and b_rowmax.is_contiguous() and b_rowmax.shape == (batch, seqlen, ngroups)
        rowmax, ready = b_rowmax, 1
    else:
        rowmax = torch.empty((batch, seqlen, ngroups), device=x_fp.device, dtype=torch.float32) if elide_zero_slabs else None
    _lib.call("lq_chunk_state_key", x_fp.device, b_rowmax=_lib.ptr(rowmax), b_rowmax_ready=ready,
              x=_lib.ptr(x_fp), x_stride_b=x_fp.stride(0), x_stride_l=x_fp.stride(1), x_stride_h=x_fp.stride(2),
              B=_lib.ptr(b_fp), B_stride_b=b_fp.stride(0), B_stride_l=b_fp.stride(1), B_stride_g=b_fp.stride(2),
              dt=_lib.ptr(dt), dA_cumsum=_lib.ptr(dA_cumsum),
              x_scale_hp=_lib.ptr(x_scale_hp), xs_stride_h=x_scale_hp.stride(0), xs_stride_p=x_scale_hp.stride(1),
              out_qscale=_lib.ptr(out_qscale), oqs_stride_h=out_qscale.stride(0), oqs_stride_p=out_qscale.stride(1),
              b_gate_scale=_lib.ptr(b_gate_scale), bgs_stride_b=bgs[0], bgs_stride_c=bgs[1], bgs_stride_h=bgs[2],
              bgs_stride_n=bgs[3],
              states=_lib.ptr(states), batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim,
              ngroups=ngroups, dstate=dstate, chunk_size=chunk_size)
    return states
