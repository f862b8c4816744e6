"""INT8 chunk scan (HIP). Call surface of linquant/kernels/mamba2/chunk_scan_v2.py:259-366."""

from __future__ import annotations

import torch

from linquant_amd import _lib
from .chunk_cumsum import _as_f32_scalar


def _quant_chunk_scan_fwd(cb_i8, x_fp, dt, dA_cumsum, q_C, C_scale, states, q_D, D_scale, state_dequant_scale, cb_scale,
                          heads_per_workgroup=0):
    """cb_i8 (B,nc,G,Q,Q) int8, x_fp (B,L,H,P) fp16 view, dt / dA_cumsum (B,H,nc,Q), q_C (B,L,G,N) int8,
    states (B,nc,H,P,N) int8 (state entering each chunk), q_D (H,) or (H,P) int8 or None, D_scale scalar,
    state_dequant_scale (H,P) fp32 view (P stride 0 allowed), cb_scale (G,). Returns fp16 (B,L,H,P).
    ``heads_per_workgroup`` (not in the reference) is a scheduling knob, 0 = automatic; the result does not depend on it."""
    _, _, nchunks, chunk_size = dt.shape
    _, _, ngroups, dstate = q_C.shape
    batch, seqlen, nheads, headdim = x_fp.shape
    dev = x_fp.device
    assert x_fp.dtype == torch.float16 and x_fp.stride(3) == 1, "x must be fp16 with unit headdim stride"
    assert q_C.dtype == torch.int8 and q_C.stride(3) == 1
    cb_i8, states = cb_i8.contiguous(), states.contiguous()
    dt, dA_cumsum = _lib.f32(dt).contiguous(), _lib.f32(dA_cumsum).contiguous()
    C_scale, cb_scale, state_dequant_scale = _lib.f32(C_scale), _lib.f32(cb_scale), _lib.f32(state_dequant_scale)
    out = torch.empty(batch, seqlen, nheads, headdim, device=dev, dtype=torch.float16)
    d_scale = None if q_D is None else _as_f32_scalar(D_scale, dev)
    if q_D is not None:
        assert q_D.dtype == torch.int8 and q_D.stride(-1) == 1
    _lib.call("lq_chunk_scan", dev,
              cb=_lib.ptr(cb_i8), x=_lib.ptr(x_fp), x_stride_b=x_fp.stride(0), x_stride_l=x_fp.stride(1),
              x_stride_h=x_fp.stride(2), dt=_lib.ptr(dt), dA_cumsum=_lib.ptr(dA_cumsum),
              C=_lib.ptr(q_C), C_stride_b=q_C.stride(0), C_stride_l=q_C.stride(1), C_stride_g=q_C.stride(2),
              C_scale=_lib.ptr(C_scale), states=_lib.ptr(states),
              states_scale=_lib.ptr(state_dequant_scale), ss_stride_h=state_dequant_scale.stride(0),
              ss_stride_p=state_dequant_scale.stride(1),
              D=_lib.ptr(q_D), D_stride_h=0 if q_D is None else q_D.stride(0),
              D_has_hdim=int(q_D is not None and q_D.dim() == 2), D_scale=_lib.ptr(d_scale),
              cb_scale=_lib.ptr(cb_scale), out=_lib.ptr(out),
              batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim, ngroups=ngroups, dstate=dstate,
              chunk_size=chunk_size, heads_hint=int(heads_per_workgroup))
    return out
