"""INT8 C.B^T per chunk with static INT8 requant (HIP). Call surface of linquant/kernels/mamba2/bmm_chunk.py:142-217."""

from __future__ import annotations

import math

import torch

from linquant_amd import _lib


def _quant_bmm_chunk_fwd(a, a_scale, b, b_scale, chunk_size, static_cb_scale, b_is_fp=False):
    """a (B,L,G,N) int8 [C], b (B,L,G,N) int8 or fp16 (b_is_fp) [B], per-group (G,) scales.
    Returns CB (B,nchunks,G,Q,Q) int8 on ``static_cb_scale``."""
    batch, seqlen, ngroups, k = a.shape
    nchunks = math.ceil(seqlen / chunk_size)
    if static_cb_scale.dtype == torch.float32 and static_cb_scale.shape == (ngroups,) and static_cb_scale.is_contiguous():
        cb_out_scale = static_cb_scale
    else:
        cb_out_scale = static_cb_scale.float().contiguous()
    assert cb_out_scale.shape == (ngroups,), f"static_cb_scale must be (ngroups,), got {cb_out_scale.shape}"
    assert a.dtype == torch.int8 and a.stride(3) == 1 and b.stride(3) == 1 and b.shape == a.shape
    assert b.dtype == (torch.float16 if b_is_fp else torch.int8)
    a_scale = a_scale if a_scale.dtype == torch.float32 and a_scale.is_contiguous() else a_scale.float().contiguous()
    b_scale = b_scale if b_scale.dtype == torch.float32 and b_scale.is_contiguous() else b_scale.float().contiguous()
    out = torch.empty((batch, nchunks, ngroups, chunk_size, chunk_size), device=a.device, dtype=torch.int8)
    _lib.call("lq_bmm_chunk", a.device,
              a=_lib.ptr(a), a_stride_b=a.stride(0), a_stride_l=a.stride(1), a_stride_g=a.stride(2),
              b=_lib.ptr(b), b_stride_b=b.stride(0), b_stride_l=b.stride(1), b_stride_g=b.stride(2),
              a_scale=_lib.ptr(a_scale), b_scale=_lib.ptr(b_scale), cb_scale=_lib.ptr(cb_out_scale),
              out=_lib.ptr(out), batch=batch, seqlen=seqlen, ngroups=ngroups, dstate=k, chunk_size=chunk_size,
              b_is_fp=int(bool(b_is_fp)))
    return out
