"""Causal depthwise conv1d (+ SiLU) on the post-in_proj xBC slab (HIP), with the call surface of
``causal_conv1d.causal_conv1d_fn`` as linquant/quantized_mamba2.py:262-268 uses it: channel-last input
``x = xBC.transpose(1, 2)`` of shape (B, D, L) with unit stride along D, weight (D, W), optional bias (D,)."""

from __future__ import annotations

import torch

from linquant_amd import _lib


def causal_conv1d_fn(x, weight, bias=None, activation=None):
    """Returns (B, D, L) fp16, the transposed view of a fresh contiguous (B, L, D) buffer."""
    assert activation in (None, "silu", "swish")
    assert x.dim() == 3 and x.dtype == torch.float16 and x.stride(1) == 1, "channel-last fp16 input (B, D, L)"
    B, D, L = x.shape
    W = weight.shape[1]
    assert weight.shape == (D, W) and 2 <= W <= 4 and D % 8 == 0
    weight = _lib.aligned(weight.to(torch.float16).contiguous())
    bias = None if bias is None else _lib.aligned(bias.to(torch.float16).contiguous())
    out = torch.empty(B, L, D, dtype=torch.float16, device=x.device)
    _lib.call("lq_causal_conv1d", x.device, x=_lib.ptr(x), x_stride_b=x.stride(0), x_stride_l=x.stride(2),
              weight=_lib.ptr(weight), bias=_lib.ptr(bias), out=_lib.ptr(out), batch=B, seqlen=L, dim=D, width=W,
              silu=int(activation is not None))
    return out.transpose(1, 2)
