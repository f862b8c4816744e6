"""Fused FP16 -> INT8 activation quantizer of the W4A8 linears (HIP), same call as linquant/w4a8_linear.py:69-98.
Only the quantizer lives here: the Marlin W4A8 GEMM itself is outside this package."""

from __future__ import annotations

import torch

from linquant_amd import _lib

_SCALE_CODES = {torch.float16: _lib.LQ_DT_F16, torch.float32: _lib.LQ_DT_F32}


def _fused_fp16_to_int8(x_2d: torch.Tensor, scale: torch.Tensor, clamp_min: float = -127.0,
                        reciprocal: bool = True) -> torch.Tensor:
    """x_2d [M, N] fp16 (unit column stride), scale a 0-dim device tensor (read on device, no host sync).
    ``reciprocal`` multiplies by 1/scale; the divide form reproduces ``x.float() / scale`` bit for bit.
    Returns int8 [M, N]."""
    assert x_2d.dim() == 2 and x_2d.dtype == torch.float16 and x_2d.stride(1) == 1
    assert scale.numel() == 1 and scale.dtype in _SCALE_CODES and scale.device == x_2d.device
    M, N = x_2d.shape
    out = torch.empty(M, N, device=x_2d.device, dtype=torch.int8)
    _lib.call("lq_fp16_to_int8", x_2d.device, x=_lib.ptr(x_2d), x_stride=x_2d.stride(0), out=_lib.ptr(out),
              scale=_lib.ptr(scale), scale_dtype=_SCALE_CODES[scale.dtype], rows=M, cols=N, clamp_min=float(clamp_min),
              reciprocal=int(bool(reciprocal)))
    return out
