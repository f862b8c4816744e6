"""Gated RMSNorm behind the Mamba-2 SSD (HIP): the `self.norm(y, z)` step at linquant/quantized_mamba2.py:354-358,
i.e. RMSNormGated with norm_before_gate = False and group_size = d_ssm / ngroups, and its fusion with the Hadamard +
INT8 quantizer of the out_proj input (linquant/quantized_mamba2.py:364)."""

from __future__ import annotations

import torch
import torch.nn as nn

from linquant_amd import _lib
from linquant_amd.hadamard_utils import _device_matrix, _kernel_scale

_W_CODES = {torch.float16: _lib.LQ_DT_F16, torch.float32: _lib.LQ_DT_F32}


def _rows(t, dim):
    t2 = t.reshape(-1, dim)
    if t2.stride(1) != 1 or t2.stride(0) % 8 != 0:
        t2 = t2.contiguous()
    return t2


def rmsnorm_gated(x, z, weight, eps=1e-5, group_size=None):
    """out = fp16(v * rsqrt(mean_group(v^2) + eps) * weight) with v = x * silu(z) (v = x when z is None), in fp32."""
    assert x.dtype == torch.float16 and weight.dtype in _W_CODES
    dim = x.shape[-1]
    group_size = dim if group_size is None else group_size
    x2 = _rows(x, dim)
    z2 = None if z is None else _rows(z, dim)
    assert z2 is None or (z2.dtype == torch.float16 and z2.shape == x2.shape)
    weight = weight.contiguous()
    out = torch.empty(x2.shape, dtype=torch.float16, device=x.device)
    if x2.shape[0]:
        _lib.call("lq_rmsnorm_gated", x.device, x=_lib.ptr(x2), x_stride=x2.stride(0), z=_lib.ptr(z2),
                  z_stride=0 if z2 is None else z2.stride(0), weight=_lib.ptr(weight),
                  weight_dtype=_W_CODES[weight.dtype], out=_lib.ptr(out), rows=x2.shape[0], dim=dim,
                  group_size=group_size, eps=float(eps))
    return out.reshape(x.shape)


def rmsnorm_gated_qhad(x, z, weight, input_scale, eps=1e-5, group_size=None, return_norm=False):
    """``qhad_transform(rmsnorm_gated(x, z, weight), input_scale)`` in one launch.
    Returns (int8, input_scale) or (int8, input_scale, fp16 normalized rows) with ``return_norm``."""
    assert x.dtype == torch.float16 and weight.dtype in _W_CODES
    dim = x.shape[-1]
    group_size = dim if group_size is None else group_size
    x2 = _rows(x, dim)
    z2 = None if z is None else _rows(z, dim)
    weight = weight.contiguous()
    out = torch.empty(x2.shape, dtype=torch.int8, device=x.device)
    normed = torch.empty(x2.shape, dtype=torch.float16, device=x.device) if return_norm else None
    if x2.shape[0]:
        _lib.call("lq_rmsnorm_gated_qhad", x.device, x=_lib.ptr(x2), x_stride=x2.stride(0), z=_lib.ptr(z2),
                  z_stride=0 if z2 is None else z2.stride(0), weight=_lib.ptr(weight),
                  weight_dtype=_W_CODES[weight.dtype], norm_out=_lib.ptr(normed), rows=x2.shape[0], dim=dim,
                  group_size=group_size, eps=float(eps), had=_lib.ptr(_device_matrix(dim, x.device)),
                  out=_lib.ptr(out), scale=_kernel_scale(dim, input_scale))
    if return_norm:
        return out.reshape(x.shape), input_scale, normed.reshape(x.shape)
    return out.reshape(x.shape), input_scale


class RMSNormGated(nn.Module):
    """Module form with the constructor of the norm the mixer receives (hidden_size, eps, group_size;
    norm_before_gate must be False, the only mode the Mamba-2 mixer uses)."""

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=False, device=None, dtype=None):
        super().__init__()
        assert not norm_before_gate, "only norm_before_gate=False is built"
        self.eps = eps
        self.group_size = hidden_size if group_size is None else group_size
        self.weight = nn.Parameter(torch.ones(hidden_size, device=device, dtype=dtype or torch.float16))

    def forward(self, x, z=None):
        return rmsnorm_gated(x, z, self.weight, self.eps, self.group_size)
