"""Kronecker-factored signed Hadamard rotation of the state axis (HIP).

Call surface of linquant/kernels/hadamard.py:106-179: y = (x * signs) . (H2 (x) H_{D/2}) per head.
"""

from __future__ import annotations

import math

import torch

from linquant_amd import _lib
from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import _SIGN_CODES, _signs_arg


def hadamard_matrix(d: int, device=None, dtype=None) -> torch.Tensor:
    """Normalized Sylvester Hadamard matrix of size d (power of two)."""
    if d & (d - 1) != 0:
        raise ValueError(f"Hadamard rotation requires d to be a power of 2, got {d}")
    H = torch.ones(1, 1, device=device, dtype=torch.float32)
    while H.shape[0] < d:
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    H = H / math.sqrt(d)
    return H if dtype is None else H.to(dtype)


def _resolve_kronecker_params(D, n_chunks, device):
    """(H_{D/n_chunks} block in bf16, 1/sqrt(n_chunks)): the factors the rotation is defined with. The HIP kernel
    evaluates the block product as a Walsh-Hadamard butterfly and only needs the block's entry magnitude."""
    return hadamard_matrix(D // n_chunks, device=device, dtype=torch.bfloat16), 1.0 / math.sqrt(n_chunks)


def kronecker_hadamard_fwd(x, signs, num_heads, n_chunks=2):
    """x (B,T,H,D) fp16 or bf16, D a power of two from 64 to 512, any batch/seq/head stride (e.g. a view of xBC);
    signs (H,D) +-1.  Returns (x * signs) @ H per head, contiguous, same dtype."""
    B, T, H, D = x.shape
    assert D >= 64, f"Kronecker Hadamard needs D >= 64, got {D}"
    assert n_chunks == 2 and D in (64, 128, 256, 512), "two-half Kronecker rotation: D a power of two, 64 .. 512"
    assert x.dtype in (torch.float16, torch.bfloat16) and x.stride(3) == 1, "x must be fp16 or bf16 with a dense last axis"
    signs = _signs_arg(signs)
    assert signs.numel() == H * D
    y = torch.empty((B, T, H, D), dtype=x.dtype, device=x.device)
    _lib.call("lq_kron_hadamard", x.device,
              x=_lib.ptr(x), x_stride_b=x.stride(0), x_stride_t=x.stride(1), x_stride_h=x.stride(2),
              y=_lib.ptr(y), signs=_lib.ptr(signs), signs_dtype=_SIGN_CODES[signs.dtype],
              batch=B, seqlen=T, nheads=H, dim=D,
              x_dtype=_lib.LQ_DT_BF16 if x.dtype == torch.bfloat16 else _lib.LQ_DT_F16)
    return y
