"""dt pipeline + chunk-local cumsum of dt*A (HIP). Call surface of linquant/kernels/mamba2/chunk_cumsum.py:77-100."""

from __future__ import annotations

import math

import torch

from linquant_amd import _lib

_DT_CODES = {torch.float16: _lib.LQ_DT_F16, torch.float32: _lib.LQ_DT_F32, torch.int8: _lib.LQ_DT_I8}


def _quant_chunk_cumsum_fwd(q_dt, dt_scale, q_A_log, A_log_scale, chunk_size, dt_bias=None, dt_softplus=False,
                            dt_limit=(0.0, float("inf"))):
    """q_dt (B,L,H) fp16/fp32/int8 with any strides, dt_scale / A_log_scale 0-dim device tensors, q_A_log (H,) int8,
    dt_bias (H,) or None. Returns (dA_cumsum, dt_out), both (B,H,nchunks,chunk_size) fp32."""
    batch, seqlen, nheads = q_dt.shape
    assert q_A_log.shape == (nheads,)
    if dt_bias is not None:
        assert dt_bias.shape == (nheads,)
    assert q_dt.dtype in _DT_CODES, f"unsupported dt dtype {q_dt.dtype}"
    assert q_A_log.dtype == torch.int8, "A_log must be INT8 codes"
    nchunks = math.ceil(seqlen / chunk_size)
    dev = q_dt.device
    dt_out = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    dA_cumsum = torch.empty(batch, nheads, nchunks, chunk_size, device=dev, dtype=torch.float32)
    dt_scale = _as_f32_scalar(dt_scale, dev)
    A_log_scale = _as_f32_scalar(A_log_scale, dev)
    bias = None if dt_bias is None else (dt_bias if dt_bias.dtype == torch.float32 else dt_bias.float())
    _lib.call("lq_chunk_cumsum", dev,
              dt=_lib.ptr(q_dt), dt_dtype=_DT_CODES[q_dt.dtype],
              dt_stride_b=q_dt.stride(0), dt_stride_l=q_dt.stride(1), dt_stride_h=q_dt.stride(2),
              dt_scale=_lib.ptr(dt_scale), A_log=_lib.ptr(q_A_log), A_log_stride_h=q_A_log.stride(0),
              A_log_scale=_lib.ptr(A_log_scale), dt_bias=_lib.ptr(bias),
              dt_bias_stride_h=0 if bias is None else bias.stride(0),
              dt_out=_lib.ptr(dt_out), dA_cumsum=_lib.ptr(dA_cumsum),
              batch=batch, seqlen=seqlen, nheads=nheads, chunk_size=chunk_size,
              dt_softplus=int(bool(dt_softplus)), dt_min=float(dt_limit[0]), dt_max=float(dt_limit[1]))
    return dA_cumsum, dt_out


def _as_f32_scalar(s, device):
    """0-dim fp32 device tensor (python numbers are staged once per call; tensors pass through)."""
    if torch.is_tensor(s):
        if s.dtype == torch.float32 and s.device == device:
            return s
        return s.to(device=device, dtype=torch.float32)
    return torch.tensor(float(s), dtype=torch.float32, device=device)
