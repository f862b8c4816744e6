"""All-INT8 fixed-point state passing (HIP). Call surface of linquant/kernels/mamba2/state_passing.py:96-121."""

from __future__ import annotations

import torch

from linquant_amd import _lib


def _fixedpoint_state_passing_fwd(states_i8, dA_chunk_cumsum, gate_shift=7):
    """states_i8 (B,nc,H,dim) int8, dA_chunk_cumsum (B,H,nc) (any strides, e.g. dA_cumsum[..., -1]).
    Returns (out_i8 (B,nc,H,dim), final_i8 (B,H,dim)); out_i8[:, c] is the state entering chunk c (zero initial)."""
    batch, nchunks, nheads, dim = states_i8.shape
    assert states_i8.dtype == torch.int8
    assert dA_chunk_cumsum.shape == (batch, nheads, nchunks)
    if dA_chunk_cumsum.dtype != torch.float32:
        dA_chunk_cumsum = dA_chunk_cumsum.float()
    out = torch.empty_like(states_i8)
    final_states = torch.empty((batch, nheads, dim), device=states_i8.device, dtype=torch.int8)
    _lib.call("lq_state_passing", states_i8.device,
              states=_lib.ptr(states_i8), states_stride_b=states_i8.stride(0), states_stride_c=states_i8.stride(1),
              states_stride_h=states_i8.stride(2), states_stride_d=states_i8.stride(3),
              dA_chunk_cumsum=_lib.ptr(dA_chunk_cumsum), dA_stride_b=dA_chunk_cumsum.stride(0),
              dA_stride_h=dA_chunk_cumsum.stride(1), dA_stride_c=dA_chunk_cumsum.stride(2),
              out=_lib.ptr(out), out_stride_b=out.stride(0), out_stride_c=out.stride(1), out_stride_h=out.stride(2),
              out_stride_d=out.stride(3),
              final_states=_lib.ptr(final_states), final_stride_b=final_states.stride(0),
              final_stride_h=final_states.stride(1), final_stride_d=final_states.stride(2),
              batch=batch, nchunks=nchunks, nheads=nheads, dim=dim, gate_shift=int(gate_shift), vec_hint=0)
    return out, final_states
