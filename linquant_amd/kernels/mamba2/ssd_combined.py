"""INT8 SSD combined forward: cumsum -> chunk state -> state passing -> C.B^T -> chunk scan.

Call surface of linquant/kernels/mamba2/ssd_combined.py:19-131. The six stage functions are module-level
names looked up at call time, so a per-stage timer can re-bind them (as the reference's component bench does).
While none of them is re-bound the five launches are issued by one C call (lq_ssd_combined) over one workspace
allocation; a re-bound stage switches the call to the stage-by-stage path, which runs the same kernels.
"""

import ctypes

import torch

from linquant_amd import _lib

from .bmm_chunk import _quant_bmm_chunk_fwd
from .chunk_cumsum import _quant_chunk_cumsum_fwd
from .chunk_scan_v2 import _quant_chunk_scan_fwd as _chunk_scan_v2
from .chunk_state import _quant_chunk_state_fwd_xfp_static_int8
from .chunk_state_keyside import _chunk_state_keyside_fwd
from .state_passing import _fixedpoint_state_passing_fwd

# Fractional bits of the fixed-point gate in the all-INT8 state passing (Q0.7).
_GATE_SHIFT = 7


def _quant_mamba_chunk_scan_combined_fwd(x_fp, q_dt, dt_scale, q_A_log, A_log_scale, q_B, B_scale, q_C, C_scale,
                                         chunk_size, q_D, D_scale, dt_bias=None, dt_softplus=True,
                                         dt_limit=(0.0, float("inf")), static_state_scale=None, static_cb_scale=None,
                                         alpha_hp=None, bscale_g=None, keyside=False, x_scale_hp=None, b_fp=None,
                                         b_gate_scale=None, b_rowmax=None):
    """fp16 x in, INT8 chunk states (value side: x quantized per tile with ``alpha_hp`` against INT8 ``q_B``; key
    side: x quantized with ``x_scale_hp`` against gated fp16 ``b_fp`` quantized with ``b_gate_scale``), INT8
    fixed-point recurrence, INT8 CB on ``static_cb_scale``, INT8 chunk scan. Returns (out fp16 (B,L,H,P), None).
    ``b_rowmax`` (not in the reference; key side, optional): the per-token max |b_fp| that the prologue can return beside
    ``b_fp``; without it the chunk state stage computes the table itself.  Same result either way."""
    batch, seqlen, nheads, headdim = x_fp.shape
    _, _, ngroups, dstate = q_B.shape

    if not _stages_rebound():
        return _one_call(x_fp, q_dt, dt_scale, q_A_log, A_log_scale, q_B, B_scale, q_C, C_scale, chunk_size, q_D, D_scale,
                         dt_bias, dt_softplus, dt_limit, static_state_scale, static_cb_scale, alpha_hp, bscale_g, keyside,
                         x_scale_hp, b_fp, b_gate_scale, b_rowmax=b_rowmax), None

    dA_cumsum, dt = _quant_chunk_cumsum_fwd(q_dt, dt_scale, q_A_log, A_log_scale, chunk_size, dt_bias=dt_bias,
                                            dt_softplus=dt_softplus, dt_limit=dt_limit)
    if keyside:
        kw = {} if b_rowmax is None else {"b_rowmax": b_rowmax}
        states_i8 = _chunk_state_keyside_fwd(x_fp, x_scale_hp, b_fp, dt, dA_cumsum, static_state_scale, b_gate_scale, **kw)
    else:
        states_i8 = _quant_chunk_state_fwd_xfp_static_int8(x_fp, q_B, dt, dA_cumsum, alpha_hp, bscale_g,
                                                           static_state_scale)
    states_flat_i8 = states_i8.reshape(batch, -1, nheads, headdim * dstate)
    sp_out_i8, _ = _fixedpoint_state_passing_fwd(states_flat_i8, dA_cumsum[:, :, :, -1], gate_shift=_GATE_SHIFT)
    states = sp_out_i8.reshape(batch, -1, nheads, headdim, dstate)
    cb_i8 = _quant_bmm_chunk_fwd(q_C, C_scale, b_fp if keyside else q_B, B_scale, chunk_size, static_cb_scale,
                                 b_is_fp=keyside)
    out = _chunk_scan_v2(cb_i8, x_fp, dt, dA_cumsum, q_C, C_scale, states, q_D, D_scale, static_state_scale,
                         static_cb_scale)
    return out, None


_STAGE_NAMES = ("_quant_chunk_cumsum_fwd", "_quant_chunk_state_fwd_xfp_static_int8", "_chunk_state_keyside_fwd",
                "_fixedpoint_state_passing_fwd", "_quant_bmm_chunk_fwd", "_chunk_scan_v2")
_STAGE_ORIGINALS = {n: globals()[n] for n in _STAGE_NAMES}


def _stages_rebound():
    g = globals()
    return any(g[n] is not f for n, f in _STAGE_ORIGINALS.items())


def combined_args(x_fp, q_dt, dt_scale, q_A_log, A_log_scale, q_B, B_scale, q_C, C_scale, chunk_size, q_D, D_scale, dt_bias,
                  dt_softplus, dt_limit, static_state_scale, static_cb_scale, alpha_hp, bscale_g, keyside, x_scale_hp, b_fp,
                  b_gate_scale, out, workspace=None, final_states=None, b_rowmax=None):
    """(lq_ssd_combined_args, keep-alive list) for one forward; the host-side checks of the stage wrappers apply."""
    from .chunk_cumsum import _DT_CODES, _as_f32_scalar
    from .chunk_state_keyside import _bgs_strides

    batch, seqlen, nheads, headdim = x_fp.shape
    _, _, ngroups, dstate = q_C.shape
    dev = x_fp.device
    assert x_fp.dtype == torch.float16 and x_fp.stride(3) == 1, "x must be fp16 with unit headdim stride"
    assert q_C.dtype == torch.int8 and q_C.stride(3) == 1
    assert q_A_log.shape == (nheads,) and q_A_log.dtype == torch.int8, "A_log must be (H,) INT8 codes"
    assert q_dt.shape == (batch, seqlen, nheads) and q_dt.dtype in _DT_CODES, f"unsupported dt {q_dt.dtype}"
    f32 = _lib.f32
    keep = [f32(t) for t in (B_scale, C_scale, static_state_scale, static_cb_scale, alpha_hp, bscale_g, x_scale_hp,
                             b_gate_scale, dt_bias)]
    Bs, Cs, sst, scb, alpha, bsg, xs, bgs, bias = keep
    assert scb.shape == (ngroups,), f"static_cb_scale must be (ngroups,), got {tuple(scb.shape)}"
    Bs, Cs, scb = Bs.contiguous(), Cs.contiguous(), scb.contiguous()
    dts, als = _as_f32_scalar(dt_scale, dev), _as_f32_scalar(A_log_scale, dev)
    dsc = None if q_D is None else _as_f32_scalar(D_scale, dev)
    keep += [Bs, Cs, scb, dts, als, dsc]
    f = dict(x=_lib.ptr(x_fp), x_stride_b=x_fp.stride(0), x_stride_l=x_fp.stride(1), x_stride_h=x_fp.stride(2),
             dt=_lib.ptr(q_dt), dt_dtype=_DT_CODES[q_dt.dtype], dt_stride_b=q_dt.stride(0), dt_stride_l=q_dt.stride(1),
             dt_stride_h=q_dt.stride(2), dt_scale=_lib.ptr(dts), A_log=_lib.ptr(q_A_log), A_log_stride_h=q_A_log.stride(0),
             A_log_scale=_lib.ptr(als), dt_bias=_lib.ptr(bias), dt_bias_stride_h=0 if bias is None else bias.stride(0),
             dt_softplus=int(bool(dt_softplus)), dt_min=float(dt_limit[0]), dt_max=float(dt_limit[1]),
             qC=_lib.ptr(q_C), qC_stride_b=q_C.stride(0), qC_stride_l=q_C.stride(1), qC_stride_g=q_C.stride(2),
             B_scale=_lib.ptr(Bs), C_scale=_lib.ptr(Cs), D=_lib.ptr(q_D), D_stride_h=0 if q_D is None else q_D.stride(0),
             D_has_hdim=int(q_D is not None and q_D.dim() == 2), D_scale=_lib.ptr(dsc),
             state_scale=_lib.ptr(sst), ss_stride_h=sst.stride(0), ss_stride_p=sst.stride(1), cb_scale=_lib.ptr(scb),
             keyside=int(bool(keyside)), gate_shift=_GATE_SHIFT, out=_lib.ptr(out), final_states=_lib.ptr(final_states),
             workspace=_lib.ptr(workspace), workspace_bytes=0 if workspace is None else workspace.numel(),
             batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim, ngroups=ngroups, dstate=dstate, chunk_size=chunk_size)
    if q_D is not None:
        assert q_D.dtype == torch.int8 and q_D.stride(-1) == 1
    if keyside:
        assert b_fp.dtype == torch.float16 and b_fp.stride(3) == 1, "b_fp must be fp16 with unit dstate stride"
        sb = _bgs_strides(bgs)
        f.update(b_fp=_lib.ptr(b_fp), bfp_stride_b=b_fp.stride(0), bfp_stride_l=b_fp.stride(1), bfp_stride_g=b_fp.stride(2),
                 x_scale_hp=_lib.ptr(xs), xs_stride_h=xs.stride(0), xs_stride_p=xs.stride(1), b_gate_scale=_lib.ptr(bgs),
                 bgs_stride_b=sb[0], bgs_stride_c=sb[1], bgs_stride_h=sb[2], bgs_stride_n=sb[3])
        if b_rowmax is not None:
            assert b_rowmax.dtype == torch.float32 and b_rowmax.is_contiguous() and b_rowmax.shape == (batch, seqlen, ngroups)
            f.update(b_rowmax=_lib.ptr(b_rowmax))
    else:
        assert q_B.dtype == torch.int8 and q_B.stride(3) == 1
        f.update(qB=_lib.ptr(q_B), qB_stride_b=q_B.stride(0), qB_stride_l=q_B.stride(1), qB_stride_g=q_B.stride(2),
                 alpha_hp=_lib.ptr(alpha), alpha_stride_h=alpha.stride(0), alpha_stride_p=alpha.stride(1),
                 bscale_g=_lib.ptr(bsg), bscale_stride_g=bsg.stride(0))
    return _lib.fill("lq_ssd_combined_args", **f), keep


def workspace_bytes(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size):
    """Bytes of device workspace lq_ssd_combined needs for these dims."""
    st = _lib.fill("lq_ssd_combined_args", batch=batch, seqlen=seqlen, nheads=nheads, headdim=headdim, ngroups=ngroups,
                   dstate=dstate, chunk_size=chunk_size)
    n = ctypes.c_int64(0)
    rc = _lib.load().lq_ssd_combined_workspace_bytes(ctypes.byref(st), ctypes.byref(n))
    if rc != 0:
        raise _lib.LinQuantHipError(f"lq_ssd_combined_workspace_bytes failed with code {rc}")
    return n.value


def _one_call(x_fp, q_dt, dt_scale, q_A_log, A_log_scale, q_B, B_scale, q_C, C_scale, chunk_size, q_D, D_scale, dt_bias,
              dt_softplus, dt_limit, static_state_scale, static_cb_scale, alpha_hp, bscale_g, keyside, x_scale_hp, b_fp,
              b_gate_scale, static=False, b_rowmax=None):
    batch, seqlen, nheads, headdim = x_fp.shape
    _, _, ngroups, dstate = q_C.shape
    out = torch.empty(batch, seqlen, nheads, headdim, device=x_fp.device, dtype=torch.float16)
    ws = None
    if not static:
        ws = torch.empty(workspace_bytes(batch, seqlen, nheads, headdim, ngroups, dstate, chunk_size), dtype=torch.uint8,
                         device=x_fp.device)
    st, keep = combined_args(x_fp, q_dt, dt_scale, q_A_log, A_log_scale, q_B, B_scale, q_C, C_scale, chunk_size, q_D, D_scale,
                             dt_bias, dt_softplus, dt_limit, static_state_scale, static_cb_scale, alpha_hp, bscale_g, keyside,
                             x_scale_hp, b_fp, b_gate_scale, out, ws, b_rowmax=b_rowmax)
    _lib.launch("lq_ssd_combined_static" if static else "lq_ssd_combined", x_fp.device, st)
    del keep
    return out
