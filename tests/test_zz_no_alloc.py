"""The allocation-free entry point lq_ssd_combined_static (scratch inside the library image) against lq_ssd_combined
(caller-supplied workspace), through the C ABI: identical output on two calls in a row, the second on a smaller
input, so that whatever the first call left in the shared scratch cannot leak into the second."""

import ctypes

import pytest
import torch

from linquant_amd import _lib
from linquant_amd.calibration import Mamba2Shape
from tests.mamba2_cases import build_case

pytestmark = pytest.mark.gpu


def _forward(case, cuda, keyside, entry, seqlen=None):
    """One forward through the C entry point ``entry`` on freshly allocated inputs (cut to ``seqlen`` tokens when given);
    returns (out, final_states)."""
    import dataclasses
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    s = case["shape"]
    p = {k: v.to(cuda) for k, v in case["params"].items()}
    sc = {k: v.to(cuda) for k, v in case["scales"].items()}
    xBC, dt_raw = case["xBC"].to(cuda), case["dt_raw"].to(cuda)
    if seqlen is not None:
        s = dataclasses.replace(s, seqlen=seqlen)
        xBC, dt_raw = xBC[:, :seqlen].contiguous(), dt_raw[:, :seqlen].contiguous()
    x, qB, qC = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                             sc["B_inv_scale"], sc["C_inv_scale"])
    gn = s.ngroups * s.dstate
    b_fp = kronecker_hadamard_fwd(xBC[..., s.d_ssm:s.d_ssm + gn].reshape(s.batch, s.seqlen, s.ngroups, s.dstate).contiguous(),
                                  p["r_signs"], s.ngroups)
    out = torch.empty(s.batch, s.seqlen, s.nheads, s.headdim, device=cuda, dtype=torch.float16)
    final = torch.empty(s.batch, s.nheads, s.headdim * s.dstate, device=cuda, dtype=torch.int8)
    ws = None
    if entry == "lq_ssd_combined":
        n = M.workspace_bytes(s.batch, s.seqlen, s.nheads, s.headdim, s.ngroups, s.dstate, s.chunk)
        ws = torch.full((n,), 0x5A, dtype=torch.uint8, device=cuda)  # garbage on entry: nothing may rely on zeros
    st, keep = M.combined_args(x, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"],
                               s.chunk, p["D"], p["D_scale"], p["dt_bias"], True, (0.0, float("inf")),
                               sc["static_state_scale"], sc["static_cb_scale"], sc["alpha_hp"], sc["bscale_g"], keyside,
                               sc["x_scale_hp"], b_fp, sc["b_gate_scale"], out, ws, final)
    _lib.launch(entry, torch.device(cuda), st)
    torch.cuda.synchronize()
    return out, final


@pytest.mark.parametrize("keyside", [True, False])
def test_static_scratch_entry_point_matches_workspace_entry_point(cuda, keyside):
    big = build_case(Mamba2Shape(batch=2, seqlen=1024, nheads=4, headdim=64, dstate=128, ngroups=1, chunk=256))
    small = build_case(Mamba2Shape(batch=1, seqlen=256, nheads=2, headdim=64, dstate=64, ngroups=1, chunk=64), seed=3)
    for name, case, L in (("first call", big, 1000), ("second, smaller call", small, None)):  # 1000: ragged last chunk
        print("[case] lq_ssd_combined_static", name, case["shape"], L, "keyside", keyside, flush=True)
        got, gfin = _forward(case, cuda, keyside, "lq_ssd_combined_static", L)
        ref, rfin = _forward(case, cuda, keyside, "lq_ssd_combined", L)
        assert torch.isfinite(got).all()
        assert torch.equal(got, ref), f"{name}: output differs from the workspace entry point"
        assert torch.equal(gfin, rfin), f"{name}: final states differ"


def test_static_scratch_entry_point_rejects_oversized_shapes(cuda):
    """Dims whose intermediates exceed the built-in scratch are refused before anything is launched."""
    st = _lib.fill("lq_ssd_combined_args", batch=4, seqlen=8192, nheads=80, headdim=64, ngroups=1, dstate=128, chunk_size=256)
    n = ctypes.c_int64(0)
    lib = _lib.load()
    assert lib.lq_ssd_combined_workspace_bytes(ctypes.byref(st), ctypes.byref(n)) == 0 and n.value > (64 << 20)
    dummy = torch.zeros(64, dtype=torch.uint8, device=cuda)
    for f in ("x", "dt", "qC", "out", "b_fp", "qB"):
        setattr(st, f, dummy.data_ptr())
    assert lib.lq_ssd_combined_static(ctypes.byref(st), None) == -22
