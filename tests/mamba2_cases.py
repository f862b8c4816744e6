"""Shared builders for the Mamba-2 SSD parity tests: seeded inputs, calibrated scales, oracle results."""

from __future__ import annotations

import numpy as np
import torch

from linquant_amd.calibration import Mamba2Shape, calibrate_mamba2, mamba2_params, mamba2_synthetic
from oracle import mamba2_ssd as O


# decay regimes: "strong" is the benchmark recipe (dt ~ 0.13, A in [-16, -1]: every 32-token slab decays by e^-4 or
# more); "weak" is what trained layers look like (dt ~ 0.011, A in [-1.3, -1]: a 256-token chunk decays by about e^-3,
# every slab factor of the scan lies strictly between 0 and 1)
REGIMES = {"strong": dict(dt_mean=-2.0, a_max=16.0), "weak": dict(dt_mean=-4.5, a_max=1.3)}


def build_case(shape: Mamba2Shape, seed=0, calib_seed=1, device="cpu", regime="strong"):
    """Inputs (seed), parameters and static scales (calibrated on a separate seed), all torch on ``device``."""
    r = REGIMES[regime]
    params = mamba2_params(shape, seed=42, device=device, a_max=r["a_max"])
    cx, cdt = mamba2_synthetic(shape, calib_seed, device, dt_mean=r["dt_mean"])
    scales = calibrate_mamba2(shape, cx, cdt, params)
    xBC, dt_raw = mamba2_synthetic(shape, seed, device, dt_mean=r["dt_mean"])
    return dict(shape=shape, params=params, scales=scales, xBC=xBC, dt_raw=dt_raw, regime=regime)


def npy(t):
    return None if t is None else t.detach().cpu().numpy()


def oracle_prologue(case, dqk=False):
    s, p, sc = case["shape"], case["params"], case["scales"]
    return O.split_rotate_quant_xBC(npy(case["xBC"]), npy(p["r_signs"]), s.nheads, s.ngroups, s.dstate, s.headdim,
                                    npy(sc["B_inv_scale"]), npy(sc["C_inv_scale"]))


def oracle_pipeline(case, keyside):
    """Runs the CPU oracle end to end; returns its dict of intermediates (numpy)."""
    s, p, sc = case["shape"], case["params"], case["scales"]
    xBC = npy(case["xBC"])
    x, qB, qC = oracle_prologue(case)
    b_fp = None
    if keyside:
        gn = s.ngroups * s.dstate
        b_lanes = xBC[..., s.d_ssm:s.d_ssm + gn].reshape(s.batch, s.seqlen, s.ngroups, s.dstate)
        b_fp = O.kron_hadamard(b_lanes, npy(p["r_signs"]))
    res = O.ssd_combined(x, npy(case["dt_raw"]), float(p["dt_scale"]), npy(p["A_log"]), float(p["A_log_scale"]),
                         qB, npy(sc["B_scale"]), qC, npy(sc["C_scale"]), s.chunk, npy(p["D"]), float(p["D_scale"]),
                         dt_bias=npy(p["dt_bias"]), dt_softplus=True,
                         static_state_scale=npy(sc["static_state_scale"]), static_cb_scale=npy(sc["static_cb_scale"]),
                         alpha_hp=npy(sc["alpha_hp"]), bscale_g=npy(sc["bscale_g"]), keyside=keyside,
                         x_scale_hp=npy(sc["x_scale_hp"]), b_fp=b_fp, b_gate_scale=npy(sc["b_gate_scale"]))
    res.update(x=x, q_B=qB, q_C=qC, b_fp=b_fp)
    return res
