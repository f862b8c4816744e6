"""Shared helpers of the zoo GPU parity tests: seeded inputs in the shapes of the reference's kernel tests
(/root/reference tests/test_kernel_simple_gla.py:8,31-37, test_kernel_gla.py:10-18, test_kernel_delta.py,
test_kernel_kda.py), calibration of the oracle's quantizer, and the reference's acceptance criterion."""

import torch

from oracle import zoo_reference as Z

CELLS = Z.CELLS


def inputs(cell, B=2, T=512, H=4, K=64, V=128, seed=0, gscale=1.0, dtype=torch.float16):
    fam, dec = CELLS[cell]
    gen = torch.Generator().manual_seed(seed)
    q = torch.nn.functional.normalize(torch.randn(B, T, H, K, generator=gen), dim=-1).to(dtype)
    k = torch.nn.functional.normalize(torch.randn(B, T, H, K, generator=gen), dim=-1).to(dtype)
    v = torch.randn(B, T, H, V, generator=gen).to(dtype)
    g = None
    if dec == "scalar":
        g = (torch.nn.functional.logsigmoid(torch.randn(B, T, H, generator=gen) * 3) / 4).float() * gscale
    elif dec == "diagonal":
        g = (torch.nn.functional.logsigmoid(torch.randn(B, T, H, K, generator=gen) * 3) / 4).float() * gscale
    beta = torch.rand(B, T, H, generator=gen).float() if fam == "delta" else None
    return q, k, v, g, beta


# The benchmark configurations (shape, cell, policy, placements) as they are stated: per-tensor operands for linear
# attention / GLA, per-token-tensor key roles with the write gate placed at sigma = 0.5 for the delta rules, per-channel
# static scales with D_QK (alpha = 0.5) for KDA; R_QK persistent on q, k (no / scalar decay) or local (diagonal decay).
CONFIGS = {
    "c2_la": dict(cell="linear_none", B=4, T=4096, H=16, policy="kernel_pt", eta=1.0, rho=1.0, dqk=False),
    "c2_gla": dict(cell="gla", B=4, T=4096, H=16, policy="kernel_pt", eta=0.0, rho=1.0, dqk=False),
    "c3_deltanet": dict(cell="deltanet", B=4, T=4096, H=16, policy="kernel_ptk", eta=1.0, rho=0.5, dqk=False),
    "c3_gdn": dict(cell="gated_deltanet", B=4, T=4096, H=16, policy="kernel_ptk", eta=1.0, rho=0.5, dqk=False),
    "c4_kda": dict(cell="kda", B=2, T=8192, H=32, policy="kernel_static", eta=0.0, rho=0.5, dqk=True),
}


def config_inputs(name, seed, K=128, V=128, heads=None, batch_row=None):
    """fp16 inputs of a benchmark configuration as the kernels receive them, optionally cut to one batch row and a list of
    heads (the cut commutes with every step here: all of them are per (batch, head)):
    (tensors, rot) with rot the local R_QK of the diagonal-decay cells (None otherwise: there q, k arrive rotated,
    materialized in fp16, as the oracle's `mat(q @ R)` does)."""
    from linquant_amd.calibration import zoo_synthetic

    cfg = CONFIGS[name]
    q, k, v, g, beta = zoo_synthetic(cfg["cell"], cfg["B"], cfg["T"], cfg["H"], K, V, seed)
    if batch_row is not None:
        sel = lambda t: None if t is None else t[batch_row:batch_row + 1][:, :, heads].contiguous()  # noqa: E731
        q, k, v, g, beta = sel(q), sel(k), sel(v), sel(g), sel(beta)
    R = Z.signed_hadamard(K, 1)
    q, k, v = q.half(), k.half(), v.half()
    if CELLS[cfg["cell"]][1] != "diagonal":
        q, k = (q.double() @ R).half(), (k.double() @ R).half()
        R = None
    return (q, k, v, g, beta), R


def apply_dqk(tensors, D):
    """q' = fp16(q * D), k' = fp16(k / D) with D (H, K) fp32: the oracle's operand prologue without a rotation."""
    from oracle import zoo_reference as Z

    q, k, v, g, beta = tensors
    qd, kd, _ = Z.rotate_operands(q, k, v, None, None, D)
    return (qd, kd, v, g, beta)


def cut(tensors, n):
    return [t[:, :n].contiguous() if t is not None else None for t in tensors]


def calibrated(cell, tensors, *, policy="kernel_static", bits=8, eta=1.0, rho=1.0, tau=1.0, rot_qk=None, rot_v=None, out_dtype=None,
               calib_tensors=None, storage=None, chunk=64):
    """Returns (qz, run): the oracle's quantizer with scales calibrated on these inputs (or on ``calib_tensors``, a
    separate batch), and a closure that evaluates the oracle on ``tensors`` under the quantizer's current arithmetic
    mode; like the kernels, the oracle materializes its output in the activation dtype unless ``out_dtype`` says
    otherwise."""
    fam, dec = CELLS[cell]
    K = tensors[0].shape[-1]
    qz = Z.ZooQuantizer.kernel_profile(policy, bits)

    def forward(t):
        q, k, v, g, beta = t
        return Z.chunk_forward(q, k, v, g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=qz, eta=eta, rho=rho,
                               tau=tau, read_post=True, C=chunk, out_dtype=out_dtype, rot_qk=rot_qk, rot_v=rot_v,
                               storage=storage or ("canonical" if rot_v is not None else "rotated"))

    qz.calibrating = True
    forward(tensors if calib_tensors is None else calib_tensors)
    qz.finalize()
    return qz, lambda: forward(tensors)


def run_kernel(cell, tensors, scales, *, eta=1.0, rho=1.0, tau=1.0, bits=8, out_dtype=None, final_state=False,
               debug=None, device="cuda", rot=None, unrot=None, chunk=64):
    from linquant_amd.kernels import zoo

    fam, dec = CELLS[cell]
    q, k, v, g, beta = [t.to(device) if t is not None else None for t in tensors]
    sc = {n: s.to(device) for n, s in scales.items()}
    K = q.shape[-1]
    kw = dict(eta=eta, scale=K ** -0.5, chunk_size=chunk, bits=bits, out_dtype=out_dtype, output_final_state=final_state,
              _debug=debug)
    if rot is not None:
        kw["rot"] = rot.to(device)
    if unrot is not None:
        kw["unrot"] = unrot.to(device)
    if fam == "linear":
        fn = zoo.chunk_gla_int8 if dec == "diagonal" else zoo.chunk_simple_gla_int8
        return fn(q, k, v, g, sc, **kw)
    fn = zoo.chunk_kda_int8 if dec == "diagonal" else zoo.chunk_delta_int8
    return fn(q, k, v, g, beta, sc, sigma=rho, tau=tau, **kw)


def errors(out, run, qz):
    """(err_max, err_mean, noise_max, noise_mean): kernel vs the oracle's kernel-arithmetic emulation, and that
    emulation vs the oracle in exact float64 arithmetic, all relative to the emulation's magnitude."""
    ref = run().float()
    qz.kernel_arith = False
    exact = run().float()
    qz.kernel_arith = True
    d, n = (out.float().cpu() - ref).abs(), (ref - exact).abs()
    rm, ra = ref.abs().max().item(), ref.abs().mean().item()
    return d.max().item() / rm, d.mean().item() / ra, n.max().item() / rm, n.mean().item() / ra


def check(out, run, qz, label):
    """Acceptance criterion of the reference's kernel tests (tests/test_kernel_simple_gla.py:11-24): the kernel
    agrees with the fake-quant emulation at least as well as the emulation agrees with exact arithmetic
    (floors 5e-3 of the output's max, 2e-4 of its mean)."""
    assert torch.isfinite(out).all(), f"{label}: non-finite output"
    err_max, err_mean, noise_max, noise_mean = errors(out, run, qz)
    assert err_max <= max(5e-3, 2 * noise_max) and err_mean <= max(2e-4, 2 * noise_mean), \
        f"{label}: rel max {err_max:.2e} rel mean {err_mean:.2e} (noise floor {noise_max:.2e} / {noise_mean:.2e})"
    return err_max, err_mean


def state_codes(qz, run):
    """INT8 codes the oracle stored after every chunk, stacked (NT, B, H, K, V)."""
    qz.trace = []
    run()
    codes = torch.stack([c.to(torch.int8) for c in qz.trace])
    qz.trace = None
    return codes


def operand_codes(qz, run):
    """INT8 operand codes the oracle formed, per role, token-major: role -> (B, T, H, D) int8 (one call per chunk and
    role; roles called more than once per chunk, like the anchored sub-block operands, are left out)."""
    qz.code_trace = {}
    run()
    trace, qz.code_trace = qz.code_trace, None
    nt = len(trace["k_write"])
    out = {}
    for role, calls in trace.items():
        if len(calls) == nt:  # [B,H,C,D] per chunk -> (B,T,H,D)
            out[role] = torch.cat([c.permute(0, 2, 1, 3) for c in calls], dim=1)
    return out
