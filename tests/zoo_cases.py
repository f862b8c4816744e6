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


def cut(tensors, n):
    return [t[:, :n].contiguous() if t is not None else None for t in tensors]


def calibrated(cell, tensors, *, policy="kernel_static", bits=8, eta=1.0, rho=1.0, tau=1.0, rot_qk=None, rot_v=None, out_dtype=None):
    """Returns (qz, run): the oracle's quantizer with scales calibrated on these inputs, and a closure that
    evaluates the oracle under the quantizer's current arithmetic mode; like the kernels, the oracle materializes its
    output in the activation dtype unless ``out_dtype`` says otherwise."""
    fam, dec = CELLS[cell]
    q, k, v, g, beta = tensors
    K = q.shape[-1]
    qz = Z.ZooQuantizer.kernel_profile(policy, bits)

    def run():
        return Z.chunk_forward(q, k, v, g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=qz, eta=eta, rho=rho,
                               tau=tau, read_post=True, C=64, out_dtype=out_dtype, rot_qk=rot_qk, rot_v=rot_v,
                               storage="canonical" if rot_v is not None else "rotated")

    qz.calibrating = True
    run()
    qz.finalize()
    return qz, run


def run_kernel(cell, tensors, scales, *, eta=1.0, rho=1.0, tau=1.0, bits=8, out_dtype=None, final_state=False,
               debug=None, device="cuda", rot=None, unrot=None):
    from linquant_amd.kernels import zoo

    fam, dec = CELLS[cell]
    q, k, v, g, beta = [t.to(device) if t is not None else None for t in tensors]
    sc = {n: s.to(device) for n, s in scales.items()}
    K = q.shape[-1]
    kw = dict(eta=eta, scale=K ** -0.5, chunk_size=64, bits=bits, out_dtype=out_dtype, output_final_state=final_state,
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
