"""GPU parity of the zoo INT8 chunk kernels (through the C ABI) against the float64 oracle, in the shapes and
with the acceptance criterion of the reference's own kernel tests (/root/reference tests/test_kernel_simple_gla.py,
test_kernel_gla.py, test_kernel_delta.py, test_kernel_kda.py, test_kernel_regimes.py).

Tolerances: outputs by the reference's criterion (tests/zoo_cases.py:check); at the two-chunk horizon also
max relative error <= 1e-3, or, where one flipped INT8 code already costs more than that, <= the oracle's own
arithmetic noise floor (its fp32-cast emulation against exact float64: 3e-3 .. 1.5e-2 at this horizon);
stored INT8 state codes within 1 LSB of the oracle's."""

import pytest
import torch

from tests import zoo_cases as zc

pytestmark = pytest.mark.gpu

DEFAULT_ETA = {"linear_none": 1.0, "mamba2": 1.0, "gla": 0.0, "deltanet": 1.0, "gated_deltanet": 1.0, "kda": 0.0}


def _go(cell, tensors, *, policy="kernel_static", bits=8, eta=None, rho=1.0, tau=1.0, label=None, rot=None, rot_v=None, **kw):
    eta = DEFAULT_ETA[cell] if eta is None else eta
    qz, run = zc.calibrated(cell, tensors, policy=policy, bits=bits, eta=eta, rho=rho, tau=tau, rot_qk=rot, rot_v=rot_v,
                            out_dtype=kw.get("out_dtype"))
    if rot_v is not None:  # the kernel receives the rotated value operand, materialized in the activation dtype
        q_, k_, v_, g_, b_ = tensors
        tensors = (q_, k_, (v_.double() @ rot_v).to(v_.dtype), g_, b_)
        kw["unrot"] = rot_v.T.contiguous()
    if rot is not None:
        kw["rot"] = rot
    B, T, H, K = tensors[0].shape
    V = tensors[2].shape[-1]
    scales = qz.kernel_scales(0, H, K, V, delta=zc.CELLS[cell][0] == "delta")
    out, ht = zc.run_kernel(cell, tensors, scales, eta=eta, rho=rho, tau=tau, bits=bits, **kw)
    torch.cuda.synchronize()
    return out, ht, qz, run


@pytest.mark.parametrize("cell", list(zc.CELLS))
@pytest.mark.parametrize("n", [128, 512])
def test_cell_matches_oracle(cuda, cell, n):
    tensors = zc.cut(zc.inputs(cell), n)
    out, _, qz, run = _go(cell, tensors)
    err_max, _ = zc.check(out, run, qz, f"{cell} T={n}")
    if n == 128:
        noise_max = zc.errors(out, run, qz)[2]
        assert err_max <= max(1e-3, noise_max), f"{cell}: two-chunk horizon rel max {err_max:.2e} (noise {noise_max:.2e})"


@pytest.mark.parametrize("cell,eta", [("mamba2", 0.0), ("mamba2", 0.5), ("gla", 0.5), ("gla", 1.0),
                                      ("gated_deltanet", 0.0), ("gated_deltanet", 0.5), ("kda", 0.5), ("kda", 1.0)])
def test_eta_split(cuda, cell, eta):
    tensors = zc.inputs(cell)
    out, _, qz, run = _go(cell, tensors, eta=eta)
    zc.check(out, run, qz, f"{cell} eta={eta}")


@pytest.mark.parametrize("cell", ["deltanet", "gated_deltanet", "kda"])
@pytest.mark.parametrize("rho,tau", [(0.5, 0.5), (0.0, 1.0), (0.0, 0.0), (0.5, 1.0)])
def test_beta_placement(cuda, cell, rho, tau):
    tensors = zc.cut(zc.inputs(cell, seed=1), 256)
    out, _, qz, run = _go(cell, tensors, rho=rho, tau=tau)
    zc.check(out, run, qz, f"{cell} sigma={rho} tau={tau}")


@pytest.mark.parametrize("cell", list(zc.CELLS))
@pytest.mark.parametrize("policy", ["kernel_pt", "kernel_ptk"])
def test_policies(cuda, cell, policy):
    tensors = zc.cut(zc.inputs(cell, seed=2), 256)
    out, _, qz, run = _go(cell, tensors, policy=policy)
    zc.check(out, run, qz, f"{cell} {policy}")


@pytest.mark.parametrize("cell", list(zc.CELLS))
def test_six_bit_codes(cuda, cell):
    tensors = zc.cut(zc.inputs(cell, seed=3), 256)
    out, _, qz, run = _go(cell, tensors, bits=6)
    zc.check(out, run, qz, f"{cell} bits=6")


@pytest.mark.parametrize("cell", ["mamba2", "gla", "gated_deltanet", "kda"])
@pytest.mark.parametrize("eta", [0.0, 0.5, 1.0])
def test_strong_decay_stays_finite(cuda, cell, eta):
    """Cumulative decay far below fp32's exp range must not produce NaN codes at any eta
    (/root/reference tests/test_kernel_simple_gla.py:63-81)."""
    tensors = zc.inputs(cell, gscale=40.0)
    out, _, qz, run = _go(cell, tensors, eta=eta)
    zc.check(out, run, qz, f"{cell} strong decay eta={eta}")


@pytest.mark.parametrize("cell", ["gla", "kda"])
@pytest.mark.parametrize("n,K", [(128, 64), (512, 64), (256, 128)])
def test_local_rqk_rotation(cuda, cell, n, K):
    """R_QK on a diagonal-decay cell is local: only the anchored operands of the off-diagonal sub-blocks are rotated
    (/root/reference tests/test_kernel_gla.py:47-60)."""
    from oracle.zoo_reference import signed_hadamard

    tensors = zc.cut(zc.inputs(cell, K=K, H=2 if K == 128 else 4), n)
    R = signed_hadamard(K, 3)
    out, _, qz, run = _go(cell, tensors, rot=R)
    zc.check(out, run, qz, f"{cell} local R_QK T={n} K={K}")


@pytest.mark.parametrize("cell", list(zc.CELLS))
@pytest.mark.parametrize("n,K,V", [(128, 64, 128), (512, 64, 128), (256, 128, 64)])
def test_canonical_storage_rv(cuda, cell, n, K, V):
    """R_V with canonical storage: v rotated outside, every product un-rotated in-kernel before it joins the fp32
    carry / the output (/root/reference tests/test_kernel_simple_gla.py:84-104, test_kernel_gla.py:63-75)."""
    from oracle.zoo_reference import signed_hadamard

    tensors = zc.cut(zc.inputs(cell, K=K, V=V, H=2 if K == 128 else 4), n)
    out, _, qz, run = _go(cell, tensors, eta=1.0, rot_v=signed_hadamard(V, 7))
    zc.check(out, run, qz, f"{cell} canonical R_V T={n} K={K} V={V}")


@pytest.mark.parametrize("cell", list(zc.CELLS))
@pytest.mark.parametrize("variant", ["plain", "rotated"])
def test_bf16_activations(cuda, cell, variant):
    """bf16 q, k, v (the dtype of the reference's timing script, /root/reference bench/zoo_kernels.py:60-63): prepared
    operands and the output are materialized in bf16, the local product stays fp16."""
    from oracle.zoo_reference import signed_hadamard

    tensors = zc.cut(zc.inputs(cell, seed=6, dtype=torch.bfloat16), 256)
    kw = {}
    if variant == "rotated":
        kw["rot_v"] = signed_hadamard(128, 7)
        if zc.CELLS[cell][1] == "diagonal":
            kw["rot"] = signed_hadamard(64, 3)
    out, _, qz, run = _go(cell, tensors, **kw)
    assert out.dtype == torch.bfloat16
    zc.check(out, run, qz, f"{cell} bf16 {variant}")


@pytest.mark.parametrize("cell", list(zc.CELLS))
def test_stored_state_codes_and_final_state(cuda, cell):
    tensors = zc.cut(zc.inputs(cell, seed=4), 256)
    dbg = {}
    out, ht, qz, run = _go(cell, tensors, debug=dbg, final_state=True)
    codes = zc.state_codes(qz, run)                      # (NT, B, H, K, V): state after each chunk
    got = dbg["h_i8"].cpu()                              # (B, NT, H, K, V): state entering each chunk
    assert (got[:, 0] == 0).all()
    NT = codes.shape[0]
    diff = (got[:, 1:].permute(1, 0, 2, 3, 4).int() - codes[: NT - 1].int()).abs()
    assert diff.max().item() <= 1, f"{cell}: stored state code off by {diff.max().item()}"
    assert (diff != 0).float().mean().item() < 0.02, f"{cell}: {(diff != 0).float().mean().item():.3%} codes differ"
    # the final fp32 carry quantizes to the last stored code
    sc = qz.kernel_scales(0, *tensors[0].shape[2:], tensors[2].shape[-1])["state"]
    last = torch.round(ht.cpu() / sc[None, :, None, :]).clamp(-127, 127)
    assert (last - codes[-1]).abs().max().item() <= 1


@pytest.mark.parametrize("cell", ["mamba2", "kda"])
def test_fp32_output_and_k128(cuda, cell):
    tensors = zc.inputs(cell, B=1, T=256, H=2, K=128, V=64, seed=5)
    out, _, qz, run = _go(cell, tensors, out_dtype=torch.float32)
    assert out.dtype == torch.float32
    zc.check(out, run, qz, f"{cell} K=128 V=64 fp32 out")


def test_rejections(cuda):
    tensors = zc.cut(zc.inputs("mamba2"), 128)
    qz, _ = zc.calibrated("mamba2", tensors)
    sc = qz.kernel_scales(0, 4, 64, 128)
    from linquant_amd.kernels import zoo

    q, k, v, g, _ = [t.cuda() if t is not None else None for t in tensors]
    sc = {n: s.cuda() for n, s in sc.items()}
    with pytest.raises(AssertionError):
        zoo.chunk_simple_gla_int8(q[:, :100], k[:, :100], v[:, :100], g[:, :100], sc)
    with pytest.raises(AssertionError):
        zoo.chunk_simple_gla_int8(q, k, v, g, sc, unrot=torch.eye(64, device="cuda", dtype=torch.float16))
