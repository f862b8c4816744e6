"""Pins the float64 zoo oracle (oracle/zoo_reference.py) against the reference's own golden vectors
(tests/golden/zoo_golden.npz, written by tests/golden/make_zoo_golden.py from linquant/reference.py), against
brute-force token-by-token recurrences, and against the invariances the reference's test suite holds
(/root/reference tests/test_reference.py:74-228)."""

import ast
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import zoo_reference as Z
from tests.golden.make_zoo_golden import B, C, CELLS, H, K, T, V, make_inputs

GOLD = np.load(Path(__file__).parent / "golden" / "zoo_golden.npz")
N_CASES = int(GOLD["n_cases"])


def _run_case(i):
    p = f"c{i:02d}_"
    cs = ast.literal_eval(str(GOLD[p + "meta"]))
    fam, dec = CELLS[cs["cell"]]
    q, k, v, g, beta = make_inputs(cs["cell"], seed=100 + i)
    sums = np.array([t.double().abs().sum().item() for t in (q, k, v, g, beta) if t is not None])
    assert np.allclose(sums, GOLD[p + "input_sum"], rtol=1e-12), "seeded input generator drifted"
    qz = Z.ZooQuantizer.kernel_profile(cs["policy"], cs["bits"])
    rq = torch.from_numpy(GOLD[p + "rot_qk"]) if "rot_qk" in cs else None
    rv = torch.from_numpy(GOLD[p + "rot_v"]) if "rot_v" in cs else None
    kw = dict(family=fam, decay=dec, scale=K ** -0.5, qz=qz, eta=cs["eta"], rho=cs["rho"], tau=cs["tau"], read_post=True,
              C=C, rot_qk=rq, rot_v=rv, storage=cs.get("storage", "rotated"), out_dtype=torch.float64)
    qz.calibrating = True
    Z.chunk_forward(q, k, v, g, beta, **kw)
    qz.finalize()
    qz.trace = []
    o = Z.chunk_forward(q, k, v, g, beta, **kw)
    return cs, qz, o, p


@pytest.mark.parametrize("i", range(N_CASES))
def test_golden_vectors_of_the_reference(i):
    cs, qz, o, p = _run_case(i)
    for (layer, role), sc in qz.scales.items():
        ref = GOLD[p + "scale_" + role]
        assert np.allclose(sc.numpy(), ref, rtol=1e-12, atol=0), (cs, role)
    codes = np.stack([c.to(torch.int8).numpy() for c in qz.trace])
    assert np.array_equal(codes, GOLD[p + "codes"]), f"{cs}: stored INT8 state codes differ"
    ref_o = GOLD[p + "o"]
    assert np.abs(o.numpy() - ref_o).max() <= 1e-9 * np.abs(ref_o).max(), cs


def test_golden_cover_every_cell_and_policy():
    seen = set()
    for i in range(N_CASES):
        cs = ast.literal_eval(str(GOLD[f"c{i:02d}_meta"]))
        seen.add((cs["cell"], cs["policy"]))
    assert {(c, p) for c in CELLS for p in ("kernel_static", "kernel_pt", "kernel_ptk")} <= seen


def test_state_pass_known_answer():
    """fp32-carry pass: the carry is never quantized, only the read copy (sc=0.5, gamma=0.9, local=0.3 x4)."""
    qz = Z.ZooQuantizer("none", 8, ["ALL"], state_bits=8)
    qz.scales[(0, "state")] = torch.full((1, 1), 0.5, dtype=torch.float64)
    S, carry, ref = torch.zeros(1, 1, 1, 1, dtype=torch.float64), None, 0.0
    for step, lc in enumerate((0.3, 0.3, 0.3, 0.3)):
        S, carry = Z._carry_update(S, carry, torch.full((1, 1, 1, 1), 0.9, dtype=torch.float64),
                                   torch.full((1, 1, 1, 1), lc, dtype=torch.float64), qz)
        ref = 0.9 * ref + lc
        assert abs(carry.item() - ref) < 1e-12 and abs(S.item() - round(ref / 0.5) * 0.5) < 1e-12
        assert np.allclose([S.item(), carry.item()], GOLD["kat_state_pass"][step], atol=1e-15)


def test_hadamard_sign_streams_and_orthogonality():
    for name in GOLD.files:
        if name.startswith("hadamard_"):
            _, n, seed = name.split("_")
            R = Z.signed_hadamard(int(n), int(seed))
            assert np.array_equal(np.sign(R.numpy()[0]), GOLD[name])
            assert torch.allclose(R @ R.T, torch.eye(int(n), dtype=R.dtype), atol=1e-12)


# ----------------------------------------------------------------------------- brute force (no quantization)
def _token_recurrence(q, k, v, g, beta, family, decay, scale):
    """S_t = Diag(exp g_t) S_{t-1} + k_t v_t^T (linear) or the (gated) delta rule; o_t = (q_t scale) S_t."""
    q, k, v = q.double(), k.double(), v.double()
    Bn, Tn, Hn, Kn = q.shape
    S = torch.zeros(Bn, Hn, Kn, v.shape[-1], dtype=torch.float64)
    out = torch.zeros(Bn, Tn, Hn, v.shape[-1], dtype=torch.float64)
    for t in range(Tn):
        if g is not None:
            gt = g[:, t].double().exp()
            S = S * (gt[..., None, None] if decay == "scalar" else gt[..., None])
        kt, vt = k[:, t], v[:, t]
        if family == "delta":
            bt = beta[:, t].double()[..., None]
            vt = bt * (vt - torch.einsum("bhk,bhkv->bhv", kt, S))
        S = S + kt[..., None] * vt[..., None, :]
        out[:, t] = torch.einsum("bhk,bhkv->bhv", q[:, t] * scale, S)
    return out


@pytest.mark.parametrize("cell", list(CELLS))
def test_unquantized_matches_token_recurrence(cell):
    fam, dec = CELLS[cell]
    q, k, v, g, beta = make_inputs(cell, seed=5)
    ref = _token_recurrence(q, k, v, g, beta, fam, dec, K ** -0.5)
    noq = Z.ZooQuantizer("none")
    for kw in (dict(), dict(eta=0.5), dict(rho=0.5, tau=0.5), dict(read_post=True), dict(C=32), dict(C=16), dict(C=128),
               dict(C=128, eta=0.5, rho=0.5, tau=0.5)):
        if dec == "none" and "eta" in kw:
            kw = {n: x for n, x in kw.items() if n != "eta"}
        o = Z.chunk_forward(q, k, v, g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=noq, out_dtype=torch.float64, **kw)
        assert (o - ref).abs().max() / ref.abs().max() < 1e-9, (cell, kw)


@pytest.mark.parametrize("cell", list(CELLS))
def test_rotation_and_storage_invariances(cell):
    fam, dec = CELLS[cell]
    q, k, v, g, beta = make_inputs(cell, seed=6)
    noq = Z.ZooQuantizer("none")
    run = lambda **kw: Z.chunk_forward(q, k, v, g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=noq,  # noqa: E731
                                       out_dtype=torch.float64, **kw)
    base = run()
    Rq, Rv = Z.signed_hadamard(K, 0), Z.signed_hadamard(V, 1)
    for kw in (dict(rot_qk=Rq), dict(rot_v=Rv), dict(rot_v=Rv, storage="canonical"), dict(rot_qk=Rq, rot_v=Rv)):
        assert (run(**kw) - base).abs().max() / base.abs().max() < 1e-9, (cell, list(kw))


def test_diagonal_key_scaling_invariance():
    for cell in ("mamba2", "gla"):
        fam, dec = CELLS[cell]
        q, k, v, g, beta = make_inputs(cell, seed=7)
        noq = Z.ZooQuantizer("none")
        D = torch.rand(H, K, generator=torch.Generator().manual_seed(2)).double() + 0.5
        base = Z.chunk_forward(q.double(), k.double(), v.double(), g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=noq)
        out = Z.chunk_forward(q.double() * D, k.double() / D, v.double(), g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=noq)
        assert (out - base).abs().max() / base.abs().max() < 1e-9


def test_kernel_profile_is_close_to_exact_and_policies_differ():
    """INT8 emulation stays within a few percent of the unquantized result; per-tensor scales are coarser."""
    q, k, v, g, beta = make_inputs("gated_deltanet", seed=8)
    exact = _token_recurrence(q, k, v, g, beta, "delta", "scalar", K ** -0.5)
    errs = {}
    for policy in ("kernel_static", "kernel_pt"):
        qz = Z.ZooQuantizer.kernel_profile(policy)
        kw = dict(family="delta", decay="scalar", scale=K ** -0.5, qz=qz, eta=1.0, read_post=True, C=C, out_dtype=torch.float64)
        qz.calibrating = True
        Z.chunk_forward(q, k, v, g, beta, **kw)
        qz.finalize()
        o = Z.chunk_forward(q, k, v, g, beta, **kw)
        errs[policy] = ((o - exact).abs().max() / exact.abs().max()).item()
        sc = qz.kernel_scales(0, H, K, V, delta=True)
        assert sc["q"].shape == (H,) and sc["kw"].shape == (H, K) and sc["state"].shape == (H, V) and sc["ew"].shape == (H, V)
        assert all(t.dtype == torch.float32 for t in sc.values())
    assert errs["kernel_static"] < 0.05 and errs["kernel_pt"] < 0.1


def test_rotate_operands_is_the_entry_rotation_of_chunk_forward():
    """The stand-alone operand prologue hands chunk_forward exactly what chunk_forward would have formed itself:
    forward(q, k, v, rot_qk=R, rot_v=Rv) == forward(*rotate_operands(q, k, v, R, Rv)) under kernel arithmetic, bit
    for bit (linquant/reference.py:40-46), and the rotation is orthogonal; D_QK scales q up and k down by the same
    factor, so the unquantized q.k products do not move (linquant/harness.py:84-87)."""
    import torch

    from oracle import zoo_reference as Z
    from tests import zoo_cases as zc

    q, k, v, g, beta = zc.cut(zc.inputs("mamba2", B=1, H=2, K=64, V=64, seed=3), 128)
    R, Rv = Z.signed_hadamard(64, 1), Z.signed_hadamard(64, 2)
    assert torch.allclose(R @ R.T, torch.eye(64, dtype=torch.float64), atol=1e-12)
    qz = Z.ZooQuantizer.kernel_profile("kernel_static", 8)
    fw = lambda a, b, c, **kw: Z.chunk_forward(a, b, c, g, None, family="linear", decay="scalar", scale=0.125, qz=qz,  # noqa: E731
                                               eta=1.0, read_post=True, C=64, **kw)
    qz.calibrating = True
    fw(q, k, v, rot_qk=R, rot_v=Rv)
    qz.finalize()
    qr, kr, vr = Z.rotate_operands(q, k, v, R, Rv)
    assert qr.dtype == q.dtype
    a = fw(q, k, v, rot_qk=R, rot_v=Rv, out_dtype=torch.float64)
    b = fw(qr, kr, vr, out_dtype=torch.float64) @ Rv.T  # rotated storage: the caller un-rotates the output
    assert torch.equal(a, b)
    D = torch.rand(2, 64) + 0.5
    qd, kd, _ = Z.rotate_operands(q, k, v, None, None, D)
    dots = (q.double() * k.double()).sum(-1)
    assert torch.allclose((qd.double() * kd.double()).sum(-1), dots, atol=5e-3)
    assert torch.equal(qd, (q.float() * D[None, None]).half())
    assert torch.equal(kd, (k.double() / D.double()[None, None]).float().half())
    # the reciprocal form k * RN(1 / D), which the division replaced, differs from it now and then: the gap is measured,
    # so that a return to it would show (the kernels divide: q0 = k r, q = q0 + fma(-q0, D, k) r)
    gen = torch.Generator().manual_seed(11)
    kk, DD = torch.randn(1, 4096, 2, 64, generator=gen).half(), torch.rand(2, 64, generator=gen) + 0.5
    div = Z.rotate_operands(kk, kk, kk, None, None, DD)[1]
    alt = (kk.float() * (1.0 / DD)[None, None]).half()
    rate = (alt != div).float().mean().item()
    assert 0.0 < rate < 1e-3, rate


def test_two_fma_quotient_of_half_precision_values_equals_ieee_division():
    """The kernels divide k by D_QK as q0 = RN(x RN(1/d)), rem = fma(-q0, d, x), q = fma(rem, RN(1/d), q0).  Over every
    finite fp16 value and every bf16 value of moderate magnitude, against many divisors, q is the IEEE fp32 quotient
    (restated in float64: the products of two fp32 values are exact there; an inexact sum that lands on an fp32 tie is
    decided exactly)."""
    import numpy as np
    from fractions import Fraction

    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    xs = [h[np.isfinite(h)].astype(np.float32)]
    b = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    xs.append(b[np.isfinite(b) & ((np.abs(b) == 0) | ((np.abs(b) > 2.0 ** -60) & (np.abs(b) < 2.0 ** 60)))])
    rng = np.random.default_rng(5)
    ds = np.concatenate([np.exp2(rng.uniform(-20, 20, 160)), rng.uniform(0.5, 1.5, 64), [1.0, 3.0, 0.1, 1.9999999, 1.0000001]]).astype(np.float32)
    for x in xs:
        for d in ds:
            r = np.float32(1.0) / d
            q0 = (x * r).astype(np.float32)
            rem = (x.astype(np.float64) - q0.astype(np.float64) * np.float64(d)).astype(np.float32)
            q = (q0.astype(np.float64) + rem.astype(np.float64) * np.float64(r)).astype(np.float32)
            ref = x / d
            for i in np.nonzero(q != ref)[0]:
                exact = Fraction(float(q0[i])) + Fraction(float(rem[i])) * Fraction(float(r))
                assert abs(exact - Fraction(float(ref[i]))) <= abs(exact - Fraction(float(q[i]))), (float(d), float(x[i]))


# ---- the remaining properties of the reference's own oracle suite (/root/reference tests/test_reference.py), each on the
# restatement: a wrong exponent, a dropped factor or a transposed operand in the delta / placement / scaling code breaks one


def _unq(cell, inputs, **kw):
    fam, dec = CELLS[cell]
    q, k, v, g, beta = inputs
    return Z.chunk_forward(q, k, v, g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=Z.ZooQuantizer("none"),
                           out_dtype=torch.float64, **kw)


@pytest.mark.parametrize("cell", ["deltanet", "gated_deltanet", "kda"])
def test_delta_gram_exponent_and_write_placement_grid_is_exact(cell):
    """Gram exponent x write placement, 3 x 3, leaves the unquantized output unchanged (test_reference.py:143-154)."""
    inp = make_inputs(cell, seed=11)
    base = _unq(cell, inp)
    for sig in (0.0, 0.5, 1.0):
        for tau in (0.0, 0.5, 1.0):
            out = _unq(cell, inp, rho=sig, tau=tau)
            assert (out - base).abs().max() / base.abs().max() < 1e-9, (cell, sig, tau)


@pytest.mark.parametrize("cell", ["linear_none", "mamba2", "gla"])
def test_linear_write_gate_placement_is_exact(cell):
    """Moving a write gate beta from v onto k in the linear cells is exact (test_reference.py:156-168)."""
    q, k, v, g, _ = make_inputs(cell, seed=12)
    beta = torch.rand(B, T, H, generator=torch.Generator().manual_seed(1)).double().unsqueeze(-1)
    base = _unq(cell, (q.double(), k.double(), v.double() * beta, g, None))
    for rho in (0.0, 0.5):
        out = _unq(cell, (q.double(), k.double() * beta ** (1 - rho), v.double() * beta ** rho, g, None))
        assert (out - base).abs().max() / base.abs().max() < 1e-9, (cell, rho)


def test_value_axis_scaling_is_exact():
    """V . Dv with the output divided by Dv is exact in every cell, the delta family included, and composes with the key
    scaling Q . D, K / D (test_reference.py:170-182, 219-228)."""
    gen = torch.Generator().manual_seed(3)
    D = torch.rand(H, K, generator=gen).double() + 0.5
    Dv = torch.rand(H, V, generator=gen).double() + 0.5
    for cell in CELLS:
        q, k, v, g, beta = make_inputs(cell, seed=13)
        base = _unq(cell, (q.double(), k.double(), v.double(), g, beta))
        out = _unq(cell, (q.double(), k.double(), v.double() * Dv, g, beta)) / Dv
        assert (out - base).abs().max() / base.abs().max() < 1e-9, cell
        if CELLS[cell][0] == "linear":
            out = _unq(cell, (q.double() * D, k.double() / D, v.double() * Dv, g, beta)) / Dv
            assert (out - base).abs().max() / base.abs().max() < 1e-9, cell


@pytest.mark.parametrize("cell", ["mamba2", "gated_deltanet"])
def test_eta_is_flat_under_per_row_dynamic_write_scales(cell):
    """Per-row dynamic scales absorb the per-token write weights, so the eta sweep is flat (test_reference.py:92-98)."""
    fam, dec = CELLS[cell]
    # float32 inputs as in the reference's test: half-precision inputs put many elements exactly on a rounding tie of the
    # per-row grid (254 x = (2 n + 1) max|x| has solutions among 11-bit mantissas), where the weight's rounding decides
    q, k, v, g, beta = make_inputs(cell, seed=14)
    gen = torch.Generator().manual_seed(14)
    q, k, v = (t.float() + 1e-3 * torch.randn(t.shape, generator=gen) for t in (q, k, v))
    outs = []
    for eta in (0.0, 1.0):
        qz = Z.ZooQuantizer("row_dyn", 8, ["k_write", "e_write", "v_write"])
        outs.append(Z.chunk_forward(q, k, v, g, beta, family=fam, decay=dec, scale=K ** -0.5, qz=qz, eta=eta,
                                    out_dtype=torch.float64))
    assert (outs[0] - outs[1]).abs().max() / outs[0].abs().max() < 1e-6


@pytest.mark.parametrize("cell", ["mamba2", "gated_deltanet", "kda"])
@pytest.mark.parametrize("policy", ["kernel_static", "kernel_pt", "kernel_ptk"])
def test_policies_with_int8_state_in_both_storage_bases_stay_close(cell, policy):
    """Every realizable policy with an INT8 stored state, rotated and canonical storage under R_V: calibrates, runs, stays
    finite and within 10 % of the unquantized result (test_reference.py:125-140)."""
    fam, dec = CELLS[cell]
    inp = make_inputs(cell, seed=15)
    q, k, v, g, beta = inp
    base = _unq(cell, inp)
    Rv = Z.signed_hadamard(V, 1)
    for storage in ("rotated", "canonical"):
        qz = Z.ZooQuantizer("pt_static", 8, ["ALL"], dict(Z.POLICIES[policy]), state_bits=8)
        kw = dict(family=fam, decay=dec, scale=K ** -0.5, qz=qz, rot_v=Rv, storage=storage, out_dtype=torch.float64)
        qz.calibrating = True
        Z.chunk_forward(q, k, v, g, beta, **kw)
        qz.finalize()
        out = Z.chunk_forward(q, k, v, g, beta, **kw)
        err = ((out - base).abs().max() / base.abs().max()).item()
        assert torch.isfinite(out).all() and err < 0.1, (cell, policy, storage, err)


def test_kernel_scales_read_the_requested_layer():
    """kernel_scales(layer) takes every operand scale from that layer, not from the quantizer's current one
    (test_reference.py:230-239)."""
    qz = Z.ZooQuantizer("none", 8, ["ALL"], state_bits=8)
    qz.layer = 1
    for layer, val in ((0, 2.0), (1, 9.0)):
        for role in ("q_read", "k_local", "k_write", "v_write", "v_local", "state"):
            qz.scales[(layer, role)] = torch.tensor(val)
    out = qz.kernel_scales(0, 1, 1, 1)
    assert all(float(t.flatten()[0]) == 2.0 for t in out.values()), {n: float(t.flatten()[0]) for n, t in out.items()}
