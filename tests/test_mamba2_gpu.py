"""GPU parity of the Mamba-2 INT8 SSD HIP kernels against the CPU oracle (through the Python call surface,
which goes through the C ABI).  Integer tensors must be bit-exact; the fp16 output stage is held to
max |err| <= 1e-3 * max |ref| against the float64 oracle."""

import math
import sys

import numpy as np
import pytest
import torch

from linquant_amd.calibration import Mamba2Shape
from oracle import mamba2_ssd as O
from tests.mamba2_cases import build_case, npy, oracle_pipeline

pytestmark = pytest.mark.gpu


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def dev(t, device):
    return None if t is None else torch.from_numpy(np.ascontiguousarray(t)).to(device)


def assert_same_codes(got, ref, name):
    got, ref = npy(got), np.asarray(ref)
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    bad = np.argwhere(got != ref)
    assert bad.size == 0, f"{name}: {len(bad)} of {ref.size} codes differ, first at {bad[0]}: got {got[tuple(bad[0])]} ref {ref[tuple(bad[0])]}"


def assert_close_out(got, ref, name, tol=1e-3):
    got, ref = npy(got).astype(np.float64), np.asarray(ref, np.float64)
    assert np.isfinite(got).all(), name
    err = np.abs(got - ref).max() / np.abs(ref).max()
    assert err <= tol, f"{name}: max err / max ref = {err:.3e} > {tol}"


SHAPES = [
    (Mamba2Shape(batch=2, seqlen=512, nheads=4, headdim=64, dstate=128, ngroups=1, chunk=256), "strong"),
    (Mamba2Shape(batch=1, seqlen=256, nheads=8, headdim=64, dstate=64, ngroups=2, chunk=64), "strong"),
    (Mamba2Shape(batch=2, seqlen=384, nheads=2, headdim=128, dstate=128, ngroups=2, chunk=128), "strong"),
    # weak decay (dt ~ 0.011, A ~ -1): the slab factors of the scan's off-diagonal path lie strictly inside (0, 1)
    (Mamba2Shape(batch=1, seqlen=512, nheads=4, headdim=64, dstate=128, ngroups=1, chunk=256), "weak"),
    (Mamba2Shape(batch=1, seqlen=384, nheads=2, headdim=64, dstate=64, ngroups=1, chunk=128), "weak"),
]


@pytest.fixture(scope="module", params=range(len(SHAPES)), ids=lambda i: f"{SHAPES[i][1]}{i}")
def case(request):
    shape, regime = SHAPES[request.param]
    c = build_case(shape, regime=regime)
    c["oracle"] = {False: oracle_pipeline(c, False), True: oracle_pipeline(c, True)}
    return c


def gpu_inputs(case, cuda):
    p = {k: v.to(cuda) for k, v in case["params"].items()}
    sc = {k: v.to(cuda) for k, v in case["scales"].items()}
    return case["xBC"].to(cuda), case["dt_raw"].to(cuda), p, sc


def test_chunk_cumsum(case, cuda):
    from linquant_amd.kernels.mamba2.chunk_cumsum import _quant_chunk_cumsum_fwd

    s = case["shape"]
    say("chunk_cumsum", s)
    _, dt_raw, p, _ = gpu_inputs(case, cuda)
    dA, dt = _quant_chunk_cumsum_fwd(dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], s.chunk, dt_bias=p["dt_bias"],
                                     dt_softplus=True)
    torch.cuda.synchronize()
    ref = case["oracle"][False]
    assert np.array_equal(npy(dt), ref["dt"]) and np.array_equal(npy(dA), ref["dA_cumsum"])


@pytest.mark.parametrize("L,Q,softplus,limit,dtype", [(300, 128, True, (0.001, 0.5), torch.float16),
                                                      (1000, 256, False, (0.0, float("inf")), torch.float32),
                                                      (64, 64, True, (0.0, float("inf")), torch.float16),
                                                      (700, 512, True, (0.0, float("inf")), torch.float16)])
def test_chunk_cumsum_ragged_strided(cuda, L, Q, softplus, limit, dtype):
    from linquant_amd.kernels.mamba2.chunk_cumsum import _quant_chunk_cumsum_fwd

    say("chunk_cumsum ragged", L, Q, softplus, limit, dtype)
    g = torch.Generator().manual_seed(5)
    B, H = 2, 6
    wide = (torch.randn(B, L, H + 10, generator=g) * 0.5 - 2).to(dtype)
    if not softplus:
        wide = wide.abs() * 0.1
    bias = torch.randn(H, generator=g) * 0.1
    a_log = torch.randint(0, 127, (H,), generator=g).to(torch.int8)
    view = wide.to(cuda)[..., 3:3 + H]  # non-contiguous slice, as the in_proj split produces
    dA, dt = _quant_chunk_cumsum_fwd(view, torch.tensor(0.9, device=cuda), a_log.to(cuda), torch.tensor(0.02, device=cuda),
                                     Q, dt_bias=bias.to(cuda), dt_softplus=softplus, dt_limit=limit)
    torch.cuda.synchronize()
    rdA, rdt = O.chunk_cumsum(npy(wide[..., 3:3 + H]), np.float32(0.9), npy(a_log), np.float32(0.02), Q, npy(bias), softplus, limit)
    assert np.array_equal(npy(dt), rdt) and np.array_equal(npy(dA), rdA)


def test_prologue_and_rotation(case, cuda):
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    s = case["shape"]
    say("prologue", s)
    xBC, _, p, sc = gpu_inputs(case, cuda)
    x, qB, qC = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                             sc["B_inv_scale"], sc["C_inv_scale"])
    torch.cuda.synchronize()
    ref = case["oracle"][True]
    assert x.data_ptr() == xBC.data_ptr() and x.shape == (s.batch, s.seqlen, s.nheads, s.headdim)
    assert_same_codes(qB, ref["q_B"], "q_B")
    assert_same_codes(qC, ref["q_C"], "q_C")
    gn = s.ngroups * s.dstate
    b_view = xBC[..., s.d_ssm:s.d_ssm + gn].view(s.batch, s.seqlen, s.ngroups, s.dstate)  # strided view
    y = kronecker_hadamard_fwd(b_view, p["r_signs"], s.ngroups)
    torch.cuda.synchronize()
    assert np.array_equal(npy(y).view(np.uint16), ref["b_fp"].view(np.uint16))


@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (128, torch.bfloat16), (256, torch.float16), (256, torch.bfloat16),
                                     (512, torch.float16), (512, torch.bfloat16)])
def test_kronecker_hadamard_widths_and_bf16(cuda, D, dtype):
    """kronecker_hadamard_fwd over the reference's whole domain (linquant/kernels/hadamard.py:141-152: fp16 / bf16, D a
    power of two >= 64; here up to 512): a strided view of a wider slab, a token count that is not a multiple of the
    rows per workgroup; bit-exact against the oracle's two-half rotation."""
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd

    say("kron hadamard", D, dtype)
    g = torch.Generator().manual_seed(D)
    B, T, H = 2, 77, 3
    slab = torch.randn(B, T, H * D + 40, generator=g).to(dtype)
    signs = (torch.randint(0, 2, (H, D), generator=g) * 2 - 1).float()
    view = slab.to(cuda)[..., 8:8 + H * D].view(B, T, H, D)  # row stride H*D + 40, 16-byte aligned start
    y = kronecker_hadamard_fwd(view, signs.to(cuda), H)
    torch.cuda.synchronize()
    assert y.dtype == dtype and y.shape == (B, T, H, D) and y.is_contiguous()
    x = slab[..., 8:8 + H * D].reshape(B, T, H, D)
    if dtype == torch.bfloat16:
        ref = O.kron_hadamard(x.float().numpy(), npy(signs), bf16=True)
        assert np.array_equal(y.float().cpu().numpy().view(np.uint32), ref.view(np.uint32))
    else:
        ref = O.kron_hadamard(npy(x), npy(signs))
        assert np.array_equal(npy(y).view(np.uint16), ref.view(np.uint16))
    # orthogonality: rotating twice with unit signs returns the row (H2 (x) H_{D/2} is symmetric), to half precision
    ones = torch.ones(H, D, device=cuda)
    back = kronecker_hadamard_fwd(kronecker_hadamard_fwd(view, ones, H), ones, H)
    assert (back.float() - view.float()).abs().max().item() <= (0.08 if dtype == torch.bfloat16 else 0.02)


def test_prologue_dqk_and_no_rotation(cuda):
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC, prepare_dqk

    s = Mamba2Shape(batch=2, seqlen=203, nheads=2, headdim=64, dstate=128, ngroups=2, chunk=64)  # T not a multiple of 16
    say("prologue dqk / no rotation", s)
    g = torch.Generator().manual_seed(11)
    xBC = torch.randn(s.batch, s.seqlen, s.xbc_dim, generator=g).half()
    signs = (torch.randint(0, 2, (s.ngroups, s.dstate), generator=g) * 2 - 1).float()
    dq = torch.rand(s.ngroups, s.dstate, generator=g) + 0.5
    binv, cinv = torch.tensor([20.0, 35.0]), torch.tensor([28.0, 31.0])
    for use_signs, use_dqk in ((True, True), (False, False), (False, True)):
        _, qB, qC = fused_split_rotate_quant_xBC(xBC.to(cuda), signs.to(cuda) if use_signs else None, s.nheads, s.ngroups,
                                                 s.dstate, s.headdim, binv.to(cuda), cinv.to(cuda),
                                                 dqk_b=(1 / dq).half().to(cuda) if use_dqk else None, dqk_c=prepare_dqk(dq).to(cuda) if use_dqk else None)
        torch.cuda.synchronize()
        _, rB, rC = O.split_rotate_quant_xBC(npy(xBC), npy(signs) if use_signs else None, s.nheads, s.ngroups, s.dstate,
                                             s.headdim, npy(binv), npy(cinv),
                                             npy(prepare_dqk(1 / dq)) if use_dqk else None, npy(prepare_dqk(dq)) if use_dqk else None)
        assert_same_codes(qB, rB, f"q_B signs={use_signs} dqk={use_dqk}")
        assert_same_codes(qC, rC, f"q_C signs={use_signs} dqk={use_dqk}")


@pytest.mark.parametrize("keyside", [False, True])
def test_chunk_state(case, cuda, keyside):
    from linquant_amd.kernels.mamba2.chunk_state import _quant_chunk_state_fwd_xfp_static_int8
    from linquant_amd.kernels.mamba2.chunk_state_keyside import _chunk_state_keyside_fwd

    s = case["shape"]
    say("chunk_state", "key" if keyside else "value", s)
    xBC, _, p, sc = gpu_inputs(case, cuda)
    ref = case["oracle"][keyside]
    x = xBC[..., :s.d_ssm].view(s.batch, s.seqlen, s.nheads, s.headdim)
    dt, dA = dev(ref["dt"], cuda), dev(ref["dA_cumsum"], cuda)
    if keyside:
        st = _chunk_state_keyside_fwd(x, sc["x_scale_hp"], dev(ref["b_fp"], cuda), dt, dA, sc["static_state_scale"],
                                      sc["b_gate_scale"])
    else:
        st = _quant_chunk_state_fwd_xfp_static_int8(x, dev(ref["q_B"], cuda), dt, dA, sc["alpha_hp"], sc["bscale_g"],
                                                    sc["static_state_scale"])
    torch.cuda.synchronize()
    assert_same_codes(st, ref["states"], "states")


@pytest.mark.parametrize("regime", ["strong", "weak"])
def test_chunk_state_key_zero_slab_elision(cuda, regime):
    """Leaving out the slabs whose gated key codes are provably zero changes nothing: same states with the elision on
    and off, and against the oracle, also when the early tokens of every chunk carry keys large enough to saturate
    their codes (slabs that a decay-only rule would have dropped), when a key is infinite, and on a ragged tail."""
    from linquant_amd.kernels.mamba2.chunk_state_keyside import _chunk_state_keyside_fwd

    s = Mamba2Shape(batch=2, seqlen=1024, nheads=4, headdim=64, dstate=128, ngroups=2, chunk=256)
    say("zero-slab elision", regime, s)
    c = build_case(s, regime=regime)
    ref = oracle_pipeline(c, True)
    sc = {k: v.to(cuda) for k, v in c["scales"].items()}
    x = c["xBC"].to(cuda)[..., :s.d_ssm].view(s.batch, s.seqlen, s.nheads, s.headdim)
    dt, dA = dev(ref["dt"], cuda), dev(ref["dA_cumsum"], cuda)
    variants = {"as drawn": ref["b_fp"].copy()}
    big = ref["b_fp"].copy()
    big.reshape(s.batch, 4, 256, s.ngroups, s.dstate)[:, :, :64] *= np.float16(3000.0)   # first slab of every chunk
    variants["large early keys"] = big
    inf = ref["b_fp"].copy()
    inf[1, 300, 1, 7] = np.float16(np.inf)
    variants["an infinite key"] = inf
    for name, b_np in variants.items():
        b_fp = dev(b_np, cuda)
        on = _chunk_state_keyside_fwd(x, sc["x_scale_hp"], b_fp, dt, dA, sc["static_state_scale"], sc["b_gate_scale"])
        off = _chunk_state_keyside_fwd(x, sc["x_scale_hp"], b_fp, dt, dA, sc["static_state_scale"], sc["b_gate_scale"],
                                       elide_zero_slabs=False)
        torch.cuda.synchronize()
        assert torch.equal(on, off), f"{name}: the elision changed the states"
        if name != "an infinite key":  # (inf * 0 is NaN on both sides; its integer conversion is not specified)
            want = O.chunk_state_key(ref["x"], npy(sc["x_scale_hp"]), b_np, ref["dt"], ref["dA_cumsum"],
                                     npy(sc["static_state_scale"]), npy(sc["b_gate_scale"]))
            assert_same_codes(on, want, f"states ({name})")
    # ragged: 1000 of the 1024 tokens
    L = 1000
    dAr, dtr = O.chunk_cumsum(npy(c["dt_raw"])[:, :L], 1.0, npy(c["params"]["A_log"]), float(c["params"]["A_log_scale"]), 256,
                              None, True)
    xr = c["xBC"][:, :L].to(cuda)[..., :s.d_ssm].view(s.batch, L, s.nheads, s.headdim)
    on = _chunk_state_keyside_fwd(xr, sc["x_scale_hp"], dev(ref["b_fp"][:, :L], cuda), dev(dtr, cuda), dev(dAr, cuda),
                                  sc["static_state_scale"], sc["b_gate_scale"])
    want = O.chunk_state_key(ref["x"][:, :L], npy(sc["x_scale_hp"]), ref["b_fp"][:, :L], dtr, dAr,
                             npy(sc["static_state_scale"]), npy(sc["b_gate_scale"]))
    torch.cuda.synchronize()
    assert_same_codes(on, want, "states (ragged)")


def test_chunk_state_scalar_scales_and_ragged(cuda):
    """Per-head scalars passed as stride-0 (H,P) views, sequence length not a multiple of the chunk."""
    from linquant_amd.kernels.mamba2.chunk_state import _quant_chunk_state_fwd_xfp_static_int8

    s = Mamba2Shape(batch=1, seqlen=384, nheads=2, headdim=64, dstate=64, ngroups=1, chunk=128)
    say("chunk_state scalar scales + ragged", s)
    c = build_case(s)
    L = 300
    ref = oracle_pipeline(c, False)
    x = npy(c["xBC"])[:, :L, :s.d_ssm].reshape(1, L, 2, 64)
    qB = ref["q_B"][:, :L]
    dA, dt = O.chunk_cumsum(npy(c["dt_raw"])[:, :L], 1.0, npy(c["params"]["A_log"]), float(c["params"]["A_log_scale"]), 128,
                            None, True)
    alpha = npy(c["scales"]["alpha_hp"]).max(1, keepdims=True)
    sout = npy(c["scales"]["static_state_scale"]).max(1, keepdims=True)
    rs = O.chunk_state_value(x, qB, dt, dA, np.broadcast_to(alpha, (2, 64)), npy(c["scales"]["bscale_g"]),
                             np.broadcast_to(sout, (2, 64)))
    xg = c["xBC"][:, :L].to(cuda)[..., :s.d_ssm].view(1, L, 2, 64)
    st = _quant_chunk_state_fwd_xfp_static_int8(xg, dev(qB, cuda), dev(dt, cuda), dev(dA, cuda),
                                                dev(alpha, cuda).expand(2, 64), c["scales"]["bscale_g"].to(cuda),
                                                dev(sout, cuda).expand(2, 64))
    torch.cuda.synchronize()
    assert_same_codes(st, rs, "states (scalar scales, ragged)")


@pytest.mark.parametrize("sign_dtype", [torch.float32, torch.float16, torch.int8])
@pytest.mark.parametrize("offset", [0, 1])
def test_prologue_sign_dtypes_and_alignment(cuda, sign_dtype, offset):
    """Signs in each accepted dtype, 16-byte aligned (fetched as whole pieces) and one element off (element-wise path),
    with and without dqk: same codes as the oracle either way."""
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC, prepare_dqk

    s = Mamba2Shape(batch=1, seqlen=77, nheads=2, headdim=64, dstate=128, ngroups=2, chunk=64)
    say("prologue sign dtype / alignment", sign_dtype, offset)
    g = torch.Generator().manual_seed(23)
    xBC = torch.randn(s.batch, s.seqlen, s.xbc_dim, generator=g).half()
    signs = (torch.randint(0, 2, (s.ngroups, s.dstate), generator=g) * 2 - 1).float()
    dq = torch.rand(s.ngroups, s.dstate, generator=g) + 0.5
    binv, cinv = torch.tensor([20.0, 35.0]), torch.tensor([28.0, 31.0])

    def shifted(t):  # the same values in a buffer whose data pointer is `offset` elements past a 256-byte boundary
        buf = torch.empty(t.numel() + offset, dtype=t.dtype, device=cuda)
        view = buf[offset:].view(t.shape)
        view.copy_(t)
        return view

    for use_dqk in (False, True):
        sg = shifted(signs.to(sign_dtype).to(cuda))
        kw = {}
        if use_dqk:
            kw = {"dqk_b": shifted((1 / dq).half().to(cuda)), "dqk_c": shifted(prepare_dqk(dq).to(cuda))}
        _, qB, qC = fused_split_rotate_quant_xBC(xBC.to(cuda), sg, s.nheads, s.ngroups, s.dstate, s.headdim, binv.to(cuda),
                                                 cinv.to(cuda), **kw)
        torch.cuda.synchronize()
        _, rB, rC = O.split_rotate_quant_xBC(npy(xBC), npy(signs), s.nheads, s.ngroups, s.dstate, s.headdim, npy(binv), npy(cinv),
                                             npy(prepare_dqk(1 / dq)) if use_dqk else None, npy(prepare_dqk(dq)) if use_dqk else None)
        assert_same_codes(qB, rB, f"q_B {sign_dtype} offset={offset} dqk={use_dqk}")
        assert_same_codes(qC, rC, f"q_C {sign_dtype} offset={offset} dqk={use_dqk}")


@pytest.mark.parametrize("dim,shift,nc", [(8192, 7, 32), (4096 + 16, 7, 5), (1000, 7, 9), (999, 5, 3), (64 * 64, 7, 1), (2048, 7, 8),
                                          (2048, 6, 16)])
def test_state_passing(cuda, dim, shift, nc):
    from linquant_amd.kernels.mamba2.state_passing import _fixedpoint_state_passing_fwd

    say("state_passing", dim, shift, nc)
    rng = np.random.default_rng(dim + nc)
    B, H = 2, 3
    states = rng.integers(-128, 128, size=(B, nc, H, dim)).astype(np.int8)
    dA_full = -rng.random((B, H, nc, 4)).astype(np.float32) * 3
    dA_full[0, 0] = 0.0
    dA_full[1, 1] = -200.0
    dA_g = dev(dA_full, cuda)
    out, fin = _fixedpoint_state_passing_fwd(dev(states, cuda), dA_g[..., -1], gate_shift=shift)
    torch.cuda.synchronize()
    rout, rfin = O.state_passing(states, dA_full[..., -1], shift)
    assert_same_codes(out, rout, "passed")
    assert_same_codes(fin, rfin, "final")


@pytest.mark.parametrize("nc", [32, 5, 1])
def test_state_passing_in_place(cuda, nc):
    """The in-place form used by the one-call forward: one buffer of nc + 1 slots, slot c + 1 holding the local state
    of chunk c on entry and the state entering chunk c + 1 on return; heads whose gates all quantize to zero are left
    untouched (their slots are already right), heads with live gates run the full recurrence."""
    from linquant_amd import _lib

    say("state_passing in place", nc)
    rng = np.random.default_rng(nc)
    B, H, dim = 2, 4, 4096
    states = rng.integers(-127, 128, size=(B, nc, H, dim)).astype(np.int8)
    dA = -rng.random((B, H, nc)).astype(np.float32) * 3
    dA[:, 0] = -200.0                      # every gate of head 0 is zero
    dA[0, 1, : max(nc - 1, 1)] = -200.0    # all but the last gate of (0, 1) are zero
    slots = torch.zeros(B, nc + 1, H, dim, dtype=torch.int8, device=cuda)
    slots[:, 0] = 77                       # garbage in the zero slot on entry
    slots[:, 1:] = dev(states, cuda)
    fin = torch.empty(B, H, dim, dtype=torch.int8, device=cuda)
    dAg = dev(dA, cuda)
    st = slots[:, 1:]
    _lib.call("lq_state_passing", slots.device, states=_lib.ptr(st), states_stride_b=st.stride(0), states_stride_c=st.stride(1),
              states_stride_h=st.stride(2), states_stride_d=1, dA_chunk_cumsum=_lib.ptr(dAg), dA_stride_b=dAg.stride(0),
              dA_stride_h=dAg.stride(1), dA_stride_c=dAg.stride(2), out=_lib.ptr(slots), out_stride_b=slots.stride(0),
              out_stride_c=slots.stride(1), out_stride_h=slots.stride(2), out_stride_d=1, final_states=_lib.ptr(fin),
              final_stride_b=fin.stride(0), final_stride_h=fin.stride(1), final_stride_d=1, batch=B, nchunks=nc, nheads=H,
              dim=dim, gate_shift=7, vec_hint=0, in_place=1)
    torch.cuda.synchronize()
    rout, rfin = O.state_passing(states, dA, 7)
    assert_same_codes(slots[:, :nc], rout, "passed (slots 0 .. nc-1)")
    assert_same_codes(fin, rfin, "final")


def test_state_passing_noncontiguous(cuda):
    from linquant_amd.kernels.mamba2.state_passing import _fixedpoint_state_passing_fwd

    say("state_passing non-contiguous")
    rng = np.random.default_rng(0)
    wide = rng.integers(-127, 128, size=(2, 6, 3, 200)).astype(np.int8)
    dA = -rng.random((2, 3, 6)).astype(np.float32)
    view = dev(wide, cuda)[..., 7:107:2]  # stride 2 on the state axis -> generic kernel
    out, fin = _fixedpoint_state_passing_fwd(view, dev(dA, cuda))
    torch.cuda.synchronize()
    rout, rfin = O.state_passing(np.ascontiguousarray(wide[..., 7:107:2]), dA)
    assert_same_codes(out, rout, "passed")
    assert_same_codes(fin, rfin, "final")


def test_documented_binding_example_runs(cuda, monkeypatch):
    """The stand-alone ctypes binding shown in the integration notes, executed as written, gives the wrapper's result."""
    from linquant_amd.kernels.mamba2.state_passing import _fixedpoint_state_passing_fwd
    from tests.test_abi import ROOT, binding_example

    say("documented ctypes binding of lq_state_passing")
    monkeypatch.chdir(ROOT)
    ns = {}
    exec(compile(binding_example(), "binding_example", "exec"), ns)
    rng = np.random.default_rng(1)
    states = dev(rng.integers(-128, 128, size=(2, 5, 3, 512)).astype(np.int8), cuda)
    dA = dev(-rng.random((2, 3, 5)).astype(np.float32), cuda)
    out, fin = ns["_fixedpoint_state_passing_fwd"](states, dA)
    rout, rfin = _fixedpoint_state_passing_fwd(states, dA)
    torch.cuda.synchronize()
    assert torch.equal(out, rout) and torch.equal(fin, rfin)


@pytest.mark.parametrize("keyside", [False, True])
def test_bmm_chunk(case, cuda, keyside):
    from linquant_amd.kernels.mamba2.bmm_chunk import _quant_bmm_chunk_fwd

    s = case["shape"]
    say("bmm_chunk", "key" if keyside else "value", s)
    _, _, _, sc = gpu_inputs(case, cuda)
    ref = case["oracle"][keyside]
    b = dev(ref["b_fp"], cuda) if keyside else dev(ref["q_B"], cuda)
    cb = _quant_bmm_chunk_fwd(dev(ref["q_C"], cuda), sc["C_scale"], b, sc["B_scale"], s.chunk, sc["static_cb_scale"],
                              b_is_fp=keyside)
    torch.cuda.synchronize()
    assert_same_codes(cb, ref["cb"], "cb")


@pytest.mark.parametrize("keyside_rowmax", [True])
def test_prologue_row_maxima_feed_the_chunk_state(case, cuda, keyside_rowmax):
    """The prologue's fifth output, max_n |b_fp| per token row, is exactly that maximum; handed to the key-side chunk state
    (alone or through the combined forward) it replaces the stage's own pre-pass: same states, same output, bit for bit."""
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.chunk_state_keyside import _chunk_state_keyside_fwd
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    s = case["shape"]
    say("prologue row maxima", s)
    xBC, dt_raw, p, sc = gpu_inputs(case, cuda)
    x, qB, qC, b_fp, rmax = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                                         sc["B_inv_scale"], sc["C_inv_scale"], return_b_fp=True,
                                                         return_b_rowmax=True)
    torch.cuda.synchronize()
    assert rmax.shape == (s.batch, s.seqlen, s.ngroups) and rmax.dtype == torch.float32
    assert torch.equal(rmax, b_fp.float().abs().amax(dim=-1))
    ref = case["oracle"][True]
    dt, dA = dev(ref["dt"], cuda), dev(ref["dA_cumsum"], cuda)
    st0 = _chunk_state_keyside_fwd(x, sc["x_scale_hp"], b_fp, dt, dA, sc["static_state_scale"], sc["b_gate_scale"])
    st1 = _chunk_state_keyside_fwd(x, sc["x_scale_hp"], b_fp, dt, dA, sc["static_state_scale"], sc["b_gate_scale"], b_rowmax=rmax)
    torch.cuda.synchronize()
    assert torch.equal(st0, st1)
    assert_same_codes(st1, ref["states"], "states")
    kw = dict(dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
              static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], keyside=True,
              x_scale_hp=sc["x_scale_hp"], b_fp=b_fp, b_gate_scale=sc["b_gate_scale"])
    args = (x, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk, p["D"], p["D_scale"])
    o0 = M._quant_mamba_chunk_scan_combined_fwd(*args, **kw)[0]
    o1 = M._quant_mamba_chunk_scan_combined_fwd(*args, b_rowmax=rmax, **kw)[0]
    torch.cuda.synchronize()
    assert torch.equal(o0, o1)


@pytest.mark.parametrize("L,Q,G,N,fp", [(2000, 256, 64, 64, True), (2048, 256, 64, 128, False), (300, 128, 3, 192, True),
                                        (1000, 64, 5, 256, False)])
def test_bmm_chunk_shapes(cuda, L, Q, G, N, fp):
    """C.B^T with many and with few groups (both workgroup orders), ragged last chunks, both B dtypes and every state
    width, against the oracle's exact integer product."""
    from linquant_amd.kernels.mamba2.bmm_chunk import _quant_bmm_chunk_fwd

    say("bmm_chunk shapes", L, Q, G, N, fp)
    g = torch.Generator().manual_seed(3)
    qC = torch.randint(-127, 128, (1, L, G, N), generator=g, dtype=torch.int8)
    C_scale = torch.rand(G, generator=g) * 0.01 + 0.01
    B_scale = torch.rand(G, generator=g) * 0.01 + 0.01
    cb_scale = torch.rand(G, generator=g) * 0.5 + 0.5
    if fp:
        b = (torch.randn(1, L, G, N, generator=g) * B_scale.view(1, 1, G, 1) * 50).half()
    else:
        b = torch.randint(-127, 128, (1, L, G, N), generator=g, dtype=torch.int8)
    cb = _quant_bmm_chunk_fwd(qC.to(cuda), C_scale.to(cuda), b.to(cuda), B_scale.to(cuda), Q, cb_scale.to(cuda), b_is_fp=fp)
    torch.cuda.synchronize()
    ref = O.bmm_chunk(npy(qC), npy(C_scale), npy(b), npy(B_scale), Q, npy(cb_scale), b_is_fp=fp)
    assert_same_codes(cb, ref, "cb")


@pytest.mark.parametrize("keyside", [False, True])
def test_chunk_scan(case, cuda, keyside):
    from linquant_amd.kernels.mamba2.chunk_scan_v2 import _quant_chunk_scan_fwd

    s = case["shape"]
    say("chunk_scan", "key" if keyside else "value", s)
    xBC, _, p, sc = gpu_inputs(case, cuda)
    ref = case["oracle"][keyside]
    x = xBC[..., :s.d_ssm].view(s.batch, s.seqlen, s.nheads, s.headdim)
    out = _quant_chunk_scan_fwd(dev(ref["cb"], cuda), x, dev(ref["dt"], cuda), dev(ref["dA_cumsum"], cuda),
                                dev(ref["q_C"], cuda), sc["C_scale"], dev(ref["passed"], cuda), p["D"], p["D_scale"],
                                sc["static_state_scale"], sc["static_cb_scale"])
    torch.cuda.synchronize()
    assert out.dtype == torch.float16 and out.is_contiguous()
    assert_close_out(out, ref["out"], "out")
    # all heads of a group in one workgroup (small shapes default to one head per workgroup)
    outg = _quant_chunk_scan_fwd(dev(ref["cb"], cuda), x, dev(ref["dt"], cuda), dev(ref["dA_cumsum"], cuda),
                                 dev(ref["q_C"], cuda), sc["C_scale"], dev(ref["passed"], cuda), p["D"], p["D_scale"],
                                 sc["static_state_scale"], sc["static_cb_scale"], heads_per_workgroup=s.nheads // s.ngroups)
    torch.cuda.synchronize()
    assert torch.equal(outg, out)
    # without the D residual, with a per-(H,P) D and with a stride-0 state scale
    out2 = _quant_chunk_scan_fwd(dev(ref["cb"], cuda), x, dev(ref["dt"], cuda), dev(ref["dA_cumsum"], cuda),
                                 dev(ref["q_C"], cuda), sc["C_scale"], dev(ref["passed"], cuda), None, None,
                                 sc["static_state_scale"], sc["static_cb_scale"])
    r2 = O.chunk_scan(ref["cb"], ref["x"], ref["dt"], ref["dA_cumsum"], ref["q_C"], npy(sc["C_scale"]), ref["passed"],
                      None, None, npy(sc["static_state_scale"]), npy(sc["static_cb_scale"]))
    assert_close_out(out2, r2, "out (no D)")
    # a small static CB scale (the chunk scan is defined for any codes and scale): S_cb * dt ~ 1e-4 is at the edge of the
    # fp16 normal range, where the reference's own fp16 weights are still accurate for all but the smallest codes
    small = (sc["static_cb_scale"] * (1.37 * 2.0 ** -6)).contiguous()
    out3 = _quant_chunk_scan_fwd(dev(ref["cb"], cuda), x, dev(ref["dt"], cuda), dev(ref["dA_cumsum"], cuda),
                                 dev(ref["q_C"], cuda), sc["C_scale"], torch.zeros_like(dev(ref["passed"], cuda)), None, None,
                                 sc["static_state_scale"], small)
    r3 = O.chunk_scan(ref["cb"], ref["x"], ref["dt"], ref["dA_cumsum"], ref["q_C"], npy(sc["C_scale"]),
                      np.zeros_like(ref["passed"]), None, None, npy(sc["static_state_scale"]), npy(small))
    assert_close_out(out3, r3, "out (small S_cb, causal path only)")


def _random_scan_case(L, Q, H, G, P, N, B=2, seed=11):
    """Arbitrary codes and scales for the chunk scan alone (dt = 0 past the sequence end, as the cumsum stage writes it)."""
    g = torch.Generator().manual_seed(seed)
    nc = (L + Q - 1) // Q
    cb = torch.randint(-127, 128, (B, nc, G, Q, Q), generator=g, dtype=torch.int8)
    x = torch.randn(B, L, H, P, generator=g).half()
    dt = torch.rand(B, H, nc, Q, generator=g) * 0.05 + 0.001
    pos = torch.arange(nc * Q).view(nc, Q)
    dt = torch.where(pos < L, dt, torch.zeros(()))
    a = -(torch.rand(H, generator=g) * 4 + 0.5)
    dA = torch.cumsum(dt * a.view(1, H, 1, 1), dim=-1)
    qC = torch.randint(-127, 128, (B, L, G, N), generator=g, dtype=torch.int8)
    states = torch.randint(-127, 128, (B, nc, H, P, N), generator=g, dtype=torch.int8)
    D = torch.randint(-127, 128, (H,), generator=g, dtype=torch.int8)
    C_scale = torch.rand(G, generator=g) * 0.01 + 0.01
    ss = torch.rand(H, P, generator=g) * 0.01 + 0.01
    cbs = torch.rand(G, generator=g) * 0.02 + 0.02
    return (cb, x, dt, dA, qC, C_scale, states, D, torch.tensor(0.01), ss, cbs)


@pytest.mark.parametrize("L,Q,H,G,P,N", [(700, 512, 4, 2, 64, 256), (200, 64, 6, 2, 64, 192), (300, 128, 4, 4, 128, 256),
                                         (40, 64, 2, 1, 64, 64), (17, 256, 3, 3, 64, 128)])
def test_chunk_scan_wide_shapes(cuda, L, Q, H, G, P, N):
    """Chunk 512, state widths 192 / 256 and sequences shorter than one chunk against the oracle, one head per workgroup
    and all heads of a group."""
    from linquant_amd.kernels.mamba2.chunk_scan_v2 import _quant_chunk_scan_fwd

    say("chunk_scan wide", L, Q, H, G, P, N)
    case = _random_scan_case(L, Q, H, G, P, N, B=1, seed=5)
    cb, x, dt, dA, qC, C_scale, states, D, D_scale, ss, cbs = case
    ref = O.chunk_scan(npy(cb), npy(x), npy(dt), npy(dA), npy(qC), npy(C_scale), npy(states), npy(D), np.float32(0.01), npy(ss), npy(cbs))
    args = tuple(t.to(cuda) for t in case)
    for hint in (1, H // G):
        say("  heads_per_workgroup", hint)
        got = _quant_chunk_scan_fwd(*args, heads_per_workgroup=hint)
        torch.cuda.synchronize()
        assert_close_out(got, ref, f"out (hint {hint})")


@pytest.mark.parametrize("L,Q,H,G,P,N", [(600, 256, 16, 2, 64, 128), (200, 64, 12, 4, 128, 64), (1024, 128, 10, 1, 64, 64)])
def test_chunk_scan_heads_per_workgroup(cuda, L, Q, H, G, P, N):
    """A workgroup of the chunk scan walks several heads of one group; how many is a scheduling choice (made from the grid
    size, so small shapes get one).  Every choice, including ones that leave a shorter last part, gives the same bits, on
    ragged last chunks too; and the one-head form is what test_chunk_scan holds against the oracle."""
    from linquant_amd.kernels.mamba2.chunk_scan_v2 import _quant_chunk_scan_fwd

    say("chunk_scan heads per workgroup", L, Q, H, G, P, N)
    args = tuple(t.to(cuda) for t in _random_scan_case(L, Q, H, G, P, N))
    one = _quant_chunk_scan_fwd(*args, heads_per_workgroup=1)
    torch.cuda.synchronize()
    assert torch.isfinite(one).all()
    hpg = H // G
    for hint in sorted({0, 2, 3, hpg - 1, hpg, hpg + 5} - {1}):
        say("  heads_per_workgroup", hint)
        got = _quant_chunk_scan_fwd(*args, heads_per_workgroup=hint)
        torch.cuda.synchronize()
        assert torch.equal(got, one), f"heads_per_workgroup={hint}"


@pytest.mark.parametrize("keyside", [False, True])
def test_pipeline_end_to_end(case, cuda, keyside):
    """The drop-in path a caller takes: prologue -> (rotation of fp B) -> combined forward."""
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    s = case["shape"]
    say("pipeline", "key" if keyside else "value", s)
    xBC, dt_raw, p, sc = gpu_inputs(case, cuda)
    x, qB, qC = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                             sc["B_inv_scale"], sc["C_inv_scale"])
    kw = {}
    if keyside:
        gn = s.ngroups * s.dstate
        b_fp = xBC[..., s.d_ssm:s.d_ssm + gn].reshape(s.batch, s.seqlen, s.ngroups, s.dstate).contiguous()
        kw = dict(keyside=True, x_scale_hp=sc["x_scale_hp"], b_fp=kronecker_hadamard_fwd(b_fp, p["r_signs"], s.ngroups),
                  b_gate_scale=sc["b_gate_scale"])
    seen = {}
    orig_sp, orig_scan = M._fixedpoint_state_passing_fwd, M._chunk_scan_v2

    def spy_sp(states, dA, gate_shift=7):  # the stage names are re-bindable module attributes
        seen["states"] = states
        r = orig_sp(states, dA, gate_shift=gate_shift)
        seen["passed"] = r[0]
        return r

    def spy_scan(cb, *a):
        seen["cb"] = cb
        return orig_scan(cb, *a)

    M._fixedpoint_state_passing_fwd, M._chunk_scan_v2 = spy_sp, spy_scan
    try:
        out, none = M._quant_mamba_chunk_scan_combined_fwd(
            x, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk,
            p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
            static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], **kw)
    finally:
        M._fixedpoint_state_passing_fwd, M._chunk_scan_v2 = orig_sp, orig_scan
    torch.cuda.synchronize()
    ref = case["oracle"][keyside]
    assert none is None
    assert_same_codes(seen["states"].reshape(ref["states"].shape), ref["states"], "states")
    assert_same_codes(seen["passed"].reshape(ref["passed"].shape), ref["passed"], "passed")
    assert_same_codes(seen["cb"], ref["cb"], "cb")
    assert_close_out(out, ref["out"], "out")


@pytest.mark.parametrize("keyside", [False, True])
def test_one_call_equals_stage_by_stage(case, cuda, keyside):
    """With no stage re-bound the combined forward is one C call (lq_ssd_combined) over one workspace; it must give
    the stage-by-stage path's output bit for bit (same kernels, same order)."""
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    s = case["shape"]
    say("one call vs staged", "key" if keyside else "value", s)
    xBC, dt_raw, p, sc = gpu_inputs(case, cuda)
    x, qB, qC = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                             sc["B_inv_scale"], sc["C_inv_scale"])
    kw = {}
    if keyside:
        gn = s.ngroups * s.dstate
        b_fp = xBC[..., s.d_ssm:s.d_ssm + gn].reshape(s.batch, s.seqlen, s.ngroups, s.dstate).contiguous()
        kw = dict(keyside=True, x_scale_hp=sc["x_scale_hp"], b_fp=kronecker_hadamard_fwd(b_fp, p["r_signs"], s.ngroups),
                  b_gate_scale=sc["b_gate_scale"])

    def fwd():
        return M._quant_mamba_chunk_scan_combined_fwd(
            x, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk,
            p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
            static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], **kw)[0]

    assert not M._stages_rebound()
    one = fwd()
    orig = M._chunk_scan_v2
    M._chunk_scan_v2 = lambda *a: orig(*a)  # any re-bound stage selects the stage-by-stage path
    try:
        assert M._stages_rebound()
        staged = fwd()
    finally:
        M._chunk_scan_v2 = orig
    torch.cuda.synchronize()
    assert torch.equal(one, staged)
    assert_close_out(one, case["oracle"][keyside]["out"], "out (one call)")


def test_hip_graph_capture_and_replay(cuda):
    """The whole key-side step (prologue + combined forward: seven launches, no allocation or synchronisation inside
    the library) captured once in a HIP graph and replayed: every replay must equal the eager result bit for bit, with
    eager work and synchronisations between the replays and with new input values written into the captured buffers."""
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    s = Mamba2Shape(batch=2, seqlen=1024, nheads=8, headdim=64, dstate=128, ngroups=1, chunk=256)
    say("HIP graph capture", s)
    c = build_case(s)
    p = {k: v.to(cuda) for k, v in c["params"].items()}
    sc = {k: v.to(cuda) for k, v in c["scales"].items()}
    xBC, dt_raw = c["xBC"].to(cuda), c["dt_raw"].to(cuda)

    def step():
        x, qB, qC, b_fp = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                                       sc["B_inv_scale"], sc["C_inv_scale"], return_b_fp=True)
        return M._quant_mamba_chunk_scan_combined_fwd(
            x, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk,
            p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
            static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], keyside=True,
            x_scale_hp=sc["x_scale_hp"], b_fp=b_fp, b_gate_scale=sc["b_gate_scale"])[0]

    eager = step().clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    torch.cuda.synchronize()
    for i in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager), f"replay {i} differs from the eager result"
        again = step()  # eager work of the program itself between replays
        torch.cuda.synchronize()
        assert torch.equal(again, eager)
    other = build_case(s, seed=5)
    xBC.copy_(other["xBC"].to(cuda))
    dt_raw.copy_(other["dt_raw"].to(cuda))
    eager2 = step().clone()
    torch.cuda.synchronize()
    assert not torch.equal(eager2, eager)
    for i in range(2):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, eager2), f"replay {i} on new inputs differs from the eager result"


def test_full_size_config5_slices(cuda):
    """Mamba-2 2.7B-shape layer (B4 L8192 H80 P64 N128 Q256) on the GPU; every integer stage is checked
    bit-exactly against the oracle on head / batch slices the oracle finishes in seconds, the output on the
    same slices, and state passing additionally through its zero-gate and copy properties at full size."""
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC
    from linquant_amd.kernels.mamba2.state_passing import _fixedpoint_state_passing_fwd
    from linquant_amd.calibration import calibrate_mamba2, mamba2_params, mamba2_synthetic

    s = Mamba2Shape(batch=4, seqlen=8192, nheads=80, headdim=64, dstate=128, ngroups=1, chunk=256)
    say("full size", s)
    p = mamba2_params(s, 42, cuda)
    cal = Mamba2Shape(batch=1, seqlen=2048, nheads=80, headdim=64, dstate=128, ngroups=1, chunk=256)
    cx, cdt = mamba2_synthetic(cal, 1, cuda)
    sc = calibrate_mamba2(cal, cx, cdt, p)
    del cx, cdt
    xBC, dt_raw = mamba2_synthetic(s, 0, cuda)
    x, qB, qC = fused_split_rotate_quant_xBC(xBC, p["r_signs"], 80, 1, 128, 64, sc["B_inv_scale"], sc["C_inv_scale"])
    b_fp = kronecker_hadamard_fwd(xBC[..., s.d_ssm:s.d_ssm + 128].view(4, 8192, 1, 128), p["r_signs"], 1)
    seen = {}
    orig_sp = M._fixedpoint_state_passing_fwd

    def spy_sp(states, dA, gate_shift=7):
        r = orig_sp(states, dA, gate_shift=gate_shift)
        seen["states"], seen["passed"], seen["dA_last"] = states, r[0], dA
        return r

    M._fixedpoint_state_passing_fwd = spy_sp
    outs = {}
    try:
        for keyside in (False, True):
            kw = dict(keyside=True, x_scale_hp=sc["x_scale_hp"], b_fp=b_fp, b_gate_scale=sc["b_gate_scale"]) if keyside else {}
            out, _ = M._quant_mamba_chunk_scan_combined_fwd(
                x, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk,
                p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
                static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], **kw)
            torch.cuda.synchronize()
            outs[keyside] = (out, seen["states"], seen["passed"])
    finally:
        M._fixedpoint_state_passing_fwd = orig_sp
    # the route the benchmark times, exactly as bench.py's step() calls it: nothing re-bound (one C call, state passing in
    # place with its zero-gate early exit), rotated fp16 B and its per-token maxima from the prologue's own launch.  It
    # must equal, bit for bit, the stage-by-stage key-side output that is checked against the oracle below.
    say("full size, one-call route as benchmarked")
    x1, qB1, qC1, b_fp1, b_rmax = fused_split_rotate_quant_xBC(xBC, p["r_signs"], 80, 1, 128, 64, sc["B_inv_scale"],
                                                               sc["C_inv_scale"], return_b_fp=True, return_b_rowmax=True)
    assert torch.equal(qB1, qB) and torch.equal(qC1, qC) and torch.equal(b_fp1, b_fp)
    out1, _ = M._quant_mamba_chunk_scan_combined_fwd(
        x1, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB1, sc["B_scale"], qC1, sc["C_scale"], s.chunk,
        p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
        static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], keyside=True,
        x_scale_hp=sc["x_scale_hp"], b_fp=b_fp1, b_gate_scale=sc["b_gate_scale"], b_rowmax=b_rmax)
    torch.cuda.synchronize()
    assert torch.equal(out1, outs[True][0]), "one-call route differs from the stage-by-stage route at full size"
    del x1, qB1, qC1, b_fp1, b_rmax, out1
    # oracle on slices: batch b, heads hs
    for keyside, b, hs in ((False, 0, [0, 79]), (True, 3, [17, 42])):
        say("full size slice check", keyside, b, hs)
        out, states, passed = outs[keyside]
        hsel = torch.tensor(hs, device=cuda)
        xs = npy(x[b:b + 1][:, :, hsel])
        sub = lambda t: npy(t[hsel])  # noqa: E731
        r = O.ssd_combined(xs, npy(dt_raw[b:b + 1][:, :, hsel]), 1.0, sub(p["A_log"]), float(p["A_log_scale"]),
                           npy(qB[b:b + 1]), npy(sc["B_scale"]), npy(qC[b:b + 1]), npy(sc["C_scale"]), 256, sub(p["D"]),
                           float(p["D_scale"]), dt_bias=sub(p["dt_bias"]), dt_softplus=True,
                           static_state_scale=sub(sc["static_state_scale"]), static_cb_scale=npy(sc["static_cb_scale"]),
                           alpha_hp=sub(sc["alpha_hp"]), bscale_g=npy(sc["bscale_g"]), keyside=keyside,
                           x_scale_hp=sub(sc["x_scale_hp"]), b_fp=npy(b_fp[b:b + 1]),
                           b_gate_scale=npy(sc["b_gate_scale"][:, :, hsel]))
        st = states.view(4, 32, 80, 64, 128)[b:b + 1][:, :, hsel]
        ps = passed.view(4, 32, 80, 64, 128)[b:b + 1][:, :, hsel]
        assert_same_codes(st, r["states"], "states slice")
        assert_same_codes(ps, r["passed"], "passed slice")
        assert_close_out(out[b:b + 1][:, :, hsel], r["out"], "out slice")
    # size-independent properties of state passing at full size
    states = outs[True][1]
    zero_gate = torch.full((4, 80, 32), -200.0, device=cuda)
    o, f = _fixedpoint_state_passing_fwd(states, zero_gate)
    torch.cuda.synchronize()
    assert torch.equal(o[:, 1:], states[:, :-1].clamp(-127, 127)) and torch.equal(f, states[:, -1].clamp(-127, 127))
    assert int(o[:, 0].abs().max()) == 0


@pytest.mark.parametrize("with_dqk", [False, True])
def test_prologue_also_returns_rotated_fp_b(case, cuda, with_dqk):
    """The optional fourth output of the prologue equals the separate rotation of the [dqk-scaled] B lanes bit for bit,
    and leaves the three reference outputs unchanged."""
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    s = case["shape"]
    xBC, dt_raw, p, sc = gpu_inputs(case, cuda)
    gn = s.ngroups * s.dstate
    kw = {}
    if with_dqk:
        gen = torch.Generator().manual_seed(5)
        from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import prepare_dqk
        kw = dict(dqk_b=prepare_dqk((0.5 + torch.rand(gn, generator=gen)).cuda()),      # fp16-rounded values, as the mixer holds them
                  dqk_c=prepare_dqk((0.5 + torch.rand(gn, generator=gen)).cuda()))
    x3, qB3, qC3 = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                                sc["B_inv_scale"], sc["C_inv_scale"], **kw)
    x4, qB4, qC4, b_fp = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                                      sc["B_inv_scale"], sc["C_inv_scale"], return_b_fp=True, **kw)
    b_lanes = xBC[..., s.d_ssm:s.d_ssm + gn]
    if with_dqk:
        b_lanes = b_lanes * kw["dqk_b"].to(xBC.dtype)
    ref = kronecker_hadamard_fwd(b_lanes.reshape(s.batch, s.seqlen, s.ngroups, s.dstate).contiguous(), p["r_signs"], s.ngroups)
    torch.cuda.synchronize()
    assert torch.equal(qB3, qB4) and torch.equal(qC3, qC4) and x4.data_ptr() == x3.data_ptr()
    assert b_fp.shape == ref.shape and torch.equal(b_fp, ref)
