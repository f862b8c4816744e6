"""GPU parity of the zoo operand prologue (lq_zoo_rotate_qkv through the C ABI) against the float64 oracle
(oracle.zoo_reference.rotate_operands: products with signed_hadamard matrices, D_QK of the reference's harness)."""

import pytest
import torch

from oracle import zoo_reference as Z
from tests import zoo_cases as zc

pytestmark = pytest.mark.gpu


def ulp_distance(a, b):
    """Distance in units of the 16-bit format between two tensors of the same half-precision dtype (same-sign or zero)."""
    ia, ib = a.view(torch.int16).int(), b.view(torch.int16).int()
    key = lambda i: torch.where(i < 0, -(i & 0x7fff), i)  # noqa: E731  sign-magnitude -> monotone integer
    return (key(ia) - key(ib)).abs()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("K,V", [(128, 128), (64, 128), (128, 64), (64, 64)])
@pytest.mark.parametrize("use_dqk", [False, True])
def test_rotate_qkv_matches_oracle(cuda, dtype, K, V, use_dqk):
    """Rotated rows equal the oracle's except where the fp32 transform and the float64 product round apart at a
    half-precision boundary: never more than one unit in the last place, fewer than 2e-3 of the elements; the D_QK
    scaling alone (one fp32 product, rounded once) is bit-exact."""
    from linquant_amd.kernels.zoo import rotate_qkv, rotation_signs

    print("[case] rotate_qkv", dtype, K, V, use_dqk, flush=True)
    gen = torch.Generator().manual_seed(K + V)
    B, T, H = 2, 203, 3  # row count not a multiple of the rows per workgroup
    q, k = torch.randn(B, T, H, K, generator=gen).to(dtype), torch.randn(B, T, H, K, generator=gen).to(dtype)
    v = torch.randn(B, T, H, V, generator=gen).to(dtype)
    D = (torch.rand(H, K, generator=gen) + 0.5) if use_dqk else None
    R, Rv = Z.signed_hadamard(K, 1), Z.signed_hadamard(V, 2)
    sq, sv = rotation_signs(R.to(cuda)), rotation_signs(Rv.to(cuda))
    got = rotate_qkv(q.to(cuda), k.to(cuda), v.to(cuda), signs_qk=sq, signs_v=sv, dqk=None if D is None else D.to(cuda))
    torch.cuda.synchronize()
    ref = Z.rotate_operands(q, k, v, R, Rv, D)
    for name, g, r in zip("qkv", got, ref):
        assert g.dtype == dtype and g.shape == r.shape
        d = ulp_distance(g.cpu(), r)
        # a sum that cancels to almost nothing has no meaningful last place: there the fp32 transform is held to its own
        # absolute accuracy instead (1e-6 on rows of N(0,1) entries)
        d = torch.where((g.cpu().float() - r.float()).abs() <= 1e-6, torch.zeros_like(d), d)
        rate = (d != 0).float().mean().item()
        print(f"[rotate] {name}: {rate:.2e} of the elements one unit apart, max {int(d.max())}", flush=True)
        assert d.max().item() <= 1 and rate < 2e-3, (name, int(d.max()), rate)
    if use_dqk:  # scaling without rotation: exact; tensors left out are skipped; in place
        qd, kd, none = rotate_qkv(q.to(cuda), k.to(cuda), None, dqk=D.to(cuda))
        rq, rk, _ = Z.rotate_operands(q, k, v, None, None, D)
        assert none is None and torch.equal(qd.cpu(), rq) and torch.equal(kd.cpu(), rk)
        vv = v.to(cuda).clone()
        rotate_qkv(None, None, vv, signs_v=sv, out=(None, None, vv))
        torch.cuda.synchronize()
        assert torch.equal(vv, got[2])


@pytest.mark.parametrize("cell", ["linear_none", "gated_deltanet"])
def test_prologue_then_kernel_matches_oracle_with_rotation(cuda, cell):
    """The whole drop-in path of a persistent R_QK: prologue kernel, then the chunk kernels on its output, against the
    oracle called with rot_qk (which rotates on entry itself)."""
    from linquant_amd.kernels.zoo import rotate_qkv, rotation_signs

    tensors = zc.cut(zc.inputs(cell, K=128, H=2, seed=12), 256)
    R = Z.signed_hadamard(128, 1)
    qz, run = zc.calibrated(cell, tensors, rot_qk=R)
    q, k, v, g, beta = tensors
    qr, kr, _ = rotate_qkv(q.to(cuda), k.to(cuda), None, signs_qk=rotation_signs(R.to(cuda)))
    fam = zc.CELLS[cell][0]
    sc = qz.kernel_scales(0, 2, 128, 128, delta=fam == "delta")
    out, _ = zc.run_kernel(cell, (qr, kr, v, g, beta), sc)
    torch.cuda.synchronize()
    zc.check(out, run, qz, f"{cell} prologue + kernel")


def test_rotate_qkv_rejections(cuda):
    from linquant_amd import _lib
    from linquant_amd.kernels.zoo import rotate_qkv

    q = torch.zeros(1, 64, 2, 96, dtype=torch.float16, device=cuda)
    with pytest.raises(AssertionError):
        rotate_qkv(q, q, None)
    q = torch.zeros(1, 64, 2, 64, dtype=torch.float32, device=cuda)
    with pytest.raises(AssertionError):
        rotate_qkv(q, q, None)
    with pytest.raises(_lib.LinQuantHipError):
        _lib.call("lq_zoo_rotate_qkv", q.device, batch=1, seqlen=1, nheads=1, kdim=64, vdim=64)


@pytest.mark.parametrize("cell", ["linear_none", "mamba2"])
@pytest.mark.parametrize("K,V,dtype,use_dqk,rot_v,eta,bits", [
    (128, 128, torch.float16, False, False, 1.0, 8),   # the benchmark's linear-attention call: R_QK on q, k only
    (128, 128, torch.float16, True, True, 0.5, 8),
    (64, 128, torch.bfloat16, False, True, 1.0, 8),
    (128, 64, torch.float16, True, False, 0.0, 6),
    (64, 64, torch.bfloat16, True, True, 0.25, 8),
])
def test_fused_prologue_equals_rotation_then_call(cuda, cell, K, V, dtype, use_dqk, rot_v, eta, bits):
    """chunk_simple_gla_int8(..., prologue=...) (one launch rotates, rescales and quantizes every operand; the output
    kernel reads codes) against rotate_qkv followed by the plain call: outputs, final state, stored state codes and the
    write codes are the same bits; the rotated activations it can export equal rotate_qkv's."""
    from linquant_amd.kernels import zoo

    print("[case] fused prologue", cell, K, V, dtype, use_dqk, rot_v, eta, bits, flush=True)
    H = 3
    q, k, v, g, _ = zc.cut(zc.inputs(cell, B=2, H=H, K=K, V=V, seed=17, dtype=dtype), 192)
    gen = torch.Generator().manual_seed(6)
    D = (torch.rand(H, K, generator=gen) + 0.5).to(cuda) if use_dqk else None
    sq = zoo.rotation_signs(Z.signed_hadamard(K, 1).to(cuda))
    sv = zoo.rotation_signs(Z.signed_hadamard(V, 2).to(cuda)) if rot_v else None
    sc = {"q": torch.rand(H, generator=gen) * 0.002 + 0.001, "k": torch.rand(H, generator=gen) * 0.01 + 0.005,
          "kw": torch.rand(H, K, generator=gen) * 0.01 + 0.004, "vw": torch.rand(H, V, generator=gen) * 0.02 + 0.02,
          "vl": torch.rand(H, V, generator=gen) * 0.02 + 0.02, "state": torch.rand(H, V, generator=gen) * 0.05 + 0.02}
    sc = {n: t.to(cuda) for n, t in sc.items()}
    dev = lambda t: None if t is None else t.to(cuda)  # noqa: E731
    kw = dict(eta=eta, scale=K ** -0.5, bits=bits, output_final_state=True)
    qr, kr, vr = zoo.rotate_qkv(dev(q), dev(k), dev(v), signs_qk=sq, signs_v=sv, dqk=D)
    d0, d1 = {}, {}
    o0, h0 = zoo.chunk_simple_gla_int8(qr, kr, vr, dev(g), sc, _debug=d0, **kw)
    o1, h1 = zoo.chunk_simple_gla_int8(dev(q), dev(k), dev(v), dev(g), sc, prologue=dict(signs_qk=sq, signs_v=sv, dqk=D),
                                       _debug=d1, **kw)
    o2, h2 = zoo.chunk_simple_gla_int8(dev(q), dev(k), dev(v), dev(g), sc, prologue=dict(signs_qk=sq, signs_v=sv, dqk=D), **kw)
    torch.cuda.synchronize()
    assert torch.isfinite(o0.float()).all() and float(o0.float().abs().max()) > 0
    assert torch.equal(o0, o1) and torch.equal(h0, h1), "fused prologue differs from rotation followed by the call"
    assert torch.equal(o0, o2) and torch.equal(h0, h2), "fused prologue without the exported activations differs"
    for name in ("h_i8", "kq", "vq"):
        assert torch.equal(d0[name], d1[name]), name
    for got, ref in zip(d1["rotated"], (qr, kr, vr)):
        assert torch.equal(got, ref)
    qmax = 2 ** (bits - 1) - 1
    assert all(int(c.abs().max()) <= qmax for c in d1["local"]) and int(d1["local"][1].abs().max()) > qmax // 4


def test_fused_prologue_falls_back_for_widths_it_is_not_built_for(cuda):
    """A key width of 48 (widened by the wrappers) with a persistent rotation of the value axis only: the call rotates
    up front and gives what the two-step route gives."""
    from linquant_amd.kernels import zoo

    q, k, v, g, _ = zc.cut(zc.inputs("mamba2", B=1, H=2, K=48, V=64, seed=5), 128)
    sv = zoo.rotation_signs(Z.signed_hadamard(64, 2).to(cuda))
    gen = torch.Generator().manual_seed(2)
    sc = {"q": torch.full((2,), 0.002), "k": torch.full((2,), 0.01), "kw": torch.full((2, 48), 0.01),
          "vw": torch.full((2, 64), 0.03), "vl": torch.full((2, 64), 0.03), "state": torch.full((2, 64), 0.05)}
    sc = {n: t.to(cuda) for n, t in sc.items()}
    dev = lambda t: t.to(cuda)  # noqa: E731
    _, _, vr = zoo.rotate_qkv(None, None, dev(v), signs_v=sv)
    o0, _ = zoo.chunk_simple_gla_int8(dev(q), dev(k), vr, dev(g), sc)
    o1, _ = zoo.chunk_simple_gla_int8(dev(q), dev(k), dev(v), dev(g), sc, prologue=dict(signs_v=sv))
    torch.cuda.synchronize()
    assert torch.equal(o0, o1)


def test_fused_prologue_with_128_token_chunks_rotates_up_front(cuda):
    """The one-launch rotation + quantization is built for 64-token chunks; with chunk_size = 128 the call rotates up front
    and gives, bit for bit, what rotate_qkv followed by the call gives."""
    from linquant_amd.kernels import zoo

    q, k, v, g, _ = zc.cut(zc.inputs("mamba2", B=1, H=2, K=64, V=64, seed=6), 256)
    sq, sv = (zoo.rotation_signs(Z.signed_hadamard(64, s).to(cuda)) for s in (1, 2))
    sc = {"q": torch.full((2,), 0.002), "k": torch.full((2,), 0.01), "kw": torch.full((2, 64), 0.01),
          "vw": torch.full((2, 64), 0.03), "vl": torch.full((2, 64), 0.03), "state": torch.full((2, 64), 0.05)}
    sc = {n: t.to(cuda) for n, t in sc.items()}
    dev = lambda t: t.to(cuda)  # noqa: E731
    qr, kr, vr = zoo.rotate_qkv(dev(q), dev(k), dev(v), signs_qk=sq, signs_v=sv)
    o0, h0 = zoo.chunk_simple_gla_int8(qr, kr, vr, dev(g), sc, chunk_size=128, output_final_state=True)
    o1, h1 = zoo.chunk_simple_gla_int8(dev(q), dev(k), dev(v), dev(g), sc, chunk_size=128, output_final_state=True,
                                       prologue=dict(signs_qk=sq, signs_v=sv))
    o64, _ = zoo.chunk_simple_gla_int8(qr, kr, vr, dev(g), sc, chunk_size=64)
    torch.cuda.synchronize()
    assert torch.equal(o0, o1) and torch.equal(h0, h1) and not torch.equal(o0, o64)
