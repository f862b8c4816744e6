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
