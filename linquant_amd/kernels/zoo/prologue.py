"""Operand prologue of the zoo calls (HIP): persistent R_QK on q, k, R_V on v and the diagonal rescaling D_QK.

The reference runs these as three bf16 GEMMs in front of the kernels (bench/zoo_kernels.py:135-140, "not fused yet") and,
in the oracle, as ``mat(q @ rot_qk)``, ``mat(k @ rot_qk)``, ``mat(v @ rot_v)`` on entry (linquant/reference.py:42-46);
D_QK is the harness's ``q' = q D, k' = k / D`` (linquant/harness.py:68-88).  Here all of it is one launch of a fast
Walsh-Hadamard transform over the rows."""

from __future__ import annotations

import torch

from linquant_amd import _lib

from . import _common as C


def rotation_signs(R: torch.Tensor) -> torch.Tensor:
    """Column signs (n,) fp32 of a signed Sylvester Hadamard rotation R = H_n / sqrt(n) . diag(signs)
    (linquant/reference.py:232-239).  Checks on the host that R has that form (a set-up step, not on the hot path)."""
    n = R.shape[0]
    assert R.shape == (n, n) and n & (n - 1) == 0, "rotation must be a square power-of-two matrix"
    Hm = torch.ones(1, 1, dtype=torch.float64)
    while Hm.shape[0] < n:
        Hm = torch.cat([torch.cat([Hm, Hm], 1), torch.cat([Hm, -Hm], 1)], 0)
    signs = torch.sign(R[0].double().cpu())
    assert torch.allclose(R.double().cpu(), Hm / n ** 0.5 * signs, atol=1e-3), "not a signed Sylvester Hadamard rotation"
    return signs.float().to(R.device)


def rotate_qkv(q=None, k=None, v=None, *, signs_qk=None, signs_v=None, dqk=None, out=None):
    """q, k [B,T,H,K], v [B,T,H,V] fp16 / bf16 (any may be None).  ``signs_qk`` (K,), ``signs_v`` (V,): +-1 column signs
    of R_QK / R_V (``rotation_signs``), None = that rotation is left out.  ``dqk`` (H,K) fp32, finite and positive: q is
    multiplied by it and k divided (the quotient rounded once, as the division of linquant/harness.py:86 rounds it).  Returns the tuple (q', k', v') of new tensors (None where the
    input was None); ``out=(q_out, k_out, v_out)`` supplies the destinations (an input itself for in-place)."""
    ref = next(t for t in (q, k, v) if t is not None)
    B, T, H = ref.shape[:3]
    K = q.shape[-1] if q is not None else (k.shape[-1] if k is not None else 0)
    V = v.shape[-1] if v is not None else 0
    for t in (q, k, v):
        assert t is None or (t.is_contiguous() and t.dtype == ref.dtype and t.shape[:3] == (B, T, H))
    assert ref.dtype in (torch.float16, torch.bfloat16), "activations: fp16 or bf16"
    assert K in (0, 64, 128) and V in (0, 64, 128), "row widths 64 and 128"
    outs = list(out) if out is not None else [None if t is None else torch.empty_like(t) for t in (q, k, v)]
    f = lambda t, n: None if t is None else _check(C.f32(t), n)  # noqa: E731
    dq = dk = None
    if dqk is not None:
        dq = _check(C.f32(dqk), H * K)
        dk = (1.0 / dq).contiguous()
    _lib.call("lq_zoo_rotate_qkv", ref.device, q=_lib.ptr(q), k=_lib.ptr(k), v=_lib.ptr(v), q_out=_lib.ptr(outs[0]),
              k_out=_lib.ptr(outs[1]), v_out=_lib.ptr(outs[2]), dq=_lib.ptr(dq), dk=_lib.ptr(dk),
              signs_qk=_lib.ptr(f(signs_qk, K)), signs_v=_lib.ptr(f(signs_v, V)), batch=B, seqlen=T, nheads=H, kdim=K,
              vdim=V, act_dtype=C.act_code(ref))
    return tuple(outs)


def _check(t, n):
    assert t.numel() == n, f"expected {n} entries, got {tuple(t.shape)}"
    return _lib.aligned(t)
