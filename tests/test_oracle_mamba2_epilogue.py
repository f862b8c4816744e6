"""Pins oracle/mamba2_epilogue.py by what mathematics fixes: the power-of-two transform against scipy's Hadamard
matrix, the chunk layout against an explicit dense Kronecker product, H^T (H x) = dim x for every size, the norm
against torch's own rms_norm and silu, and the host-side matrix constructions of the package."""

import math

import numpy as np
import pytest
import scipy.linalg
import torch

from linquant_amd import hadamard_utils as HU
from oracle import mamba2_epilogue as O


@pytest.mark.parametrize("m", [1, 2, 4, 12, 20, 24, 28, 40, 64])
def test_package_matrices_are_hadamard(m):
    H = HU.hadamard_matrix(m).astype(np.int64)
    assert set(np.unique(H)) <= {-1, 1}
    assert np.array_equal(H @ H.T, m * np.eye(m, dtype=np.int64))


def test_sylvester_is_scipys():
    for n in (1, 2, 16, 128):
        assert np.array_equal(O.sylvester(n), scipy.linalg.hadamard(n))
        assert np.array_equal(HU.sylvester(n), scipy.linalg.hadamard(n))


def test_branch_order_and_chunk_matrix():
    # 5120 matches 40N and 20N: the 40N branch must win (patches/ssdi8.patch:2157-2170)
    assert HU.small_order(5120) == 40 and HU.small_order(2560) == 40 and HU.small_order(3584) == 28 and HU.small_order(20) == 20
    assert HU.small_order(1536) == 12 and HU.small_order(3072) == 12 and HU.small_order(4096) == 1
    assert np.array_equal(HU.chunk_matrix(4096), scipy.linalg.hadamard(32))
    HU.register_hadamard(12, HU.hadamard_matrix(12))
    G = HU.chunk_matrix(3072).astype(np.int64)               # 3072 = 12 * 256: H_12 (x) H_2 across the 24 chunks
    assert np.array_equal(G, np.kron(HU.hadamard_matrix(12).astype(np.int64), scipy.linalg.hadamard(2)))
    with pytest.raises(AssertionError):
        HU.register_hadamard(12, np.ones((12, 12)))


def test_power_of_two_transform_is_the_textbook_one():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 1024)).astype(np.float16)
    got = O.hadamard_rows(x, O.sylvester(8))
    ref = x.astype(np.float64) @ scipy.linalg.hadamard(1024).astype(np.float64)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("m,dim", [(12, 1536), (20, 2560), (40, 5120)])
def test_chunk_layout_against_dense_kron(m, dim):
    """out = H x with H = H_m (x) H_(dim/m): H_m acts across contiguous chunks, Sylvester inside."""
    rng = np.random.default_rng(1)
    Hm = HU.hadamard_matrix(m).astype(np.int64)
    G = np.kron(Hm, O.sylvester(dim // (m * 128)))
    x = rng.standard_normal((3, dim)).astype(np.float16)
    dense = np.kron(Hm, O.sylvester(dim // m)).astype(np.float64)
    assert np.array_equal(O.hadamard_rows(x, G), x.astype(np.float64) @ dense.T)
    # one non-symmetric probe: a unit vector in chunk 1 must come out as column 1 of H_m across chunks
    e = np.zeros((1, dim), np.float16)
    e[0, dim // m] = 1
    out = O.hadamard_rows(e, G).reshape(m, dim // m)
    assert np.array_equal(out[:, 0], Hm[:, 1].astype(np.float64))
    # orthogonality: H^T (H x) = dim x
    back = O.hadamard_rows(x, G) @ dense
    assert np.allclose(back, dim * x.astype(np.float64), rtol=0, atol=1e-7 * dim)


def test_qhad_rounding_and_saturation():
    G = O.sylvester(1)
    x = np.zeros((1, 128), np.float16)
    x[0, 0] = 1.0                                  # H x = all ones
    for scale, want in [(0.5, 1), (1.5, 2), (2.5, 3), (-0.5, -1), (-2.5, -3), (0.49, 0), (126.5, 127), (500.0, 127), (-500.0, -127)]:
        q = O.qhad_transform(x, G, scale)
        assert (q == want).all(), (scale, q[0, :4])


@pytest.mark.parametrize("gate,groups,wdt", [(True, 1, np.float16), (True, 8, np.float32), (False, 4, np.float16)])
def test_rmsnorm_gated_against_torch(gate, groups, wdt):
    rng = np.random.default_rng(2)
    rows, dim = 7, 1024
    x = (rng.standard_normal((rows, dim)) * 3).astype(np.float16)
    z = rng.standard_normal((rows, dim)).astype(np.float16) if gate else None
    w = (1 + 0.1 * rng.standard_normal(dim)).astype(wdt)
    got = O.rmsnorm_gated(x, z, w, 1e-5, dim // groups).astype(np.float64)
    xt = torch.from_numpy(x).double()
    if gate:
        xt = xt * torch.nn.functional.silu(torch.from_numpy(z).double())
    ref = torch.nn.functional.rms_norm(xt.view(rows, groups, dim // groups), (dim // groups,), eps=1e-5).view(rows, dim)
    ref = (ref * torch.from_numpy(w).double()).numpy()
    assert (np.abs(got - ref) <= np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64) * 0.51 + 1e-7).all()


def test_one_add_rounding_is_round_half_away():
    """The HIP quantizer rounds with trunc(y + copysign(0.5 - 2^-25, y)); it must equal round-half-away-from-zero on
    every tie, on the neighbours of every tie and integer, and on random values (the restatement uses floor(|y| + 0.5))."""
    F = np.float32
    c = F(0.5) - F(2.0 ** -25)
    assert c == F(float.fromhex("0x1.fffffep-2"))

    def trick(y):
        return np.trunc((y + np.copysign(c, y).astype(F)).astype(F))

    def ref(y):
        y64 = y.astype(np.float64)
        return np.sign(y64) * np.floor(np.abs(y64) + 0.5)

    k = np.arange(0, 1 << 16, dtype=np.float64)
    cands = []
    for base in (k + 0.5, k, k + 0.25):
        b = base.astype(F)
        cands += [b, np.nextafter(b, F(np.inf)), np.nextafter(b, F(-np.inf))]
    y = np.concatenate(cands)
    y = np.concatenate([y, -y])
    assert np.array_equal(trick(y), ref(y))
    rng = np.random.default_rng(0)
    y = (rng.standard_normal(2_000_000) * np.exp(rng.uniform(-10, 12, 2_000_000))).astype(F)
    assert np.array_equal(trick(y), ref(y))
