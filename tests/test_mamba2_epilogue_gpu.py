"""GPU parity (through the C ABI) of the stages behind the Mamba-2 SSD: gated RMSNorm (fp16 output within one unit in
the last place of the numpy restatement: hardware exp2 / reciprocal and the fp32 summation order differ) and the
Hadamard + INT8 quantizer (codes equal to the float64-exact restatement except where the fp32 transform lands within
its own rounding error of a .5 boundary; never more than one code apart)."""

import numpy as np
import pytest
import torch

from oracle import mamba2_epilogue as O

pytestmark = pytest.mark.gpu

DIMS = [128, 1536, 2048, 3072, 3584, 4096, 5120, 8192]


def _register():
    from linquant_amd import hadamard_utils as HU

    for m in (12, 20, 28, 40):
        HU.register_hadamard(m, HU.hadamard_matrix(m))
    return HU


def _check_codes(got, x, G, scale, max_rate):
    ref, v = O.qhad_transform(x, G, scale, return_float=True)
    diff = got.astype(np.int32) - ref.astype(np.int32)
    assert np.abs(diff).max() <= 1, np.abs(diff).max()
    bad = diff != 0
    if bad.any():
        # a differing code must sit at a rounding boundary of the exact value (fp32 accumulation error of the row)
        frac = np.abs(np.abs(v[bad].astype(np.float64)) % 1.0 - 0.5)
        tol = 64 * np.spacing(np.abs(v).max(axis=None).astype(np.float32)).astype(np.float64) + 1e-6
        assert frac.max() <= tol, (frac.max(), tol)
    assert bad.mean() <= max_rate, bad.mean()


@pytest.mark.parametrize("dim", DIMS)
def test_qhad_transform(cuda, dim):
    HU = _register()
    rng = np.random.default_rng(dim)
    rows = 37
    x = (rng.standard_normal((rows, dim)) * 2).astype(np.float16)
    x[3] = 0
    x[5, ::7] *= 30                                           # outliers
    input_scale = float(np.abs(O.hadamard_rows(x, HU.chunk_matrix(dim))).max() / np.sqrt(dim) / 127)
    got, s = HU.qhad_transform(torch.from_numpy(x).cuda(), input_scale)
    torch.cuda.synchronize()
    assert s == input_scale and got.dtype == torch.int8 and got.shape == x.shape
    _check_codes(got.cpu().numpy(), x, HU.chunk_matrix(dim), (1.0 / np.sqrt(dim)) / input_scale, 1e-3)


def test_qhad_exact_on_integer_rows(cuda):
    """Small-integer rows make every fp32 sum exact: the codes must then match bit for bit, including the .5 ties
    (round half away from zero) and the saturation at +-127."""
    HU = _register()
    rng = np.random.default_rng(1)
    for dim in (1536, 4096, 5120):
        x = rng.integers(-3, 4, (64, dim)).astype(np.float16)
        for scale_val in (0.5, 0.25, 1 / 64):
            input_scale = (1.0 / np.sqrt(dim)) / scale_val   # kernel scale == scale_val up to the fp32 cast
            got, _ = HU.qhad_transform(torch.from_numpy(x).cuda(), input_scale)
            ref = O.qhad_transform(x, HU.chunk_matrix(dim), np.float32((1.0 / np.sqrt(dim)) / input_scale))
            assert np.array_equal(got.cpu().numpy(), ref), (dim, scale_val)
            assert (np.abs(ref) == 127).any() or scale_val < 0.5


def test_qhad_views_scale_tensor_and_rows(cuda):
    HU = _register()
    rng = np.random.default_rng(2)
    dim = 5120
    G = HU.chunk_matrix(dim)
    for rows in (1, 3, 4, 5, 1001):
        big = (rng.standard_normal((rows, dim + 64))).astype(np.float16)
        xt = torch.from_numpy(big).cuda()[:, 8:8 + dim]                      # strided rows, 16-byte aligned
        scale_t = torch.tensor(0.05, dtype=torch.float16).cuda()
        got, s = HU.qhad_transform(xt.view(1, rows, dim), scale_t)
        assert s is scale_t and got.shape == (1, rows, dim)
        _check_codes(got.cpu().numpy().reshape(rows, dim), big[:, 8:8 + dim], G,
                     (1.0 / np.sqrt(dim)) / float(scale_t.float().item()), 1e-3)
    empty, _ = HU.qhad_transform(torch.empty(0, dim, dtype=torch.float16, device="cuda"), 0.1)
    assert empty.shape == (0, dim)


def test_qhad_rejections(cuda):
    from linquant_amd import _lib
    HU = _register()
    with pytest.raises(_lib.LinQuantHipError):
        HU.qhad_transform(torch.zeros(2, 2560, dtype=torch.float16, device="cuda"), 0.1)   # 40 * 64: chunk of 64
    with pytest.raises(_lib.LinQuantHipError):
        HU.qhad_transform(torch.zeros(2, 16384, dtype=torch.float16, device="cuda"), 0.1)  # g = 128
    x = torch.zeros(4, 256, dtype=torch.float16, device="cuda")
    out = torch.empty(4, 256, dtype=torch.int8, device="cuda")
    had = torch.ones(2, 2, dtype=torch.int8, device="cuda")
    with pytest.raises(_lib.LinQuantHipError):
        _lib.call("lq_qhad_transform", x.device, x=_lib.ptr(x), x_stride=100, had=_lib.ptr(had), out=_lib.ptr(out),
                  rows=4, dim=256, scale=1.0)
    with pytest.raises(_lib.LinQuantHipError):
        _lib.call("lq_qhad_transform", x.device, x=_lib.ptr(x), x_stride=256, had=None, out=_lib.ptr(out),
                  rows=4, dim=256, scale=1.0)


@pytest.mark.parametrize("dim,groups", [(5120, 1), (5120, 8), (4096, 1), (8192, 8), (1536, 4), (128, 1)])
@pytest.mark.parametrize("gate", [True, False])
def test_rmsnorm_gated(cuda, dim, groups, gate):
    from linquant_amd.norm import rmsnorm_gated

    rng = np.random.default_rng(dim + groups)
    rows = 19
    x = (rng.standard_normal((rows, dim)) * 2).astype(np.float16)
    z = (rng.standard_normal((rows, dim)) * 2).astype(np.float16) if gate else None
    wdt = np.float32 if groups == 8 else np.float16
    w = (1 + 0.2 * rng.standard_normal(dim)).astype(wdt)
    got = rmsnorm_gated(torch.from_numpy(x).cuda(), None if z is None else torch.from_numpy(z).cuda(),
                        torch.from_numpy(w).cuda(), 1e-5, dim // groups)
    torch.cuda.synchronize()
    ref = O.rmsnorm_gated(x, z, w, 1e-5, dim // groups)
    g = got.cpu().numpy()
    diff = np.abs(g.astype(np.float64) - ref.astype(np.float64))
    assert (diff <= np.spacing(np.abs(ref)).astype(np.float64)).all(), "more than one fp16 ulp apart"
    assert (g != ref).mean() < 2e-2


@pytest.mark.parametrize("dim,groups", [(5120, 1), (5120, 8), (4096, 1), (3072, 1), (8192, 8)])
def test_fused_norm_qhad_equals_the_two_stages(cuda, dim, groups):
    """The fused launch rounds the normalized row to fp16 exactly as the separate stage stores it, so its codes are
    the codes of qhad_transform applied to its own normalized rows, bit for bit."""
    from linquant_amd.norm import rmsnorm_gated, rmsnorm_gated_qhad
    HU = _register()

    rng = np.random.default_rng(dim * 3 + groups)
    rows = 41
    x = torch.from_numpy((rng.standard_normal((2, rows, dim)) * 2).astype(np.float16)).cuda()
    z = torch.from_numpy((rng.standard_normal((2, rows, dim)) * 2).astype(np.float16)).cuda()
    w = torch.from_numpy((1 + 0.2 * rng.standard_normal(dim)).astype(np.float16)).cuda()
    q, s, normed = rmsnorm_gated_qhad(x, z, w, 0.03, 1e-5, dim // groups, return_norm=True)
    q2, _ = rmsnorm_gated_qhad(x, z, w, 0.03, 1e-5, dim // groups)
    two_a = rmsnorm_gated(x, z, w, 1e-5, dim // groups)
    two_b, _ = HU.qhad_transform(two_a, 0.03)
    torch.cuda.synchronize()
    assert s == 0.03 and q.shape == x.shape and torch.equal(q, q2)
    assert torch.equal(normed, two_a)
    assert torch.equal(q, two_b)
    # and against the restatement end to end
    ref_norm = O.rmsnorm_gated(x.cpu().numpy().reshape(-1, dim), z.cpu().numpy().reshape(-1, dim), w.cpu().numpy(),
                               1e-5, dim // groups)
    _check_codes(q.cpu().numpy().reshape(-1, dim), normed.cpu().numpy().reshape(-1, dim), HU.chunk_matrix(dim),
                 (1.0 / np.sqrt(dim)) / 0.03, 1e-3)
    assert (normed.cpu().numpy().reshape(-1, dim) != ref_norm).mean() < 2e-2
