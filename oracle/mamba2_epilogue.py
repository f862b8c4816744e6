"""TEST INFRASTRUCTURE ONLY (CPU checker; never imported by the product package).

The two stages behind the Mamba-2 SSD, restated in numpy.

Follows (reference file:line):
  rmsnorm_gated    the `self.norm(y, z)` call at linquant/quantized_mamba2.py:354-358.  The module is the norm of the
                   wrapped mixer (RMSNormGated of mamba-ssm / its SSDi8 twin, scripts/mamba2_w4a8.py:92), absent from
                   the reference tree; this restates its published algorithm with norm_before_gate = False:
                   v = x * (z * sigmoid(z)); y = v * rsqrt(mean_group(v^2) + eps) * weight, fp32, stored as fp16.
  qhad_transform   linquant/hadamard_utils.py:9-19 calling SSDi8's quant_hadamard kernels (absent); their epilogue is
                   patches/ssdi8.patch:101-112: q = saturate(roundf(v * scale)) to +-127, roundf = half away from zero,
                   v the fp32 Hadamard transform of the fp16 row, scale = (1 / sqrt(dim)) / input_scale taken in 64-bit
                   and passed as fp32.  Chunk layout of the m * 2^k sizes (H_m across contiguous chunks, Sylvester
                   inside a chunk, out = H x): the published fast-hadamard-transform algorithm.

Parity status: both functions are PARITY UNPINNED against the third-party kernels' bits (the order of their fp32
additions and the order-12/20/28/40 matrices themselves live in packages the reference tree does not hold; the
product takes that matrix as an argument).  What pins the restatement: the power-of-two case against
scipy.linalg.hadamard, H^T (H x) = dim x for every size, the kron identity against an explicit dense matrix, and
torch's own rms_norm / silu for the norm (tests/test_oracle_mamba2_epilogue.py).  The transform is evaluated in
float64 (exact for fp16 inputs up to the last bit of a 53-bit sum), so it is the correctly rounded value the fp32
kernels approximate; GPU parity is therefore "codes equal except at rounding boundaries, never more than one apart".
"""

from __future__ import annotations

import numpy as np

F = np.float32


def sylvester(n):
    i = np.arange(n)
    bits = i[:, None] & i[None, :]
    par = np.zeros((n, n), np.int64)
    while bits.any():
        par ^= bits & 1
        bits >>= 1
    return 1 - 2 * par


def rmsnorm_gated(x, z, weight, eps=1e-5, group_size=None):
    """x, z fp16 (rows, dim) (z may be None); weight (dim,) fp16 or fp32.  Returns fp16 (rows, dim)."""
    rows, dim = x.shape
    group_size = dim if group_size is None else group_size
    v = x.astype(np.float16).astype(F)
    if z is not None:
        zf = z.astype(np.float16).astype(F)
        v = v * (zf * (F(1.0) / (F(1.0) + np.exp(-zf, dtype=F))))
    vg = v.reshape(rows, dim // group_size, group_size)
    var = (vg.astype(np.float64) ** 2).mean(axis=2, keepdims=True).astype(F)
    rstd = F(1.0) / np.sqrt(var + F(eps), dtype=F)
    y = ((vg * rstd).reshape(rows, dim) * weight.astype(F)).astype(F)
    return y.astype(np.float16)


def hadamard_rows(x, had):
    """float64 (H x) per row for H = had (x) H_128: x fp16 (rows, dim), had (g, g) +-1 with dim = 128 g."""
    rows, dim = x.shape
    g = dim // 128
    assert had.shape == (g, g) and dim == 128 * g
    X = x.astype(np.float16).astype(np.float64).reshape(rows, g, 128)
    Y = np.einsum("pc,rci->rpi", had.astype(np.float64), X)
    Y = Y @ sylvester(128).astype(np.float64)  # symmetric
    return Y.reshape(rows, dim)


def qhad_transform(x, had, scale, return_float=False):
    """int8 (rows, dim) = saturate(round_half_away(fp32(H x) * fp32(scale)), +-127)."""
    v = hadamard_rows(x, had).astype(F) * F(scale)
    r = np.sign(v) * np.floor(np.abs(v).astype(np.float64) + 0.5)
    q = np.clip(r, -127, 127).astype(np.int8)
    return (q, v) if return_float else q
