"""TEST INFRASTRUCTURE ONLY (CPU checker; never imported by the product package).

fp32 arithmetic helpers shared by the kernel-lineage oracles: every function is a fixed sequence of
individually rounded IEEE fp32 operations in numpy, the same sequences the HIP kernels execute
(linquant_amd/csrc/lq_common.h), so INT8 code tensors can be compared bit for bit.

The reference's Triton kernels use `tl.exp` / `tl.log` (hardware approximations whose last bits are not
specified: linquant/kernels/mamba2/chunk_cumsum.py:12,71, chunk_state.py:209, state_passing.py:69); this
checker fixes one concrete, accurate evaluation (|rel err| < 2e-7, pinned against float64 in tests).
"""

from __future__ import annotations

import numpy as np

F = np.float32


def f32(x):
    return np.asarray(x, dtype=np.float32)


def lq_expf(x):
    """exp(x) in fp32: Cody-Waite reduction, degree-7 Taylor, exponent-bit scaling; x <= -86 -> 0, x > 88 -> inf."""
    x = f32(x)
    with np.errstate(all="ignore"):
        xc = np.clip(x, F(-86.0), F(88.0))
        t = xc * F(1.44269502162933349609375)
        n = np.rint(t)
        r = xc - n * F(0.693145751953125)
        r = r - n * F(1.42860676533018704504e-06)
        p = F(1.98412701138295233250e-04)
        for c in (1.38888892251998186111e-03, 8.33333376795053482056e-03, 4.16666679084300994873e-02,
                  1.66666671633720397949e-01, 0.5, 1.0, 1.0):
            p = p * r + F(c)
        e = ((n.astype(np.int32) + 127) << 23).astype(np.int32).view(np.float32)
        res = p * e
    res = np.where(x > F(-86.0), res, F(0.0))
    res = np.where(x > F(88.0), F(np.inf), res)
    res = np.where(np.isnan(x), x, res)
    return res.astype(np.float32)


def lq_logf(y):
    """log(y) for normal y > 0 in fp32 (atanh series on the reduced mantissa)."""
    y = f32(y)
    bits = y.view(np.int32)
    e = ((bits >> 23) & 0xFF) - 127
    m = ((bits & 0x007FFFFF) | 0x3F800000).astype(np.int32).view(np.float32)
    big = m > F(1.41421353816986083984375)
    m = np.where(big, m * F(0.5), m)
    e = np.where(big, e + 1, e)
    s = (m - F(1.0)) / (m + F(1.0))
    s2 = s * s
    p = F(9.09090936183929443359e-02)
    for c in (1.11111111938953399658e-01, 1.42857149243354797363e-01, 2.00000002980232238770e-01,
              3.33333343267440795898e-01, 1.0):
        p = p * s2 + F(c)
    lm = (s + s) * p
    fe = e.astype(np.float32)
    return (fe * F(0.693145751953125) + (fe * F(1.42860676533018704504e-06) + lm)).astype(np.float32)


def rha(y):
    """Round half away from zero, as floor(y+.5) / ceil(y-.5) evaluated in fp32 (returns float32 integers)."""
    y = f32(y)
    return np.trunc(y + np.copysign(F(0.5), y)).astype(np.float32)


def q_rha(y, qmax):
    """clamp(rha(y), -qmax, qmax) -> int32 codes (linquant/kernels/zoo/simple_gla.py:15-20)."""
    r = np.clip(rha(y), -qmax, qmax)
    return np.where(np.isnan(r), 0, r).astype(np.int32)


def q_rint(y, lo, hi):
    """clamp(rint(y), lo, hi) with round-half-even -> int32 codes (libdevice.rint lineage)."""
    r = np.clip(np.rint(f32(y)), lo, hi)
    return np.where(np.isnan(r), lo, r).astype(np.int32)


def bf16_round(x):
    """fp32 -> bf16 -> fp32, round to nearest even (finite inputs)."""
    u = f32(x).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def fp16_round(x):
    return f32(x).astype(np.float16).astype(np.float32)


def int_dot_exact(a, b):
    """Exact integer matmul a @ b of small-integer-valued arrays via BLAS: fp32 when every partial sum stays
    below 2^24, float64 otherwise. Returns int32."""
    k = a.shape[-1]
    amax = float(np.abs(a).max(initial=0)) * float(np.abs(b).max(initial=0)) * k
    dt = np.float32 if amax < 2**24 else np.float64
    return np.matmul(a.astype(dt), b.astype(dt)).astype(np.int32)
