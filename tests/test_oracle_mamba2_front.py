"""Pins oracle/mamba2_front.py: the fp16 -> int8 quantizer against exact rational arithmetic, the causal conv1d + SiLU
against a float64 evaluation of the published formula."""

from fractions import Fraction

import numpy as np

from oracle import mamba2_front as O


def test_fp16_to_int8_divide_form_is_exact_division():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((4, 64)) * 3).astype(np.float16)
    s = np.float32(0.0371)
    got = O.fp16_to_int8(x, s, clamp_min=-128.0, reciprocal=False)
    for xv, g in zip(x.ravel(), got.ravel()):
        q = Fraction(float(xv)) / Fraction(float(s))
        y = np.float32(float(xv)) / s                      # IEEE division: correctly rounded quotient
        assert abs(Fraction(float(y)) - q) <= abs(q) * Fraction(1, 2 ** 23)
        r = int(np.clip(np.rint(y), -128, 127))
        assert g == r


def test_fp16_to_int8_ties_clamps_and_reciprocal():
    s = np.float32(0.5)
    x = np.array([[0.25, 0.75, 1.25, -0.25, -0.75, 100.0, -100.0, 63.5]], np.float16)
    assert O.fp16_to_int8(x, s).tolist() == [[0, 2, 2, 0, -2, 127, -127, 127]]      # half to even, +-127
    assert O.fp16_to_int8(x, s, clamp_min=-128.0).tolist()[0][6] == -128
    # reciprocal and divide forms differ only where x * fl(1/s) and x / s round differently
    rng = np.random.default_rng(1)
    xb = (rng.standard_normal((64, 128)) * 2).astype(np.float16)
    s3 = np.float32(1.0 / 3.0)
    a, b = O.fp16_to_int8(xb, s3, reciprocal=True), O.fp16_to_int8(xb, s3, reciprocal=False)
    assert np.abs(a.astype(int) - b.astype(int)).max() <= 1


def test_causal_conv1d_silu_against_float64():
    rng = np.random.default_rng(2)
    B, L, D, W = 2, 37, 16, 4
    x = rng.standard_normal((B, L, D)).astype(np.float16)
    w = (rng.standard_normal((D, W)) * 0.5).astype(np.float16)
    bias = (rng.standard_normal(D) * 0.1).astype(np.float16)
    got = O.causal_conv1d_silu(x, w, bias).astype(np.float64)
    xp = np.concatenate([np.zeros((B, W - 1, D)), x.astype(np.float64)], axis=1)
    acc = np.broadcast_to(bias.astype(np.float64), (B, L, D)).copy()
    for j in range(W):
        acc += w[:, j].astype(np.float64) * xp[:, j:j + L]
    ref = acc / (1 + np.exp(-acc))
    assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()          # fp16 output spacing
    lin = O.causal_conv1d_silu(x, w, None, silu=False).astype(np.float64)
    acc0 = sum(w[:, j].astype(np.float64) * xp[:, j:j + L] for j in range(W))
    assert np.abs(lin - acc0).max() <= 2e-3 * max(np.abs(acc0).max(), 1)
    # causality: output at t depends on inputs <= t only
    x2 = x.copy()
    x2[:, 20:] = 0
    assert np.array_equal(O.causal_conv1d_silu(x2, w, bias)[:, :20], O.causal_conv1d_silu(x, w, bias)[:, :20])


def test_two_fma_quotient_equals_ieee_division():
    """The HIP quantizer divides by a uniform scale as q0 = RN(x * RN(1/s)), r = fma(-q0, s, x), q = fma(r, RN(1/s), q0).
    Restated here in float64 (every product of two fp32 values is exact there; the one inexact sum is checked for
    fp32 ties) over every finite fp16 value and scales of many magnitudes: q must be the IEEE fp32 quotient."""
    bits = np.arange(65536, dtype=np.uint16).view(np.float16)
    x = bits[np.isfinite(bits)].astype(np.float32)
    rng = np.random.default_rng(3)
    scales = np.concatenate([np.exp2(rng.uniform(-59, 59, 64)), np.exp2(rng.uniform(-12, 6, 192)),
                             [1.0, 0.1, 1 / 3, 0.0313, 1.9999999, 1.0000001]]).astype(np.float32)
    for s in scales:
        inv = np.float32(1.0) / s
        q0 = (x * inv).astype(np.float32)
        rem64 = x.astype(np.float64) - q0.astype(np.float64) * np.float64(s)
        rem = rem64.astype(np.float32)    # float64 holds x - q0 * s exactly (at most 26 significant bits): one rounding, as the fma
        sum64 = q0.astype(np.float64) + rem.astype(np.float64) * np.float64(inv)
        q = sum64.astype(np.float32)
        ref = x / s
        differ = q != ref
        if differ.any():
            # a float64 sum that landed on an fp32 tie was rounded twice: decide those exactly
            from fractions import Fraction
            for i in np.nonzero(differ)[0]:
                exact = Fraction(float(q0[i])) + Fraction(float(rem[i])) * Fraction(float(inv))
                assert abs(exact - Fraction(float(ref[i]))) <= abs(exact - Fraction(float(q[i]))), (float(s), float(x[i]))
