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
