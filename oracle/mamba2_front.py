"""TEST INFRASTRUCTURE ONLY (CPU checker; never imported by the product package).

The two element-wise stages in front of the Mamba-2 SSD prologue, restated in numpy with individually rounded fp32
operations (oracle/kernel_arith.py), the same sequences the HIP kernels execute.

Follows (reference file:line):
  fp16_to_int8         linquant/w4a8_linear.py:36-98 (_fused_fp16_to_int8: rint(x * (1/s)) or rint(x / s), clamp, int8)
  causal_conv1d_silu   the call linquant/quantized_mamba2.py:262-268 makes into causal-conv1d==1.5.3.post1
                       (`causal_conv1d_fn(x, weight, bias, activation="silu")`, channel-last layout); the package is
                       absent from the reference tree, so this restates its published algorithm:
                       y[t, c] = silu(bias[c] + sum_j weight[c, j] * x[t - (W-1) + j, c]), fp32 accumulate, fp16 out.

Parity status: fp16_to_int8 is a closed form (IEEE division / multiplication, round-half-even) and pinned exactly by
brute force in tests/test_oracle_mamba2_front.py.  causal_conv1d_silu is PARITY UNPINNED against the third-party CUDA
kernel's bits (its multiply-add contraction and expf are not specified by any file of the reference); it is pinned
against a float64 evaluation of the same formula at the fp16 output spacing.  The HIP kernel evaluates the SiLU on the
hardware exp2 / reciprocal units, so GPU tests compare its fp16 output to this restatement within one unit in the last place.
"""

from __future__ import annotations

import numpy as np

from .kernel_arith import F, f32, lq_expf


def fp16_to_int8(x, scale, clamp_min=-127.0, reciprocal=True):
    """x fp16 (M, N); scale scalar.  Returns int8 (M, N)."""
    xf = x.astype(np.float16).astype(F)
    s = F(scale)
    y = xf * (F(1.0) / s) if reciprocal else xf / s
    return np.clip(np.rint(y), F(clamp_min), F(127.0)).astype(np.int8)


def causal_conv1d_silu(x, weight, bias=None, silu=True):
    """x fp16 (B, L, D), weight fp16 (D, W), bias fp16 (D,) or None.  Returns fp16 (B, L, D)."""
    B, L, D = x.shape
    W = weight.shape[1]
    xf = np.concatenate([np.zeros((B, W - 1, D), F), x.astype(np.float16).astype(F)], axis=1)
    wf = weight.astype(np.float16).astype(F)
    acc = np.zeros((B, L, D), F) if bias is None else np.broadcast_to(bias.astype(np.float16).astype(F), (B, L, D)).copy()
    for j in range(W):
        acc = f32(acc + f32(wf[:, j] * xf[:, j:j + L]))
    if silu:
        acc = f32(acc / f32(F(1.0) + lq_expf(-acc)))
    return acc.astype(np.float16)
