"""Fused Hadamard transform + INT8 quantization of the out_proj input (HIP), same call as
linquant/hadamard_utils.py:9-19 (`qhad_transform(w, input_scale) -> (w_int8, input_scale)`).

The transform of a row of ``dim = m * 2^k`` channels is ``H_m (x) H_(2^k)`` with ``H_m`` acting across the ``m``
contiguous chunks of ``2^k`` channels and the Sylvester matrix inside a chunk -- the layout of the
``fast_hadamard_transform_{12N,20N,28N,40N}`` kernels the reference calls, with the same branch order
(12N, 40N, 20N, 28N, power of two).  The order-``m`` factor of a non-power-of-two size is not unique: the activations
must be rotated with the very matrix that was folded into ``out_proj.weight``.  ``register_hadamard`` installs it;
``hadamard_matrix`` offers Paley constructions for builds that fold their own weights with this package.
"""

from __future__ import annotations

import math

import numpy as np
import torch

from linquant_amd import _lib

_SMALL = {}        # order -> int8 numpy (m, m), entries +-1
_DEVICE_CACHE = {}  # (dim, device) -> int8 tensor (g, g)


def sylvester(n: int) -> np.ndarray:
    """Sylvester Hadamard matrix of order n (a power of two): H[i, j] = (-1)^popcount(i & j)."""
    assert n >= 1 and n & (n - 1) == 0
    i = np.arange(n)
    bits = i[:, None] & i[None, :]
    par = np.zeros((n, n), np.int64)
    while bits.any():
        par ^= bits & 1
        bits >>= 1
    return (1 - 2 * par).astype(np.int8)


def _legendre(a: int, q: int) -> int:
    a %= q
    if a == 0:
        return 0
    return 1 if pow(a, (q - 1) // 2, q) == 1 else -1


def hadamard_matrix(m: int) -> np.ndarray:
    """A Hadamard matrix of order m for m in {1, 2, 4, ...} and m = 12, 20, 28, 40 (and their doublings):
    Paley's first construction for q = m - 1 prime, q = 3 mod 4 (12, 20); his second for m = 2 (q + 1),
    q prime, q = 1 mod 4 (28 from q = 13); Sylvester doubling otherwise (40 = 2 * 20)."""
    if m >= 1 and m & (m - 1) == 0:
        return sylvester(m)
    q = m - 1
    if q % 4 == 3 and all(q % d for d in range(2, int(math.isqrt(q)) + 1)):
        Q = np.array([[_legendre(i - j, q) for j in range(q)] for i in range(q)], np.int64)
        S = np.zeros((m, m), np.int64)
        S[0, 1:] = 1
        S[1:, 0] = -1
        S[1:, 1:] = Q
        return (np.eye(m, dtype=np.int64) + S).astype(np.int8)
    if m % 2 == 0:
        q = m // 2 - 1
        if q % 4 == 1 and all(q % d for d in range(2, int(math.isqrt(q)) + 1)):
            Q = np.array([[_legendre(i - j, q) for j in range(q)] for i in range(q)], np.int64)
            C = np.zeros((q + 1, q + 1), np.int64)
            C[0, 1:] = 1
            C[1:, 0] = 1
            C[1:, 1:] = Q
            one = np.array([[1, -1], [-1, -1]], np.int64)
            two = np.array([[1, 1], [1, -1]], np.int64)
            H = np.kron(C, two) + np.kron(np.eye(q + 1, dtype=np.int64), one)
            return H.astype(np.int8)
        return np.kron(sylvester(2).astype(np.int64), hadamard_matrix(m // 2).astype(np.int64)).astype(np.int8)
    raise ValueError(f"no construction for a Hadamard matrix of order {m}")


def register_hadamard(order: int, matrix) -> None:
    """Install the order-``order`` factor used for dims ``order * 2^k``: ``out_chunk[i] = sum_j matrix[i, j] chunk[j]``."""
    H = np.asarray(matrix.cpu() if isinstance(matrix, torch.Tensor) else matrix)
    assert H.shape == (order, order) and np.isin(H, (-1, 1)).all(), "entries must be +1 / -1"
    Hi = H.astype(np.int64)
    assert np.array_equal(Hi @ Hi.T, order * np.eye(order, dtype=np.int64)), "rows must be orthogonal"
    _SMALL[order] = H.astype(np.int8)
    _DEVICE_CACHE.clear()


def _is_pow2(n: int) -> bool:
    return n >= 1 and n & (n - 1) == 0


def small_order(dim: int) -> int:
    """Order of the non-power-of-two factor, in the branch order of get_qhad_fn (patches/ssdi8.patch:2153-2178)."""
    for m in (12, 40, 20, 28):
        if dim % m == 0 and _is_pow2(dim // m):
            return m
    assert _is_pow2(dim), f"dim {dim} is none of 12, 40, 20, 28 times a power of two, nor a power of two"
    return 1


def chunk_matrix(dim: int) -> np.ndarray:
    """The (dim/128, dim/128) matrix that acts across the 128-channel chunks of a row."""
    m = small_order(dim)
    if dim % 128 != 0 or dim // m < 128 or dim // 128 > 64:
        raise _lib.LinQuantHipError(f"qhad_transform: dim {dim} is outside the built range (128 * g, g <= 64, "
                                    f"power-of-two part >= 128)")
    if m == 1:
        return sylvester(dim // 128)
    if m not in _SMALL:
        raise _lib.LinQuantHipError(
            f"qhad_transform: dim {dim} needs the order-{m} Hadamard factor that out_proj.weight was folded with; "
            f"install it with linquant_amd.hadamard_utils.register_hadamard({m}, H)")
    return np.kron(_SMALL[m].astype(np.int64), sylvester(dim // (m * 128)).astype(np.int64)).astype(np.int8)


def _device_matrix(dim: int, device) -> torch.Tensor:
    key = (dim, str(device))
    if key not in _DEVICE_CACHE:
        _DEVICE_CACHE[key] = torch.from_numpy(np.ascontiguousarray(chunk_matrix(dim))).to(device)
    return _DEVICE_CACHE[key]


def _kernel_scale(dim: int, input_scale) -> float:
    # the reference keeps had_scale / input_scale in 64-bit on the host (linquant/hadamard_utils.py:17-18)
    scale_val = input_scale.float().item() if isinstance(input_scale, torch.Tensor) else float(input_scale)
    return (1.0 / math.sqrt(dim)) / scale_val


def qhad_transform(w, input_scale):
    """Hadamard-rotate ``w`` (..., dim) fp16 and quantize to INT8 in one launch. Returns (w_int8, input_scale)."""
    assert w.dtype == torch.float16
    dim = w.shape[-1]
    x = w.reshape(-1, dim)
    if x.stride(1) != 1 or x.stride(0) % 8 != 0:
        x = x.contiguous()
    out = torch.empty(x.shape, dtype=torch.int8, device=w.device)
    if x.shape[0]:
        _lib.call("lq_qhad_transform", w.device, x=_lib.ptr(x), x_stride=x.stride(0),
                  had=_lib.ptr(_device_matrix(dim, w.device)), out=_lib.ptr(out), rows=x.shape[0], dim=dim,
                  scale=_kernel_scale(dim, input_scale))
    return out.reshape(w.shape), input_scale
