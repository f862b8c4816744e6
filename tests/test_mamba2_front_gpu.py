"""GPU parity (through the C ABI) of the fp16 -> int8 quantizer (bit-exact against the numpy restatement) and the
causal conv1d + SiLU (bit-exact without the activation; with SiLU the hardware exp2 / reciprocal leave at most one
fp16 unit in the last place at rounding boundaries)."""

import numpy as np
import pytest
import torch

from oracle import mamba2_front as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("reciprocal", [True, False])
@pytest.mark.parametrize("clamp_min", [-127.0, -128.0])
@pytest.mark.parametrize("scale_dtype", [torch.float32, torch.float16])
def test_fused_fp16_to_int8(cuda, reciprocal, clamp_min, scale_dtype):
    from linquant_amd.w4a8_linear import _fused_fp16_to_int8

    gen = torch.Generator().manual_seed(0)
    big = (torch.randn(300, 2560 + 64, generator=gen) * 4).half()
    x = big[:, :2560]                                    # strided rows
    scale = torch.tensor(0.0313, dtype=scale_dtype)
    got = _fused_fp16_to_int8(x.cuda(), scale.cuda(), clamp_min=clamp_min, reciprocal=reciprocal)
    torch.cuda.synchronize()
    ref = O.fp16_to_int8(x.numpy(), np.float32(scale.float().item()), clamp_min, reciprocal)
    assert got.dtype == torch.int8 and np.array_equal(got.cpu().numpy(), ref)


def test_fused_fp16_to_int8_every_fp16_value(cuda):
    """The divide form must equal IEEE x / s for every finite or infinite fp16 input, at scales of every magnitude the
    fast correctly-rounded quotient covers and at the extremes where the kernel falls back to the plain divide."""
    from linquant_amd.w4a8_linear import _fused_fp16_to_int8

    bits = np.arange(65536, dtype=np.uint16).view(np.float16)
    vals = bits[~np.isnan(bits)]
    vals = np.concatenate([vals, vals[: (-len(vals)) % 64]]).reshape(-1, 64)
    x = torch.from_numpy(vals.copy()).cuda()
    rng = np.random.default_rng(7)
    scales = np.concatenate([np.exp2(rng.uniform(-12, 6, 48)), [1.0, 0.1, 1 / 3, 0.0313, 2.0 ** -70, 2.0 ** 70,
                                                                 np.float32(1.9999999), np.float32(1.0000001)]]).astype(np.float32)
    for sc in scales:
        for clamp_min in (-127.0, -128.0):
            got = _fused_fp16_to_int8(x, torch.tensor(sc, dtype=torch.float32).cuda(), clamp_min=clamp_min, reciprocal=False)
            with np.errstate(over="ignore", invalid="ignore"):
                ref = O.fp16_to_int8(vals, sc, clamp_min, False)
            bad = got.cpu().numpy() != ref
            assert not bad.any(), (float(sc), vals[bad][:4], got.cpu().numpy()[bad][:4], ref[bad][:4])


@pytest.mark.parametrize("width,bias,act", [(4, True, "silu"), (4, False, "silu"), (3, True, None), (2, True, "silu")])
@pytest.mark.parametrize("L", [1, 37, 512])
def test_causal_conv1d(cuda, width, bias, act, L):
    from linquant_amd.kernels.mamba2.causal_conv1d import causal_conv1d_fn

    gen = torch.Generator().manual_seed(1)
    B, D = 2, 5376 // 4
    proj = torch.randn(B, L, D + 40, generator=gen).half()           # xBC is a slice of the in_proj output
    xBC = proj[..., 8:8 + D]
    w = (torch.randn(D, width, generator=gen) * 0.5).half()
    bs = (torch.randn(D, generator=gen) * 0.1).half() if bias else None
    out = causal_conv1d_fn(xBC.cuda().transpose(1, 2), w.cuda(), None if bs is None else bs.cuda(), activation=act)
    torch.cuda.synchronize()
    assert out.shape == (B, D, L)
    ref = O.causal_conv1d_silu(xBC.numpy(), w.numpy(), None if bs is None else bs.numpy(), silu=act is not None)
    got = out.transpose(1, 2).cpu().numpy()
    if act is None:
        assert np.array_equal(got, ref)
    else:
        diff = np.abs(got.astype(np.float64) - ref.astype(np.float64))
        assert (diff <= np.spacing(np.abs(ref)).astype(np.float64)).all(), "more than one fp16 ulp apart"
        assert (got != ref).mean() < 1e-2


def test_causal_conv1d_parameter_views(cuda):
    """Taps and bias that are views into a larger parameter tensor (first byte off the 16-byte grid) give the same output
    as freshly allocated ones through the wrapper, and the C entry point itself rejects such pointers with LQ_E_SHAPE."""
    from linquant_amd import _lib
    from linquant_amd.kernels.mamba2.causal_conv1d import causal_conv1d_fn

    gen = torch.Generator().manual_seed(2)
    B, L, D, W = 1, 96, 256, 4
    x = torch.randn(B, L, D, generator=gen).half().cuda()
    wbig = (torch.randn(D + 1, W, generator=gen) * 0.5).half().cuda()
    bbig = (torch.randn(D + 4, generator=gen) * 0.1).half().cuda()
    w_view, b_view = wbig[1:], bbig[4:]                              # 8 bytes past a 16-byte boundary
    assert w_view.data_ptr() % 16 == 8 and b_view.data_ptr() % 16 == 8 and w_view.is_contiguous()
    ref = causal_conv1d_fn(x.transpose(1, 2), w_view.clone(), b_view.clone(), activation="silu")
    got = causal_conv1d_fn(x.transpose(1, 2), w_view, b_view, activation="silu")
    torch.cuda.synchronize()
    assert torch.equal(got, ref)
    out = torch.empty(B, L, D, dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.LinQuantHipError):
        _lib.call("lq_causal_conv1d", x.device, x=_lib.ptr(x), x_stride_b=x.stride(0), x_stride_l=x.stride(1),
                  weight=_lib.ptr(w_view), bias=None, out=_lib.ptr(out), batch=B, seqlen=L, dim=D, width=W, silu=1)
