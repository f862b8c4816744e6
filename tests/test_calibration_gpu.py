"""GPU test of the device-side absmax collectors: maxima are exact, so every comparison is bit for bit."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("scheme", ["pc_static", "ph_static", "pt_static"])
def test_absmax_schemes_and_running_maximum(cuda, dtype, scheme):
    from linquant_amd.calibration import absmax_update

    gen = torch.Generator().manual_seed(0)
    B, T, H, D = 2, 300, 6, 64                      # a ragged last slab of rows
    out = None
    ref = None
    for batch in range(3):                          # running maximum over calibration batches
        big = (torch.randn(B, T, H, D + 16, generator=gen) * (1 + batch)).to(dtype).cuda()
        x = big[..., 8:8 + D] if dtype != torch.float32 else big[..., 4:4 + D]      # strided, 16-byte aligned view
        a = x.float().abs()
        r = {"pc_static": a.amax(dim=(0, 1)).reshape(-1), "ph_static": a.amax(dim=(0, 1, 3)), "pt_static": a.amax().reshape(1)}[scheme]
        ref = r if ref is None else torch.maximum(ref, r)
        if out is None:
            out = torch.zeros_like(r)
        absmax_update(out, x, scheme)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)


def test_absmax_reference_layout_gate_and_groups(cuda):
    """The three SSD observers: plain x per (H, P), x * gate per (H, P), and B * gate per (H, N) with B broadcast from
    its group to the heads -- against the torch expressions scripts/nemotron_h_calibration.py evaluates."""
    from linquant_amd.calibration import AbsmaxCollector, absmax_update

    gen = torch.Generator().manual_seed(1)
    B, L, H, P, G, N = 2, 512, 8, 64, 2, 128
    xBC = torch.randn(B, L, H * P + 2 * G * N, generator=gen).half().cuda()
    x = xBC[..., :H * P].view(B, L, H, P)
    Bm = xBC[..., H * P:H * P + G * N].view(B, L, G, N)
    gate = torch.rand(B, H, L // 64, 64, generator=gen).cuda()           # (B, H, nchunks, Q) as the cumsum stage stores it
    gate_blh = gate.permute(0, 2, 3, 1).reshape(B, L, H)                 # a view: no copy
    x_hp = torch.zeros(H * P, device="cuda")
    xs_hp = torch.zeros(H * P, device="cuda")
    bg_hn = torch.zeros(H * N, device="cuda")
    absmax_update(x_hp, x, "pc_static")
    absmax_update(xs_hp, x, "pc_static", gate=gate_blh)
    absmax_update(bg_hn, Bm, "pc_static", gate=gate_blh, heads_per_group=H // G)
    torch.cuda.synchronize()
    g = gate_blh.unsqueeze(-1)
    assert torch.equal(x_hp.view(H, P), x.float().abs().amax(dim=(0, 1)))
    assert torch.equal(xs_hp.view(H, P), (x.float() * g).abs().amax(dim=(0, 1)))
    b_per_head = Bm[:, :, torch.arange(H, device="cuda") // (H // G)]
    assert torch.equal(bg_hn.view(H, N), (b_per_head.float() * g).abs().amax(dim=(0, 1)))

    # the reference's operand layout [B, H, rows, D] through the collector, two roles with different schemes
    col = AbsmaxCollector("pc_static", {"q": "ph_static"})
    q = torch.randn(B, H, L, P, generator=gen).half().cuda()
    k = torch.randn(B, L, H, P, generator=gen).half().cuda().permute(0, 2, 1, 3)     # a permuted view with unit D stride
    col("q", q), col("k", k), col("k", k * 2)
    torch.cuda.synchronize()
    sc = col.scales(127)
    assert torch.equal(sc["q"], (q.float().abs().amax(dim=(0, 2, 3)) / 127).clamp_min(1e-12))
    assert torch.equal(sc["k"].view(H, P), ((k * 2).float().abs().amax(dim=(0, 2)) / 127).clamp_min(1e-12))


def test_absmax_rejections(cuda):
    from linquant_amd import _lib
    from linquant_amd.calibration import absmax_update

    x = torch.zeros(1, 4, 2, 12, dtype=torch.float16, device="cuda")            # D not a multiple of 8
    with pytest.raises(_lib.LinQuantHipError):
        absmax_update(torch.zeros(24, device="cuda"), x, "pc_static")
    x = torch.zeros(1, 4, 2, 24, dtype=torch.float16, device="cuda")[..., 4:20]  # misaligned view
    with pytest.raises(_lib.LinQuantHipError):
        absmax_update(torch.zeros(32, device="cuda"), x, "pc_static")


@pytest.mark.parametrize("b_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("N", [64, 128, 256])
def test_chunk_state_observer(cuda, b_dtype, N):
    """The chunk-state observer (scripts/nemotron_h_calibration.py:602-651: amax over (batch, chunk, N) of the unquantized
    chunk states per (H, P)) against a float64 einsum of the same operands, over two calibration batches, with a ragged
    last chunk, x as a strided view, B shared by the heads of a group.  fp32 sums of up to 128 terms: 1e-5 relative."""
    from linquant_amd.calibration import absmax_chunk_state_update

    gen = torch.Generator().manual_seed(0)
    Bn, L, H, G, P, Q = 2, 450, 8, 2, 128, 128
    out = torch.zeros(H * P, device=cuda)
    ref = torch.zeros(H, P, dtype=torch.float64)
    for batch in range(2):
        big = (torch.randn(Bn, L, H * P + 64, generator=gen) * (1 + batch)).half()
        x = big[..., 32:32 + H * P].view(Bn, L, H, P)
        Bt = torch.randn(Bn, L, G, N, generator=gen).to(b_dtype)
        gate = torch.rand(Bn, L, H, generator=gen) * 0.3
        absmax_chunk_state_update(out, x.cuda(), Bt.cuda(), gate.cuda(), Q)
        nc = (L + Q - 1) // Q
        pad = nc * Q - L
        xg = torch.nn.functional.pad((x.double() * gate.double()[..., None]), (0, 0, 0, 0, 0, pad)).view(Bn, nc, Q, H, P)
        Bh = torch.nn.functional.pad(Bt.double(), (0, 0, 0, 0, 0, pad)).view(Bn, nc, Q, G, N).repeat_interleave(H // G, dim=3)
        st = torch.einsum("bcqhp,bcqhn->bchpn", xg, Bh)
        ref = torch.maximum(ref, st.abs().amax(dim=(0, 1, 4)))
    torch.cuda.synchronize()
    got = out.view(H, P).cpu().double()
    assert ((got - ref).abs() / ref).max().item() < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Q", [64, 256])
def test_cb_observer(cuda, dtype, Q):
    """The C.B^T observer (scripts/nemotron_h_w4a8.py:126-169: amax over (batch, chunk, Q, Q) per group, every (m, k)
    pair of a chunk) against a float64 einsum; ragged last chunk, two batches."""
    from linquant_amd.calibration import absmax_cb_update

    gen = torch.Generator().manual_seed(1)
    Bn, L, G, N = 2, 600, 3, 128
    out = torch.zeros(G, device=cuda)
    ref = torch.zeros(G, dtype=torch.float64)
    for batch in range(2):
        C = (torch.randn(Bn, L, G, N, generator=gen) * (1 + batch)).to(dtype)
        Bt = torch.randn(Bn, L, G, N, generator=gen).to(dtype)
        absmax_cb_update(out, C.cuda(), Bt.cuda(), Q)
        nc = (L + Q - 1) // Q
        for c in range(nc):
            cc, bb = C[:, c * Q:(c + 1) * Q].double(), Bt[:, c * Q:(c + 1) * Q].double()
            cb = torch.einsum("bmgn,bkgn->bgmk", cc, bb)
            ref = torch.maximum(ref, cb.abs().amax(dim=(0, 2, 3)))
    torch.cuda.synchronize()
    got = out.cpu().double()
    assert ((got - ref).abs() / ref).max().item() < 1e-5


def test_calibrate_mamba2_on_the_device_matches_the_torch_expressions(cuda):
    """calibrate_mamba2 runs its observers as device reductions on GPU tensors and as torch expressions on CPU tensors:
    the two give the same scales up to what torch's own CPU and GPU evaluations of the gate differ by (the chunk-local
    cumulative sum of dt * A is an fp32 sum of 256 terms in a different order on each: about 1e-5 of the exponent)."""
    from linquant_amd.calibration import Mamba2Shape, calibrate_mamba2, mamba2_params, mamba2_synthetic

    s = Mamba2Shape(batch=1, seqlen=1024, nheads=8, headdim=64, dstate=128, ngroups=2, chunk=256)
    p_cpu = mamba2_params(s, 42, "cpu")
    x, dt = mamba2_synthetic(s, 1, "cpu")
    ref = calibrate_mamba2(s, x, dt, p_cpu)
    p_gpu = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in p_cpu.items()}
    got = calibrate_mamba2(s, x.cuda(), dt.cuda(), p_gpu)
    for name, r in ref.items():
        g = got[name].cpu()
        assert g.shape == r.shape, name
        assert ((g - r).abs() / r.abs().clamp_min(1e-12)).max().item() < 2e-4, name


def test_calibrate_mamba2_on_the_device_at_a_shape_the_reductions_do_not_take(cuda):
    """A state width the device observers are not built for (N = 32) and a head width of 32: calibrate_mamba2 on GPU
    tensors evaluates its torch expressions there instead of raising, and agrees with the CPU evaluation."""
    from linquant_amd.calibration import Mamba2Shape, calibrate_mamba2, mamba2_params, mamba2_synthetic

    s = Mamba2Shape(batch=1, seqlen=256, nheads=4, headdim=32, dstate=32, ngroups=1, chunk=64)
    p_cpu = mamba2_params(s, 42, "cpu")
    x, dt = mamba2_synthetic(s, 1, "cpu")
    ref = calibrate_mamba2(s, x, dt, p_cpu)
    p_gpu = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in p_cpu.items()}
    got = calibrate_mamba2(s, x.cuda(), dt.cuda(), p_gpu)
    for name, r in ref.items():
        g = got[name].cpu()
        assert g.shape == r.shape, name
        assert ((g - r).abs() / r.abs().clamp_min(1e-12)).max().item() < 2e-4, name
