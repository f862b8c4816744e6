"""Concurrent calls on two streams of default priority: the library keeps no mutable state between calls (the
allocation-free entry point aside), so a Mamba-2 SSD forward on one stream and a KDA chunk forward on another, issued
alternately so that their kernels interleave on the device, must give the bits of the same calls issued one after the
other."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_two_streams_interleaved(cuda):
    from linquant_amd.calibration import Mamba2Shape
    from linquant_amd.kernels import zoo
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC
    from tests import mamba2_cases as mc

    s = Mamba2Shape(batch=2, seqlen=4096, nheads=16, headdim=64, dstate=128, ngroups=1, chunk=256)
    case = mc.build_case(s, device=cuda, regime="weak")
    p, sc, xBC, dt_raw = case["params"], case["scales"], case["xBC"], case["dt_raw"]

    def ssd():
        x, qB, qC, b_fp, b_rmax = fused_split_rotate_quant_xBC(xBC, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                                               sc["B_inv_scale"], sc["C_inv_scale"], return_b_fp=True,
                                                               return_b_rowmax=True)
        out, _ = M._quant_mamba_chunk_scan_combined_fwd(
            x, dt_raw, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk,
            p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
            static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], keyside=True,
            x_scale_hp=sc["x_scale_hp"], b_fp=b_fp, b_gate_scale=sc["b_gate_scale"], b_rowmax=b_rmax)
        return out

    B, T, H, K, V = 2, 4096, 8, 128, 128
    gen = torch.Generator(device=cuda).manual_seed(3)
    q = torch.randn(B, T, H, K, generator=gen, device=cuda, dtype=torch.float16)
    k = torch.randn(B, T, H, K, generator=gen, device=cuda, dtype=torch.float16)
    k = k / k.float().norm(dim=-1, keepdim=True).clamp_min(1e-6).half()
    v = torch.randn(B, T, H, V, generator=gen, device=cuda, dtype=torch.float16)
    g = torch.nn.functional.logsigmoid(torch.randn(B, T, H, K, generator=gen, device=cuda) + 1.0)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen, device=cuda))
    full = lambda shape, val: torch.full(shape, val, device=cuda, dtype=torch.float32)  # noqa: E731
    zs = {"q": full((H,), 4.0 / 127 * K ** -0.5), "k": full((H,), 0.4 / 127), "w": full((H,), 0.8 / 127),
          "kw": full((H, K), 0.4 / 127), "el": full((H, V), 8.0 / 127), "ew": full((H, V), 8.0 / 127),
          "state": full((H, V), 0.05)}

    def kda():
        return zoo.chunk_kda_int8(q, k, v, g, beta, zs, sigma=0.5, eta=0.0)[0]

    ref_ssd, ref_kda = ssd(), kda()
    torch.cuda.synchronize()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    for _ in range(6):
        with torch.cuda.stream(sa):
            outs_a.append(ssd())
        with torch.cuda.stream(sb):
            outs_b.append(kda())
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(outs_a, outs_b)):
        assert torch.equal(a, ref_ssd), f"SSD forward {i} on its own stream differs"
        assert torch.equal(b, ref_kda), f"KDA forward {i} on its own stream differs"
