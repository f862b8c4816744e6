"""Tensors with more than 2^31 elements (and more than 2^32 bytes): every (batch row, head) is an independent recurrence
in both lineages, so a launch over many batch rows must reproduce, bit for bit, a launch on one batch row cut out of
the same inputs.  The rows compared sit below 2^31 elements, across that boundary and at the far end of the tensors,
where a 32-bit element or byte offset anywhere in a kernel would read or write the wrong place.  Inputs are drawn on
the device (the host generator would take minutes at these sizes); no oracle is involved, the small launch is the
reference and is itself covered by the oracle tests at the same per-row shape."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _rows(batch):
    return sorted({0, batch // 2 - 1, batch // 2, batch - 1})


def test_mamba2_ssd_beyond_2_31_elements(cuda):
    from linquant_amd.calibration import Mamba2Shape, calibrate_mamba2, mamba2_params, mamba2_synthetic
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    B, L = 52, 8192                                            # x and out: 52 * 8192 * 80 * 64 = 2.18e9 elements
    s = Mamba2Shape(batch=B, seqlen=L, nheads=80, headdim=64, dstate=128, ngroups=1, chunk=256)
    assert B * L * s.nheads * s.headdim > 2 ** 31
    p = mamba2_params(s, 42, cuda)
    cal = Mamba2Shape(batch=1, seqlen=2048, nheads=s.nheads, headdim=s.headdim, dstate=s.dstate, ngroups=1, chunk=256)
    cx, cdt = mamba2_synthetic(cal, 1, cuda)
    sc = calibrate_mamba2(cal, cx, cdt, p)
    gen = torch.Generator(device=cuda).manual_seed(0)
    xBC = torch.randn(B, L, s.xbc_dim, generator=gen, device=cuda, dtype=torch.float16)
    dt_raw = (torch.randn(B, L, s.nheads, generator=gen, device=cuda) * 0.5 - 2.0).half()

    def forward(xb, dtb):
        x, qB, qC, b_fp, b_rmax = fused_split_rotate_quant_xBC(xb, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                                               sc["B_inv_scale"], sc["C_inv_scale"], return_b_fp=True,
                                                               return_b_rowmax=True)
        out, _ = M._quant_mamba_chunk_scan_combined_fwd(
            x, dtb, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk,
            p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
            static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], keyside=True,
            x_scale_hp=sc["x_scale_hp"], b_fp=b_fp, b_gate_scale=sc["b_gate_scale"], b_rowmax=b_rmax)
        return out

    print("mamba2 large: full launch", flush=True)
    full = forward(xBC, dt_raw)
    torch.cuda.synchronize()
    assert full.numel() > 2 ** 31 and torch.isfinite(full[-1]).all()
    for b in _rows(B):
        print("mamba2 large: row", b, flush=True)
        one = forward(xBC[b:b + 1], dt_raw[b:b + 1])
        assert torch.equal(full[b:b + 1], one), f"batch row {b} of the {B}-row launch differs from its own launch"


@pytest.mark.parametrize("cell", ["linear_none", "gla", "gated_deltanet", "kda"])
def test_zoo_beyond_2_31_elements(cuda, cell):
    from linquant_amd.kernels import zoo

    B, T, H, K, V = 34, 8192, 64, 128, 128                     # q, k, v: 34 * 8192 * 64 * 128 = 2.28e9 elements each
    assert B * T * H * K > 2 ** 31
    gen = torch.Generator(device=cuda).manual_seed(0)
    q = torch.randn(B, T, H, K, generator=gen, device=cuda, dtype=torch.float16)
    k = torch.randn(B, T, H, K, generator=gen, device=cuda, dtype=torch.float16)
    k = k / k.float().norm(dim=-1, keepdim=True).clamp_min(1e-6).half()
    v = torch.randn(B, T, H, V, generator=gen, device=cuda, dtype=torch.float16)
    full = lambda shape, val: torch.full(shape, val, device=cuda, dtype=torch.float32)  # noqa: E731
    sc = {"q": full((H,), 4.0 / 127 * K ** -0.5), "k": full((H,), 0.4 / 127), "w": full((H,), 0.8 / 127),
          "kw": full((H, K), 0.4 / 127), "vw": full((H, V), 4.0 / 127), "vl": full((H, V), 4.0 / 127),
          "el": full((H, V), 8.0 / 127), "ew": full((H, V), 8.0 / 127), "state": full((H, V), 0.05)}
    if cell in ("kda", "gla"):
        g = torch.nn.functional.logsigmoid(torch.randn(B, T, H, K, generator=gen, device=cuda) + 1.0)
    if cell in ("kda", "gated_deltanet"):
        beta = torch.sigmoid(torch.randn(B, T, H, generator=gen, device=cuda))
    if cell == "kda":
        def forward(sl):
            return zoo.chunk_kda_int8(q[sl], k[sl], v[sl], g[sl], beta[sl], sc, sigma=0.5, eta=0.0, output_final_state=True)
    elif cell == "gla":
        def forward(sl):
            return zoo.chunk_gla_int8(q[sl], k[sl], v[sl], g[sl], sc, eta=0.0, output_final_state=True)
    elif cell == "gated_deltanet":
        gs = torch.nn.functional.logsigmoid(torch.randn(B, T, H, generator=gen, device=cuda) + 2.0)

        def forward(sl):
            return zoo.chunk_delta_int8(q[sl], k[sl], v[sl], gs[sl], beta[sl], sc, sigma=0.5, eta=1.0, output_final_state=True)
    else:
        def forward(sl):
            return zoo.chunk_simple_gla_int8(q[sl], k[sl], v[sl], None, sc, eta=1.0, output_final_state=True)

    print("zoo large", cell, ": full launch", flush=True)
    o_full, ht_full = forward(slice(0, B))
    torch.cuda.synchronize()
    assert o_full.numel() > 2 ** 31 and torch.isfinite(o_full[-1]).all()
    for b in _rows(B):
        print("zoo large", cell, ": row", b, flush=True)
        o_one, ht_one = forward(slice(b, b + 1))
        assert torch.equal(o_full[b:b + 1], o_one), f"{cell}: batch row {b} of the {B}-row launch differs from its own launch"
        assert torch.equal(ht_full[b:b + 1], ht_one), f"{cell}: final state of batch row {b} differs"


def test_front_and_epilogue_stages_beyond_2_31_elements(cuda):
    """Activation quantizer, causal conv1d + SiLU and the fused gated RMSNorm + Hadamard + INT8 stage on tensors of more
    than 2^31 elements: slices at the start, across the 2^31-element mark and at the end equal the launch on the slice."""
    from linquant_amd import hadamard_utils as HU
    from linquant_amd.kernels.mamba2.causal_conv1d import causal_conv1d_fn
    from linquant_amd.norm import rmsnorm_gated_qhad
    from linquant_amd.w4a8_linear import _fused_fp16_to_int8

    gen = torch.Generator(device=cuda).manual_seed(0)
    # ---- activation quantizer: 900 000 rows x 2560
    M, N = 900_000, 2560
    assert M * N > 2 ** 31
    x = torch.randn(M, N, generator=gen, device=cuda, dtype=torch.float16)
    scale = torch.tensor(4.0 / 127, device=cuda)
    print("large: fp16_to_int8", flush=True)
    q = _fused_fp16_to_int8(x, scale)
    mark = 2 ** 31 // N
    for r0 in (0, mark - 8, M - 1000):
        assert torch.equal(q[r0:r0 + 1000], _fused_fp16_to_int8(x[r0:r0 + 1000], scale)), f"rows from {r0}"
    del x, q
    # ---- conv1d + SiLU: 52 batch rows of the c5 layer's xBC slice inside the in_proj output
    B, L, D = 52, 8192, 5376
    assert B * L * D > 2 ** 31
    proj = torch.randn(B, L, D + 80, generator=gen, device=cuda, dtype=torch.float16)
    xin = proj[..., :D].transpose(1, 2)                        # (B, D, L) channel-last view with a padded row stride
    w = (torch.randn(D, 4, generator=gen, device=cuda) * 0.5).half()
    bias = (torch.randn(D, generator=gen, device=cuda) * 0.1).half()
    print("large: conv1d", flush=True)
    y = causal_conv1d_fn(xin, w, bias, activation="silu")
    for b in _rows(B):
        assert torch.equal(y[b:b + 1], causal_conv1d_fn(xin[b:b + 1], w, bias, activation="silu")), f"conv batch row {b}"
    del proj, xin, y
    # ---- gated RMSNorm + Hadamard + INT8: 450 000 rows x 5120
    R, d_ssm = 450_000, 5120
    assert R * d_ssm > 2 ** 31
    HU.register_hadamard(40, HU.hadamard_matrix(40))
    yv = torch.randn(R, d_ssm, generator=gen, device=cuda, dtype=torch.float16)
    zv = torch.randn(R, d_ssm, generator=gen, device=cuda, dtype=torch.float16)
    wn = (1 + 0.1 * torch.randn(d_ssm, generator=gen, device=cuda)).half()
    print("large: norm + hadamard", flush=True)
    qo = rmsnorm_gated_qhad(yv, zv, wn, 4.0 / 127, 1e-5, d_ssm)
    codes = qo[0] if isinstance(qo, tuple) else qo
    mark = 2 ** 31 // d_ssm
    for r0 in (0, mark - 8, R - 512):
        part = rmsnorm_gated_qhad(yv[r0:r0 + 512], zv[r0:r0 + 512], wn, 4.0 / 127, 1e-5, d_ssm)
        part = part[0] if isinstance(part, tuple) else part
        assert torch.equal(codes[r0:r0 + 512], part), f"norm rows from {r0}"


def test_long_sequences(cuda):
    """262 144 tokens per sequence (1024 Mamba-2 chunks, 4096 zoo chunks): two batch rows holding the same data give the
    same bits although the second lies beyond 2^31 elements, and the causal prefix equals a launch on the prefix alone."""
    from linquant_amd.calibration import Mamba2Shape, calibrate_mamba2, mamba2_params, mamba2_synthetic
    from linquant_amd.kernels import zoo
    from linquant_amd.kernels.mamba2 import ssd_combined as M
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC

    L = 262_144
    s = Mamba2Shape(batch=2, seqlen=L, nheads=80, headdim=64, dstate=128, ngroups=1, chunk=256)
    p = mamba2_params(s, 42, cuda, a_max=1.3)                  # weak decay: the state carries across many chunks
    cal = Mamba2Shape(batch=1, seqlen=2048, nheads=s.nheads, headdim=s.headdim, dstate=s.dstate, ngroups=1, chunk=256)
    cx, cdt = mamba2_synthetic(cal, 1, cuda, dt_mean=-4.5)
    sc = calibrate_mamba2(cal, cx, cdt, p)
    gen = torch.Generator(device=cuda).manual_seed(0)
    row = torch.randn(1, L, s.xbc_dim, generator=gen, device=cuda, dtype=torch.float16)
    dt_row = (torch.randn(1, L, s.nheads, generator=gen, device=cuda) * 0.5 - 4.5).half()
    xBC, dt_raw = row.repeat(2, 1, 1), dt_row.repeat(2, 1, 1)
    assert xBC.numel() > 2 ** 31
    del row

    def forward(xb, dtb):
        x, qB, qC, b_fp, b_rmax = fused_split_rotate_quant_xBC(xb, p["r_signs"], s.nheads, s.ngroups, s.dstate, s.headdim,
                                                               sc["B_inv_scale"], sc["C_inv_scale"], return_b_fp=True,
                                                               return_b_rowmax=True)
        out, _ = M._quant_mamba_chunk_scan_combined_fwd(
            x, dtb, p["dt_scale"], p["A_log"], p["A_log_scale"], qB, sc["B_scale"], qC, sc["C_scale"], s.chunk,
            p["D"], p["D_scale"], dt_bias=p["dt_bias"], dt_softplus=True, static_state_scale=sc["static_state_scale"],
            static_cb_scale=sc["static_cb_scale"], alpha_hp=sc["alpha_hp"], bscale_g=sc["bscale_g"], keyside=True,
            x_scale_hp=sc["x_scale_hp"], b_fp=b_fp, b_gate_scale=sc["b_gate_scale"], b_rowmax=b_rmax)
        return out

    print("long: mamba2", flush=True)
    out = forward(xBC, dt_raw)
    assert torch.isfinite(out[1, -256:]).all()
    assert torch.equal(out[0], out[1]), "two batch rows with the same data differ"
    short = forward(xBC[:1, :8192], dt_raw[:1, :8192])
    assert torch.equal(out[:1, :8192], short), "causal prefix differs from the launch on the prefix"
    del out, short, xBC, dt_raw

    B, T, H, K, V = 3, L, 24, 128, 128
    assert B * T * H * K > 2 ** 31
    q1 = torch.randn(1, T, H, K, generator=gen, device=cuda, dtype=torch.float16)
    k1 = torch.randn(1, T, H, K, generator=gen, device=cuda, dtype=torch.float16)
    k1 = k1 / k1.float().norm(dim=-1, keepdim=True).clamp_min(1e-6).half()
    v1 = torch.randn(1, T, H, V, generator=gen, device=cuda, dtype=torch.float16)
    g1 = torch.nn.functional.logsigmoid(torch.randn(1, T, H, K, generator=gen, device=cuda) + 1.0)
    b1 = torch.sigmoid(torch.randn(1, T, H, generator=gen, device=cuda))
    q, k, v, g, beta = (t.repeat(B, *([1] * (t.dim() - 1))) for t in (q1, k1, v1, g1, b1))
    del q1, k1, v1, g1, b1
    full = lambda shape, val: torch.full(shape, val, device=cuda, dtype=torch.float32)  # noqa: E731
    zs = {"q": full((H,), 4.0 / 127 * K ** -0.5), "k": full((H,), 0.4 / 127), "w": full((H,), 0.8 / 127),
          "kw": full((H, K), 0.4 / 127), "el": full((H, V), 8.0 / 127), "ew": full((H, V), 8.0 / 127),
          "state": full((H, V), 0.05)}
    print("long: kda", flush=True)
    o, ht = zoo.chunk_kda_int8(q, k, v, g, beta, zs, sigma=0.5, eta=0.0, output_final_state=True)
    assert torch.isfinite(o[-1, -64:]).all() and torch.isfinite(ht).all()
    assert torch.equal(o[0], o[2]) and torch.equal(ht[0], ht[2]), "batch rows with the same data differ"
    o_s, _ = zoo.chunk_kda_int8(q[:1, :4096], k[:1, :4096], v[:1, :4096], g[:1, :4096], beta[:1, :4096], zs, sigma=0.5, eta=0.0)
    assert torch.equal(o[:1, :4096], o_s), "causal prefix differs from the launch on the prefix"
