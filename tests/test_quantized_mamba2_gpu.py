"""GPU test of the mixer module: every stage is checked against the CPU restatements on the tensors the module itself
fed it (captured through the ``_debug`` hook), so a wrong slice, stride, scale or argument order in the glue shows up
at the stage where it happens.  The two fp16 GEMMs are torch's; they are compared with an fp32 numpy product."""

import numpy as np
import pytest
import torch

from oracle import mamba2_epilogue as OE
from oracle import mamba2_front as OF
from oracle import mamba2_ssd as OS

pytestmark = pytest.mark.gpu


def npy(t):
    return None if t is None else t.detach().cpu().numpy()


def build(keyside=False, ngroups=1, nheads=8, chunk=64, seqlen=256, d_state=128):
    from linquant_amd.quantized_mamba2 import random_calibrated_mixer

    return random_calibrated_mixer(d_model=256, nheads=nheads, headdim=64, d_state=d_state, ngroups=ngroups,
                                   chunk_size=chunk, batch=2, seqlen=seqlen, keyside=keyside, seed=3)


def gemm_close(got, a, w, name):
    ref = a.astype(np.float32) @ w.astype(np.float32).T
    g = npy(got).astype(np.float32).reshape(ref.shape)
    tol = 4 * np.spacing(np.abs(ref).astype(np.float16)).astype(np.float32) + 1e-3 * np.abs(ref).max()
    assert (np.abs(g - ref) <= tol).all(), name


@pytest.mark.parametrize("keyside,ngroups", [(False, 1), (True, 1), (False, 2)])
def test_mixer_stage_by_stage(cuda, keyside, ngroups):
    from linquant_amd import hadamard_utils as HU

    m, hidden = build(keyside=keyside, ngroups=ngroups)
    gen = torch.Generator().manual_seed(11)
    hidden = (torch.randn(hidden.shape, generator=gen) * 0.9).half().cuda()    # not the calibration batch
    m.register_buffer("comp_out", (torch.randn(m.d_model, generator=gen) * 0.01).half().cuda())
    dbg = {}
    out = m(hidden, _debug=dbg)
    torch.cuda.synchronize()
    B, L, _ = hidden.shape
    d_ssm, gn, H = m.d_ssm, m.ngroups * m.d_state, m.nheads
    assert out.shape == (B, L, m.d_model) and out.dtype == torch.float16 and torch.isfinite(out).all()

    # 1. activation quantizer (bit-exact) and in_proj
    s_in = np.float32(m.in_proj.input_scale.item())
    h_ref = OF.fp16_to_int8(npy(hidden).reshape(-1, m.d_model), s_in, -128.0, False)
    assert np.array_equal(npy(dbg["h_i8"]).reshape(-1, m.d_model), h_ref)
    a_in = (h_ref.astype(np.float32) * s_in).astype(np.float16)
    gemm_close(dbg["projected"], a_in, npy(m.in_proj.weight), "in_proj")

    # 2. conv + SiLU on the xBC slice of the module's own projection
    proj = npy(dbg["projected"])
    z, xBC_raw, dt = proj[..., :d_ssm], proj[..., d_ssm:d_ssm + m.conv_dim], proj[..., d_ssm + m.conv_dim:]
    assert dt.shape[-1] == H
    conv_ref = OF.causal_conv1d_silu(xBC_raw, npy(m.conv1d.weight).reshape(m.conv_dim, -1), npy(m.conv1d.bias))
    xBC = npy(dbg["xBC"])
    assert (np.abs(xBC.astype(np.float64) - conv_ref.astype(np.float64)) <= np.spacing(np.abs(conv_ref)).astype(np.float64)).all()

    # 3. prologue on the module's own conv output: codes bit-exact, x a view
    x_ref, qB_ref, qC_ref = OS.split_rotate_quant_xBC(xBC, npy(m.r_signs), H, m.ngroups, m.d_state, m.headdim,
                                                      npy(m.B_inv_scale), npy(m.C_inv_scale))
    assert np.array_equal(npy(dbg["q_B"]), qB_ref) and np.array_equal(npy(dbg["q_C"]), qC_ref)
    assert np.array_equal(npy(dbg["x_fp"]), x_ref)
    b_fp = None
    if keyside:
        b_fp = OS.kron_hadamard(xBC[..., d_ssm:d_ssm + gn].reshape(B, L, m.ngroups, m.d_state), npy(m.r_signs))
        assert np.array_equal(npy(dbg["b_fp"]), b_fp)

    # 4. SSD
    ref = OS.ssd_combined(x_ref, dt, 1.0, npy(m.A_log), float(m.A_log_scale), qB_ref, npy(m.B_scale), qC_ref,
                          npy(m.C_scale), m.chunk_size, npy(m.D), float(m.D_scale), dt_bias=npy(m.dt_bias),
                          dt_softplus=True, static_state_scale=npy(m.static_state_scale),
                          static_cb_scale=npy(m.static_cb_scale), alpha_hp=npy(m.alpha_hp), bscale_g=npy(m.bscale_g),
                          keyside=keyside, x_scale_hp=npy(getattr(m, "x_quant_scale_hp", None)), b_fp=b_fp,
                          b_gate_scale=npy(getattr(m, "b_gate_scale", None)))
    y = npy(dbg["y"]).astype(np.float64)
    y_ref = np.asarray(ref["out"], np.float64).reshape(y.shape)
    assert np.abs(y - y_ref).max() <= 1e-3 * np.abs(y_ref).max()

    # 5 + 6. gated norm + Hadamard + INT8 on the module's own y and z
    s_out = float(m.out_proj.input_scale.item())
    normed = OE.rmsnorm_gated(npy(dbg["y"]).reshape(-1, d_ssm), z.reshape(-1, d_ssm), npy(m.norm.weight), m.norm.eps,
                              m.norm.group_size)
    q_ref = OE.qhad_transform(normed, HU.chunk_matrix(d_ssm), (1.0 / np.sqrt(d_ssm)) / s_out)
    q = npy(dbg["y_i8"]).reshape(-1, d_ssm)
    diff = np.abs(q.astype(np.int32) - q_ref.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 2e-2
    assert np.abs(q).max() >= 100, "the calibrated out_proj scale should use the INT8 range"

    # out_proj + compensation
    a_out = (q.astype(np.float32) * np.float32(s_out)).astype(np.float16)
    gemm_close(out - m.comp_out, a_out, npy(m.out_proj.weight), "out_proj")


def test_fused_and_two_launch_routes_agree(cuda):
    from linquant_amd.quantized_mamba2 import _Unfused

    m, hidden = build()
    d1, d2 = {}, {}
    out1 = m(hidden, _debug=d1)
    plain = m.norm
    m.norm = _Unfused(plain)
    out2 = m(hidden, _debug=d2)
    m.norm = plain
    torch.cuda.synchronize()
    assert d1["normed"] is None and d2["normed"] is not None
    assert torch.equal(d1["y_i8"], d2["y_i8"]) and torch.equal(out1, out2)


def test_attention_mask_and_errors(cuda):
    m, hidden = build()
    B, L, _ = hidden.shape
    mask = torch.ones(B, L, dtype=torch.float16, device="cuda")
    mask[1, : L // 4] = 0                                  # left padding on the second sequence
    dbg = {}
    out = m(hidden, attention_mask=mask, _debug=dbg)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    assert (dbg["xBC"][1, : L // 4] == 0).all() and (dbg["q_B"][1, : L // 4] == 0).all()
    # the unpadded sequence is untouched by the mask of the other one
    out_ref = m(hidden)
    assert torch.equal(out[0], out_ref[0])
    with pytest.raises(NotImplementedError, match="prefill-only"):
        m(hidden, past_key_values=object())
    with pytest.raises(NotImplementedError, match="prefill-only"):
        m(hidden, inference_params=object())
    del m.alpha_hp
    with pytest.raises(RuntimeError, match="not calibrated"):
        m(hidden)


def test_stage_names_are_rebindable(cuda):
    """Per-stage timing scripts wrap the stage functions through the importing module's namespace."""
    import linquant_amd.quantized_mamba2 as QM

    m, hidden = build()
    seen = []
    names = ["_fused_fp16_to_int8", "causal_conv1d_fn", "fused_split_rotate_quant_xBC",
             "_quant_mamba_chunk_scan_combined_fwd", "rmsnorm_gated_qhad"]
    saved = {n: getattr(QM, n) for n in names}

    def wrap(n):
        def f(*a, **k):
            seen.append(n)
            return saved[n](*a, **k)
        return f

    try:
        for n in names:
            setattr(QM, n, wrap(n))
        m(hidden)
    finally:
        for n in names:
            setattr(QM, n, saved[n])
    assert seen == names
