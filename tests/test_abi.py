"""CPU checks of the drop-in boundary: the C-ABI library loads, exports every symbol the public header
declares, its struct layouts agree with the binding, and the Python wrappers enforce the reference's host-side
contracts before any launch (no compute call is made here)."""

import ctypes
import re
from pathlib import Path

import pytest
import torch

from linquant_amd import _lib

ROOT = Path(__file__).resolve().parents[1]


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    header = (ROOT / "include" / "linquant_hip.h").read_text()
    declared = re.findall(r"^\s*int\s+(lq_\w+)\s*\(", header, flags=re.M)
    assert len(declared) >= 10 and set(declared) == set(_lib.FUNCTIONS)
    for name in declared:
        assert getattr(lib, name) is not None, name
    assert lib.lq_abi_version() == _lib.ABI_VERSION


def test_struct_layouts_match_the_library():
    lib = _lib.load()
    assert len(_lib.STRUCTS) >= 8
    for name, st in _lib.STRUCTS.items():
        assert lib.lq_args_size(name.encode()) == ctypes.sizeof(st), name
    assert lib.lq_args_size(b"no_such_struct") < 0


def test_every_declaration_cites_the_reference():
    header = (ROOT / "include" / "linquant_hip.h").read_text()
    for m in re.finditer(r"/\*((?:(?!\*/).)*?)\*/\s*typedef struct", header, flags=re.S):
        text = m.group(1)
        assert re.search(r"(linquant|scripts|bench)/[\w/]+\.py:\d+", text) or "no counterpart in the reference" in text, text[:80]


def test_null_and_shape_errors_without_launch():
    """Argument validation happens on the host before anything touches a device."""
    lib = _lib.load()
    st = _lib.STRUCTS["lq_state_passing_args"]()
    assert lib.lq_state_passing(ctypes.byref(st), None) == -14  # missing pointers
    st2 = _lib.STRUCTS["lq_chunk_cumsum_args"]()
    assert lib.lq_chunk_cumsum(ctypes.byref(st2), None) == -14
    buf = (ctypes.c_char * 64)()
    for f in ("dt", "dt_scale", "A_log", "A_log_scale", "dt_out", "dA_cumsum"):
        setattr(st2, f, ctypes.addressof(buf))
    st2.batch, st2.seqlen, st2.nheads, st2.chunk_size = 1, 64, 1, 48  # chunk not a multiple of 64
    assert lib.lq_chunk_cumsum(ctypes.byref(st2), None) == -22


def test_one_call_forward_validates_every_stage_limit_before_the_first_launch():
    """lq_ssd_combined / lq_ssd_combined_static check the intersection of their five stages' limits up front: a call
    that one of the later stages would refuse returns its code without having queued a kernel (no device is touched
    here: the buffers are host memory, and a launch on them would fail differently)."""
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    ptrs = ("x", "dt", "qC", "out", "b_fp", "qB", "dt_scale", "A_log", "A_log_scale", "state_scale", "cb_scale", "C_scale",
            "B_scale", "alpha_hp", "bscale_g", "x_scale_hp", "b_gate_scale", "workspace")

    def args(**kw):
        st = _lib.fill("lq_ssd_combined_args", batch=1, seqlen=512, nheads=4, headdim=64, ngroups=1, dstate=128,
                       chunk_size=256, gate_shift=7, workspace_bytes=1 << 40)
        for f in ptrs:
            setattr(st, f, ctypes.addressof(buf))
        for k, v in kw.items():
            setattr(st, k, v)
        return st

    for entry in (lib.lq_ssd_combined, lib.lq_ssd_combined_static):
        assert entry(ctypes.byref(args(chunk_size=1024)), None) == -22     # only the chunk scan refuses it
        assert entry(ctypes.byref(args(chunk_size=192)), None) == -22
        assert entry(ctypes.byref(args(dstate=320)), None) == -22
        assert entry(ctypes.byref(args(headdim=48)), None) == -22
        assert entry(ctypes.byref(args(nheads=3, ngroups=2)), None) == -22
        assert entry(ctypes.byref(args(gate_shift=16)), None) == -22
        for missing in ("state_scale", "cb_scale", "C_scale", "B_scale", "dt_scale", "A_log"):
            assert entry(ctypes.byref(args(**{missing: None})), None) == -14, missing
        assert entry(ctypes.byref(args(keyside=1, x_scale_hp=None)), None) == -14
        assert entry(ctypes.byref(args(keyside=0, alpha_hp=None)), None) == -14
        assert entry(ctypes.byref(args(D=ctypes.addressof(buf), D_scale=None)), None) == -14


def test_zoo_chunk_size_128_is_taken_where_it_is_built_and_refused_elsewhere():
    """128-token chunks exist for raw operands: the entry points refuse every other combination on the host (the buffers here are host memory: a call that passed
    validation would launch, so only refusals are exercised)."""
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    a = ctypes.addressof(buf)
    dims = dict(batch=1, seqlen=256, nheads=1, kdim=64, vdim=64, qmax=127, act_dtype=_lib.LQ_DT_F16)

    def rc(fn, **kw):
        known = {n for n, _ in _lib.STRUCTS[fn + "_args"]._fields_}
        return getattr(lib, fn)(ctypes.byref(_lib.fill(fn + "_args", **{k: v for k, v in {**dims, **kw}.items() if k in known})), None)

    wc = dict(key=a, kqT=a, ev=a, gam=a, skw=a, val=a, vqT=a, svw=a, g=a, chunk_size=128)
    assert rc("lq_zoo_write_codes", **{**wc, "seqlen": 192}, decay=1) == -22        # not a whole number of chunks
    assert rc("lq_zoo_write_codes", **{**wc, "chunk_size": 320, "seqlen": 640}, decay=1) == -22
    assert rc("lq_zoo_write_codes", **{**wc, "chunk_size": 256, "seqlen": 512}, decay=2, logenv=a) == -22   # per-channel decay: up to 128
    stt = dict(kqT=a, gam=a, h_i8=a, skw=a, svw=a, ss=a, vqT=a, chunk_size=128)
    assert rc("lq_zoo_state", **{**stt, "seqlen": 192}, family=0) == -22
    out = dict(h_i8=a, o=a, sq=a, svl=a, ss=a, q=a, k=a, v=a, sk=a, g=a, chunk_size=128, scale=1.0)
    assert rc("lq_zoo_output", **out, decay=1) == -14                                         # no cross workspace
    assert rc("lq_zoo_output", **out, decay=2, A=a, qg=a, cross=a) == -14                     # per-channel decay: no A_cross
    assert rc("lq_zoo_output", **out, decay=1, cross=a, qc=a, kc=a, vc=a) == -22              # ready-made codes
    assert rc("lq_zoo_output", **{**out, "seqlen": 192}, decay=1, cross=a) == -22
    # 192 and 256 tokens: linear family with no / scalar decay in rotated storage only
    assert rc("lq_zoo_state", **{**stt, "chunk_size": 256, "seqlen": 512}, family=1, wq=a, u=a, fw=a, ev=a, e_out=a, sw=a) == -22
    assert rc("lq_zoo_output", **{**out, "chunk_size": 192, "seqlen": 384}, decay=2, A=a, qg=a, cross=a, A_cross=a) == -22
    assert rc("lq_zoo_output", **{**out, "chunk_size": 256, "seqlen": 512}, decay=1, cross=a, unrot=a) == -22
    ga = dict(q=a, k=a, g=a, A=a, sq=a, sk=a, chunk_size=128, scale=1.0)
    assert rc("lq_zoo_gla_A", **ga) == -14                                                    # no A_cross
    assert rc("lq_zoo_gla_A", **{**ga, "seqlen": 192}, A_cross=a) == -22
    wy = dict(k=a, v=a, beta=a, Hw=a, W=a, U=a, fw=a, g=a, chunk_size=128, decay=1)
    assert rc("lq_zoo_wy_prep", **wy, kqT=a, wq=a, ev=a, gam=a, skw=a, sw=a) == -22           # no write codes at 128
    assert rc("lq_zoo_wy_prep", **{**wy, "W": None}) == -14
    assert rc("lq_zoo_wy_prep", **{**wy, "seqlen": 192}) == -22
    cs = dict(g=a, gc=a, logenv=a, chunk_size=128)
    assert rc("lq_zoo_cumsum", **cs, kqT=a, k=a, v=a, vqT=a, ev=a, gam=a, skw=a, svw=a) == -22   # no write codes at 128
    assert rc("lq_zoo_cumsum", **{**cs, "chunk_size": 96}) == -22


def test_every_entry_point_rejects_an_empty_argument_struct():
    """A zeroed argument struct (every pointer NULL, every size 0) and a NULL struct pointer come back as an error code
    from every entry point: nothing is launched and no device is touched."""
    lib = _lib.load()
    checked = 0
    for fn in _lib.FUNCTIONS:
        sname = _lib._SHARED_ARGS.get(fn, fn + "_args")
        if sname not in _lib.STRUCTS:
            continue
        f = getattr(lib, fn)
        if fn == "lq_ssd_combined_workspace_bytes":   # (args, int64_t* bytes)
            f.argtypes = [ctypes.POINTER(_lib.STRUCTS[sname]), ctypes.c_void_p]
        st = _lib.STRUCTS[sname]()
        assert f(ctypes.byref(st), None) in (-14, -22), fn
        assert f(None, None) in (-14, -22), fn
        checked += 1
    assert checked >= 20


def test_wrapper_contracts_raise_assertion_errors():
    from linquant_amd.kernels.hadamard import kronecker_hadamard_fwd
    from linquant_amd.kernels.mamba2.bmm_chunk import _quant_bmm_chunk_fwd
    from linquant_amd.kernels.mamba2.chunk_cumsum import _quant_chunk_cumsum_fwd
    from linquant_amd.kernels.mamba2.chunk_state_keyside import _bgs_strides
    from linquant_amd.kernels.mamba2.fused_split_rotate_xBC import fused_split_rotate_quant_xBC, prepare_dqk

    one = torch.ones(())
    with pytest.raises(AssertionError):  # xBC_dim mismatch (fused_split_rotate_xBC.py:270)
        fused_split_rotate_quant_xBC(torch.zeros(1, 8, 100, dtype=torch.float16), None, 1, 1, 64, 64, one, one)
    with pytest.raises(AssertionError):  # A_log shape (chunk_cumsum.py:79)
        _quant_chunk_cumsum_fwd(torch.zeros(1, 64, 2), one, torch.zeros(3, dtype=torch.int8), one, 64)
    with pytest.raises(AssertionError):  # dt_bias shape (chunk_cumsum.py:81)
        _quant_chunk_cumsum_fwd(torch.zeros(1, 64, 2), one, torch.zeros(2, dtype=torch.int8), one, 64, dt_bias=torch.zeros(3))
    with pytest.raises(AssertionError):  # D >= 64 (hadamard.py:152)
        kronecker_hadamard_fwd(torch.zeros(1, 4, 1, 32, dtype=torch.float16), torch.ones(1, 32), 1)
    with pytest.raises(AssertionError):  # static_cb_scale shape (bmm_chunk.py:174)
        _quant_bmm_chunk_fwd(torch.zeros(1, 64, 2, 64, dtype=torch.int8), torch.ones(2), torch.zeros(1, 64, 2, 64, dtype=torch.int8),
                             torch.ones(2), 64, torch.ones(3))
    with pytest.raises(AssertionError):  # 4-D b_gate_scale (chunk_state_keyside.py:338)
        _bgs_strides(torch.ones(2, 64))
    assert _bgs_strides(torch.ones(1, 1, 4, 64)) == (0, 0, 64, 1)
    d = prepare_dqk(torch.tensor([[1.0001, 2.0]]))
    assert d.dtype == torch.float32 and d.shape == (2,) and float(d[0]) == float(torch.tensor(1.0001).half())


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.LinQuantHipError):
        _lib.load()


def binding_example():
    """The ctypes binding example of the integration notes (the fenced block that defines lq_state_passing_args), as
    source text."""
    text = (ROOT / "INTEGRATION.md").read_text()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    (block,) = [b for b in blocks if "class lq_state_passing_args" in b]
    return block


def test_documented_binding_example_matches_the_library(monkeypatch):
    """The documented stub is executed as written: it loads the library by its in-tree path, checks the ABI version
    and passes its own lq_args_size assertion; its struct has the header's field names in the header's order."""
    monkeypatch.chdir(ROOT)
    ns = {}
    exec(compile(binding_example(), "binding_example", "exec"), ns)
    st = ns["lq_state_passing_args"]
    assert [n for n, _ in st._fields_] == [n for n, _ in _lib.STRUCTS["lq_state_passing_args"]._fields_]
    assert ctypes.sizeof(st) == ctypes.sizeof(_lib.STRUCTS["lq_state_passing_args"])
    assert callable(ns["_fixedpoint_state_passing_fwd"])
