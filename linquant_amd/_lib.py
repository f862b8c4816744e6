"""ctypes binding of liblinquant_hip.so.

The args structs are generated from ``include/linquant_hip.h`` at import, so the Python side cannot drift
from the C ABI.  There is no fallback path: if the library is missing or a call fails, an exception is raised.
"""

from __future__ import annotations

import ctypes
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parent
HEADER = ROOT.parent / "include" / "linquant_hip.h"
LIB_PATH = ROOT / "csrc" / "liblinquant_hip.so"
ABI_VERSION = 18

LQ_DT_F16, LQ_DT_F32, LQ_DT_I8, LQ_DT_BF16 = 0, 1, 2, 3

_CTYPES = {"int64_t": ctypes.c_int64, "int32_t": ctypes.c_int32, "float": ctypes.c_float, "int": ctypes.c_int}
_ERRORS = {-14: "a required pointer is missing (LQ_E_NULL)",
           -22: "unsupported size / stride / alignment / flag (LQ_E_SHAPE)",
           -5: "kernel launch failed (LQ_E_LAUNCH)",
           -11: "set-up needed that cannot run now: stream under graph capture (LQ_E_STATE)"}


class LinQuantHipError(RuntimeError):
    pass


def parse_header(text: str | None = None):
    """Returns ({struct name: [(field, ctype)]}, [function names]) from the public header."""
    text = HEADER.read_text() if text is None else text
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    structs = {}
    for body, name in re.findall(r"typedef\s+struct\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        fields = []
        for decl in body.split(";"):
            decl = decl.strip()
            if not decl:
                continue
            m = re.match(r"(const\s+)?(\w+)\s*(\*?)\s*(.*)", decl, flags=re.S)
            base, star, names = m.group(2), m.group(3), m.group(4)
            for nm in names.split(","):
                nm = nm.strip()
                ptr = bool(star) or nm.startswith("*")
                nm = nm.lstrip("*").strip()
                fields.append((nm, ctypes.c_void_p if ptr else _CTYPES[base]))
        structs[name] = fields
    funcs = re.findall(r"^\s*int\s+(lq_\w+)\s*\(", text, flags=re.M)
    return structs, funcs


_structs, _funcs = parse_header()
STRUCTS = {name: type(name, (ctypes.Structure,), {"_fields_": fields}) for name, fields in _structs.items()}
FUNCTIONS = tuple(_funcs)

# entry points whose first argument is another function's args struct
_SHARED_ARGS = {"lq_ssd_combined_static": "lq_ssd_combined_args", "lq_ssd_combined_workspace_bytes": "lq_ssd_combined_args",
                "lq_zoo_simple_gla_workspace_bytes": "lq_zoo_simple_gla_args",
                "lq_zoo_chunk_forward_workspace_bytes": "lq_zoo_chunk_forward_args"}

_lib = None


def load():
    """Load the shared library (once). Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise LinQuantHipError(
            f"{LIB_PATH} is missing: build it with `python -m linquant_amd.build` (there is no fallback path)")
    lib = ctypes.CDLL(str(LIB_PATH))
    for fn in FUNCTIONS:
        f = getattr(lib, fn)
        f.restype = ctypes.c_int
        sname = _SHARED_ARGS.get(fn, fn + "_args")
        if sname in STRUCTS:
            f.argtypes = [ctypes.POINTER(STRUCTS[sname]), ctypes.c_void_p]
        elif fn == "lq_args_size":
            f.argtypes = [ctypes.c_char_p]
        else:
            f.argtypes = []
    ver = lib.lq_abi_version()
    if ver != ABI_VERSION:
        raise LinQuantHipError(f"liblinquant_hip.so has ABI version {ver}, the Python side expects {ABI_VERSION}: rebuild")
    for name, st in STRUCTS.items():
        size = lib.lq_args_size(name.encode())
        if size != ctypes.sizeof(st):
            raise LinQuantHipError(f"{name}: library sizeof {size} != binding sizeof {ctypes.sizeof(st)}")
    _lib = lib
    return lib


def ptr(t):
    """Device pointer of a torch tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


def f32(t):
    """``t`` itself when it is fp32 (or None), else an fp32 copy: the kernels read scale tensors as fp32, where the
    reference's kernels convert on load, so an fp16 / fp64 scale buffer must not be reinterpreted."""
    import torch

    return t if t is None or t.dtype == torch.float32 else t.float()


def aligned(t, nbytes=16):
    """``t`` itself when its first byte sits on an ``nbytes`` boundary (or it is None), else a fresh copy: kernels that
    fetch small parameter tables as whole 16-byte pieces need this, and a view into a larger tensor need not have it."""
    return t if t is None or t.data_ptr() % nbytes == 0 else t.clone()


def current_stream(device):
    import torch

    return torch.cuda.current_stream(device).cuda_stream


def fill(struct_name: str, **fields):
    """An instance of the named args struct with the given fields set (unknown names raise KeyError)."""
    st = STRUCTS[struct_name]()
    known = {n for n, _ in st._fields_}
    for k, v in fields.items():
        if k not in known:
            raise KeyError(f"{struct_name} has no field {k!r}")
        setattr(st, k, v)
    return st


def launch(fn: str, device, st):
    """Call entry point ``fn`` with an already filled args struct on the current stream of ``device``."""
    lib = load()
    import torch

    with torch.cuda.device(device):
        rc = getattr(lib, fn)(ctypes.byref(st), current_stream(device))
    if rc != 0:
        raise LinQuantHipError(f"{fn} failed with code {rc}: {_ERRORS.get(rc, 'unknown error')}")


_FIELD_NAMES = {}


def call(fn: str, device, **fields):
    """Fill ``<fn>_args`` from keyword fields and launch on the current stream of ``device``."""
    lib = _lib if _lib is not None else load()
    sname = _SHARED_ARGS.get(fn, fn + "_args")
    cls = STRUCTS[sname]
    known = _FIELD_NAMES.get(sname)
    if known is None:
        known = _FIELD_NAMES[sname] = frozenset(n for n, _ in cls._fields_)
    st = cls()
    for k, v in fields.items():
        if k not in known:
            raise KeyError(f"{fn}_args has no field {k!r}")
        setattr(st, k, v)
    import torch

    # (the device guard costs several microseconds a launch: it is entered only when the tensors' device is not the current one)
    idx = device.index if getattr(device, "index", None) is not None else torch.cuda.current_device()
    if idx == torch.cuda.current_device():
        rc = getattr(lib, fn)(ctypes.byref(st), torch.cuda.current_stream(idx).cuda_stream)
    else:
        with torch.cuda.device(device):
            rc = getattr(lib, fn)(ctypes.byref(st), current_stream(device))
    if rc != 0:
        raise LinQuantHipError(f"{fn} failed with code {rc}: {_ERRORS.get(rc, 'unknown error')}")
