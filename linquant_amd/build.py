"""Build liblinquant_hip.so (all HIP kernels + the C ABI) for gfx950 with hipcc.

``python -m linquant_amd.build`` compiles in-tree; the library lands next to the sources so it travels with
the repository snapshot.  hipcc cross-compiles without a GPU.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_PATH = CSRC / "liblinquant_hip.so"
ARCH = "gfx950"

# -ffp-contract=off: every fp32 multiply/add that feeds an INT8 code is rounded on its own (the CPU checker
# restates the same sequences); the packed-fp32 feature is switched off for the device pass.
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built")
    return exe


def _compile(src: Path, obj: Path) -> None:
    cmd = [_hipcc(), *FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stderr}")


def build(force: bool = True, jobs: int | None = None, verbose: bool = False) -> Path:
    """Compile every .hip source and link the shared library. Returns the library path."""
    srcs = sources()
    objdir = CSRC / "build"
    objdir.mkdir(exist_ok=True)
    headers = list(CSRC.glob("*.h")) + [CSRC.parents[1] / "include" / "linquant_hip.h"]
    newest_hdr = max(h.stat().st_mtime for h in headers)
    todo = []
    for s in srcs:
        o = objdir / (s.stem + ".o")
        if force or not o.exists() or o.stat().st_mtime < max(s.stat().st_mtime, newest_hdr):
            todo.append((s, o))
    jobs = jobs or min(8, max(1, (os.cpu_count() or 2)))
    if verbose:
        print(f"[linquant_amd.build] compiling {len(todo)}/{len(srcs)} sources with {jobs} jobs", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _compile(*so), todo))
    objs = [str(objdir / (s.stem + ".o")) for s in srcs]
    cmd = [_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", str(LIB_PATH)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--incremental" not in sys.argv, verbose=True)
    print(path)
