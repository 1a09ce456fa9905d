"""Compiles the package's HIP libraries for gfx950 with hipcc (cross-compiles without a GPU).  ``libjacobiforcing.so`` is the
Jacobi loop body; ``libjf_layers.so`` holds the layer kernels of the models whose forward is not stock PyTorch.  Each is built
from its own sources only, so a process that needs one does not wait for the other."""
from __future__ import annotations

import os
import shutil
import subprocess
import tempfile
from pathlib import Path

_PKG = Path(__file__).resolve().parent
ROOT = _PKG.parent
CSRC = _PKG / "csrc"
LIB_DIR = _PKG / "lib"
# every translation unit is compiled without packed-fp32 instructions (the flag is for the device pass; the host pass warns)
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

LAYERS_SRCS = sorted((CSRC / "layers").glob("*.hip"))
LAYERS_DEPS = LAYERS_SRCS + [CSRC / "layers" / "jl_common.h", ROOT / "include" / "jf_layers.h"]
LAYERS_LIB = LIB_DIR / "libjf_layers.so"


def hipcc() -> str:
    return shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def stale(target: Path, deps) -> bool:
    return (not target.exists()) or target.stat().st_mtime < max(Path(d).stat().st_mtime for d in deps)


def build_layers(force: bool = False) -> Path:
    """One object per source, compiled side by side, linked into ``lib/libjf_layers.so`` (written under a temporary name and
    renamed, so that a process that starts meanwhile never loads half a file)."""
    if not (force or stale(LAYERS_LIB, LAYERS_DEPS)):
        return LAYERS_LIB
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    with tempfile.TemporaryDirectory(dir=LIB_DIR) as tmp:
        inc = [f"-I{ROOT / 'include'}", f"-I{CSRC / 'layers'}"]
        jobs = [(subprocess.Popen([hipcc(), *HIP_FLAGS, *inc, "-c", str(s), "-o", f"{tmp}/{s.stem}.o"], stderr=subprocess.PIPE, text=True), s)
                for s in LAYERS_SRCS]
        for p, s in jobs:
            _, err = p.communicate()
            if p.returncode:
                raise RuntimeError(f"hipcc failed on {s.name}:\n{err[-4000:]}")
        out = f"{tmp}/libjf_layers.so"
        subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *[f"{tmp}/{s.stem}.o" for s in LAYERS_SRCS], "-o", out])
        os.replace(out, LAYERS_LIB)
    return LAYERS_LIB
