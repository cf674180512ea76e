"""Compile the sdv2kv HIP sources into streamdiffusionv2_amd/_lib/libsdv2kv.so.

hipcc cross-compiles for gfx950 without a GPU.  Run as
``python -m streamdiffusionv2_amd.build_ext`` or call :func:`build`.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_ROOT = PKG_DIR.parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "_lib"
LIB_PATH = LIB_DIR / "libsdv2kv.so"
SOURCES = ["sdv2kv_api.hip", "kv_append_rope.hip", "swa_attn_fwd.hip", "swa_attn_fwd_f32.hip", "sink_similarity.hip",
           "cache_relayout.hip", "rms_norm.hip", "mfma_ceiling.hip"]

# -packed-fp32-ops is switched off: the compiler would otherwise form
# v_pk_*_f32 from ordinary float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the sdv2kv extension needs ROCm's hipcc to build")
    return exe


def build(verbose: bool = False, keep_temps: bool = False) -> Path:
    """Compile every source for gfx950 and link the shared library."""
    LIB_DIR.mkdir(exist_ok=True)
    work = REPO_ROOT / "build" / "sdv2kv"
    work.mkdir(parents=True, exist_ok=True)
    objects = []
    for src in SOURCES:
        obj = work / (Path(src).stem + ".o")
        cmd = [hipcc_path(), *HIPCC_FLAGS, f"-I{REPO_ROOT / 'include'}", f"-I{CSRC}",
               "-c", str(CSRC / src), "-o", str(obj)]
        if keep_temps:
            cmd.append("-save-temps=obj")
        _run(cmd, verbose)
        objects.append(str(obj))
    tmp = LIB_DIR / "libsdv2kv.so.tmp"
    _run([hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", str(tmp)], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def ensure_built(verbose: bool = False) -> Path:
    """Build the library only when none is there.  For the entry points around
    the package (smoke run, benchmark, GPU test session): the package itself
    never builds behind the caller's back, it raises when the library is
    missing."""
    return LIB_PATH if LIB_PATH.exists() else build(verbose)


GPU_CALLER_SRC = REPO_ROOT / "tests" / "c_abi" / "gpu_caller.cpp"
GPU_CALLER_BIN = REPO_ROOT / "tests" / "c_abi" / "_bin" / "gpu_caller"


def build_gpu_caller(verbose: bool = False) -> Path:
    """The stand-alone C++ program of the GPU test suite that drives the
    library through include/sdv2kv.h with nothing but the HIP runtime; built
    here so that a GPU box only has to run it."""
    GPU_CALLER_BIN.parent.mkdir(exist_ok=True)
    _run([hipcc_path(), "-O2", "-std=c++17", "-Wno-unused-command-line-argument", "-Wno-unused-result",
          f"-I{REPO_ROOT / 'include'}", str(GPU_CALLER_SRC), "-o", str(GPU_CALLER_BIN), f"-L{LIB_DIR}", "-lsdv2kv",
          "-Wl,-rpath,$ORIGIN/../../../streamdiffusionv2_amd/_lib"], verbose)
    return GPU_CALLER_BIN


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{' '.join(cmd)}\n{res.stdout}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


if __name__ == "__main__":
    print(build(verbose=True, keep_temps="--keep-temps" in sys.argv))
    print(build_gpu_caller(verbose=True))
