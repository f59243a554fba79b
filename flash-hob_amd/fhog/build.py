"""Build libfhog_hip.so (gfx950) in-tree with hipcc.

The shared library is the only native artefact of the package: HIP kernels plus the C ABI
declared in ``include/fhog_hip.h``.  It is compiled ahead of time (hipcc cross-compiles
without a GPU); nothing is JIT-compiled at run time.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent            # .../flash-hob_amd/fhog
CSRC = PKG_DIR.parent / "csrc"
INCLUDE = PKG_DIR.parent.parent / "include"
LIB_PATH = PKG_DIR / "libfhog_hip.so"
SOURCES = ["fhog_abi.hip", "fhog_fp32.hip", "fhog_bf16.hip", "fhog_bf16_pc.hip", "fhog_bf16_ddo.hip", "fhog_attn.hip", "fhog_attn_fp32.hip", "fhog_probe.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed-fp32 VALU forms are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
] + os.environ.get("FHOG_EXTRA", "").split()   # extra hipcc flags for experiments


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libfhog_hip.so cannot be built")
    return exe


def build(verbose: bool = True, jobs: int = 7) -> Path:
    """Compile every source and link ``libfhog_hip.so`` next to this file. Always recompiles."""
    objdir = PKG_DIR.parent / "build"
    objdir.mkdir(exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = objdir / (src + ".o")
        objs.append(str(obj))
        cmd = [hipcc(), *HIPCC_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs, verbose)
    _drain(procs, verbose)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


def _drain(procs, verbose):
    for src, pr in procs:
        out, _ = pr.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
        if pr.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n" + "\n".join(lines))
        if verbose and lines:
            print("\n".join(lines), flush=True)
    procs.clear()


if __name__ == "__main__":
    build()
    print("built", LIB_PATH)
    sys.exit(0)
