"""Builds libkinetics_amd.so (HIP kernels + C ABI) for gfx950, in-tree.

Run as ``python -m kinetics_amd.build``.  hipcc cross-compiles without a GPU.
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
INCLUDE = REPO_ROOT / "include"
LIB_PATH = PKG_DIR / "libkinetics_amd.so"
OBJ_DIR = PKG_DIR / "build"

SOURCES = ["kin_api.hip", "kin_append.hip", "kin_score_topk.hip", "kin_decode.hip", "kin_step.hip", "kin_token_topk.hip",
           "kin_table.hip", "kin_layer.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-result",
    # Keep the compiler from forming packed-FP32 instructions.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # The host pass does not know the packed-fp32 feature and says so; drop that line.
    out = "\n".join(ln for ln in proc.stdout.splitlines() if "is not a recognized feature" not in ln)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def build_library(verbose: bool = True) -> Path:
    """Compile every HIP source and link the shared library.  Always rebuilds."""
    hipcc = _hipcc()
    OBJ_DIR.mkdir(exist_ok=True)
    objs = []
    for src in SOURCES:
        obj = OBJ_DIR / (Path(src).stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print("[kinetics_amd.build]", " ".join(cmd), file=sys.stderr)
        _run(cmd)
        objs.append(str(obj))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(tmp)])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[kinetics_amd.build] wrote {LIB_PATH}", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
