"""Builds libkinetics_amd.so (HIP kernels + C ABI) for gfx950, in-tree.

Run as ``python -m kinetics_amd.build``.  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_ROOT = PKG_DIR.parent
CSRC = PKG_DIR / "csrc"
INCLUDE = REPO_ROOT / "include"
LIB_PATH = PKG_DIR / "libkinetics_amd.so"
OBJ_DIR = PKG_DIR / "build"
# The same sources with the fused step's clock stamps compiled in (-DKIN_TUNE): a diagnostic
# build for kinetics_amd/phase_timeline.py, never loaded by the operators.
PHASES_LIB_PATH = PKG_DIR / "libkinetics_amd_phases.so"

SOURCES = ["kin_api.hip", "kin_append.hip", "kin_score_topk.hip", "kin_decode.hip", "kin_step.hip", "kin_token_topk.hip", "kin_token_topk_small.hip",
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


def build_library(verbose: bool = True, defines: tuple = (), lib_path: Path = LIB_PATH, obj_dir: Path = OBJ_DIR,
                  jobs: int = 8) -> Path:
    """Compile every HIP source (``jobs`` at a time) and link the shared library.  Always rebuilds."""
    hipcc = _hipcc()
    obj_dir.mkdir(exist_ok=True)

    def compile_one(src: str) -> str:
        obj = obj_dir / (Path(src).stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *[f"-D{d}" for d in defines], f"-I{INCLUDE}", f"-I{CSRC}", "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print("[kinetics_amd.build]", " ".join(cmd), file=sys.stderr)
        _run(cmd)
        return str(obj)

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp = lib_path.with_suffix(".so.tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(tmp)])
    os.replace(tmp, lib_path)
    if verbose:
        print(f"[kinetics_amd.build] wrote {lib_path}", file=sys.stderr)
    return lib_path


def build_phases_library(verbose: bool = True) -> Path:
    """The diagnostic build with phase stamps (see PHASES_LIB_PATH)."""
    return build_library(verbose, defines=("KIN_TUNE",), lib_path=PHASES_LIB_PATH, obj_dir=PKG_DIR / "build_phases")


if __name__ == "__main__":
    build_library()
    build_phases_library()
