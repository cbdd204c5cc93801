"""Builds libmi355vit.so (gfx950) in-tree with hipcc.

Usage: ``python -m mi355_vit.build`` (with ``multimodal-training_amd`` on ``sys.path``) or call
``build_library()``.  The library lands next to this file so that it travels with the source tree.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR.parent / "csrc"
LIB_PATH = PKG_DIR / "libmi355vit.so"
SOURCES = ["planners.cpp", "block.cpp", "bandwidth.hip", "gemm.hip", "attention.hip", "optimizer.hip", "pixels.hip"]

# packed-fp32 instructions are switched off for every device translation unit
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or put /opt/rocm/bin on PATH)")


def build_library(verbose: bool = True, extra_flags: list[str] | None = None) -> Path:
    """Compile every translation unit and link the shared library.  Always rebuilds."""
    hipcc = hipcc_path()
    obj_dir = PKG_DIR.parent / "build"
    obj_dir.mkdir(exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = obj_dir / (src.rsplit(".", 1)[0] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *(extra_flags or [])]
        if src.endswith(".cpp"):
            cmd += ["-x", "hip"]
        cmd += ["-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print("[build]", " ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(str(obj))
    failed = []
    for src, proc in procs:
        out, _ = proc.communicate()
        lines = [ln for ln in out.splitlines() if "packed-fp32-ops" not in ln and ln.strip()]
        if proc.returncode != 0:
            failed.append(src)
            print("\n".join(lines), file=sys.stderr)
        elif verbose and lines:
            print("\n".join(lines))
    if failed:
        raise RuntimeError(f"hipcc failed for {failed}")
    tmp = LIB_PATH.with_suffix(".so.tmp")
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(tmp)]
    if verbose:
        print("[build]", " ".join(link), flush=True)
    subprocess.run(link, check=True)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
