"""Builds the HIP library (libmi355_moe.so) for gfx950 in-tree."""
from __future__ import annotations

import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libmi355_moe.so")
SOURCES = ["moe_api.hip", "pack.hip", "router.hip", "dispatch.hip", "gemm.hip", "norm.hip", "yardstick.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # hipcc -O3 may form packed fp32 ops from plain float code; keep them off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _compile(src: str, verbose: bool, extra: list[str] | None) -> str:
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [c for c in [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj] if c != "-shared"]
    cmd += extra or []
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return obj


def build_lib(verbose: bool = True, extra: list[str] | None = None) -> str:
    # one hipcc per source file, side by side (the GEMM's template instances dominate)
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1, 8)) as ex:
        objs = list(ex.map(lambda src: _compile(src, verbose, extra), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build_lib()
