"""Builds libsjvp.so (the gfx950 attention-JVP kernels + C ABI) in-tree with hipcc."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libsjvp.so")
SOURCES = [os.path.join(CSRC, "sjvp_api.hip")]
HEADERS = sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith(".hpp")) + [
    os.path.join(os.path.dirname(PKG_DIR), "include", "sjvp.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-shared",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (expected on PATH or at /opt/rocm/bin/hipcc)")


def build(verbose: bool = False) -> str:
    """Compile unconditionally; returns the path of the shared library."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-o", LIB_PATH + ".tmp", *SOURCES]
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout + res.stderr)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


def is_stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(s) > t for s in SOURCES + HEADERS)


if __name__ == "__main__":
    print(build(verbose=True))
