"""Builds libsjvp.so (the gfx950 attention-JVP kernels + C ABI) in-tree with hipcc.

The kernels are instantiated in several translation units (one per kernel family and element type)
that are compiled in parallel and linked into one shared library."""
from __future__ import annotations

import hashlib
import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_PATH = os.path.join(PKG_DIR, "libsjvp.so")
# (source, element types it is compiled for: the unit instantiates its kernels for -DSJVP_T=<type>)
UNITS = [(name, ("Bf16", "Fp16") if name.startswith("sjvp_tu_") else (None,))
         for name in sorted(os.listdir(CSRC)) if name.endswith(".hip")]
SOURCES = [os.path.join(CSRC, name) for name, _ in UNITS]
HEADERS = sorted(os.path.join(CSRC, n) for n in os.listdir(CSRC) if n.endswith(".hpp")) + [
    os.path.join(os.path.dirname(PKG_DIR), "include", "sjvp.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# Flags of single units.  The row-owned and column-owned backward kernels gain about 1 % from the
# scheduler that orders for instruction-level parallelism (measured on the MI355X at head dimensions 64 and
# 128); the single-launch backward loses 2 % with it and the forward is unchanged, so they keep the default.
UNIT_FLAGS = {"sjvp_tu_pair16.hip": ["-mllvm", "-amdgpu-sched-strategy=max-ilp"]}


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (expected on PATH or at /opt/rocm/bin/hipcc)")


def source_id() -> str:
    """Identifier of the sources the library is built from: a hash of their contents and the flags."""
    h = hashlib.sha256((" ".join(HIPCC_FLAGS) + repr(sorted(UNIT_FLAGS.items()))).encode())
    for path in SOURCES + HEADERS:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def built_id(path: str = LIB_PATH) -> str | None:
    """The source identifier embedded in a built library (read from the file, nothing is loaded)."""
    try:
        with open(path, "rb") as f:
            m = re.search(rb"SJVP_BUILD_ID=([0-9a-f]{16})", f.read())
    except OSError:
        return None
    return m.group(1).decode() if m else None


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)


def build(verbose: bool = False, jobs: int | None = None) -> str:
    """Compile every translation unit unconditionally and link; returns the path of the library."""
    hipcc = hipcc_path()
    os.makedirs(OBJ_DIR, exist_ok=True)
    cmds, objs = [], []
    build_id = f'-DSJVP_BUILD_ID="SJVP_BUILD_ID={source_id()}"'
    for name, types in UNITS:
        for t in types:
            obj = os.path.join(OBJ_DIR, name[:-4] + (f"_{t}" if t else "") + ".o")
            define = [f"-DSJVP_T={t}"] if t else ([build_id] if name == "sjvp_api.hip" else [])
            cmds.append([hipcc, *HIPCC_FLAGS, *UNIT_FLAGS.get(name, []), *define, "-c", os.path.join(CSRC, name),
                         "-o", obj])
            objs.append(obj)
    jobs = jobs or min(len(cmds), os.cpu_count() or 4, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH + ".tmp", *objs], verbose)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


def is_stale() -> bool:
    """True when no library is built or it was built from other sources than the ones in the tree
    (compared by content, so copying or checking out the tree does not matter)."""
    return built_id() != source_id()


if __name__ == "__main__":
    print(build(verbose=True))
