"""Compiles the HIP sources under csrc/ into lib/libuniql_amd.so for gfx950.

    python -m uniql_amd.build

hipcc cross-compiles without a GPU.  The library is built in-tree so that it
travels with the source tree; nothing is installed.
"""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libuniql_amd.so")

ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared",
    # keep fp32 arithmetic scalar: packed fp32 forms are not wanted on this target
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC)")


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = True, jobs: int | None = None) -> str:
    """Always recompiles every source (one hipcc per file, a few at a time, into a temporary
    directory), links, and returns the path of the shared library."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = find_hipcc()
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    srcs = sources()
    jobs = jobs or max(1, min(len(srcs), (os.cpu_count() or 2) // 2, 8))
    with tempfile.TemporaryDirectory(prefix="uniql_build_") as tmpdir:
        objs = [os.path.join(tmpdir, os.path.basename(src)[:-4] + ".o") for src in srcs]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(lambda so: _run([hipcc, *compile_flags, f"-I{INCLUDE}", f"-I{CSRC}", "-c", so[0], "-o", so[1]],
                                          verbose), zip(srcs, objs)))
        tmp = LIB_PATH + ".tmp"
        _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", tmp], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build())
