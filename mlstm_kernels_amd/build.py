"""Builds libmlstm_hip.so (gfx950 only) in-tree with plain hipcc: one object per kernel translation unit,
compiled in parallel, then one shared library with the C ABI declared in include/mlstm_hip.h."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libmlstm_hip.so")
OBJ_DIR = os.path.join(PKG_DIR, "build")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffast-math" if False else "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP library cannot be built on this machine")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    if out.strip():
        print(out, file=sys.stderr)


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def build(verbose: bool = True, jobs: int = 8) -> str:
    """Compile every HIP source for gfx950 and link libmlstm_hip.so.  Always recompiles."""
    hipcc = _hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(OBJ_DIR, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        if verbose:
            print(f"[mlstm_kernels_amd.build] hipcc {os.path.basename(src)}", file=sys.stderr)
        _run([hipcc, *HIPCC_FLAGS, "-c", src, "-o", obj])

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(compile_one, zip(srcs, objs)))
    tmp = LIB_PATH + ".tmp"
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[mlstm_kernels_amd.build] linked {LIB_PATH}", file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    build()
