"""Builds libcastle_hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m lookahead_keys_attention_amd.build

No torch headers are involved: the library is plain HIP behind the C ABI declared in
include/castle_hip.h and is loaded with ctypes.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libcastle_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ("castle_fwd.hip", "castle_bwd.hip", "castle_decode.hip", "castle_profile.hip", "castle_abi.hip")
ARCH = "gfx950"
# packed fp32 VALU instructions stay disabled on purpose (hipcc's host pass warns that it
# does not know the feature; that warning is harmless)
HIPCC_FLAGS = (
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l and "warning" not in l.lower() or "error" in l.lower())
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    return err


def build(verbose: bool = False, jobs: int | None = None) -> str:
    """Compile every HIP source and link the shared library; returns its path."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 8)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", LIB_PATH, *objs]
    if verbose:
        print(" ".join(link), flush=True)
    _run(link)
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose="-q" not in sys.argv)
    print(path)
