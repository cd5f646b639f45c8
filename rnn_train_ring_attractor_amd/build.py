"""Build recipe of libringattr.so: hipcc, gfx950 only, in-tree output next to this file.

Usage:  python -m rnn_train_ring_attractor_amd.build   (or build_library() from Python).
Cross-compiles without a GPU.  The counterpart of the reference's JIT loader
(cpp/rnn_cuda.py:59-91), which drives nvcc through torch.utils.cpp_extension.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libringattr.so")
SOURCES = ["ring_kernels.hip", "ring_res256.hip", "ring_dw.hip", "ringattr_api.hip"]
ARCH = os.environ.get("RINGATTR_ARCH", "gfx950")

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or put /opt/rocm/bin on PATH)")


def build_library(verbose: bool = False, extra_flags=(), out_path: str = LIB_PATH) -> str:
    """Compile every HIP source into libringattr.so; raises on any compiler error."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, f"-I{INCLUDE}", f"-I{CSRC}",
           *[os.path.join(CSRC, s) for s in SOURCES], "-o", out_path + ".tmp"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + log)
    os.replace(out_path + ".tmp", out_path)
    if verbose and log.strip():
        print(log)
    return out_path


if __name__ == "__main__":
    print(build_library(verbose=True, extra_flags=sys.argv[1:]))
