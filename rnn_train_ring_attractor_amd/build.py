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
SOURCES = ["ring_kernels.hip", "ring_res256.hip", "ring_cluster.hip", "ring_dw.hip", "ring_loss.hip", "ring_gain.hip", "ring_bign.hip", "ring_block.hip", "ring_aux.hip", "ringattr_api.hip"]
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


# Per-source additions.  ring_res256.hip: accumulators of the time-loop MFMAs live in architectural
# VGPRs (the AGPR file is full of weights there), which spares one v_accvgpr_read per result register.
PER_SOURCE_FLAGS = {
    "ring_res256.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "ring_cluster.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def build_library(verbose: bool = False, extra_flags=(), out_path: str = LIB_PATH, per_source=None) -> str:
    """Compile every HIP source to an object (in parallel), link libringattr.so; raises on any compiler error."""
    per_source = PER_SOURCE_FLAGS if per_source is None else per_source
    hipcc = hipcc_path()
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    noise = "is not a recognized feature for this target"
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    jobs = []
    for src in SOURCES:
        obj = os.path.join(obj_dir, f"{os.path.basename(out_path)}.{src}.o")
        cmd = [hipcc, *compile_flags, *extra_flags, *per_source.get(src, []), f"-I{INCLUDE}", f"-I{CSRC}",
               "-c", os.path.join(CSRC, src), "-o", obj]
        jobs.append((cmd, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    logs, failed = [], None
    for cmd, obj, proc in jobs:
        out, _ = proc.communicate()
        logs.append("\n".join(l for l in out.splitlines() if noise not in l))
        if proc.returncode != 0 and failed is None:
            failed = cmd
    log = "\n".join(l for l in logs if l.strip())
    if failed is not None:
        raise RuntimeError("hipcc failed:\n" + " ".join(failed) + "\n" + log)
    link = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *[obj for _, obj, _ in jobs], "-o", out_path + ".tmp"]
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + " ".join(link) + "\n" + proc.stdout + proc.stderr)
    os.replace(out_path + ".tmp", out_path)
    if verbose and log.strip():
        print(log)
    return out_path


C_CONSUMER_SRC = os.path.join(os.path.dirname(PKG_DIR), "tests", "c_abi", "ring_c_consumer.c")
C_CONSUMER_LIB = os.path.join(os.path.dirname(PKG_DIR), "tests", "c_abi", "libring_c_consumer.so")


def build_c_consumer() -> str:
    """The plain-C consumer of the C ABI that the GPU tests run in-process: C99, compiled by the host C compiler
    against include/ringattr.h, the built library and the HIP runtime (no C++, no torch)."""
    cc = shutil.which("gcc") or shutil.which("cc")
    if not cc:
        raise RuntimeError("no C compiler found for tests/c_abi/ring_c_consumer.c")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [cc, "-std=c99", "-Wall", "-Wextra", "-O2", "-fPIC", "-shared", "-fvisibility=hidden", f"-I{INCLUDE}",
           f"-I{rocm}/include", C_CONSUMER_SRC, "-o", C_CONSUMER_LIB, f"-L{PKG_DIR}", "-lringattr", f"-L{rocm}/lib",
           "-lamdhip64", "-lm", "-Wl,-rpath,$ORIGIN/../../rnn_train_ring_attractor_amd", f"-Wl,-rpath,{rocm}/lib"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("C consumer build failed:\n" + " ".join(cmd) + "\n" + proc.stdout + proc.stderr)
    return C_CONSUMER_LIB


if __name__ == "__main__":
    print(build_library(verbose=True, extra_flags=sys.argv[1:]))
    print(build_c_consumer())
