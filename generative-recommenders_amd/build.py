"""Compile ``csrc/`` into ``csrc/libhstu_hip.so`` and ``csrc/libhstu_linear.so`` with hipcc for gfx950 (cross-compiles
without a GPU)."""

import os
import shutil
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(_HERE), "include")
LIB_PATH = os.path.join(CSRC, "libhstu_hip.so")
LINEAR_LIB_PATH = os.path.join(CSRC, "libhstu_linear.so")  # separate: it links hipBLASLt, the attention library does not

# -packed-fp32-ops off: hipcc must not fuse scalar float code into v_pk_*_f32 on this hardware pool.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-fPIC",
    "-shared",
]


def build_library(verbose: bool = False) -> str:
    """Always recompiles; returns the path of the shared library."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc] + HIPCC_FLAGS + ["-I", INCLUDE, "-I", CSRC, os.path.join(CSRC, "hstu_api.hip"), "-o", LIB_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout + proc.stderr)
    if verbose:
        print(" ".join(cmd))
    cmd = [hipcc] + HIPCC_FLAGS + ["-I", INCLUDE, "-I", CSRC, os.path.join(CSRC, "hstu_linear.hip"), "-o", LINEAR_LIB_PATH, "-lhipblaslt"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout + proc.stderr)
    if verbose:
        print(" ".join(cmd))
    return LIB_PATH
