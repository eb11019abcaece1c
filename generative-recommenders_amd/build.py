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


def _run(cmd, verbose):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + proc.stdout + proc.stderr)
    if verbose:
        print(" ".join(cmd))


def build_library(verbose: bool = False) -> str:
    """Always recompiles; returns the path of the attention library.  The translation units compile side by side
    (forward, backward, dense steps), then libhstu_hip.so is linked from the first two."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    common = [hipcc] + [f for f in HIPCC_FLAGS if f != "-shared"] + ["-I", INCLUDE, "-I", CSRC]
    objs = [os.path.join(CSRC, "hstu_api.o"), os.path.join(CSRC, "hstu_bwd_api.o")]
    jobs = [
        common + ["-c", os.path.join(CSRC, "hstu_api.hip"), "-o", objs[0]],
        common + ["-c", os.path.join(CSRC, "hstu_bwd_api.hip"), "-o", objs[1]],
        common + ["-shared", os.path.join(CSRC, "hstu_linear.hip"), "-o", LINEAR_LIB_PATH, "-lhipblaslt"],
    ]
    with ThreadPoolExecutor(max_workers=3) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB_PATH], verbose)
    for o in objs:
        os.remove(o)
    return LIB_PATH
