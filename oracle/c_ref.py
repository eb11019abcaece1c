"""ctypes loader for ``libhstu_ref.so`` (built from ``hstu_ref.c``).  TEST INFRASTRUCTURE ONLY."""

import ctypes
import os
import subprocess
from typing import Optional

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhstu_ref.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-s", "-C", _HERE, "-B"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.hstu_ref_mask.argtypes = [ctypes.c_int] * 5 + [ctypes.c_void_p]
        _lib.hstu_ref_mask.restype = None
        _lib.hstu_ref_count_pairs.argtypes = [ctypes.c_int] * 6
        _lib.hstu_ref_count_pairs.restype = ctypes.c_longlong
        _lib.hstu_ref_fwd.argtypes = (
            [ctypes.c_void_p] * 6 + [ctypes.c_int] * 5 + [ctypes.c_float] + [ctypes.c_int] * 4
        )
        _lib.hstu_ref_fwd.restype = ctypes.c_int
    return _lib


def mask(n: int, c: int = 0, t: Optional[int] = None, w: int = 0, f: int = 0) -> np.ndarray:
    out = np.zeros((n, n), dtype=np.uint8)
    lib().hstu_ref_mask(n, c, -1 if t is None else t, w, f, out.ctypes.data)
    return out.astype(bool)


def count_pairs(n: int, c: int = 0, t: Optional[int] = None, w: int = 0, f: int = 0, delta_size: int = 0) -> int:
    return int(lib().hstu_ref_count_pairs(n, c, -1 if t is None else t, w, f, delta_size))


def fwd(
    max_seq_len: int,
    alpha: float,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    seq_offsets: torch.Tensor,
    num_targets: Optional[torch.Tensor] = None,
    max_attn_len: int = 0,
    contextual_seq_len: int = 0,
    min_full_attn_seq_len: int = 0,
    delta_size: int = 0,
) -> torch.Tensor:
    q32 = q.detach().to(torch.float32).contiguous()
    k32 = k.detach().to(torch.float32).contiguous()
    v32 = v.detach().to(torch.float32).contiguous()
    offs = seq_offsets.detach().to(torch.int64).contiguous()
    tg = None if num_targets is None else num_targets.detach().to(torch.int64).contiguous()
    H, dqk, dv = q32.shape[1], q32.shape[2], v32.shape[2]
    assert dv <= 1024
    out = torch.zeros((q32.shape[0], H, dv), dtype=torch.float32)
    rc = lib().hstu_ref_fwd(
        q32.data_ptr(),
        k32.data_ptr(),
        v32.data_ptr(),
        out.data_ptr(),
        offs.data_ptr(),
        None if tg is None else tg.data_ptr(),
        offs.numel() - 1,
        H,
        dqk,
        dv,
        max_seq_len,
        alpha,
        max_attn_len,
        contextual_seq_len,
        min_full_attn_seq_len,
        delta_size,
    )
    if rc != 0:
        raise ValueError("hstu_ref_fwd: a sequence is longer than max_seq_len or shorter than delta_size")
    return out
