"""Shared helpers of the test-suite: random jagged cases and the parity criteria."""

from typing import Optional

import numpy as np
import torch

# Stated tolerance of the bf16/fp16 path against the fp32 oracle.
MAX_ABS_TOL = 2e-2
MEAN_ABS_TOL = 2e-3
# Outputs are O(1e-3), so the absolute bounds alone would accept an all-zero result; this relative
# bound (Frobenius) is what actually bites.  bf16 rounding of P and of the output gives about 3e-3.
REL_FRO_TOL = 1e-2


def make_case(
    seed: int,
    lengths,
    heads: int,
    dqk: int,
    dv: Optional[int] = None,
    targets=None,
    dtype: torch.dtype = torch.bfloat16,
    scale: float = 0.1,
    delta_size: int = 0,
):
    g = torch.Generator().manual_seed(seed)
    lengths = torch.as_tensor(lengths, dtype=torch.int64)
    B = lengths.numel()
    offs = torch.zeros(B + 1, dtype=torch.int64)
    offs[1:] = torch.cumsum(lengths, 0)
    L = int(offs[-1])
    dv = dqk if dv is None else dv
    q = (torch.randn((L, heads, dqk), generator=g) * scale).to(dtype)
    k = (torch.randn((L, heads, dqk), generator=g) * scale).to(dtype)
    v = (torch.randn((L, heads, dv), generator=g) * scale).to(dtype)
    if delta_size > 0:
        q = (torch.randn((B * delta_size, heads, dqk), generator=g) * scale).to(dtype)
    t = None if targets is None else torch.as_tensor(targets, dtype=torch.int64)
    return q, k, v, offs, t


def assert_parity(out: torch.Tensor, ref: torch.Tensor, what: str = "", rel_tol: float = REL_FRO_TOL) -> None:
    out = out.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert out.shape == ref.shape, f"{what}: shape {tuple(out.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(out).all(), f"{what}: non-finite output"
    if out.numel() == 0:
        return
    err = (out - ref).abs()
    max_abs, mean_abs = float(err.max()), float(err.mean())
    denom = float(ref.norm())
    rel = float((out - ref).norm()) / denom if denom > 0 else float((out - ref).norm())
    assert max_abs <= MAX_ABS_TOL, f"{what}: max-abs {max_abs:.3e} > {MAX_ABS_TOL}"
    assert mean_abs <= MEAN_ABS_TOL, f"{what}: mean-abs {mean_abs:.3e} > {MEAN_ABS_TOL}"
    assert rel <= rel_tol, f"{what}: relative Frobenius error {rel:.3e} > {rel_tol} (max-abs {max_abs:.3e})"


def random_lengths(rng: np.random.Generator, batch: int, lo: int, hi: int):
    return rng.integers(lo, hi + 1, size=batch)
