"""Host-side helpers mirrored from ``generative_recommenders/common.py`` of the reference."""

from enum import Enum, unique

import torch


@unique
class HammerKernel(Enum):
    """Same members as ``common.py:112-119`` so call sites keep compiling, plus ``HIP``.

    This build has exactly one backend.  Every value selects the gfx950 HIP kernels; the
    argument exists only so that ``hstu_mha(..., kernel=...)`` call sites need no edit.
    """

    TRITON = "TRITON"
    TLX = "TLX"
    PYTORCH = "PYTORCH"
    CUDA = "CUDA"
    TRITON_CC = "TRITON_CC"
    CUTEDSL = "CUTEDSL"
    HIP = "HIP"


def switch_to_contiguous_if_needed(x: torch.Tensor) -> torch.Tensor:
    """``common.py:262-269``: only the innermost dimension has to be dense."""
    if x.stride(-1) == 1:
        return x
    return x.contiguous()


def generate_sparse_seq_len(size: int, max_seq_len: int, sparsity: float, device: torch.device) -> torch.Tensor:
    """Length generator of ``common.py:185-213`` (uniform in a band set by ``sparsity``)."""
    if sparsity == 0.0:
        return torch.zeros(size=(size,), device=device, dtype=torch.int)
    if sparsity == 1.0:
        return torch.ones(size=(size,), device=device, dtype=torch.int) * max_seq_len
    if sparsity >= 0.5:
        lo, hi = int((2 * sparsity - 1.0) * max_seq_len), max_seq_len
    else:
        lo, hi = 0, int(2 * sparsity * max_seq_len)
    return torch.randint(low=lo, high=hi, size=(size,), device=device, dtype=torch.int)


def apply_sampling(lengths: torch.Tensor, alpha: float, max_seq_len: int) -> torch.Tensor:
    """Stochastic-length sampling of ``common.py:216-228``."""
    threshold = int(max_seq_len ** (alpha / 2))
    no_sample_prob = (max_seq_len**alpha) / torch.pow(lengths, 2)
    users_to_sample = torch.logical_and(lengths > threshold, torch.rand_like(no_sample_prob) < 1 - no_sample_prob)
    return torch.where(users_to_sample, threshold, lengths)
