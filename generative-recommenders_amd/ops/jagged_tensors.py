"""``concat_2D_jagged`` / ``split_2D_jagged`` with the reference's signatures, plus the in-place K/V-cache form.

Mirrors ``generative_recommenders/ops/jagged_tensors.py`` of the reference (``concat_2D_jagged`` at lines 55-100,
``split_2D_jagged`` at lines 102-167; semantics ``ops/pytorch/pt_jagged_tensors.py:31-173``): the per-batch
concatenation of two jagged (or dense-per-batch) 2-D tensors and its inverse -- what ``STULayer`` uses to put
cached and new K/V rows together for ``delta_hstu_mha`` (``modules/stu.py:84-173``).  Device tensors only, one backend
(``kernel`` is accepted and ignored).  Differentiable as in the reference (``ops/triton/triton_jagged_tensors.py:
_Concat2DJaggedFunction / _Split2DJaggedFunction``): the gradient of the concatenation is the split of the incoming
gradient and the other way round, run by the same two kernels.  Output sizes follow the reference's GPU backend
(``ops/triton/triton_jagged_tensors.py:546-568, 650-682``): the concatenation has
``values_left.shape[0] + values_right.shape[0]`` rows, which assumes the caller contract "no sequence longer than
``max_len_*``".
"""

from typing import Optional, Tuple

import torch

from ..common import HammerKernel, switch_to_contiguous_if_needed
from . import hip_backend


def _needs_grad(*tensors: torch.Tensor) -> bool:
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def _concat_rows(left, right, offsets_left, offsets_right, batch, max_len_left, max_len_right) -> torch.Tensor:
    left = switch_to_contiguous_if_needed(left.detach())
    right = switch_to_contiguous_if_needed(right.detach())
    out = torch.empty((left.shape[0] + right.shape[0], left.shape[1]), dtype=left.dtype, device=left.device)
    if out.numel() > 0:
        hip_backend.jagged_copy(False, left, right, out, offsets_left, offsets_right, batch, max_len_left, max_len_right)
    return out


def _split_rows(values, total_left, total_right, offsets_left, offsets_right, batch, max_len_left, max_len_right):
    joined = switch_to_contiguous_if_needed(values.detach())
    left = torch.empty((total_left, values.shape[1]), dtype=values.dtype, device=values.device)
    right = torch.empty((total_right, values.shape[1]), dtype=values.dtype, device=values.device)
    if values.shape[0] > 0 and values.shape[1] > 0:
        hip_backend.jagged_copy(True, left, right, joined, offsets_left, offsets_right, batch, max_len_left, max_len_right)
    return left, right


class _ConcatFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, left, right, offsets_left, offsets_right, batch, max_len_left, max_len_right):
        ctx.meta = (left.shape[0], right.shape[0], offsets_left, offsets_right, batch, max_len_left, max_len_right)
        return _concat_rows(left, right, offsets_left, offsets_right, batch, max_len_left, max_len_right)

    @staticmethod
    def backward(ctx, d_out):
        d_left, d_right = _split_rows(d_out, *ctx.meta)
        return d_left, d_right, None, None, None, None, None


class _SplitFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values, total_left, total_right, offsets_left, offsets_right, batch, max_len_left, max_len_right):
        ctx.meta = (offsets_left, offsets_right, batch, max_len_left, max_len_right)
        return _split_rows(values, total_left, total_right, offsets_left, offsets_right, batch, max_len_left, max_len_right)

    @staticmethod
    def backward(ctx, d_left, d_right):
        return (_concat_rows(d_left, d_right, *ctx.meta),) + (None,) * 7


def _max_len(offsets: torch.Tensor) -> int:
    # as the reference (pt_jagged_tensors.py:98-113): a missing max_len costs a host synchronisation
    return int((offsets[1:] - offsets[:-1]).max().item())


def _index_tensor(x: Optional[torch.Tensor], name: str) -> Optional[torch.Tensor]:
    if x is None:
        return None
    torch._assert(x.dtype in (torch.int32, torch.int64), f"{name} must be int32 or int64")
    torch._assert(x.is_cuda, f"{name} must be CUDA tensor")
    return x.contiguous()


def concat_2D_jagged(
    max_seq_len: int,
    values_left: torch.Tensor,
    values_right: torch.Tensor,
    max_len_left: Optional[int] = None,
    max_len_right: Optional[int] = None,
    offsets_left: Optional[torch.Tensor] = None,
    offsets_right: Optional[torch.Tensor] = None,
    kernel: HammerKernel = HammerKernel.HIP,
) -> torch.Tensor:
    """Per batch: rows of ``values_left`` followed by rows of ``values_right``; returns ``[L_left + L_right, D]``.

    A side without offsets is dense: exactly ``max_len_*`` rows per batch."""
    torch._assert(values_left.dim() == 2, "values_left must be 2D")
    torch._assert(values_right.dim() == 2, "values_right must be 2D")
    torch._assert(
        values_right.shape[1] == values_left.shape[1],
        f"values_left shape[1] must be equal to values_right shape[1] {values_left.shape[1]} vs {values_right.shape[1]}",
    )
    torch._assert(values_left.is_cuda and values_right.is_cuda, "values must be CUDA tensors")
    torch._assert(values_left.dtype == values_right.dtype, "values_left and values_right must have the same dtype")
    offsets_left = _index_tensor(offsets_left, "offsets_left")
    offsets_right = _index_tensor(offsets_right, "offsets_right")
    if offsets_left is None:
        assert max_len_left is not None
        batch = values_left.shape[0] // max_len_left if max_len_left > 0 else 0
    else:
        batch = offsets_left.shape[0] - 1
    if offsets_right is None:
        assert max_len_right is not None
        batch = values_right.shape[0] // max_len_right if max_len_right > 0 else batch
    else:
        batch = offsets_right.shape[0] - 1
    if max_len_left is None:
        max_len_left = _max_len(offsets_left)
    if max_len_right is None:
        max_len_right = _max_len(offsets_right)
    if _needs_grad(values_left, values_right):
        return _ConcatFunction.apply(values_left, values_right, offsets_left, offsets_right, batch, max_len_left, max_len_right)
    return _concat_rows(values_left, values_right, offsets_left, offsets_right, batch, max_len_left, max_len_right)


def split_2D_jagged(
    max_seq_len: int,
    values: torch.Tensor,
    total_len_left: Optional[int] = None,
    total_len_right: Optional[int] = None,
    max_len_left: Optional[int] = None,
    max_len_right: Optional[int] = None,
    offsets_left: Optional[torch.Tensor] = None,
    offsets_right: Optional[torch.Tensor] = None,
    kernel: HammerKernel = HammerKernel.HIP,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Inverse of ``concat_2D_jagged``: returns ``(values_left, values_right)``."""
    torch._assert(values.dim() == 2, "values must be 2D")
    torch._assert(
        offsets_left is not None or offsets_right is not None,
        "offsets_left and offsets_right cannot be None at the same time",
    )
    if offsets_left is None:
        torch._assert(max_len_left is not None, "max_len_left must be provided when offsets_left is None")
    if offsets_right is None:
        torch._assert(max_len_right is not None, "max_len_right must be provided when offsets_right is None")
    if offsets_left is not None and offsets_right is not None:
        torch._assert(
            offsets_left.shape[0] == offsets_right.shape[0],
            "offsets_left shape[0] must be equal to offsets_right shape[0]",
        )
    torch._assert(values.is_cuda, "values must be CUDA tensor")
    offsets_left = _index_tensor(offsets_left, "offsets_left")
    offsets_right = _index_tensor(offsets_right, "offsets_right")
    total = values.shape[0]
    # sizes of the two parts as ops/triton/triton_jagged_tensors.py:650-675 of the reference derives them
    if offsets_left is None:
        batch = offsets_right.shape[0] - 1
        total_left = max_len_left * batch
        total_right = total - total_left
    elif offsets_right is None:
        batch = offsets_left.shape[0] - 1
        total_right = max_len_right * batch
        total_left = total - total_right
    else:
        batch = offsets_left.shape[0] - 1
        if total_len_left is not None and total_len_right is not None:
            assert total_len_left + total_len_right == total
            total_left, total_right = total_len_left, total_len_right
        else:
            total_left = int(offsets_left[-1].item())
            total_right = total - total_left
    if max_len_left is None:
        max_len_left = _max_len(offsets_left)
    if max_len_right is None:
        max_len_right = _max_len(offsets_right)
    if _needs_grad(values):
        return _SplitFunction.apply(values, total_left, total_right, offsets_left, offsets_right, batch, max_len_left, max_len_right)
    return _split_rows(values, total_left, total_right, offsets_left, offsets_right, batch, max_len_left, max_len_right)


def write_kv_tail(full_values: torch.Tensor, full_offsets: torch.Tensor, delta_values: torch.Tensor) -> torch.Tensor:
    """In-place ``_construct_full_kv`` (``modules/stu.py:133-173`` of the reference) for a cache that keeps
    ``delta_size`` spare rows behind every sequence's history.

    ``full_values`` is ``[sum(history_b + delta_size), D]`` with ``full_offsets = kv_caching_offsets +
    delta_size * arange(B + 1)``; ``delta_values`` is ``[B * delta_size, D]``.  The last ``delta_size`` rows of every
    sequence are overwritten with its block of ``delta_values``; the history rows are not touched, so the next
    micro-batch of candidates only repeats this call.  Returns ``full_values``.
    """
    torch._assert(full_values.dim() == 2 and delta_values.dim() == 2, "values must be 2D")
    torch._assert(full_values.shape[1] == delta_values.shape[1], "row widths must match")
    torch._assert(full_values.dtype == delta_values.dtype, "dtypes must match")
    torch._assert(full_values.is_cuda and delta_values.is_cuda, "values must be CUDA tensors")
    torch._assert(full_values.stride(1) == 1 and delta_values.stride(1) == 1, "innermost stride must be 1")
    full_offsets = _index_tensor(full_offsets, "full_offsets")
    batch = full_offsets.shape[0] - 1
    torch._assert(batch > 0 and delta_values.shape[0] % batch == 0, "delta_values must hold the same number of rows per batch")
    hip_backend.jagged_write_tail(full_values, full_offsets, delta_values, batch, delta_values.shape[0] // batch)
    return full_values
