"""CPU restatement of ``concat_2D_jagged`` / ``split_2D_jagged`` -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline may import this module; the product
package never does.

Two statements of the same index copy:

* ``concat_padded`` / ``split_padded`` follow the reference's algorithm step by step
  (``generative_recommenders/ops/pytorch/pt_jagged_tensors.py:31-62`` and ``:117-140``): pad both sides to dense
  ``[B, max_len, D]`` (the closed form of ``fbgemm.jagged_to_padded_dense``: ``dense[b, i] = values[off[b] + i]`` for
  ``i < min(len_b, max_len)``, else 0), concatenate along the length axis, select rows with the boolean mask.
* ``concat_by_batch`` / ``split_by_batch`` are the textbook definition: a Python loop with ``torch.cat`` per batch.

Pinned by: the two forms agree on random cases incl. dense sides and empty sequences (all within the caller
contract ``len_b <= max_len``; beyond it the reference's mask selects padding rows, which the step-by-step form
reproduces and a hand-computed case checks); ``split(concat(a, b)) == (a, b)``; a dense side equals a jagged side with
``max_len * arange`` offsets (``pt_jagged_tensors.py:73-90``); the reference holds no golden vectors for these ops
(its tests compare its Triton and PyTorch backends, ``ops/tests/jagged_tensors_test.py:38-240``).
``fbgemm_gpu`` (absent here, not version-locked by the reference) only moves data in these functions.
"""

from typing import Optional, Tuple

import torch


def _dense_offsets(max_len: int, batch: int) -> torch.Tensor:
    return max_len * torch.arange(batch + 1, dtype=torch.int64)


def _pad(values: torch.Tensor, offsets: torch.Tensor, max_len: int) -> torch.Tensor:
    """Closed form of ``fbgemm.jagged_to_padded_dense`` with padding value 0."""
    B = offsets.numel() - 1
    out = torch.zeros((B, max_len, values.shape[1]), dtype=values.dtype)
    for b in range(B):
        s, e = int(offsets[b]), int(offsets[b + 1])
        n = min(e - s, max_len)
        out[b, :n] = values[s : s + n]
    return out


def concat_padded(
    values_left: torch.Tensor,
    values_right: torch.Tensor,
    max_len_left: Optional[int],
    max_len_right: Optional[int],
    offsets_left: Optional[torch.Tensor],
    offsets_right: Optional[torch.Tensor],
) -> torch.Tensor:
    """``pytorch_concat_2D_jagged`` (pt_jagged_tensors.py:64-114) on CPU tensors."""
    if offsets_left is None:
        offsets_left = _dense_offsets(max_len_left, values_left.shape[0] // max_len_left)
    if offsets_right is None:
        offsets_right = _dense_offsets(max_len_right, values_right.shape[0] // max_len_right)
    len_l = offsets_left[1:] - offsets_left[:-1]
    len_r = offsets_right[1:] - offsets_right[:-1]
    if max_len_left is None:
        max_len_left = int(len_l.max())
    if max_len_right is None:
        max_len_right = int(len_r.max())
    dense = torch.cat([_pad(values_left, offsets_left, max_len_left), _pad(values_right, offsets_right, max_len_right)], dim=1)
    pos = torch.arange(max_len_left + max_len_right).view(1, -1)
    mask = (pos < len_l.view(-1, 1)) | ((pos >= max_len_left) & (pos < max_len_left + len_r.view(-1, 1)))
    return dense.flatten(0, 1)[mask.view(-1)]


def split_padded(
    max_seq_len: int,
    values: torch.Tensor,
    max_len_left: Optional[int],
    max_len_right: Optional[int],
    offsets_left: Optional[torch.Tensor],
    offsets_right: Optional[torch.Tensor],
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``pytorch_split_2D_jagged`` (pt_jagged_tensors.py:117-173) on CPU tensors."""
    if offsets_left is None:
        offsets_left = max_len_left * torch.arange(offsets_right.shape[0], dtype=torch.int64)
    if offsets_right is None:
        offsets_right = max_len_right * torch.arange(offsets_left.shape[0], dtype=torch.int64)
    padded = _pad(values, offsets_left + offsets_right, max_seq_len).flatten(0, 1)
    len_l = (offsets_left[1:] - offsets_left[:-1]).view(-1, 1)
    len_r = (offsets_right[1:] - offsets_right[:-1]).view(-1, 1)
    pos = torch.arange(max_seq_len).view(1, -1)
    return padded[(pos < len_l).view(-1)], padded[((pos >= len_l) & (pos < len_l + len_r)).view(-1)]


def concat_by_batch(values_left, values_right, offsets_left, offsets_right) -> torch.Tensor:
    """Textbook form: for every batch the left rows, then the right rows."""
    parts = []
    for b in range(offsets_left.numel() - 1):
        parts.append(values_left[int(offsets_left[b]) : int(offsets_left[b + 1])])
        parts.append(values_right[int(offsets_right[b]) : int(offsets_right[b + 1])])
    return torch.cat(parts, dim=0) if parts else values_left[:0]


def split_by_batch(values, offsets_left, offsets_right) -> Tuple[torch.Tensor, torch.Tensor]:
    lefts, rights = [], []
    for b in range(offsets_left.numel() - 1):
        start = int(offsets_left[b]) + int(offsets_right[b])
        nl = int(offsets_left[b + 1] - offsets_left[b])
        nr = int(offsets_right[b + 1] - offsets_right[b])
        lefts.append(values[start : start + nl])
        rights.append(values[start + nl : start + nl + nr])
    return torch.cat(lefts, dim=0), torch.cat(rights, dim=0)
