"""PyTorch-on-CPU oracle for ``hstu_mha`` / ``delta_hstu_mha``.  TEST INFRASTRUCTURE ONLY.

Restates ``generative_recommenders/ops/pytorch/pt_hstu_attention.py`` of the
reference (cited below as ``PT:<line>``) without ``fbgemm_gpu``.  The shipped
package never imports this file; the HIP path raises when its library is missing.

How each function is pinned (none by re-typing its own formula):

* ``jagged_to_padded_dense`` / ``dense_to_jagged`` (stand-ins for the two fbgemm
  ops at PT:97-125,183-187): pure index copies; pinned by the round trip
  ``unpad(pad(x)) == x`` and by an explicit Python loop over ``(b, i)``.
* ``get_valid_attn_mask`` (PT:32-84): pinned against ``hstu_ref_mask`` in
  ``hstu_ref.c`` -- a scalar formulation by *position class* (contextual /
  history / target rows with explicit column ranges, the way
  ``ops/cpp/hstu_attention/mask.h`` states it) that shares no arithmetic with
  the id formula -- exhaustively over small ``(n, c, t, w, f)``, and against the
  closed-form special cases (lower-triangular, identity, all-ones).
* ``pytorch_hstu_mha`` / ``pytorch_cached_hstu_mha`` (PT:129-251): pinned
  against ``hstu_ref_fwd`` (scalar C, double accumulation, its own mask), against
  the textbook reduction ``tril(silu(alpha QK^T)) / N @ V`` when the mask is
  lower-triangular, and by the invariants the reference's own tests state:
  delta output == last rows of the full output
  (``ops/tests/hstu_attention_test.py:382-488``), target permutation
  equivariance (``modules/tests/stu_test.py:180-321``), batch/head
  independence and exact ``N1/N2`` rescaling under a change of ``max_seq_len``.
* ``hstu_mha_per_sequence`` / ``cached_hstu_mha_per_sequence``: same mathematics
  evaluated per sequence at its own length (no ``[B, H, N, N]`` tensor); pinned
  against the dense-as-written functions above on every small test case.
* The reference holds no golden vectors or fixture files for this path, so none
  are checked.  ``fbgemm_gpu`` is not importable here; the reference module was
  not imported or run.
"""

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def jagged_to_padded_dense(
    values: torch.Tensor, offsets: torch.Tensor, max_len: int, padding_value: float = 0.0
) -> torch.Tensor:
    """``[L, D]`` jagged rows -> ``[B, max_len, D]``; rows past ``max_len`` are dropped.

    Stand-in for ``torch.ops.fbgemm.jagged_to_padded_dense`` as called at PT:97-125.
    """
    B = offsets.numel() - 1
    D = values.shape[1]
    lengths = (offsets[1:] - offsets[:-1]).to(torch.int64)
    pos = torch.arange(max_len, dtype=torch.int64).view(1, max_len)
    valid = pos < lengths.view(B, 1)
    src = (offsets[:-1].to(torch.int64).view(B, 1) + pos)[valid]
    dense = torch.full((B, max_len, D), padding_value, dtype=values.dtype)
    dense[valid] = values[src]
    return dense


def dense_to_jagged(dense: torch.Tensor, offsets: torch.Tensor, total_len: int) -> torch.Tensor:
    """``[B, N, D]`` -> ``[L, D]`` keeping the first ``n_b`` rows of each batch (PT:183-187)."""
    B, N, _ = dense.shape
    lengths = (offsets[1:] - offsets[:-1]).to(torch.int64)
    pos = torch.arange(N, dtype=torch.int64).view(1, N)
    valid = pos < lengths.view(B, 1)
    out = dense[valid]
    assert out.shape[0] == total_len, (out.shape, total_len)
    return out


def get_valid_attn_mask(
    causal: bool,
    N: int,
    seq_lengths: torch.Tensor,
    num_targets: Optional[torch.Tensor] = None,
    max_attn_len: int = 0,
    contextual_seq_len: int = 0,
    min_full_attn_seq_len: int = 0,
) -> torch.Tensor:
    """Boolean mask ``[B or 1, N, N]`` of PT:32-84, same operations in the same order."""
    ids = torch.arange(0, N).view(1, N)
    max_ids = seq_lengths.view(-1, 1, 1)
    if contextual_seq_len > 0:
        ids = torch.clamp(ids - contextual_seq_len + 1, min=0)
        max_ids = max_ids - contextual_seq_len + 1
    if num_targets is not None:
        max_ids = max_ids - num_targets.view(-1, 1, 1)
        ids = torch.clamp(ids, max=max_ids)
        row_ids = ids.view(-1, N, 1).expand(-1, N, N)
        col_ids = ids.view(-1, 1, N).expand(-1, N, N)
    else:
        row_ids = ids.view(N, 1).expand(N, N)
        col_ids = row_ids.t()
        row_ids = row_ids.view(1, N, N)
        col_ids = col_ids.view(1, N, N)
    dist = row_ids - col_ids
    mask = torch.eye(N, dtype=torch.bool).view(1, N, N)
    if not causal:
        dist = torch.where(dist > 0, dist, -dist)
    mask = torch.logical_or(mask, dist > 0)
    if max_attn_len > 0:
        if min_full_attn_seq_len > 0:
            mask = torch.logical_and(
                mask,
                torch.logical_or(dist <= max_attn_len, row_ids >= max_ids - min_full_attn_seq_len),
            )
        else:
            mask = torch.logical_and(mask, dist <= max_attn_len)
    if contextual_seq_len > 0:
        mask = torch.logical_or(mask, torch.logical_and(row_ids == 0, col_ids < max_ids))
    return mask


def _pad_qkv(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_offsets: torch.Tensor, N: int
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """PT:87-126: jagged ``[L, H, D]`` -> padded ``[B, H, N, D]``."""
    L, H, D = q.shape
    V = v.shape[2]
    pq = jagged_to_padded_dense(q.reshape(L, H * D), seq_offsets, N).view(-1, N, H, D).transpose(1, 2)
    pk = jagged_to_padded_dense(k.reshape(L, H * D), seq_offsets, N).view(-1, N, H, D).transpose(1, 2)
    pv = jagged_to_padded_dense(v.reshape(L, H * V), seq_offsets, N).view(-1, N, H, V).transpose(1, 2)
    return pq, pk, pv


def pytorch_hstu_mha(
    max_seq_len: int,
    alpha: float,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    seq_offsets: torch.Tensor,
    causal: bool = True,
    dropout_pr: float = 0.0,
    training: bool = True,
    num_targets: Optional[torch.Tensor] = None,
    attn_scale: Optional[torch.Tensor] = None,
    max_attn_len: int = 0,
    contextual_seq_len: int = 0,
    min_full_attn_seq_len: int = 0,
) -> torch.Tensor:
    """Dense-as-written restatement of ``pytorch_hstu_mha`` (PT:129-187)."""
    L, H, _ = q.shape
    V = v.shape[2]
    pq, pk, pv = _pad_qkv(q, k, v, seq_offsets, max_seq_len)
    qk_attn = torch.einsum("bhxa,bhya->bhxy", pq, pk) * alpha
    if attn_scale is not None:
        if attn_scale.ndim > 0:
            attn_scale = (
                jagged_to_padded_dense(attn_scale.unsqueeze(-1), seq_offsets, max_seq_len)
                .unsqueeze(1)
                .to(qk_attn.dtype)
            )
        qk_attn = F.silu(qk_attn) * attn_scale
    else:
        qk_attn = F.silu(qk_attn) / max_seq_len
    mask = get_valid_attn_mask(
        causal=causal,
        N=max_seq_len,
        seq_lengths=seq_offsets[1:] - seq_offsets[:-1],
        num_targets=num_targets,
        max_attn_len=max_attn_len,
        contextual_seq_len=contextual_seq_len,
        min_full_attn_seq_len=min_full_attn_seq_len,
    )
    qk_attn = qk_attn * mask.unsqueeze(1)
    if dropout_pr > 0.0:
        qk_attn = F.dropout(qk_attn, p=dropout_pr, training=training)
    attn_dense = torch.einsum("bhxd,bhdv->bhxv", qk_attn, pv)
    return dense_to_jagged(attn_dense.transpose(1, 2).flatten(2, 3), seq_offsets, L).view(L, H, V)


def pytorch_cached_hstu_mha(
    max_seq_len: int,
    alpha: float,
    delta_q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    seq_offsets: torch.Tensor,
    num_targets: Optional[torch.Tensor] = None,
    max_attn_len: int = 0,
    contextual_seq_len: int = 0,
) -> torch.Tensor:
    """Dense-as-written restatement of ``pytorch_cached_hstu_mha`` (PT:190-251)."""
    L, H, D = delta_q.shape
    V = v.shape[2]
    B = seq_offsets.numel() - 1
    delta_size = L // B
    dq = delta_q.view(B, -1, H, D).transpose(1, 2)
    full_k = (
        jagged_to_padded_dense(k.reshape(-1, H * D), seq_offsets, max_seq_len).view(B, -1, H, D).transpose(1, 2)
    )
    full_v = (
        jagged_to_padded_dense(v.reshape(-1, H * V), seq_offsets, max_seq_len).view(B, -1, H, V).transpose(1, 2)
    )
    qk_attn = torch.einsum("bhxa,bhya->bhxy", dq, full_k) * alpha
    qk_attn = F.silu(qk_attn) / max_seq_len
    seq_lengths = seq_offsets[1:] - seq_offsets[:-1]
    full_mask = get_valid_attn_mask(
        causal=True,
        N=max_seq_len,
        seq_lengths=seq_lengths,
        num_targets=num_targets,
        max_attn_len=max_attn_len,
        contextual_seq_len=contextual_seq_len,
    )
    pos = torch.arange(max_seq_len).view(1, -1)
    rows = torch.logical_and(pos >= (seq_lengths - delta_size).view(-1, 1), pos < seq_lengths.view(-1, 1))
    mask = full_mask.expand(B, -1, -1).flatten(0, 1)[rows.view(-1), :].view(-1, delta_size, max_seq_len)
    qk_attn = qk_attn * mask.unsqueeze(1)
    out = torch.einsum("bhxd,bhdv->bhxv", qk_attn, full_v)
    return out.transpose(1, 2).reshape(-1, H, V)


def _seq_mask_rows(
    n: int,
    r0: int,
    r1: int,
    t: Optional[int],
    max_attn_len: int,
    contextual_seq_len: int,
    min_full_attn_seq_len: int,
) -> torch.Tensor:
    """Rows ``[r0, r1)`` of the ``n x n`` mask of one sequence (id formula of PT:43-83)."""
    ids = torch.arange(n)
    max_id = n
    if contextual_seq_len > 0:
        ids = torch.clamp(ids - contextual_seq_len + 1, min=0)
        max_id = max_id - contextual_seq_len + 1
    if t is not None:
        max_id = max_id - t
        ids = torch.clamp(ids, max=max_id)
    row_ids = ids[r0:r1].view(-1, 1)
    col_ids = ids.view(1, -1)
    dist = row_ids - col_ids
    mask = torch.arange(r0, r1).view(-1, 1) == torch.arange(n).view(1, -1)
    mask = mask | (dist > 0)
    if max_attn_len > 0:
        if min_full_attn_seq_len > 0:
            mask = mask & ((dist <= max_attn_len) | (row_ids >= max_id - min_full_attn_seq_len))
        else:
            mask = mask & (dist <= max_attn_len)
    if contextual_seq_len > 0:
        mask = mask | ((row_ids == 0) & (col_ids < max_id))
    return mask


def hstu_mha_per_sequence(
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
    row_chunk: int = 1024,
    compute_dtype: torch.dtype = torch.float32,
    sequences: Optional[list] = None,
    row_ranges: Optional[list] = None,
    attn_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Same mathematics as PT:129-251, one sequence at a time at its own length.

    ``delta_size == 0``: ``q`` is jagged like ``k`` and the result is ``[L, H, Dv]``.
    ``delta_size > 0``: ``q`` is ``[B * delta_size, H, Dqk]`` holding the last
    ``delta_size`` positions of each sequence; the result is ``[B * delta_size, H, Dv]``.
    ``sequences`` restricts the work to those batch indices (other rows stay zero).
    ``row_ranges`` (a list of ``(r0, r1)`` in query-row indices of a sequence, clipped to its rows) restricts it
    further to those query rows; a row's result does not depend on which other rows are evaluated with it.
    ``attn_scale`` (PT:152-165, full form only): 0-dim, or one value per query row (jagged like ``q``); it multiplies
    ``silu`` in place of ``1 / max_seq_len``.
    """
    H = q.shape[1]
    V = v.shape[2]
    B = seq_offsets.numel() - 1
    out = torch.zeros((q.shape[0], H, V), dtype=compute_dtype)
    offs = [int(x) for x in seq_offsets.tolist()]
    tg = None if num_targets is None else [int(x) for x in num_targets.tolist()]
    for b in range(B) if sequences is None else sequences:
        s0, s1 = offs[b], offs[b + 1]
        n = s1 - s0
        if n == 0:
            continue
        kb = k[s0:s1].to(compute_dtype).transpose(0, 1)  # [H, n, D]
        vb = v[s0:s1].to(compute_dtype).transpose(0, 1)  # [H, n, V]
        if delta_size > 0:
            rows0, q0 = n - delta_size, b * delta_size
            nq = delta_size
        else:
            rows0, q0 = 0, s0
            nq = n
        spans = [(0, nq)] if row_ranges is None else [(max(0, a), min(nq, z)) for a, z in row_ranges]
        chunks = [(c0, min(z, c0 + row_chunk)) for a, z in spans for c0 in range(a, z, row_chunk)]
        for c0, c1 in chunks:
            qb = q[q0 + c0 : q0 + c1].to(compute_dtype).transpose(0, 1)  # [H, m, D]
            s = torch.matmul(qb, kb.transpose(1, 2)) * alpha
            if attn_scale is None:
                s = F.silu(s) / max_seq_len
            elif attn_scale.ndim == 0:
                s = F.silu(s) * attn_scale.to(compute_dtype)
            else:
                s = F.silu(s) * attn_scale[q0 + c0 : q0 + c1].to(compute_dtype).view(1, -1, 1)
            m = _seq_mask_rows(
                n,
                rows0 + c0,
                rows0 + c1,
                None if tg is None else tg[b],
                max_attn_len,
                contextual_seq_len,
                min_full_attn_seq_len,
            )
            s = s * m.unsqueeze(0)
            out[q0 + c0 : q0 + c1] = torch.matmul(s, vb).transpose(0, 1)
    return out


def cached_hstu_mha_per_sequence(
    max_seq_len: int,
    alpha: float,
    delta_q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    seq_offsets: torch.Tensor,
    num_targets: Optional[torch.Tensor] = None,
    max_attn_len: int = 0,
    contextual_seq_len: int = 0,
    **kw,
) -> torch.Tensor:
    """Per-sequence form of ``pytorch_cached_hstu_mha`` (PT:190-251)."""
    B = seq_offsets.numel() - 1
    return hstu_mha_per_sequence(
        max_seq_len,
        alpha,
        delta_q,
        k,
        v,
        seq_offsets,
        num_targets=num_targets,
        max_attn_len=max_attn_len,
        contextual_seq_len=contextual_seq_len,
        delta_size=delta_q.shape[0] // B,
        **kw,
    )
