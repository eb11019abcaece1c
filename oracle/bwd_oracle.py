"""CPU statements of the backward of ``hstu_mha`` -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline may import this module; the product
package never does.

The reference defines the gradients by autograd through ``pytorch_hstu_mha``
(``generative_recommenders/ops/tests/hstu_attention_test.py:118-165`` compares its Triton backward,
``ops/triton/triton_hstu_attention.py:1905-2229``, with exactly that).  Two statements here:

* ``autograd_grads``: autograd through ``hstu_oracle.pytorch_hstu_mha`` (the dense-as-written restatement of the
  forward, pinned on its own) -- small inputs only, the intermediate is ``[B, H, N, N]``;
* ``closed_form_grads``: the formulas written out per sequence,
      P = M * silu(alpha S) / N,   dV = P^T dO,   dP = dO V^T,
      dS = M * dP * silu'(alpha S) / N,   silu'(x) = sigmoid(x) * (1 + x * (1 - sigmoid(x))),
      dQ = alpha * dS K,   dK = alpha * dS^T Q,
  which is what ``_hstu_attn_bwd_one_block`` computes (``triton_hstu_attention.py:1966-2006``); usable at any size.

Pinned by: the two against each other over the mask parameters; ``torch.autograd.gradcheck`` (finite differences in
fp64) on the forward restatement; ``silu'`` special values (1/2 at 0, -> 1 and -> 0 at +-inf) and its finite
difference; linearity in ``dout``.  The reference holds no golden vectors for the gradients.
"""

from typing import Optional, Tuple

import torch

from . import hstu_oracle


def silu_slope(x: torch.Tensor) -> torch.Tensor:
    sig = torch.sigmoid(x)
    return sig * (1 + x * (1 - sig))


def autograd_grads(
    max_seq_len: int, alpha: float, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_offsets: torch.Tensor, dout: torch.Tensor,
    num_targets: Optional[torch.Tensor] = None, max_attn_len: int = 0, contextual_seq_len: int = 0, min_full_attn_seq_len: int = 0,
    dtype: torch.dtype = torch.float64, attn_scale: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    q, k, v = (t.detach().to(dtype).requires_grad_() for t in (q, k, v))
    out = hstu_oracle.pytorch_hstu_mha(
        max_seq_len, alpha, q, k, v, seq_offsets, num_targets=num_targets, max_attn_len=max_attn_len,
        contextual_seq_len=contextual_seq_len, min_full_attn_seq_len=min_full_attn_seq_len,
        attn_scale=None if attn_scale is None else attn_scale.to(dtype),
    )
    out.backward(dout.to(dtype))
    return q.grad, k.grad, v.grad


def closed_form_grads(
    max_seq_len: int, alpha: float, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seq_offsets: torch.Tensor, dout: torch.Tensor,
    num_targets: Optional[torch.Tensor] = None, max_attn_len: int = 0, contextual_seq_len: int = 0, min_full_attn_seq_len: int = 0,
    dtype: torch.dtype = torch.float32, row_chunk: int = 1024, sequences: Optional[list] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``sequences`` restricts the work to those batch indices (other rows stay zero)."""
    dq = torch.zeros(q.shape, dtype=dtype)
    dk = torch.zeros(k.shape, dtype=dtype)
    dv = torch.zeros(v.shape, dtype=dtype)
    offs = [int(x) for x in seq_offsets.tolist()]
    tg = None if num_targets is None else [int(x) for x in num_targets.tolist()]
    for b in range(len(offs) - 1) if sequences is None else sequences:
        s0, s1 = offs[b], offs[b + 1]
        n = s1 - s0
        if n == 0:
            continue
        kb = k[s0:s1].to(dtype).transpose(0, 1)  # [H, n, D]
        vb = v[s0:s1].to(dtype).transpose(0, 1)  # [H, n, V]
        dkb = torch.zeros_like(kb)
        dvb = torch.zeros_like(vb)
        for c0 in range(0, n, row_chunk):
            c1 = min(n, c0 + row_chunk)
            qb = q[s0 + c0 : s0 + c1].to(dtype).transpose(0, 1)      # [H, m, D]
            dob = dout[s0 + c0 : s0 + c1].to(dtype).transpose(0, 1)  # [H, m, V]
            m = hstu_oracle._seq_mask_rows(
                n, c0, c1, None if tg is None else tg[b], max_attn_len, contextual_seq_len, min_full_attn_seq_len
            ).unsqueeze(0)
            x = torch.matmul(qb, kb.transpose(1, 2)) * alpha
            p = torch.nn.functional.silu(x) / max_seq_len * m
            dvb += torch.matmul(p.transpose(1, 2), dob)
            ds = torch.matmul(dob, vb.transpose(1, 2)) * silu_slope(x) / max_seq_len * m
            dq[s0 + c0 : s0 + c1] = (alpha * torch.matmul(ds, kb)).transpose(0, 1)
            dkb += alpha * torch.matmul(ds.transpose(1, 2), qb)
        dk[s0:s1] = dkb.transpose(0, 1)
        dv[s0:s1] = dvb.transpose(0, 1)
    return dq, dk, dv
