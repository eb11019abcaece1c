"""CPU restatement of ``hstu_compute_uqvk`` -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline may import this module; the product
package never does.

``compute_uqvk`` follows ``generative_recommenders/ops/hstu_compute.py:54-104`` with the PyTorch backend
(``ops/pytorch/pt_layer_norm.py:24-39``: statistics and affine transform in fp32, result cast back to the input
type; ``torch.addmm``; split; ``silu(u)``), evaluated in fp32 or fp64 on whatever the caller passes.

Pinned by: ``layer_norm_by_hand`` (mean and biased variance written out in fp64) against ``F.layer_norm``; the
invariances of a layer norm (x -> a*x + c leaves the result unchanged for a > 0); the projection against a plain
fp64 ``@``; SiLU special values; the split against column indices written out by hand.  The reference holds no
golden vectors for this function (its test file covers ``hstu_compute_output`` only,
``ops/tests/hstu_compute_test.py:38-79``).
"""

from typing import Tuple

import torch
import torch.nn.functional as F


def layer_norm_by_hand(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    x = x.double()
    mean = x.mean(dim=1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight.double() + bias.double()


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    """pt_layer_norm.py:24-39: fp32 inside, input dtype outside."""
    return F.layer_norm(x.float(), (x.shape[1],), weight.float(), bias.float(), eps).to(x.dtype)


def compute_uqvk(
    x: torch.Tensor, norm_weight, norm_bias, norm_eps: float, num_heads: int, attn_dim: int, hidden_dim: int, uvqk_weight,
    uvqk_bias, round_normed_to: torch.dtype = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """fp32 throughout; ``round_normed_to`` reproduces the one rounding the reference's low-precision path has
    before the GEMM (the layer norm's result is cast to the input type)."""
    normed = F.layer_norm(x.float(), (x.shape[1],), norm_weight.float(), norm_bias.float(), norm_eps)
    if round_normed_to is not None:
        normed = normed.to(round_normed_to).float()
    uvqk = torch.addmm(uvqk_bias.float(), normed, uvqk_weight.float())
    hu, ha = hidden_dim * num_heads, attn_dim * num_heads
    u, v, q, k = torch.split(uvqk, [hu, hu, ha, ha], dim=1)
    return F.silu(u), q.reshape(-1, num_heads, attn_dim), k.reshape(-1, num_heads, attn_dim), v.reshape(-1, num_heads, hidden_dim)
