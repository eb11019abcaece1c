"""CPU restatement of ``hstu_compute_output`` -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline may import this module; the product
package never does.

``norm_mul`` follows ``pytorch_norm_mul_dropout`` (``generative_recommenders/ops/pytorch/pt_hstu_linear.py:24-85``)
without its dropout (inference: ``F.dropout(training=False)`` is the identity); ``compute_output`` follows
``pytorch_hstu_compute_output`` (``pt_hstu_linear.py:88-124``), the PyTorch backend behind ``hstu_compute_output``
(``ops/hstu_compute.py:107-214``).  fp32 on whatever the caller passes.

Pinned by: ``group_norm_by_hand`` / ``uqvk_oracle.layer_norm_by_hand`` (mean and biased variance written out in
fp64) against the library calls used here; the column blocks of the concatenation against the inputs they copy;
a one-hot ``output_weight`` that turns the GEMM into a column selection (so a swapped or dropped block shows);
``sigmoid`` / ``silu`` special values.  The reference holds no golden vectors for this function: its test compares
two of its own backends on a GPU (``ops/tests/hstu_compute_test.py:38-79``), with inputs drawn uniformly from
[-0.1, 0.1] -- the distribution the GPU tests here use as well.
"""

import torch
import torch.nn.functional as F


def group_norm_by_hand(x: torch.Tensor, num_heads: int, linear_dim: int, weight: torch.Tensor, bias: torch.Tensor, eps: float):
    """Each head's ``linear_dim`` columns normalised on their own; one weight and one bias per head."""
    x = x.double().view(-1, num_heads, linear_dim)
    mean = x.mean(dim=2, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=2, keepdim=True)
    y = (x - mean) / torch.sqrt(var + eps) * weight.double().view(1, -1, 1) + bias.double().view(1, -1, 1)
    return y.view(-1, num_heads * linear_dim)


def norm_mul(
    attn: torch.Tensor, u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, silu_u: bool = False,
    concat_u: bool = False, concat_x: bool = False, mul_u_activation_type: str = "none", group_norm: bool = False,
    num_heads: int = 1, linear_dim: int = -1,
) -> torch.Tensor:
    """fp32 result, not yet rounded to the input type (pt_hstu_linear.py:40-85)."""
    x = attn.float()
    u = u.float()
    if group_norm:  # :43-56
        if silu_u:
            u = F.silu(u)
        y = u * F.group_norm(
            x.view(-1, num_heads, linear_dim), num_groups=num_heads, weight=weight.float(), bias=bias.float(), eps=eps
        ).view(-1, num_heads * linear_dim)
        if concat_u and concat_x:
            y = torch.cat([u, x, y], dim=1)
        return y
    mul_u = u  # :57-79
    if mul_u_activation_type == "sigmoid":
        mul_u = torch.sigmoid(u)
    elif mul_u_activation_type == "silu":
        mul_u = F.silu(u)
    y = mul_u * F.layer_norm(x, (x.shape[-1],), weight.float(), bias.float(), eps)
    if concat_u:
        if silu_u:
            u = F.silu(u)
        y = torch.cat([u, x, y], dim=1) if concat_x else torch.cat([u, y], dim=1)
    elif concat_x:
        y = torch.cat([x, y], dim=1)
    return y


def compute_output(
    attn: torch.Tensor, u: torch.Tensor, x: torch.Tensor, norm_weight, norm_bias, output_weight, eps: float, silu_u: bool = False,
    concat_u: bool = False, concat_x: bool = False, mul_u_activation_type: str = "none", group_norm: bool = False,
    num_heads: int = 1, linear_dim: int = -1, round_joined_to: torch.dtype = None,
) -> torch.Tensor:
    """``x + norm_mul(...) @ output_weight`` in fp32; ``round_joined_to`` reproduces the one rounding the reference's
    low-precision path has before the GEMM (``norm_mul``'s result is cast to the input type, pt_hstu_linear.py:85)."""
    y = norm_mul(attn, u, norm_weight, norm_bias, eps, silu_u, concat_u, concat_x, mul_u_activation_type, group_norm, num_heads, linear_dim)
    if round_joined_to is not None:
        y = y.to(round_joined_to).float()
    return torch.addmm(x.float(), y, output_weight.float())
