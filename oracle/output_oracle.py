"""CPU restatement of ``hstu_compute_output`` -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU baseline may import this module; the product
package never does.

``norm_mul`` follows ``pytorch_norm_mul_dropout`` (``generative_recommenders/ops/pytorch/pt_hstu_linear.py:24-85``);
its dropout (``F.dropout(y, p, training)``, :80-84: zero with probability p, survivors times ``1 / (1 - p)``, over the
whole concatenation, in fp32) takes its mask from ``dropout_keep``: the reference draws it from the framework's
generator, whose stream nothing outside the framework can reproduce, so the mask is this build's own -- Philox4x32-10
keyed by (seed, offset, element position), stated in ``include/hstu_linear.h`` -- and what is checked against the
reference is the arithmetic around it.  ``compute_output`` follows
``pytorch_hstu_compute_output`` (``pt_hstu_linear.py:88-124``), the PyTorch backend behind ``hstu_compute_output``
(``ops/hstu_compute.py:107-214``).  fp32 on whatever the caller passes.

Pinned by: ``group_norm_by_hand`` / ``uqvk_oracle.layer_norm_by_hand`` (mean and biased variance written out in
fp64) against the library calls used here; the column blocks of the concatenation against the inputs they copy;
a one-hot ``output_weight`` that turns the GEMM into a column selection (so a swapped or dropped block shows);
``sigmoid`` / ``silu`` special values.  The reference holds no golden vectors for this function: its test compares
two of its own backends on a GPU (``ops/tests/hstu_compute_test.py:38-79``), with inputs drawn uniformly from
[-0.1, 0.1] -- the distribution the GPU tests here use as well.  ``philox4x32_10`` is pinned by the known-answer
vectors of its authors' library (Random123, ``kat_vectors``: zero, all-ones and the digits of pi as counter and key).
"""

import numpy as np
import torch
import torch.nn.functional as F


def group_norm_by_hand(x: torch.Tensor, num_heads: int, linear_dim: int, weight: torch.Tensor, bias: torch.Tensor, eps: float):
    """Each head's ``linear_dim`` columns normalised on their own; one weight and one bias per head."""
    x = x.double().view(-1, num_heads, linear_dim)
    mean = x.mean(dim=2, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=2, keepdim=True)
    y = (x - mean) / torch.sqrt(var + eps) * weight.double().view(1, -1, 1) + bias.double().view(1, -1, 1)
    return y.view(-1, num_heads * linear_dim)


def philox4x32_10(counter: np.ndarray, key: np.ndarray) -> np.ndarray:
    """Salmon et al., "Parallel random numbers: as easy as 1, 2, 3" (SC'11): ``counter [n, 4]`` and ``key [n, 2]`` (or
    ``[2]``) of uint32 -> ``[n, 4]`` uint32.  Ten rounds of: two 32x32 -> 64-bit products of counter words 0 and 2 with
    fixed multipliers; the high halves, xor-ed with words 1 and 3 and the key, become words 0 and 2, the low halves
    words 1 and 3; the key is bumped by two Weyl constants between rounds."""
    c = np.array(counter, dtype=np.uint64).reshape(-1, 4).copy()
    k = np.broadcast_to(np.array(key, dtype=np.uint64).reshape(-1, 2), (c.shape[0], 2)).copy()
    m32 = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c[:, 0]
        p1 = np.uint64(0xCD9E8D57) * c[:, 2]
        n0 = (p1 >> np.uint64(32)) ^ c[:, 1] ^ k[:, 0]
        n2 = (p0 >> np.uint64(32)) ^ c[:, 3] ^ k[:, 1]
        c = np.stack([n0, p1 & m32, n2, p0 & m32], axis=1)
        k[:, 0] = (k[:, 0] + np.uint64(0x9E3779B9)) & m32
        k[:, 1] = (k[:, 1] + np.uint64(0xBB67AE85)) & m32
    return c.astype(np.uint32)


def dropout_keep(ratio: float, seed: int, offset: int, rows: int, width: int) -> np.ndarray:
    """``[rows, width]`` bool: element (r, c) survives when word ``c % 4`` of Philox(counter = (g lo, g hi, offset lo,
    offset hi), key = (seed lo, seed hi)), ``g = (r * width + c) // 4``, is at least ``floor(ratio * 2^32)``."""
    assert width % 4 == 0
    groups = np.arange(rows * width // 4, dtype=np.uint64)
    m32 = np.uint64(0xFFFFFFFF)
    ctr = np.stack([groups & m32, groups >> np.uint64(32), np.full_like(groups, offset & 0xFFFFFFFF), np.full_like(groups, offset >> 32)], axis=1)
    words = philox4x32_10(ctr, np.array([seed & 0xFFFFFFFF, seed >> 32]))
    return (words.reshape(rows, width) >= np.uint32(int(float(np.float32(ratio)) * 4294967296.0)))


def dropout(y: torch.Tensor, ratio: float, seed: int, offset: int) -> torch.Tensor:
    """pt_hstu_linear.py:80-84 on the fp32 concatenation: survivors times ``1 / (1 - p)`` (formed in fp32), the rest zero."""
    keep = torch.from_numpy(dropout_keep(ratio, seed, offset, y.shape[0], y.shape[1]))
    scale = np.float32(1.0) / (np.float32(1.0) - np.float32(ratio))
    return torch.where(keep, y.float() * float(scale), torch.zeros((), dtype=torch.float32))


def norm_mul(
    attn: torch.Tensor, u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, silu_u: bool = False,
    concat_u: bool = False, concat_x: bool = False, mul_u_activation_type: str = "none", group_norm: bool = False,
    num_heads: int = 1, linear_dim: int = -1,
) -> torch.Tensor:
    """fp32 result before dropout, not yet rounded to the input type (pt_hstu_linear.py:40-79)."""
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
    num_heads: int = 1, linear_dim: int = -1, round_joined_to: torch.dtype = None, dropout_state=None,
) -> torch.Tensor:
    """``x + dropout(norm_mul(...)) @ output_weight`` in fp32; ``round_joined_to`` reproduces the one rounding the
    reference's low-precision path has before the GEMM (``norm_mul``'s result is cast to the input type,
    pt_hstu_linear.py:85); ``dropout_state = (ratio, seed, offset)`` or None (inference)."""
    y = norm_mul(attn, u, norm_weight, norm_bias, eps, silu_u, concat_u, concat_x, mul_u_activation_type, group_norm, num_heads, linear_dim)
    if dropout_state is not None:
        y = dropout(y, *dropout_state)
    if round_joined_to is not None:
        y = y.to(round_joined_to).float()
    return torch.addmm(x.float(), y, output_weight.float())
