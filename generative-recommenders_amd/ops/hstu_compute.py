"""``hstu_compute_uqvk`` with the reference's signature: layer norm + uvqk projection + split + SiLU(u).

Mirrors ``generative_recommenders/ops/hstu_compute.py:54-104`` of the reference.  The layer norm is a hand-written
gfx950 kernel; the projection is a plain GEMM and runs on hipBLASLt with the bias and, for the u columns, the SiLU
in its epilogue (``csrc/hstu_uqvk.hip``, ``include/hstu_uqvk.h``).  ``u, q, k, v`` come back as column slices of one
``[L, (2*hidden + 2*attn) * H]`` buffer, which ``hstu_mha`` / ``delta_hstu_mha`` read in place.
Forward only, device tensors only, bf16 or fp16; ``kernel`` is accepted and ignored.
"""

import ctypes
import os
from typing import Optional, Tuple

import torch

from ..build import UQVK_LIB_PATH
from ..common import HammerKernel


class HstuUqvkArgs(ctypes.Structure):
    """Mirror of ``HstuUqvkArgs`` in include/hstu_uqvk.h (field order and types must match)."""

    _fields_ = [
        ("x", ctypes.c_void_p),
        ("x_row_stride", ctypes.c_int64),
        ("norm_weight", ctypes.c_void_p),
        ("norm_bias", ctypes.c_void_p),
        ("norm_eps", ctypes.c_float),
        ("uvqk_weight", ctypes.c_void_p),
        ("uvqk_bias", ctypes.c_void_p),
        ("uvqk", ctypes.c_void_p),
        ("rows", ctypes.c_int64),
        ("d_model", ctypes.c_int32),
        ("heads", ctypes.c_int32),
        ("attn_dim", ctypes.c_int32),
        ("hidden_dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_int64),
    ]


EXPORTS = ("hstu_uqvk_workspace_bytes", "hstu_uqvk_forward", "hstu_uqvk_layer_norm", "hstu_uqvk_last_error")

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """Load libhstu_uqvk.so.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(UQVK_LIB_PATH):
            raise RuntimeError(f"{UQVK_LIB_PATH} is missing: build it with __graft_entry__.build().  There is no fallback.")
        L = ctypes.CDLL(UQVK_LIB_PATH)
        L.hstu_uqvk_workspace_bytes.restype = ctypes.c_size_t
        L.hstu_uqvk_workspace_bytes.argtypes = [ctypes.POINTER(HstuUqvkArgs)]
        L.hstu_uqvk_forward.restype = ctypes.c_int
        L.hstu_uqvk_forward.argtypes = [ctypes.POINTER(HstuUqvkArgs), ctypes.c_void_p]
        L.hstu_uqvk_layer_norm.restype = ctypes.c_int
        L.hstu_uqvk_layer_norm.argtypes = [
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_int64,
            ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p,
        ]
        L.hstu_uqvk_last_error.restype = ctypes.c_char_p
        _lib = L
    return _lib


_STATUS = {-1: ValueError, -2: RuntimeError, -4: RuntimeError, -5: ValueError, -6: NotImplementedError, -7: RuntimeError, -9: RuntimeError}


def _raise_for_status(rc: int) -> None:
    if rc != 0:
        extra = lib().hstu_uqvk_last_error().decode()
        raise _STATUS.get(rc, RuntimeError)(f"hstu_uqvk: status {rc}" + (f" ({extra})" if extra else ""))


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return 0
    if dt == torch.float16:
        return 1
    raise RuntimeError(f"hstu_uqvk only supports bf16 and fp16, got {dt}")


def _check(x: torch.Tensor, *others: torch.Tensor) -> None:
    torch._assert(x.is_cuda, "x must be CUDA tensor")
    for t in others:
        torch._assert(t.is_cuda and t.dtype == x.dtype, "all tensors must be CUDA tensors of x's dtype")
    if torch.is_grad_enabled() and any(t.requires_grad for t in (x,) + others):
        raise NotImplementedError(
            "the HIP backend implements the forward pass only; call it under torch.no_grad() or detach the inputs"
        )


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """``layer_norm`` over the last dimension of a 2-D tensor with fp32 statistics
    (``ops/pytorch/pt_layer_norm.py:24-39`` of the reference)."""
    torch._assert(x.dim() == 2, "x must be 2-D")
    _check(x, weight, bias)
    x = x.detach()
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
        x = x.contiguous()
    out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device).cuda_stream
        rc = lib().hstu_uqvk_layer_norm(
            x.data_ptr(), x.stride(0), weight.detach().contiguous().data_ptr(), bias.detach().contiguous().data_ptr(), eps,
            out.data_ptr(), out.stride(0), x.shape[0], x.shape[1], _dtype_code(x.dtype), ctypes.c_void_p(stream),
        )
    _raise_for_status(rc)
    return out


def hstu_compute_uqvk(
    x: torch.Tensor,
    norm_weight: torch.Tensor,
    norm_bias: torch.Tensor,
    norm_eps: float,
    num_heads: int,
    attn_dim: int,
    hidden_dim: int,
    uvqk_weight: torch.Tensor,
    uvqk_bias: torch.Tensor,
    kernel: HammerKernel = HammerKernel.HIP,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(u, q, k, v)``: ``u [L, hidden*H]`` already through SiLU, ``q, k [L, H, attn]``, ``v [L, H, hidden]``,
    all views of one buffer."""
    torch._assert(x.dim() == 2, "x must be 2-D")
    n_out = (2 * hidden_dim + 2 * attn_dim) * num_heads
    torch._assert(uvqk_weight.shape == (x.shape[1], n_out), "uvqk_weight must be [d_model, (2*hidden + 2*attn) * heads]")
    torch._assert(uvqk_bias.shape == (n_out,), "uvqk_bias must be [(2*hidden + 2*attn) * heads]")
    _check(x, norm_weight, norm_bias, uvqk_weight, uvqk_bias)
    x = x.detach()
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
        x = x.contiguous()
    uvqk = torch.empty((x.shape[0], n_out), dtype=x.dtype, device=x.device)
    a = HstuUqvkArgs()
    a.x, a.x_row_stride = x.data_ptr(), x.stride(0)
    nw, nb = norm_weight.detach().contiguous(), norm_bias.detach().contiguous()
    w, b = uvqk_weight.detach().contiguous(), uvqk_bias.detach().contiguous()
    a.norm_weight, a.norm_bias, a.norm_eps = nw.data_ptr(), nb.data_ptr(), norm_eps
    a.uvqk_weight, a.uvqk_bias, a.uvqk = w.data_ptr(), b.data_ptr(), uvqk.data_ptr()
    a.rows, a.d_model = x.shape[0], x.shape[1]
    a.heads, a.attn_dim, a.hidden_dim = num_heads, attn_dim, hidden_dim
    a.dtype = _dtype_code(x.dtype)
    if x.shape[0] > 0:
        need = lib().hstu_uqvk_workspace_bytes(ctypes.byref(a))
        workspace = torch.empty(need + 256, dtype=torch.uint8, device=x.device)
        base = (workspace.data_ptr() + 255) & ~255
        a.workspace, a.workspace_bytes = base, need
        with torch.cuda.device(x.device):
            stream = torch.cuda.current_stream(x.device).cuda_stream
            rc = lib().hstu_uqvk_forward(ctypes.byref(a), ctypes.c_void_p(stream))
        _raise_for_status(rc)
    u, v, q, k = torch.split(
        uvqk, [hidden_dim * num_heads, hidden_dim * num_heads, attn_dim * num_heads, attn_dim * num_heads], dim=1
    )
    return u, q.view(-1, num_heads, attn_dim), k.view(-1, num_heads, attn_dim), v.view(-1, num_heads, hidden_dim)
