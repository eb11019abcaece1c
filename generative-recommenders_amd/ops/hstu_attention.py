"""``hstu_mha`` / ``delta_hstu_mha`` with the reference's signatures, running on gfx950 HIP kernels.

Mirrors ``generative_recommenders/ops/hstu_attention.py`` of the reference (``hstu_mha``
at lines 101-207, ``delta_hstu_mha`` at lines 210-284): same argument names, defaults, assertion
messages and output shapes.  Differences, all explicit:

* there is one backend, so ``kernel`` / ``enable_tma`` are accepted and ignored; ``sort_by_length`` is, as in
  the reference, a scheduling hint (long sequences are started first) that never changes the result;
* ``hstu_mha`` is differentiable for bf16 / fp16 / fp32 inputs (``dq, dk, dv`` come from the backward kernels through
  an autograd function, as ``_AttentionFunction`` does in the reference, ``triton_hstu_attention.py:2978-3093``; for
  fp32 inputs the backward runs on bf16 copies and widens its results); ``delta_hstu_mha`` and the fp8 form are
  forward only -- inputs that require grad under ``torch.enable_grad()`` raise ``NotImplementedError`` there;
* tensors must live on a HIP device; there is no CPU or PyTorch fallback;
* fp32 q/k/v are rounded to fp16 inside the library (11-bit significand; the reference's Triton path multiplies in
  tf32) and give an fp32 result;
* fp8 (``torch.float8_e4m3fn``) q/k/v take per-tensor scales through ``q_scale``/``k_scale``/``v_scale``
  and give bf16 output, as the reference's native op does (``flash_common.cpp:596-607``);
* ``tile_config`` / ``kv_splits`` choose the kernel and the split of the kv range over workgroups (0 = automatic);
  they change the schedule, and with a split the fp32 summation order, never the mask or the scaling.
"""

import functools
from typing import Optional

import torch

from ..common import HammerKernel, switch_to_contiguous_if_needed
from . import hip_backend


def _kernel_layout(x: torch.Tensor) -> torch.Tensor:
    """Dense innermost dim (``common.py:262-269``) and 16-byte aligned rows, copying only if needed."""
    x = switch_to_contiguous_if_needed(x)
    per16 = 16 // x.element_size()
    if x.data_ptr() % 16 != 0 or x.stride(0) % per16 != 0 or x.stride(1) % per16 != 0:
        x = x.contiguous()
        if x.data_ptr() % 16 != 0:
            x = x.clone(memory_format=torch.contiguous_format)
    return x


def _index_tensor(x: torch.Tensor, name: str) -> torch.Tensor:
    torch._assert(x.dtype in (torch.int32, torch.int64), f"{name} must be int32 or int64")
    return x.contiguous()


def _check_forward_only(*tensors: torch.Tensor) -> None:
    if torch.is_grad_enabled() and any(t.requires_grad for t in tensors):
        raise NotImplementedError(
            "the HIP backend implements the forward pass only; call it under torch.no_grad() "
            "or detach the inputs"
        )


class _HstuMhaFunction(torch.autograd.Function):
    """Forward and backward through the C ABI; saves only the inputs (the backward recomputes the scores)."""

    @staticmethod
    def forward(ctx, q, k, v, seq_offsets, num_targets, max_seq_len, alpha, max_attn_len, contextual_seq_len,
                min_full_attn_seq_len, sort_by_length, tile_config, kv_splits, attn_scale, bwd_workspace):
        q, k, v = _kernel_layout(q.detach()), _kernel_layout(k.detach()), _kernel_layout(v.detach())
        out = torch.empty((v.shape[0], v.shape[1], v.shape[2]), dtype=v.dtype, device=v.device)
        if out.numel() > 0:
            hip_backend.mha_fwd(
                q, k, v, out, seq_offsets, num_targets, max_seq_len=max_seq_len, alpha=alpha, delta_size=0,
                max_attn_len=max_attn_len, contextual_seq_len=contextual_seq_len, min_full_attn_seq_len=min_full_attn_seq_len,
                tile_config=tile_config, sort_by_length=sort_by_length, kv_splits=kv_splits, attn_scale=attn_scale,
            )
        ctx.save_for_backward(q, k, v, seq_offsets, *([] if num_targets is None else [num_targets]))
        ctx.has_targets = num_targets is not None
        ctx.attn_scale = attn_scale  # a constant of the call (no gradient flows into it)
        ctx.bwd_workspace = bwd_workspace  # the caller's dS scratch, or None: the backward recomputes the scores
        ctx.params = (max_seq_len, alpha, max_attn_len, contextual_seq_len, min_full_attn_seq_len)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, seq_offsets = ctx.saved_tensors[:4]
        num_targets = ctx.saved_tensors[4] if ctx.has_targets else None
        max_seq_len, alpha, max_attn_len, contextual_seq_len, min_full_attn_seq_len = ctx.params
        # fp32 inputs: the backward kernels take 16-bit operands, so they run on bf16 copies (fp32's range, 8 bits of
        # mantissa; the products accumulate in fp32 as always) and the gradients are widened again -- the counterpart
        # of the forward's fp16 copies, with the range of dout, which can be tiny, kept whole
        wide = q.dtype == torch.float32
        if wide:
            q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
        # the kernels write the gradient of every row of every sequence that keeps the contract; rows past max_seq_len of
        # a sequence that breaks it come back uninitialised, like the forward's (HSTU_HIP_CHECK_CONTRACT=1 raises instead)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        if q.numel() > 0:
            if ctx.attn_scale is not None:
                # out = attn_scale[row] * N * (the result with 1 / N), so the gradients are those of the plain call for
                # dout scaled the same way
                factor = ctx.attn_scale * float(max_seq_len)
                dout = dout.detach().float() * (factor.view(-1, 1, 1) if factor.dim() > 0 else factor)
            dout = _kernel_layout(dout.detach().to(q.dtype))
            hip_backend.mha_bwd(
                dout, q, k, v, dq, dk, dv, seq_offsets, num_targets, max_seq_len, alpha, max_attn_len, contextual_seq_len,
                min_full_attn_seq_len, workspace=ctx.bwd_workspace,
            )
        if wide:
            dq, dk, dv = dq.float(), dk.float(), dv.float()
        return (dq, dk, dv) + (None,) * 12


def _require_device(t: torch.Tensor, name: str) -> None:
    # same wording as hstu_attention.py:132-135 of the reference
    torch._assert(t.is_cuda, f"{name} must be CUDA tensor")


def _profiled(name: str):
    """Runs the operator inside a ``torch.profiler.record_function`` range, so that it shows up by name in a trace as the
    reference's ranges around the same calls do (``modules/stu.py:303,392``)."""

    def decorate(fn):
        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            with torch.profiler.record_function(name):
                return fn(*args, **kwargs)

        return wrapper

    return decorate


@_profiled("hstu_mha")
def hstu_mha(
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
    sort_by_length: bool = False,
    kernel: HammerKernel = HammerKernel.HIP,
    enable_tma: bool = False,
    q_scale: float = 1.0,
    k_scale: float = 1.0,
    v_scale: float = 1.0,
    tile_config: int = 0,
    kv_splits: int = 0,
    bwd_workspace: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Jagged HSTU attention forward; returns ``[L, H, Dv]``.

    ``out[r] = sum_s M(r, s) * silu(alpha * q_r . k_s) / max_seq_len * v_s`` per sequence and head
    (``attn_scale``, one factor or one per row of ``q``, takes the place of ``1 / max_seq_len``).

    Caller contract, as in the reference: ``0 <= n_b <= max_seq_len``, ``0 <= num_targets[b] <= n_b``,
    ``n_b - num_targets[b] >= contextual_seq_len``.  It is not checked by default (that would read the offsets back);
    rows of a sequence that breaks it may come back UNINITIALISED (the output is ``torch.empty``).  Set
    ``HSTU_HIP_CHECK_CONTRACT=1`` in the environment to have every call validated on the device first and raise
    ``ValueError`` instead.

    The backward recomputes the scores and allocates nothing that grows with ``max_seq_len``.  ``bwd_workspace`` (uint8,
    ``hip_backend.mha_bwd_workspace_bytes`` bytes, kept by the caller across steps) selects the faster form that stores
    dS there; the choice never depends on how much device memory is free.
    """
    torch._assert(max_seq_len > 0, "max_seq_len must be larger than 0")
    torch._assert(q.dim() == 3, "q must be 3-D")
    torch._assert(k.shape == q.shape, "k must be the same shape as q")
    torch._assert(v.dim() == 3, "v must be 3-D")
    torch._assert(v.shape[0] == q.shape[0], "wrong v shape[0]")
    torch._assert(v.shape[1] == q.shape[1], "wrong v shape[1]")
    torch._assert(causal, "only support causal attention")
    _require_device(q, "q")
    _require_device(k, "k")
    _require_device(v, "v")
    _require_device(seq_offsets, "seq_offsets")
    torch._assert(dropout_pr < 1e-6, "dropout for triton path not implemented")
    if attn_scale is not None:
        # pt_hstu_attention.py:152-165: one factor (0-dim) or one per query row, in place of 1 / max_seq_len
        _require_device(attn_scale, "attn_scale")
        torch._assert(attn_scale.dim() == 0 or (attn_scale.dim() == 1 and attn_scale.shape[0] == q.shape[0]),
                      "attn_scale must be 0-dim or hold one value per row of q")
        if torch.is_grad_enabled() and attn_scale.requires_grad:
            raise NotImplementedError("the HIP backend has no gradient for attn_scale; detach it")
        attn_scale = attn_scale.detach().to(torch.float32).contiguous()
    torch._assert(k.dtype == q.dtype and v.dtype == q.dtype, "q, k and v must have the same dtype")
    if num_targets is not None:
        _require_device(num_targets, "num_targets")
        torch._assert(num_targets.numel() == seq_offsets.numel() - 1, "num_targets must have one entry per sequence")
        num_targets = _index_tensor(num_targets, "num_targets")
    seq_offsets = _index_tensor(seq_offsets, "seq_offsets")
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v)):
        if q.dtype not in (torch.bfloat16, torch.float16, torch.float32):
            _check_forward_only(q, k, v)
        return _HstuMhaFunction.apply(
            q, k, v, seq_offsets, num_targets, max_seq_len, alpha, max_attn_len, contextual_seq_len, min_full_attn_seq_len,
            sort_by_length, tile_config, kv_splits, attn_scale, bwd_workspace,
        )

    q = _kernel_layout(q.detach())
    k = _kernel_layout(k.detach())
    v = _kernel_layout(v.detach())
    out_dtype = torch.bfloat16 if q.dtype == torch.float8_e4m3fn else v.dtype
    out = torch.empty((v.shape[0], v.shape[1], v.shape[2]), dtype=out_dtype, device=v.device)
    if out.numel() == 0:
        return out
    hip_backend.mha_fwd(
        q,
        k,
        v,
        out,
        seq_offsets,
        num_targets,
        max_seq_len=max_seq_len,
        alpha=alpha,
        delta_size=0,
        max_attn_len=max_attn_len,
        contextual_seq_len=contextual_seq_len,
        min_full_attn_seq_len=min_full_attn_seq_len,
        q_scale=q_scale,
        k_scale=k_scale,
        v_scale=v_scale,
        tile_config=tile_config,
        sort_by_length=sort_by_length,
        kv_splits=kv_splits,
        attn_scale=attn_scale,
    )
    return out


@_profiled("delta_hstu_mha")
def delta_hstu_mha(
    max_seq_len: int,
    alpha: float,
    delta_q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    seq_offsets: torch.Tensor,
    num_targets: Optional[torch.Tensor] = None,
    max_attn_len: int = 0,
    contextual_seq_len: int = 0,
    kernel: HammerKernel = HammerKernel.HIP,
    enable_tma: bool = False,
    q_scale: float = 1.0,
    k_scale: float = 1.0,
    v_scale: float = 1.0,
    tile_config: int = 0,
    kv_splits: int = 0,
) -> torch.Tensor:
    """Cached-KV (M-FALCON) forward: ``delta_q`` holds the last ``L // B`` positions of every sequence.

    Returns ``[B * delta_size, H, Dv]`` in the dtype of ``delta_q`` (bf16 for fp8 inputs).
    """
    torch._assert(delta_q.dim() == 3, "delta_q must be 3-D")
    L, H, D = delta_q.shape
    B = seq_offsets.size(0) - 1
    torch._assert(B > 0, "seq_offsets must hold at least one sequence")
    delta_size = L // B
    torch._assert(max_seq_len > 0, "max_seq_len must be larger than 0")
    torch._assert(L % B == 0, "delta_q must be padded")
    torch._assert(k.dim() == 3, "k must be 3-D")
    torch._assert(k.shape[1] == H, "wrong k shape[1]")
    torch._assert(k.shape[2] == D, "wrong k shape[2]")
    torch._assert(v.dim() == 3, "v must be 3-D")
    torch._assert(v.shape[1] == H, "wrong v shape[1]")
    torch._assert(v.shape[0] == k.shape[0], "wrong v shape[0]")
    _require_device(delta_q, "q")
    _require_device(k, "k")
    _require_device(v, "v")
    _require_device(seq_offsets, "seq_offsets")
    torch._assert(k.dtype == delta_q.dtype and v.dtype == delta_q.dtype, "q, k and v must have the same dtype")
    if num_targets is not None:
        _require_device(num_targets, "num_targets")
        torch._assert(num_targets.numel() == B, "num_targets must have one entry per sequence")
        num_targets = _index_tensor(num_targets, "num_targets")
    _check_forward_only(delta_q, k, v)
    seq_offsets = _index_tensor(seq_offsets, "seq_offsets")

    delta_q = _kernel_layout(delta_q.detach())
    k = _kernel_layout(k.detach())
    v = _kernel_layout(v.detach())
    out_dtype = torch.bfloat16 if delta_q.dtype == torch.float8_e4m3fn else delta_q.dtype
    out = torch.empty((L, H, v.shape[2]), dtype=out_dtype, device=delta_q.device)
    if out.numel() == 0:
        return out
    hip_backend.mha_fwd(
        delta_q,
        k,
        v,
        out,
        seq_offsets,
        num_targets,
        max_seq_len=max_seq_len,
        alpha=alpha,
        delta_size=delta_size,
        max_attn_len=max_attn_len,
        contextual_seq_len=contextual_seq_len,
        min_full_attn_seq_len=0,
        q_scale=q_scale,
        k_scale=k_scale,
        v_scale=v_scale,
        tile_config=tile_config,
        kv_splits=kv_splits,
    )
    return out
