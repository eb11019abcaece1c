"""``torch.ops.hstu.hstu_mha`` / ``torch.ops.hstu.hstu_mha_fwd`` on the HIP kernels.

The reference's TorchScript path and its ``cuda_hstu_mha`` wrappers call the dispatcher operator
``hstu::hstu_mha`` with 27 positional arguments (``generative_recommenders/ops/hstu_attention.py:50-98``,
``ops/cpp/cuda_hstu_attention.py:136-196``); the schemas are those of
``ops/cpp/hstu_attention/flash_api_cpu.cpp:142-235``, the host checks those of ``flash_common.cpp:394-724``.
Importing this module defines the same two schemas (unless an extension has defined them already) and registers
implementations for device tensors that forward to the C ABI (``hstu_hip_mha_fwd`` / ``hstu_hip_mha_bwd``).
What the C ABI has no kernel for is refused with the exception class the reference's ``TORCH_CHECK`` raises
(``RuntimeError``), never silently ignored:

* dense ``[B, S, H, D]`` inputs (``seq_offsets=None``), cross attention (``seq_offsets_q`` / ``max_q_len``), softmax
  heads, more than one group and the per-group tensors;
* fp8 descale tensors with more than one element (the kernels take one scale per tensor; a one-element tensor is read
  on the host, which synchronises).

``deterministic``, ``sm_margin``, ``training`` and ``use_bf16_dq_accum`` change nothing here: the kernels are always
deterministic, leave no compute units aside, have no dropout and accumulate dq in fp32.
"""

from typing import Optional, Tuple

import torch

from . import hip_backend

_FWD_ARGS = (
    "SymInt max_seq_len, float alpha, Tensor q, Tensor k, Tensor v, Tensor? seq_offsets, bool causal, "
    "Tensor? num_targets, Tensor? attn_scale, int max_attn_len, int min_full_attn_seq_len, int contextual_seq_len, "
    "Tensor? q_descale, Tensor? k_descale, Tensor? v_descale, "
)
_TAIL_ARGS = (
    "int sm_margin = 0, SymInt max_q_len = 0, Tensor? seq_offsets_q = None, int num_softmax_heads = 0, "
    "bool training = True, Tensor? max_seq_len_tensor = None, Tensor? contextual_seq_len_tensor = None, "
    "Tensor? max_attn_len_tensor = None, Tensor? min_full_attn_seq_len_tensor = None, int num_groups = 1"
)
SCHEMA_HSTU_MHA_FWD = "hstu_mha_fwd(" + _FWD_ARGS + _TAIL_ARGS + ") -> (Tensor, Tensor?)"
SCHEMA_HSTU_MHA = (
    "hstu_mha(" + _FWD_ARGS + "bool sort_by_length, bool deterministic, " + _TAIL_ARGS + ", bool use_bf16_dq_accum = False) -> Tensor"
)


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _scale_of(descale: Optional[torch.Tensor], name: str) -> float:
    if descale is None:
        return 1.0
    _check(descale.numel() == 1, f"{name}: one scale per tensor is built (got {descale.numel()} elements)")
    return float(descale.float().reshape(()))


def _forward(
    max_seq_len, alpha, q, k, v, seq_offsets, causal, num_targets, attn_scale, max_attn_len, min_full_attn_seq_len,
    contextual_seq_len, q_descale, k_descale, v_descale, sort_by_length, max_q_len, seq_offsets_q, num_softmax_heads,
    per_group_tensors, num_groups,
) -> torch.Tensor:
    from .hstu_attention import _index_tensor, _kernel_layout

    _check(q.dim() == 3 and seq_offsets is not None, "hstu_mha: only the jagged [total, heads, dim] layout with seq_offsets is built")
    _check(causal, "hstu_mha: only causal attention is built")
    _check(seq_offsets_q is None and int(max_q_len) in (0, int(max_seq_len)), "hstu_mha: cross attention (seq_offsets_q) is not built")
    _check(num_softmax_heads == 0, "hstu_mha: softmax heads are not built")
    _check(num_groups == 1 and all(t is None for t in per_group_tensors), "hstu_mha: one group only")
    # flash_common.cpp:428-452
    _check(q.dtype in (torch.float16, torch.bfloat16, torch.float8_e4m3fn), "FlashAttention only supports fp16, bf16, and fp8_e4m3 data type")
    _check(k.dtype == q.dtype, "query and key must have the same dtype")
    _check(v.dtype == q.dtype, "query and value must have the same dtype")
    _check(k.shape == q.shape and v.shape[:2] == q.shape[:2], "hstu_mha: q, k, v shapes disagree")
    _check(q.is_cuda and k.is_cuda and v.is_cuda and seq_offsets.is_cuda, "hstu_mha: tensors must be on the GPU")
    q, k, v = _kernel_layout(q), _kernel_layout(k), _kernel_layout(v)
    seq_offsets = _index_tensor(seq_offsets, "seq_offsets")
    if num_targets is not None:
        num_targets = _index_tensor(num_targets, "num_targets")
    if attn_scale is not None:
        _check(attn_scale.numel() in (1, q.shape[0]), "attn_scale: one element, or one per row of q")
        if torch.is_grad_enabled() and attn_scale.requires_grad:
            # (as generative_recommenders_amd.hstu_mha does: silently returning no gradient would be worse)
            raise NotImplementedError("hstu_mha: no gradient is computed for attn_scale; pass it detached")
        attn_scale = attn_scale.detach().to(torch.float32)
        attn_scale = attn_scale.reshape(()) if attn_scale.numel() == 1 else attn_scale.reshape(-1).contiguous()
    out_dtype = torch.bfloat16 if q.dtype == torch.float8_e4m3fn else q.dtype  # flash_common.cpp:596-607
    out = torch.empty((q.shape[0], q.shape[1], v.shape[2]), dtype=out_dtype, device=q.device)
    if out.numel() == 0:
        return out
    hip_backend.mha_fwd(
        q, k, v, out, seq_offsets, num_targets, max_seq_len=int(max_seq_len), alpha=float(alpha), delta_size=0,
        max_attn_len=int(max_attn_len), contextual_seq_len=int(contextual_seq_len), min_full_attn_seq_len=int(min_full_attn_seq_len),
        q_scale=_scale_of(q_descale, "q_descale"), k_scale=_scale_of(k_descale, "k_descale"), v_scale=_scale_of(v_descale, "v_descale"),
        sort_by_length=bool(sort_by_length), attn_scale=attn_scale,
    )
    return out


def _hstu_mha_fwd(
    max_seq_len, alpha, q, k, v, seq_offsets, causal, num_targets, attn_scale, max_attn_len, min_full_attn_seq_len,
    contextual_seq_len, q_descale, k_descale, v_descale, sm_margin=0, max_q_len=0, seq_offsets_q=None, num_softmax_heads=0,
    training=True, max_seq_len_tensor=None, contextual_seq_len_tensor=None, max_attn_len_tensor=None,
    min_full_attn_seq_len_tensor=None, num_groups=1,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    out = _forward(
        max_seq_len, alpha, q, k, v, seq_offsets, causal, num_targets, attn_scale, max_attn_len, min_full_attn_seq_len,
        contextual_seq_len, q_descale, k_descale, v_descale, False, max_q_len, seq_offsets_q, num_softmax_heads,
        (max_seq_len_tensor, contextual_seq_len_tensor, max_attn_len_tensor, min_full_attn_seq_len_tensor), num_groups,
    )
    return out, None  # the second result is the softmax statistics of softmax heads


def _hstu_mha(
    max_seq_len, alpha, q, k, v, seq_offsets, causal, num_targets, attn_scale, max_attn_len, min_full_attn_seq_len,
    contextual_seq_len, q_descale, k_descale, v_descale, sort_by_length, deterministic, sm_margin=0, max_q_len=0,
    seq_offsets_q=None, num_softmax_heads=0, training=True, max_seq_len_tensor=None, contextual_seq_len_tensor=None,
    max_attn_len_tensor=None, min_full_attn_seq_len_tensor=None, num_groups=1, use_bf16_dq_accum=False,
) -> torch.Tensor:
    return _forward(
        max_seq_len, alpha, q, k, v, seq_offsets, causal, num_targets, attn_scale, max_attn_len, min_full_attn_seq_len,
        contextual_seq_len, q_descale, k_descale, v_descale, sort_by_length, max_q_len, seq_offsets_q, num_softmax_heads,
        (max_seq_len_tensor, contextual_seq_len_tensor, max_attn_len_tensor, min_full_attn_seq_len_tensor), num_groups,
    )


def _setup_context(ctx, inputs, output) -> None:
    (max_seq_len, alpha, q, k, v, seq_offsets, _causal, num_targets, attn_scale, max_attn_len, min_full_attn_seq_len,
     contextual_seq_len) = inputs[:12]
    ctx.save_for_backward(q, k, v, seq_offsets, *([] if num_targets is None else [num_targets]),
                          *([] if attn_scale is None else [attn_scale]))
    ctx.has_targets, ctx.has_scale = num_targets is not None, attn_scale is not None
    ctx.params = (int(max_seq_len), float(alpha), int(max_attn_len), int(contextual_seq_len), int(min_full_attn_seq_len))
    ctx.n_inputs = len(inputs)


def _backward(ctx, dout) -> Tuple[Optional[torch.Tensor], ...]:
    from .hstu_attention import _kernel_layout

    saved = list(ctx.saved_tensors)
    q, k, v, seq_offsets = saved[:4]
    num_targets = saved[4] if ctx.has_targets else None
    attn_scale = saved[-1] if ctx.has_scale else None
    max_seq_len, alpha, max_attn_len, contextual_seq_len, min_full_attn_seq_len = ctx.params
    _check(q.dtype in (torch.float16, torch.bfloat16), "hstu_mha backward: fp16 and bf16 only")
    q, k, v = _kernel_layout(q.detach()), _kernel_layout(k.detach()), _kernel_layout(v.detach())
    # (as the other autograd path: the kernels write every row of every sequence that keeps the caller's contract)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if q.numel() > 0:
        if attn_scale is not None:
            factor = attn_scale.detach().float() * float(max_seq_len)
            dout = dout.detach().float() * (factor.reshape(-1, 1, 1) if factor.numel() > 1 else factor.reshape(()))
        dout = _kernel_layout(dout.detach().to(q.dtype))
        hip_backend.mha_bwd(dout, q, k, v, dq, dk, dv, seq_offsets.contiguous(), None if num_targets is None else num_targets.contiguous(),
                            max_seq_len, alpha, max_attn_len, contextual_seq_len, min_full_attn_seq_len)
    return (None, None, dq, dk, dv) + (None,) * (ctx.n_inputs - 5)


_lib: Optional[torch.library.Library] = None


def register() -> None:
    """Define (if nobody has) and implement the two operators; safe to call more than once."""
    global _lib
    if _lib is not None:
        return
    lib = torch.library.Library("hstu", "FRAGMENT")
    for name, schema in (("hstu_mha_fwd", SCHEMA_HSTU_MHA_FWD), ("hstu_mha", SCHEMA_HSTU_MHA)):
        try:
            torch._C._dispatch_find_schema_or_throw(f"hstu::{name}", "")
        except RuntimeError:
            lib.define(schema)
    lib.impl("hstu_mha_fwd", _hstu_mha_fwd, "CUDA")
    lib.impl("hstu_mha", _hstu_mha, "CUDA")
    torch.library.register_autograd("hstu::hstu_mha", _backward, setup_context=_setup_context, lib=lib)
    _lib = lib


register()
