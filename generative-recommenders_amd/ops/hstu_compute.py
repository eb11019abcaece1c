"""``hstu_compute_uqvk``, ``hstu_compute_output`` and ``hstu_preprocess_and_attention`` with the reference's
signatures (``generative_recommenders/ops/hstu_compute.py:54-104``, ``:107-214``, ``:217-334``).

``hstu_compute_uqvk``: layer norm + uvqk projection + split + SiLU(u).  The layer norm is a hand-written gfx950
kernel; the projection is a plain GEMM and runs on hipBLASLt with the bias and, for the u columns, the SiLU in its
epilogue.  ``u, q, k, v`` come back as column slices of one ``[L, (2*hidden + 2*attn) * H]`` buffer, which
``hstu_mha`` / ``delta_hstu_mha`` read in place.

``hstu_compute_output``: ``x + [u | attn | act(u) * norm(attn)] @ output_weight``.  One hand-written kernel
normalises, multiplies and writes the concatenated operand; the product, with the residual as the GEMM's C operand,
runs on hipBLASLt.  (``csrc/hstu_linear.hip``, ``include/hstu_linear.h``.)

Device tensors only, bf16 or fp16; ``kernel`` is accepted and ignored.  The forward runs on the kernels above; the
gradients come from a recomputation with the framework's operators (see ``_grads_by_recomputation``).
"""

import ctypes
import os
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from ..build import LINEAR_LIB_PATH
from ..common import HammerKernel


class HstuUqvkArgs(ctypes.Structure):
    """Mirror of ``HstuUqvkArgs`` in include/hstu_linear.h (field order and types must match)."""

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
        ("path", ctypes.c_int32),
        ("qkv_fp8", ctypes.c_void_p),
        ("v_scale", ctypes.c_float),
        ("q_scale", ctypes.c_float),
        ("k_scale", ctypes.c_float),
        ("qkv_absmax", ctypes.c_void_p),
    ]


class HstuOutputArgs(ctypes.Structure):
    """Mirror of ``HstuOutputArgs`` in include/hstu_linear.h (field order and types must match)."""

    _fields_ = [
        ("attn", ctypes.c_void_p),
        ("attn_row_stride", ctypes.c_int64),
        ("u", ctypes.c_void_p),
        ("u_row_stride", ctypes.c_int64),
        ("x", ctypes.c_void_p),
        ("x_row_stride", ctypes.c_int64),
        ("norm_weight", ctypes.c_void_p),
        ("norm_bias", ctypes.c_void_p),
        ("norm_eps", ctypes.c_float),
        ("output_weight", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("rows", ctypes.c_int64),
        ("d_out", ctypes.c_int32),
        ("heads", ctypes.c_int32),
        ("linear_dim", ctypes.c_int32),
        ("concat_u", ctypes.c_int32),
        ("concat_x", ctypes.c_int32),
        ("group_norm", ctypes.c_int32),
        ("silu_u", ctypes.c_int32),
        ("mul_u_activation", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_int64),
        ("path", ctypes.c_int32),
        ("dropout_ratio", ctypes.c_float),
        ("dropout_seed", ctypes.c_uint64),
        ("dropout_offset", ctypes.c_uint64),
    ]


EXPORTS = (
    "hstu_uqvk_workspace_bytes", "hstu_uqvk_forward", "hstu_uqvk_layer_norm", "hstu_output_workspace_bytes", "hstu_output_forward",
    "hstu_output_norm_mul", "hstu_output_dropout_mask", "hstu_linear_last_error", "hstu_linear_version",
)
MUL_U_ACTIVATIONS = {"none": 0, "sigmoid": 1, "silu": 2}

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """Load libhstu_linear.so.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LINEAR_LIB_PATH):
            raise RuntimeError(f"{LINEAR_LIB_PATH} is missing: build it with __graft_entry__.build().  There is no fallback.")
        L = ctypes.CDLL(LINEAR_LIB_PATH)
        L.hstu_uqvk_workspace_bytes.restype = ctypes.c_size_t
        L.hstu_uqvk_workspace_bytes.argtypes = [ctypes.POINTER(HstuUqvkArgs)]
        L.hstu_uqvk_forward.restype = ctypes.c_int
        L.hstu_uqvk_forward.argtypes = [ctypes.POINTER(HstuUqvkArgs), ctypes.c_void_p]
        L.hstu_uqvk_layer_norm.restype = ctypes.c_int
        L.hstu_uqvk_layer_norm.argtypes = [
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_int64,
            ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p,
        ]
        L.hstu_output_workspace_bytes.restype = ctypes.c_size_t
        L.hstu_output_workspace_bytes.argtypes = [ctypes.POINTER(HstuOutputArgs)]
        L.hstu_output_forward.restype = ctypes.c_int
        L.hstu_output_forward.argtypes = [ctypes.POINTER(HstuOutputArgs), ctypes.c_void_p]
        L.hstu_output_norm_mul.restype = ctypes.c_int
        L.hstu_output_norm_mul.argtypes = [ctypes.POINTER(HstuOutputArgs), ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        L.hstu_output_dropout_mask.restype = ctypes.c_int
        L.hstu_output_dropout_mask.argtypes = [ctypes.c_float, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int64, ctypes.c_int64,
                                               ctypes.c_void_p, ctypes.c_void_p]
        L.hstu_linear_last_error.restype = ctypes.c_char_p
        L.hstu_linear_version.restype = ctypes.c_int
        if L.hstu_linear_version() != 101:
            raise RuntimeError(f"{LINEAR_LIB_PATH} is version {L.hstu_linear_version()}, this binding expects 101: rebuild it")
        _lib = L
    return _lib


_STATUS = {-1: ValueError, -2: RuntimeError, -4: RuntimeError, -5: ValueError, -6: NotImplementedError, -7: RuntimeError, -9: RuntimeError}


def _raise_for_status(rc: int) -> None:
    if rc != 0:
        extra = lib().hstu_linear_last_error().decode()
        raise _STATUS.get(rc, RuntimeError)(f"hstu_linear: status {rc}" + (f" ({extra})" if extra else ""))


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return 0
    if dt == torch.float16:
        return 1
    raise RuntimeError(f"hstu_compute only supports bf16 and fp16, got {dt}")


def _dense16(t: torch.Tensor) -> torch.Tensor:
    """Detached, contiguous and 16-byte aligned (a slice of a larger parameter may start anywhere)."""
    t = t.detach().contiguous()
    return t.clone() if t.data_ptr() % 16 != 0 else t


def _check(x: torch.Tensor, *others: torch.Tensor) -> None:
    torch._assert(x.is_cuda, "x must be CUDA tensor")
    for t in others:
        torch._assert(t.is_cuda and t.dtype == x.dtype, "all tensors must be CUDA tensors of x's dtype")


def _needs_grad(*tensors: torch.Tensor) -> bool:
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


# ---- gradients of the dense steps -----------------------------------------------------------------------------------
# The forward of every function below runs on this package's kernels.  Their gradients are NOT hand-written: the
# backward recomputes the step with the framework's own operators (layer / group norm, addmm on hipBLASLt) in the
# arithmetic of the reference's PyTorch backend (fp32 norm and product with u, result rounded to the input type, then the
# product with the weight: ops/pytorch/pt_layer_norm.py:24-39, pt_hstu_linear.py:24-124, ops/hstu_compute.py:54-104) and
# lets autograd differentiate that -- nothing but the inputs is saved, which is what the reference's recompute_* flags
# ask for.  It is there so that a training step can run through the package.

def _layer_norm_math(x, weight, bias, eps):
    return F.layer_norm(x.float(), (x.shape[-1],), weight.float(), bias.float(), eps).to(x.dtype)


def _uqvk_math(x, norm_weight, norm_bias, eps, u_cols, weight, bias):
    uvqk = torch.addmm(bias, _layer_norm_math(x, norm_weight, norm_bias, eps), weight)
    return torch.cat([F.silu(uvqk[:, :u_cols]), uvqk[:, u_cols:]], dim=1)


def _norm_mul_math(attn, u, weight, bias, eps, silu_u, concat_u, concat_x, act, group_norm, heads, linear_dim, keep_scaled=None):
    """The output step's first half with the framework's operators (for the backward's recomputation).  ``keep_scaled``:
    the dropout mask times ``1 / (1 - p)`` in fp32, applied to the whole concatenation before it is rounded."""
    a32, u32, w32, b32 = attn.float(), u.float(), weight.float(), bias.float()
    if group_norm:
        if silu_u:
            u32 = F.silu(u32)
        # written out: the framework's group-norm backward on this device returned wrong weight / bias gradients for
        # (rows, heads, linear_dim) inputs with one group per head (fp32, checked against the CPU)
        xh = a32.view(-1, heads, linear_dim)
        centred = xh - xh.mean(dim=-1, keepdim=True)
        normed = centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + eps)
        y = u32 * (normed * w32.view(1, heads, 1) + b32.view(1, heads, 1)).reshape(a32.shape)
        parts = [u32, a32, y] if (concat_u and concat_x) else [y]
    else:
        gate = torch.sigmoid(u32) if act == "sigmoid" else F.silu(u32) if act == "silu" else u32
        y = gate * F.layer_norm(a32, (a32.shape[-1],), w32, b32, eps)
        parts = ([F.silu(u32) if silu_u else u32] if concat_u else []) + ([a32] if concat_x else []) + [y]
    joined = torch.cat(parts, dim=1) if len(parts) > 1 else parts[0]
    if keep_scaled is not None:
        joined = joined * keep_scaled
    return joined.to(attn.dtype)


def _grads_by_recomputation(fn, tensors, d_out):
    """d(fn(*tensors)) / d(tensor) contracted with ``d_out``, for the tensors that want a gradient (None for the others)."""
    with torch.enable_grad():
        leaves = [t.detach().requires_grad_(t.requires_grad) for t in tensors]
        wanted = [t for t in leaves if t.requires_grad]
        got = iter(torch.autograd.grad(fn(*leaves), wanted, d_out)) if wanted else iter(())
    return tuple(next(got) if t.requires_grad else None for t in leaves)


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """``layer_norm`` over the last dimension of a 2-D tensor with fp32 statistics
    (``ops/pytorch/pt_layer_norm.py:24-39`` of the reference)."""
    torch._assert(x.dim() == 2, "x must be 2-D")
    _check(x, weight, bias)
    if _needs_grad(x, weight, bias):
        return _LayerNormFunction.apply(x, weight, bias, eps)
    x = x.detach()
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
        x = x.contiguous()
    out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    weight, bias = _dense16(weight), _dense16(bias)
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device).cuda_stream
        rc = lib().hstu_uqvk_layer_norm(
            x.data_ptr(), x.stride(0), weight.data_ptr(), bias.data_ptr(), eps,
            out.data_ptr(), out.stride(0), x.shape[0], x.shape[1], _dtype_code(x.dtype), ctypes.c_void_p(stream),
        )
    _raise_for_status(rc)
    return out


class _LayerNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        ctx.save_for_backward(x, weight, bias)
        ctx.eps = eps
        with torch.no_grad():
            return layer_norm(x, weight, bias, eps)

    @staticmethod
    def backward(ctx, d_out):
        eps = ctx.eps
        return _grads_by_recomputation(lambda x, w, b: _layer_norm_math(x, w, b, eps), ctx.saved_tensors, d_out) + (None,)


class _UqvkFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, norm_weight, norm_bias, uvqk_weight, uvqk_bias, norm_eps, num_heads, attn_dim, hidden_dim, path):
        ctx.save_for_backward(x, norm_weight, norm_bias, uvqk_weight, uvqk_bias)
        ctx.cfg = (norm_eps, hidden_dim * num_heads)
        return _uqvk_buffer(x, norm_weight, norm_bias, norm_eps, num_heads, attn_dim, hidden_dim, uvqk_weight, uvqk_bias, path)

    @staticmethod
    def backward(ctx, d_uvqk):
        eps, u_cols = ctx.cfg
        fn = lambda x, nw, nb, w, b: _uqvk_math(x, nw, nb, eps, u_cols, w, b)  # noqa: E731
        return _grads_by_recomputation(fn, ctx.saved_tensors, d_uvqk.contiguous()) + (None,) * 5


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
    path: int = 0,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(u, q, k, v)``: ``u [L, hidden*H]`` already through SiLU, ``q, k [L, H, attn]``, ``v [L, H, hidden]``,
    all views of one buffer.  ``path``: 0 = the fused kernel where the shape allows, else the layer-norm kernel +
    hipBLASLt; 1 = layer-norm kernel + hipBLASLt; 2 = the fused kernel; 3 = layer-norm kernel + hand-written GEMM
    (d_model a multiple of 64, hidden * H and the output width multiples of 256; slower than 1 at the sizes measured);
    2 and 3 raise ``NotImplementedError`` where they do not apply."""
    torch._assert(x.dim() == 2, "x must be 2-D")
    n_out = (2 * hidden_dim + 2 * attn_dim) * num_heads
    torch._assert(uvqk_weight.shape == (x.shape[1], n_out), "uvqk_weight must be [d_model, (2*hidden + 2*attn) * heads]")
    torch._assert(uvqk_bias.shape == (n_out,), "uvqk_bias must be [(2*hidden + 2*attn) * heads]")
    _check(x, norm_weight, norm_bias, uvqk_weight, uvqk_bias)
    if _needs_grad(x, norm_weight, norm_bias, uvqk_weight, uvqk_bias):
        uvqk = _UqvkFunction.apply(x, norm_weight, norm_bias, uvqk_weight, uvqk_bias, norm_eps, num_heads, attn_dim, hidden_dim, path)
    else:
        uvqk = _uqvk_buffer(x, norm_weight, norm_bias, norm_eps, num_heads, attn_dim, hidden_dim, uvqk_weight, uvqk_bias, path)
    u, v, q, k = torch.split(
        uvqk, [hidden_dim * num_heads, hidden_dim * num_heads, attn_dim * num_heads, attn_dim * num_heads], dim=1
    )
    return u, q.view(-1, num_heads, attn_dim), k.view(-1, num_heads, attn_dim), v.view(-1, num_heads, hidden_dim)


def _uqvk_buffer(x, norm_weight, norm_bias, norm_eps, num_heads, attn_dim, hidden_dim, uvqk_weight, uvqk_bias, path, fp8=None) -> torch.Tensor:
    """The ``[L, (2*hidden + 2*attn) * H]`` buffer ``u | v | q | k`` (u through SiLU) from the kernels; no autograd.
    ``fp8 = (qkv8, absmax, v_scale, q_scale, k_scale)``: the fused kernel's e4m3 copy of ``v | q | k`` as well."""
    n_out = (2 * hidden_dim + 2 * attn_dim) * num_heads
    x = x.detach()
    if x.stride(1) != 1 or x.stride(0) % 8 != 0 or x.data_ptr() % 16 != 0:
        x = x.contiguous()
    uvqk = torch.empty((x.shape[0], n_out), dtype=x.dtype, device=x.device)
    a = HstuUqvkArgs()
    a.x, a.x_row_stride = x.data_ptr(), x.stride(0)
    nw, nb = _dense16(norm_weight), _dense16(norm_bias)
    w, b = _dense16(uvqk_weight), _dense16(uvqk_bias)
    a.norm_weight, a.norm_bias, a.norm_eps = nw.data_ptr(), nb.data_ptr(), norm_eps
    a.uvqk_weight, a.uvqk_bias, a.uvqk = w.data_ptr(), b.data_ptr(), uvqk.data_ptr()
    a.rows, a.d_model = x.shape[0], x.shape[1]
    a.heads, a.attn_dim, a.hidden_dim = num_heads, attn_dim, hidden_dim
    a.dtype = _dtype_code(x.dtype)
    a.path = path
    if fp8 is not None:
        qkv8, absmax, a.v_scale, a.q_scale, a.k_scale = fp8
        a.qkv_fp8, a.qkv_absmax = qkv8.data_ptr(), absmax.data_ptr()
    if x.shape[0] > 0:
        need = lib().hstu_uqvk_workspace_bytes(ctypes.byref(a))
        if need > 0:
            workspace = torch.empty(need + 256, dtype=torch.uint8, device=x.device)
            a.workspace, a.workspace_bytes = (workspace.data_ptr() + 255) & ~255, need
        with torch.cuda.device(x.device):
            stream = torch.cuda.current_stream(x.device).cuda_stream
            rc = lib().hstu_uqvk_forward(ctypes.byref(a), ctypes.c_void_p(stream))
        _raise_for_status(rc)
    return uvqk


def hstu_compute_uqvk_fp8(
    x: torch.Tensor,
    norm_weight: torch.Tensor,
    norm_bias: torch.Tensor,
    norm_eps: float,
    num_heads: int,
    attn_dim: int,
    hidden_dim: int,
    uvqk_weight: torch.Tensor,
    uvqk_bias: torch.Tensor,
    q_scale: float,
    k_scale: float,
    v_scale: float,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``hstu_compute_uqvk`` for the fp8 attention path (inference; no autograd): returns ``(u, q8, k8, v8, absmax)``.
    ``q8, k8 [L, H, attn]`` and ``v8 [L, H, hidden]`` are float8_e4m3fn views of one buffer the fused kernel fills in the
    same pass, ``x8 = e4m3(x * (1 / x_scale))`` with the caller's per-tensor scales (pass the same scales to
    ``hstu_mha``); ``absmax`` = fp32 ``[v, q, k]``: the largest magnitudes of THIS batch, from which the caller derives
    the next batch's scales (``absmax / 448``) without another pass over the data -- the hand-off the reference makes
    with its fp8 producer (``ops/cpp/cuda_hstu_preprocess_and_attention.py:262-282``).  ``NotImplementedError`` for
    shapes the fused kernel does not take (d_model 128 / 256 / 384 / 512, hidden * H and the output width multiples of
    128)."""
    torch._assert(x.dim() == 2, "x must be 2-D")
    n_out = (2 * hidden_dim + 2 * attn_dim) * num_heads
    torch._assert(uvqk_weight.shape == (x.shape[1], n_out), "uvqk_weight must be [d_model, (2*hidden + 2*attn) * heads]")
    torch._assert(uvqk_bias.shape == (n_out,), "uvqk_bias must be [(2*hidden + 2*attn) * heads]")
    torch._assert(min(q_scale, k_scale, v_scale) > 0.0, "the scales must be positive")
    _check(x, norm_weight, norm_bias, uvqk_weight, uvqk_bias)
    n8 = (hidden_dim + 2 * attn_dim) * num_heads
    qkv8 = torch.empty((x.shape[0], n8), dtype=torch.float8_e4m3fn, device=x.device)
    absmax = torch.zeros(3, dtype=torch.float32, device=x.device)
    uvqk = _uqvk_buffer(x, norm_weight, norm_bias, norm_eps, num_heads, attn_dim, hidden_dim, uvqk_weight, uvqk_bias, 0,
                        fp8=(qkv8, absmax, float(v_scale), float(q_scale), float(k_scale)))
    u = uvqk[:, : hidden_dim * num_heads]
    v8, q8, k8 = torch.split(qkv8, [hidden_dim * num_heads, attn_dim * num_heads, attn_dim * num_heads], dim=1)
    return u, q8.view(-1, num_heads, attn_dim), k8.view(-1, num_heads, attn_dim), v8.view(-1, num_heads, hidden_dim), absmax


def _rows_ok(t: torch.Tensor) -> torch.Tensor:
    t = t.detach()
    if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) % 8 != 0) or t.data_ptr() % 16 != 0:
        t = t.contiguous()
    return t


def _output_args(attn, u, norm_weight, norm_bias, norm_eps, num_heads, linear_dim, concat_u, concat_x, mul_u_activation_type,
                 group_norm, silu_u) -> Tuple[HstuOutputArgs, tuple, int]:
    torch._assert(attn.dim() == 2 and u.shape == attn.shape, "attn and u must be 2-D and of one shape")
    torch._assert(attn.shape[1] == num_heads * linear_dim, "attn.shape[1] must equal num_heads * linear_dim")
    torch._assert(mul_u_activation_type in MUL_U_ACTIVATIONS, "mul_u_activation_type must be none, sigmoid or silu")
    norm_len = num_heads if group_norm else attn.shape[1]
    torch._assert(norm_weight.shape == (norm_len,) and norm_bias.shape == (norm_len,), "norm_weight / norm_bias have the wrong length")
    attn, u = _rows_ok(attn), _rows_ok(u)
    nw, nb = _dense16(norm_weight), _dense16(norm_bias)
    a = HstuOutputArgs()
    a.attn, a.attn_row_stride = attn.data_ptr(), max(attn.stride(0), attn.shape[1])
    a.u, a.u_row_stride = u.data_ptr(), max(u.stride(0), u.shape[1])
    a.norm_weight, a.norm_bias, a.norm_eps = nw.data_ptr(), nb.data_ptr(), norm_eps
    a.rows, a.heads, a.linear_dim = attn.shape[0], num_heads, linear_dim
    a.concat_u, a.concat_x, a.group_norm, a.silu_u = int(concat_u), int(concat_x), int(group_norm), int(silu_u)
    a.mul_u_activation = MUL_U_ACTIVATIONS[mul_u_activation_type]
    a.dtype = _dtype_code(attn.dtype)
    if group_norm:
        blocks = 3 if (concat_u and concat_x) else 1
    else:
        blocks = 1 + int(concat_u) + int(concat_x)
    return a, (attn, u, nw, nb), blocks


def _dropout_state(dropout_ratio: float, training: bool, elements: int, device: torch.device, seed) -> Optional[Tuple[float, int, int]]:
    """``None`` when nothing is dropped, else ``(ratio, seed, offset)`` of the Philox stream the kernel draws the mask from:
    the caller's ``seed = (seed, offset)``, or the device's default generator, advanced past the words this call uses (one
    word per element) as the framework's own dropout would advance it."""
    if not training or dropout_ratio <= 0.0:
        return None
    torch._assert(dropout_ratio < 1.0, "dropout_ratio must be below 1")
    if seed is not None:
        return float(dropout_ratio), int(seed[0]), int(seed[1])
    gen = torch.cuda.default_generators[device.index if device.index is not None else torch.cuda.current_device()]
    offset = gen.get_offset()
    gen.set_offset(offset + ((elements + 3) // 4 + 3) // 4 * 4)
    return float(dropout_ratio), gen.initial_seed(), offset


def dropout_keep_mask(state: Tuple[float, int, int], rows: int, width: int, device: torch.device) -> torch.Tensor:
    """``[rows, width]`` uint8, 1 where the dropout of a call with this ``(ratio, seed, offset)`` kept the element: the mask
    is a pure function of these and of the element's position, regenerated on the device whenever it is needed."""
    keep = torch.empty((rows, width), dtype=torch.uint8, device=device)
    if keep.numel() > 0:
        with torch.cuda.device(device):
            stream = torch.cuda.current_stream(device).cuda_stream
            rc = lib().hstu_output_dropout_mask(state[0], state[1], state[2], rows, width, keep.data_ptr(), ctypes.c_void_p(stream))
        _raise_for_status(rc)
    return keep


def _keep_scaled(state, rows: int, width: int, device: torch.device) -> Optional[torch.Tensor]:
    if state is None:
        return None
    # the kernel's factor: 1 / (1 - p) in fp32
    scale = (torch.ones((), dtype=torch.float32) / (torch.ones((), dtype=torch.float32) - torch.tensor(state[0], dtype=torch.float32))).item()
    return dropout_keep_mask(state, rows, width, device).float() * scale


def _set_dropout(a: HstuOutputArgs, state) -> None:
    if state is not None:
        a.dropout_ratio, a.dropout_seed, a.dropout_offset = state


class _NormMulFunction(torch.autograd.Function):
    """Saves the inputs and the dropout stream's ``(ratio, seed, offset)``; the backward recomputes ``joined`` with the
    mask regenerated on the device."""

    @staticmethod
    def forward(ctx, x, u, weight, bias, eps, state, *flags):
        ctx.save_for_backward(x, u, weight, bias)
        ctx.cfg = (eps,) + flags
        ctx.state = state
        with torch.no_grad():
            return _norm_mul_forward(x, u, weight, bias, eps, state, *flags)

    @staticmethod
    def backward(ctx, d_out):
        cfg = ctx.cfg
        x = ctx.saved_tensors[0]
        mask = _keep_scaled(ctx.state, d_out.shape[0], d_out.shape[1], x.device)
        fn = lambda x, u, w, b: _norm_mul_math(x, u, w, b, *cfg, keep_scaled=mask)  # noqa: E731
        return _grads_by_recomputation(fn, ctx.saved_tensors, d_out.contiguous()) + (None,) * 9


class _OutputFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, attn, u, x, norm_weight, norm_bias, output_weight, norm_eps, num_heads, linear_dim, concat_u, concat_x, act,
                group_norm, path, state):
        ctx.save_for_backward(attn, u, x, norm_weight, norm_bias, output_weight)
        ctx.cfg = (norm_eps, False, concat_u, concat_x, act, group_norm, num_heads, linear_dim)
        ctx.state = state
        with torch.no_grad():
            return _output_forward(attn, u, x, norm_weight, norm_bias, norm_eps, output_weight, num_heads, linear_dim, concat_u,
                                   concat_x, act, group_norm, path, state)

    @staticmethod
    def backward(ctx, d_out):
        cfg = ctx.cfg
        attn, w = ctx.saved_tensors[0], ctx.saved_tensors[5]
        mask = _keep_scaled(ctx.state, attn.shape[0], w.shape[0], attn.device)
        fn = lambda attn, u, x, nw, nb, w: torch.addmm(x, _norm_mul_math(attn, u, nw, nb, *cfg, keep_scaled=mask), w)  # noqa: E731
        return _grads_by_recomputation(fn, ctx.saved_tensors, d_out.contiguous()) + (None,) * 9


def _norm_mul_forward(x, u, weight, bias, eps, state, silu_u, concat_u, concat_x, act, group_norm, num_heads, linear_dim) -> torch.Tensor:
    a, keep, blocks = _output_args(x, u, weight, bias, eps, num_heads, linear_dim, concat_u, concat_x, act, group_norm, silu_u)
    _set_dropout(a, state)
    joined = torch.empty((x.shape[0], blocks * x.shape[1]), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device).cuda_stream
        rc = lib().hstu_output_norm_mul(ctypes.byref(a), joined.data_ptr(), joined.shape[1], ctypes.c_void_p(stream))
    _raise_for_status(rc)
    return joined


def _blocks(concat_u: bool, concat_x: bool, group_norm: bool) -> int:
    return (3 if (concat_u and concat_x) else 1) if group_norm else 1 + int(concat_u) + int(concat_x)


def norm_mul_dropout(
    x: torch.Tensor, u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, dropout_ratio: float, training: bool,
    silu_u: bool = False, concat_u: bool = False, concat_x: bool = False, mul_u_activation_type: str = "none",
    group_norm: bool = False, num_heads: int = 1, linear_dim: int = -1, seed: Optional[Tuple[int, int]] = None,
) -> torch.Tensor:
    """``dropout(act(u) * norm(x) joined with the copied blocks)`` (``ops/pytorch/pt_hstu_linear.py:24-85`` of the
    reference).  Dropout runs when ``training`` and ``dropout_ratio > 0``, over the whole concatenation, in fp32 before the
    result is rounded; its mask comes from a Philox stream -- ``seed = (seed, offset)``, or the device's default
    generator -- and is regenerated, not stored, for the backward."""
    _check(x, u, weight, bias)
    if not group_norm:
        num_heads, linear_dim = 1, x.shape[1]
    state = _dropout_state(dropout_ratio, training, x.shape[0] * x.shape[1] * _blocks(concat_u, concat_x, group_norm), x.device, seed)
    flags = (silu_u, concat_u, concat_x, mul_u_activation_type, group_norm, num_heads, linear_dim)
    if _needs_grad(x, u, weight, bias):
        return _NormMulFunction.apply(x, u, weight, bias, eps, state, *flags)
    return _norm_mul_forward(x, u, weight, bias, eps, state, *flags)


def hstu_compute_output(
    attn: torch.Tensor,
    u: torch.Tensor,
    x: torch.Tensor,
    norm_weight: torch.Tensor,
    norm_bias: torch.Tensor,
    norm_eps: float,
    output_weight: torch.Tensor,
    num_heads: int,
    linear_dim: int,
    dropout_ratio: float,
    training: bool,
    concat_u: bool,
    concat_x: bool,
    mul_u_activation_type: str,
    group_norm: bool,
    recompute_y_in_backward: bool,
    kernel: HammerKernel = HammerKernel.HIP,
    path: int = 0,
    seed: Optional[Tuple[int, int]] = None,
) -> torch.Tensor:
    """Returns ``x + dropout(joined) @ output_weight`` of shape ``[L, d_model]``.  The backward always recomputes ``joined``
    (what ``recompute_y_in_backward=True`` asks for), so the flag changes nothing.  ``path``: 1 = the norm-mul kernel
    writes ``joined`` and hipBLASLt multiplies it; 2 = the norm-mul kernel writes ``y`` alone and a hand-written GEMM
    reads ``u`` and ``attn`` where they are (``NotImplementedError`` if the shape does not fit: d_model a multiple of 256,
    heads * linear_dim a multiple of 64 -- or with dropout, whose mask covers the copied blocks too); 0 = whichever is
    faster for the shape (2 where it fits, rows >= 32768 and nothing is dropped).  Dropout as in ``norm_mul_dropout``."""
    torch._assert(x.dim() == 2 and x.shape[0] == attn.shape[0], "x must be 2-D with attn's row count")
    _check(x, attn, u, norm_weight, norm_bias, output_weight)
    torch._assert(mul_u_activation_type in MUL_U_ACTIVATIONS, "mul_u_activation_type must be none, sigmoid or silu")
    state = _dropout_state(dropout_ratio, training, attn.shape[0] * attn.shape[1] * _blocks(concat_u, concat_x, group_norm), attn.device, seed)
    if _needs_grad(x, attn, u, norm_weight, norm_bias, output_weight):
        return _OutputFunction.apply(attn, u, x, norm_weight, norm_bias, output_weight, norm_eps, num_heads, linear_dim, concat_u,
                                     concat_x, mul_u_activation_type, group_norm, path, state)
    return _output_forward(attn, u, x, norm_weight, norm_bias, norm_eps, output_weight, num_heads, linear_dim, concat_u, concat_x,
                           mul_u_activation_type, group_norm, path, state)


def _output_forward(attn, u, x, norm_weight, norm_bias, norm_eps, output_weight, num_heads, linear_dim, concat_u, concat_x,
                    mul_u_activation_type, group_norm, path, state) -> torch.Tensor:
    a, keep, blocks = _output_args(attn, u, norm_weight, norm_bias, norm_eps, num_heads, linear_dim, concat_u, concat_x,
                                   mul_u_activation_type, group_norm, False)
    _set_dropout(a, state)
    torch._assert(output_weight.shape == (blocks * attn.shape[1], x.shape[1]), "output_weight must be [blocks * heads * linear_dim, d_model]")
    xr, w = _rows_ok(x), _dense16(output_weight)
    out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    a.x, a.x_row_stride = xr.data_ptr(), max(xr.stride(0), xr.shape[1])
    a.output_weight, a.out, a.d_out = w.data_ptr(), out.data_ptr(), x.shape[1]
    a.path = int(path)
    if x.shape[0] > 0:
        need = lib().hstu_output_workspace_bytes(ctypes.byref(a))
        if need > 0:  # the library path: `joined` and the GEMM's scratch
            workspace = torch.empty(need + 256, dtype=torch.uint8, device=x.device)
            a.workspace, a.workspace_bytes = (workspace.data_ptr() + 255) & ~255, need
        with torch.cuda.device(x.device):
            stream = torch.cuda.current_stream(x.device).cuda_stream
            rc = lib().hstu_output_forward(ctypes.byref(a), ctypes.c_void_p(stream))
        _raise_for_status(rc)
    return out


def hstu_preprocess_and_attention(
    x: torch.Tensor,
    norm_weight: torch.Tensor,
    norm_bias: torch.Tensor,
    norm_eps: float,
    num_heads: int,
    attn_dim: int,
    hidden_dim: int,
    uvqk_weight: torch.Tensor,
    uvqk_bias: torch.Tensor,
    max_seq_len: int,
    seq_offsets: torch.Tensor,
    attn_alpha: float,
    causal: bool,
    num_targets: Optional[torch.Tensor],
    max_attn_len: int,
    contextual_seq_len: int,
    recompute_uvqk_in_backward: bool,
    recompute_normed_x_in_backward: bool,
    sort_by_length: bool,
    prefill: bool = False,
    kernel: HammerKernel = HammerKernel.HIP,
    enable_tma: Optional[bool] = None,
) -> Tuple[torch.Tensor, torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """``hstu_compute_uqvk`` followed by ``hstu_mha`` on the views it returns; returns ``(u, attn_output, k, v)`` with
    ``attn_output [L, hidden * H]``.  Differentiable through its two parts; both always recompute in the backward (what
    the ``recompute_*`` flags ask for), so the flags change nothing."""
    from .hstu_attention import hstu_mha

    torch._assert(max_seq_len > 0, "max_seq_len must be larger than 0")
    torch._assert(x.dim() == 2, "x must be 2-D")
    torch._assert(x.shape[1] == uvqk_weight.shape[0], "x.shape[1] must equal uvqk_weight.shape[0]")
    torch._assert(
        uvqk_weight.shape[1] == 2 * num_heads * (hidden_dim + attn_dim),
        "uvqk_weight.shape[1] must equal 2 * num_heads * (hidden_dim + attn_dim)",
    )
    torch._assert(causal is True, "only causal attention is supported.")
    u, q, k, v = hstu_compute_uqvk(x, norm_weight, norm_bias, norm_eps, num_heads, attn_dim, hidden_dim, uvqk_weight, uvqk_bias, kernel)
    attn_output = hstu_mha(
        max_seq_len=max_seq_len, alpha=attn_alpha, q=q, k=k, v=v, seq_offsets=seq_offsets, causal=causal, dropout_pr=0.0,
        training=False, num_targets=num_targets, max_attn_len=max_attn_len, contextual_seq_len=contextual_seq_len,
        sort_by_length=sort_by_length, kernel=kernel,
    ).view(-1, hidden_dim * num_heads)
    return u, attn_output, k, v
