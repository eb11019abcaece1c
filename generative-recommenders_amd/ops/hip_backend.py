"""ctypes binding of ``libhstu_hip.so`` (C ABI declared in ``include/hstu_hip.h``)."""

import ctypes
import os
from typing import Optional

import torch

from ..build import LIB_PATH

HSTU_BF16, HSTU_FP16, HSTU_FP8_E4M3, HSTU_FP32 = 0, 1, 2, 3


class HstuFwdArgs(ctypes.Structure):
    """Field-for-field mirror of ``struct HstuFwdArgs``."""

    _fields_ = [
        ("q", ctypes.c_void_p),
        ("k", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("q_row_stride", ctypes.c_int64),
        ("q_head_stride", ctypes.c_int64),
        ("k_row_stride", ctypes.c_int64),
        ("k_head_stride", ctypes.c_int64),
        ("v_row_stride", ctypes.c_int64),
        ("v_head_stride", ctypes.c_int64),
        ("o_row_stride", ctypes.c_int64),
        ("o_head_stride", ctypes.c_int64),
        ("seq_offsets", ctypes.c_void_p),
        ("num_targets", ctypes.c_void_p),
        ("seq_offsets_i64", ctypes.c_int32),
        ("num_targets_i64", ctypes.c_int32),
        ("batch", ctypes.c_int32),
        ("heads", ctypes.c_int32),
        ("dqk", ctypes.c_int32),
        ("dv", ctypes.c_int32),
        ("total_q", ctypes.c_int64),
        ("total_kv", ctypes.c_int64),
        ("max_seq_len", ctypes.c_int32),
        ("delta_size", ctypes.c_int32),
        ("alpha", ctypes.c_float),
        ("max_attn_len", ctypes.c_int32),
        ("contextual_seq_len", ctypes.c_int32),
        ("min_full_attn_seq_len", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("q_scale", ctypes.c_float),
        ("k_scale", ctypes.c_float),
        ("v_scale", ctypes.c_float),
        ("tile_config", ctypes.c_int32),
        ("sort_by_length", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_int64),
        ("kv_splits", ctypes.c_int32),
        ("attn_scale", ctypes.c_void_p),
        ("attn_scale_per_row", ctypes.c_int32),
    ]


class HstuBwdGrads(ctypes.Structure):
    """Mirror of ``HstuBwdGrads`` in include/hstu_hip.h (field order and types must match)."""

    _fields_ = [
        ("dout", ctypes.c_void_p),
        ("dq", ctypes.c_void_p),
        ("dk", ctypes.c_void_p),
        ("dv", ctypes.c_void_p),
        ("do_row_stride", ctypes.c_int64),
        ("do_head_stride", ctypes.c_int64),
        ("dq_row_stride", ctypes.c_int64),
        ("dq_head_stride", ctypes.c_int64),
        ("dk_row_stride", ctypes.c_int64),
        ("dk_head_stride", ctypes.c_int64),
        ("dv_row_stride", ctypes.c_int64),
        ("dv_head_stride", ctypes.c_int64),
    ]


class HstuJaggedCopyArgs(ctypes.Structure):
    """Mirror of ``HstuJaggedCopyArgs`` in include/hstu_hip.h (field order and types must match)."""

    _fields_ = [
        ("left", ctypes.c_void_p),
        ("right", ctypes.c_void_p),
        ("joined", ctypes.c_void_p),
        ("left_row_stride", ctypes.c_int64),
        ("right_row_stride", ctypes.c_int64),
        ("joined_row_stride", ctypes.c_int64),
        ("row_bytes", ctypes.c_int64),
        ("offsets_left", ctypes.c_void_p),
        ("offsets_right", ctypes.c_void_p),
        ("offsets_left_i64", ctypes.c_int32),
        ("offsets_right_i64", ctypes.c_int32),
        ("batch", ctypes.c_int32),
        ("max_len_left", ctypes.c_int32),
        ("max_len_right", ctypes.c_int32),
        ("total_left", ctypes.c_int64),
        ("total_right", ctypes.c_int64),
    ]


EXPORTS = (
    "hstu_hip_version",
    "hstu_hip_status_string",
    "hstu_hip_last_error",
    "hstu_hip_check_args",
    "hstu_hip_mha_fwd",
    "hstu_hip_mha_fwd_noalloc",
    "hstu_hip_check_contract",
    "hstu_hip_mha_bwd",
    "hstu_hip_mha_bwd_workspace_bytes",
    "hstu_hip_workspace_bytes",
    "hstu_hip_plan",
    "hstu_hip_tile_configs",
    "hstu_hip_tile_config_name",
    "hstu_hip_concat_2d_jagged",
    "hstu_hip_split_2d_jagged",
    "hstu_hip_jagged_write_tail",
)

_lib: Optional[ctypes.CDLL] = None


def library_path() -> str:
    return LIB_PATH


def lib() -> ctypes.CDLL:
    """Load the shared library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with __graft_entry__.build() "
                "(hipcc --offload-arch=gfx950).  There is no CPU or PyTorch fallback."
            )
        L = ctypes.CDLL(LIB_PATH)
        L.hstu_hip_version.restype = ctypes.c_int
        L.hstu_hip_status_string.restype = ctypes.c_char_p
        L.hstu_hip_status_string.argtypes = [ctypes.c_int]
        L.hstu_hip_last_error.restype = ctypes.c_char_p
        L.hstu_hip_check_args.restype = ctypes.c_int
        L.hstu_hip_check_args.argtypes = [ctypes.POINTER(HstuFwdArgs)]
        L.hstu_hip_mha_fwd.restype = ctypes.c_int
        L.hstu_hip_mha_fwd.argtypes = [ctypes.POINTER(HstuFwdArgs), ctypes.c_void_p]
        L.hstu_hip_mha_fwd_noalloc.restype = ctypes.c_int
        L.hstu_hip_mha_fwd_noalloc.argtypes = [ctypes.POINTER(HstuFwdArgs), ctypes.c_void_p]
        L.hstu_hip_check_contract.restype = ctypes.c_int
        L.hstu_hip_check_contract.argtypes = [ctypes.POINTER(HstuFwdArgs), ctypes.c_void_p, ctypes.c_void_p]
        L.hstu_hip_mha_bwd.restype = ctypes.c_int
        L.hstu_hip_mha_bwd.argtypes = [ctypes.POINTER(HstuFwdArgs), ctypes.POINTER(HstuBwdGrads), ctypes.c_void_p]
        L.hstu_hip_mha_bwd_workspace_bytes.restype = ctypes.c_size_t
        L.hstu_hip_mha_bwd_workspace_bytes.argtypes = [ctypes.POINTER(HstuFwdArgs)]
        L.hstu_hip_plan.restype = ctypes.c_int
        L.hstu_hip_plan.argtypes = [ctypes.POINTER(HstuFwdArgs), ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]
        L.hstu_hip_workspace_bytes.restype = ctypes.c_size_t
        L.hstu_hip_workspace_bytes.argtypes = [ctypes.POINTER(HstuFwdArgs)]
        L.hstu_hip_tile_configs.restype = ctypes.c_int
        L.hstu_hip_tile_config_name.restype = ctypes.c_char_p
        L.hstu_hip_tile_config_name.argtypes = [ctypes.c_int]
        for name in ("hstu_hip_concat_2d_jagged", "hstu_hip_split_2d_jagged"):
            fn = getattr(L, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.POINTER(HstuJaggedCopyArgs), ctypes.c_void_p]
        L.hstu_hip_jagged_write_tail.restype = ctypes.c_int
        L.hstu_hip_jagged_write_tail.argtypes = [
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int64,
            ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p,
        ]
        _lib = L
    return _lib


_STATUS_EXC = {
    -1: ValueError,
    -2: RuntimeError,  # the reference raises RuntimeError via TORCH_CHECK for dtype / layout problems
    -3: RuntimeError,
    -4: RuntimeError,
    -5: ValueError,
    -6: NotImplementedError,
    -7: RuntimeError,
    -8: RuntimeError,
    -9: RuntimeError,
    -10: RuntimeError,
}


def raise_for_status(rc: int) -> None:
    if rc == 0:
        return
    L = lib()
    msg = L.hstu_hip_status_string(rc).decode()
    extra = L.hstu_hip_last_error().decode()
    if extra:
        msg = f"{msg} ({extra})"
    raise _STATUS_EXC.get(rc, RuntimeError)(f"hstu_hip: {msg} [status {rc}]")


def tile_config_names() -> list:
    L = lib()
    return [L.hstu_hip_tile_config_name(i + 1).decode() for i in range(L.hstu_hip_tile_configs())]


def plan_for(batch, heads, dqk, dv, total_q, total_kv, max_seq_len, delta_size=0, tile_config=0, kv_splits=0,
             sort_by_length=False, dtype=HSTU_BF16):
    """(tile configuration, kv runs) the library would choose for a call of these sizes when given the workspace it
    asks for.  Touches no device memory."""
    a = HstuFwdArgs()
    a.batch, a.heads, a.dqk, a.dv = batch, heads, dqk, dv
    a.total_q, a.total_kv, a.max_seq_len, a.delta_size = total_q, total_kv, max_seq_len, delta_size
    a.tile_config, a.kv_splits, a.sort_by_length, a.dtype = tile_config, kv_splits, 1 if sort_by_length else 0, dtype
    # sizes only: the pointers are checked for presence and alignment, never followed
    a.q = a.k = a.v = a.out = a.seq_offsets = 256
    a.q_row_stride = a.k_row_stride = heads * dqk
    a.v_row_stride = a.o_row_stride = heads * dv
    a.q_head_stride = a.k_head_stride = dqk
    a.v_head_stride = a.o_head_stride = dv
    need = lib().hstu_hip_workspace_bytes(ctypes.byref(a))
    a.workspace, a.workspace_bytes = (256, need) if need else (None, 0)
    cfg, splits = ctypes.c_int32(0), ctypes.c_int32(0)
    raise_for_status(lib().hstu_hip_plan(ctypes.byref(a), ctypes.byref(cfg), ctypes.byref(splits)))
    return cfg.value, splits.value


def contract_checks_enabled() -> bool:
    """``HSTU_HIP_CHECK_CONTRACT=1`` in the environment: every forward call first validates the caller contract on the
    device and raises instead of computing (costs a small kernel and a host synchronisation; off by default)."""
    return os.environ.get("HSTU_HIP_CHECK_CONTRACT", "0") not in ("", "0")


_CONTRACT_BITS = (
    (1, "seq_offsets decrease"), (2, "a sequence is longer than max_seq_len"), (4, "num_targets outside [0, length]"),
    (8, "fewer non-target positions than contextual_seq_len"), (16, "a sequence is shorter than delta_size"),
)


def check_contract(a: "HstuFwdArgs", device: torch.device) -> None:
    """Run ``hstu_hip_check_contract`` for ``a`` and raise ``ValueError`` naming what is broken (synchronises)."""
    report = torch.empty(4, dtype=torch.int32, device=device)
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        raise_for_status(lib().hstu_hip_check_contract(ctypes.byref(a), ctypes.c_void_p(report.data_ptr()), ctypes.c_void_p(stream)))
    bad, first, what, ends = (int(x) for x in report.cpu())
    if bad or ends:
        why = [text for bit, text in _CONTRACT_BITS if what & bit]
        if ends:
            why.append("seq_offsets[0] != 0 or seq_offsets[-1] != number of k/v rows")
        raise ValueError(f"hstu_hip: caller contract broken by {bad} sequence(s), first at index {first}: " + "; ".join(why))


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return HSTU_BF16
    if dt == torch.float16:
        return HSTU_FP16
    if dt == torch.float8_e4m3fn:
        return HSTU_FP8_E4M3
    if dt == torch.float32:
        return HSTU_FP32
    raise RuntimeError(f"hstu_hip only supports fp16, bf16, fp8_e4m3 and fp32 data type, got {dt}")


def mha_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    seq_offsets: torch.Tensor,
    num_targets: Optional[torch.Tensor],
    max_seq_len: int,
    alpha: float,
    delta_size: int,
    max_attn_len: int,
    contextual_seq_len: int,
    min_full_attn_seq_len: int,
    q_scale: float = 1.0,
    k_scale: float = 1.0,
    v_scale: float = 1.0,
    tile_config: int = 0,
    sort_by_length: bool = False,
    kv_splits: int = 0,
    workspace_bytes: Optional[int] = None,
    noalloc: bool = False,
    attn_scale: Optional[torch.Tensor] = None,
    check_contract_first: bool = False,
) -> None:
    """Fill ``out`` on the current stream of ``q.device``.  All tensors are device tensors.

    ``workspace_bytes``: scratch to hand to the library; ``None`` = as much as it asks for.  With less it skips
    the scheduling options that do not fit (the result is the same).
    ``noalloc``: go through ``hstu_hip_mha_fwd_noalloc``, which keeps its scratch in a fixed area inside the library
    instead (no allocation here or there; calls that overlap in time on one device must not use it together).
    ``check_contract_first`` (or ``HSTU_HIP_CHECK_CONTRACT=1`` in the environment): validate the caller contract on the
    device before launching and raise ``ValueError`` if it is broken.  Without it, rows of a sequence that breaks the
    contract (longer than ``max_seq_len``, shorter than ``delta_size``, ...) may be left UNWRITTEN in ``out``."""
    a = HstuFwdArgs()
    a.q, a.k, a.v, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.q_row_stride, a.q_head_stride = q.stride(0), q.stride(1)
    a.k_row_stride, a.k_head_stride = k.stride(0), k.stride(1)
    a.v_row_stride, a.v_head_stride = v.stride(0), v.stride(1)
    a.o_row_stride, a.o_head_stride = out.stride(0), out.stride(1)
    a.seq_offsets = seq_offsets.data_ptr()
    a.seq_offsets_i64 = 1 if seq_offsets.dtype == torch.int64 else 0
    if num_targets is not None:
        a.num_targets = num_targets.data_ptr()
        a.num_targets_i64 = 1 if num_targets.dtype == torch.int64 else 0
    else:
        a.num_targets = None
    a.batch = seq_offsets.numel() - 1
    a.heads = q.shape[1]
    a.dqk = q.shape[2]
    a.dv = v.shape[2]
    a.total_q = q.shape[0]
    a.total_kv = k.shape[0]
    a.max_seq_len = max_seq_len
    a.delta_size = delta_size
    a.alpha = alpha
    a.max_attn_len = max_attn_len
    a.contextual_seq_len = contextual_seq_len
    a.min_full_attn_seq_len = min_full_attn_seq_len
    a.dtype = _dtype_code(q.dtype)
    a.q_scale, a.k_scale, a.v_scale = q_scale, k_scale, v_scale
    a.tile_config = tile_config
    a.sort_by_length = 1 if sort_by_length else 0
    a.kv_splits = kv_splits
    if attn_scale is not None:
        # fp32 on the device, 0-dim (one factor) or [total_q] (one per query row); the caller keeps it alive
        a.attn_scale = attn_scale.data_ptr()
        a.attn_scale_per_row = 1 if attn_scale.dim() > 0 else 0
    if contract_checks_enabled() or check_contract_first:
        check_contract(a, q.device)
    workspace = None
    need = lib().hstu_hip_workspace_bytes(ctypes.byref(a))
    if workspace_bytes is not None:
        need = min(need, workspace_bytes)
    if noalloc:
        with torch.cuda.device(q.device):
            stream = torch.cuda.current_stream(q.device).cuda_stream
            rc = lib().hstu_hip_mha_fwd_noalloc(ctypes.byref(a), ctypes.c_void_p(stream))
        raise_for_status(rc)
        return
    if need > 0:
        # scratch for the schedule; the caching allocator keeps it alive until the stream has consumed it
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        a.workspace = workspace.data_ptr()
        a.workspace_bytes = need
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        rc = lib().hstu_hip_mha_fwd(ctypes.byref(a), ctypes.c_void_p(stream))
    raise_for_status(rc)


def mha_bwd_workspace_bytes(total_rows: int, batch: int, heads: int, max_seq_len: int) -> int:
    """Bytes of scratch with which ``mha_bwd`` stores dS instead of recomputing the scores for dq."""
    a = HstuFwdArgs()
    a.total_q, a.batch, a.heads, a.max_seq_len = total_rows, batch, heads, max_seq_len
    return int(lib().hstu_hip_mha_bwd_workspace_bytes(ctypes.byref(a)))


def mha_bwd(
    dout: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    dq: torch.Tensor,
    dk: torch.Tensor,
    dv: torch.Tensor,
    seq_offsets: torch.Tensor,
    num_targets: Optional[torch.Tensor],
    max_seq_len: int,
    alpha: float,
    max_attn_len: int,
    contextual_seq_len: int,
    min_full_attn_seq_len: int,
    sort_by_length: bool = True,
    store_ds: bool = False,
    workspace: Optional[torch.Tensor] = None,
) -> None:
    """Fill ``dq``, ``dk``, ``dv`` on the current stream of ``q.device`` (full attention only).  ``sort_by_length``
    starts the long sequences first; it never changes the result.

    Two forms, chosen by the caller and by nothing else (not by how much device memory happens to be free).  The
    default recomputes the scores for dq and needs no scratch beyond ``4 * batch`` bytes for the sort.  The stored
    form lets the kernel that forms dk and dv write dS to scratch memory (2 bytes per query row, head and key position
    up to ``max_seq_len``; ``mha_bwd_workspace_bytes`` says how much), so that dq is one streamed product instead of a
    second pass over the scores: it runs when the caller passes a ``workspace`` of that size (uint8, 256-byte aligned;
    a smaller one selects the recomputed form) or asks for a fresh allocation with ``store_ds=True``."""
    a = HstuFwdArgs()
    a.q, a.k, a.v, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), None
    a.q_row_stride, a.q_head_stride = q.stride(0), q.stride(1)
    a.k_row_stride, a.k_head_stride = k.stride(0), k.stride(1)
    a.v_row_stride, a.v_head_stride = v.stride(0), v.stride(1)
    a.seq_offsets = seq_offsets.data_ptr()
    a.seq_offsets_i64 = 1 if seq_offsets.dtype == torch.int64 else 0
    if num_targets is not None:
        a.num_targets = num_targets.data_ptr()
        a.num_targets_i64 = 1 if num_targets.dtype == torch.int64 else 0
    else:
        a.num_targets = None
    a.batch = seq_offsets.numel() - 1
    a.heads, a.dqk, a.dv = q.shape[1], q.shape[2], v.shape[2]
    a.total_q, a.total_kv = q.shape[0], k.shape[0]
    a.max_seq_len, a.delta_size, a.alpha = max_seq_len, 0, alpha
    a.max_attn_len, a.contextual_seq_len, a.min_full_attn_seq_len = max_attn_len, contextual_seq_len, min_full_attn_seq_len
    a.dtype = _dtype_code(q.dtype)
    a.q_scale = a.k_scale = a.v_scale = 1.0
    if workspace is not None:
        torch._assert(workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.device == q.device,
                      "workspace must be a contiguous uint8 tensor on the inputs' device")
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel()
        a.sort_by_length = 1 if sort_by_length else 0
    else:
        need = 4 * a.batch if sort_by_length and a.batch >= 2 else 0
        if store_ds and a.total_q > 0 and a.batch > 0:
            need = lib().hstu_hip_mha_bwd_workspace_bytes(ctypes.byref(a))
        if need:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
            a.workspace, a.workspace_bytes, a.sort_by_length = workspace.data_ptr(), need, 1 if sort_by_length else 0
    g = HstuBwdGrads()
    g.dout, g.dq, g.dk, g.dv = dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    g.do_row_stride, g.do_head_stride = dout.stride(0), dout.stride(1)
    g.dq_row_stride, g.dq_head_stride = dq.stride(0), dq.stride(1)
    g.dk_row_stride, g.dk_head_stride = dk.stride(0), dk.stride(1)
    g.dv_row_stride, g.dv_head_stride = dv.stride(0), dv.stride(1)
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        rc = lib().hstu_hip_mha_bwd(ctypes.byref(a), ctypes.byref(g), ctypes.c_void_p(stream))
    raise_for_status(rc)


def _offsets_ptr(offsets: Optional[torch.Tensor]):
    if offsets is None:
        return None, 0
    return offsets.data_ptr(), 1 if offsets.dtype == torch.int64 else 0


def jagged_copy(
    split: bool,
    left: torch.Tensor,
    right: torch.Tensor,
    joined: torch.Tensor,
    offsets_left: Optional[torch.Tensor],
    offsets_right: Optional[torch.Tensor],
    batch: int,
    max_len_left: int,
    max_len_right: int,
) -> None:
    """``left``, ``right`` -> ``joined`` (``split=False``) or back (``split=True``) on the current stream.
    2-D device tensors of one dtype and row width, innermost stride 1."""
    a = HstuJaggedCopyArgs()
    es = joined.element_size()
    a.left, a.right, a.joined = left.data_ptr(), right.data_ptr(), joined.data_ptr()
    a.left_row_stride = (left.stride(0) if left.shape[0] > 1 else left.shape[1]) * es
    a.right_row_stride = (right.stride(0) if right.shape[0] > 1 else right.shape[1]) * es
    a.joined_row_stride = (joined.stride(0) if joined.shape[0] > 1 else joined.shape[1]) * es
    a.row_bytes = joined.shape[1] * es
    a.offsets_left, a.offsets_left_i64 = _offsets_ptr(offsets_left)
    a.offsets_right, a.offsets_right_i64 = _offsets_ptr(offsets_right)
    a.batch = batch
    a.max_len_left, a.max_len_right = max_len_left, max_len_right
    a.total_left, a.total_right = left.shape[0], right.shape[0]
    with torch.cuda.device(joined.device):
        stream = torch.cuda.current_stream(joined.device).cuda_stream
        fn = lib().hstu_hip_split_2d_jagged if split else lib().hstu_hip_concat_2d_jagged
        rc = fn(ctypes.byref(a), ctypes.c_void_p(stream))
    raise_for_status(rc)


def jagged_write_tail(joined: torch.Tensor, offsets: torch.Tensor, tail: torch.Tensor, batch: int, tail_len: int) -> None:
    """``joined[offsets[b+1] - tail_len + i] = tail[b * tail_len + i]`` in place, on the current stream."""
    es = joined.element_size()
    optr, i64 = _offsets_ptr(offsets)
    with torch.cuda.device(joined.device):
        stream = torch.cuda.current_stream(joined.device).cuda_stream
        rc = lib().hstu_hip_jagged_write_tail(
            joined.data_ptr(), joined.stride(0) * es, optr, i64, tail.data_ptr(), tail.stride(0) * es, joined.shape[1] * es,
            batch, tail_len, ctypes.c_void_p(stream),
        )
    raise_for_status(rc)
