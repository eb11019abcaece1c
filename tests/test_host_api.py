"""CPU tests of the host side: the C-ABI library loads and exports what include/hstu_hip.h declares,
argument validation returns the documented status codes, the Python mirror keeps the reference's
assertions, and the work counts used by the benchmark are exact.  No kernel is launched."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import c_ref

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def backend():
    from generative_recommenders_amd.ops import hip_backend

    if not os.path.exists(hip_backend.library_path()):
        import __graft_entry__

        __graft_entry__.build()
    return hip_backend


def test_library_exports_every_declared_symbol(backend):
    header = open(os.path.join(ROOT, "include", "hstu_hip.h")).read()
    declared = set(re.findall(r"\b(hstu_hip_\w+)\s*\(", header))
    assert declared == set(backend.EXPORTS), declared ^ set(backend.EXPORTS)
    lib = ctypes.CDLL(backend.library_path())
    for name in declared:
        assert hasattr(lib, name), name
    assert backend.lib().hstu_hip_version() >= 100
    assert backend.tile_config_names() == ["m128n64w4", "m256n64w8pp", "m128n64w4pl"]


@pytest.mark.parametrize("struct", ["HstuFwdArgs", "HstuJaggedCopyArgs", "HstuBwdGrads"])
def test_struct_mirror_has_the_header_fields_in_order(backend, struct):
    header = open(os.path.join(ROOT, "include", "hstu_hip.h")).read()
    body = header[header.index(f"typedef struct {struct} {{") : header.index(f"}} {struct};")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S).replace(f"typedef struct {struct} {{", "")
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        parts = decl.split(",")
        names.append(re.findall(r"(\w+)\s*$", parts[0].strip())[0])
        names += [p.strip() for p in parts[1:]]
    assert names == [f[0] for f in getattr(backend, struct)._fields_]


def test_backward_argument_checks(backend):
    """Validation of hstu_hip_mha_bwd runs before anything touches the device."""
    L = backend.lib()
    a, g = backend.HstuFwdArgs(), backend.HstuBwdGrads()
    assert L.hstu_hip_mha_bwd(None, ctypes.byref(g), None) == -1
    assert L.hstu_hip_mha_bwd(ctypes.byref(a), None, None) == -1
    a.batch, a.heads, a.dqk, a.dv, a.total_q, a.total_kv, a.max_seq_len, a.dtype = 2, 2, 64, 64, 0, 0, 16, 0
    assert L.hstu_hip_mha_bwd(ctypes.byref(a), ctypes.byref(g), None) == 0  # nothing to do
    a.delta_size, a.total_q, a.total_kv = 4, 8, 32
    a.q = a.k = a.v = a.seq_offsets = 4096  # never dereferenced: the call is refused first
    a.q_row_stride = a.k_row_stride = a.v_row_stride = 128
    a.q_head_stride = a.k_head_stride = a.v_head_stride = 64
    assert L.hstu_hip_mha_bwd(ctypes.byref(a), ctypes.byref(g), None) == -6  # delta mode has no backward
    a.delta_size, a.total_q, a.dtype = 0, 32, 2
    assert L.hstu_hip_mha_bwd(ctypes.byref(a), ctypes.byref(g), None) == -6  # nor has fp8
    a.dtype = 0
    assert L.hstu_hip_mha_bwd(ctypes.byref(a), ctypes.byref(g), None) == -1  # gradient pointers missing
    g.dout = g.dq = g.dk = g.dv = 4096
    g.do_row_stride = 127
    assert L.hstu_hip_mha_bwd(ctypes.byref(a), ctypes.byref(g), None) == -4


def test_backward_workspace_bytes(backend):
    """The dS scratch: 4 * batch bytes for the sequence order rounded up to 256, then (rows + 32 per sequence) x heads x
    (max_seq_len rounded up to 128) x 2 bytes -- 17.3 GB at the size of the headline benchmark."""
    assert backend.mha_bwd_workspace_bytes(100, 3, 2, 200) == 256 + (100 + 96) * 2 * 256 * 2
    assert backend.mha_bwd_workspace_bytes(524288, 128, 4, 4096) == 512 + (524288 + 4096) * 4 * 4096 * 2
    assert backend.mha_bwd_workspace_bytes(0, 3, 2, 200) == 0
    assert backend.lib().hstu_hip_mha_bwd_workspace_bytes(None) == 0


def test_jagged_copy_argument_checks(backend):
    """Validation of the jagged copy entry points runs before anything touches the device."""
    a = backend.HstuJaggedCopyArgs()
    L = backend.lib()
    assert L.hstu_hip_concat_2d_jagged(None, None) == -1
    a.batch, a.row_bytes, a.max_len_left, a.max_len_right = 2, 64, 4, 4
    a.left_row_stride = a.right_row_stride = a.joined_row_stride = 64
    a.total_left, a.total_right = 8, 7  # both sides dense: totals must be batch * max_len
    assert L.hstu_hip_concat_2d_jagged(ctypes.byref(a), None) == -5
    a.total_right = 8
    assert L.hstu_hip_concat_2d_jagged(ctypes.byref(a), None) == -1  # pointers missing
    a.joined_row_stride = 32  # narrower than a row
    assert L.hstu_hip_split_2d_jagged(ctypes.byref(a), None) == -5
    a.total_left = a.total_right = a.max_len_left = a.max_len_right = 0
    a.joined_row_stride = 64
    assert L.hstu_hip_concat_2d_jagged(ctypes.byref(a), None) == 0  # nothing to copy
    assert L.hstu_hip_jagged_write_tail(None, 64, None, 1, None, 64, 64, 3, 0, None) == 0
    assert L.hstu_hip_jagged_write_tail(None, 64, None, 1, None, 64, 64, 3, 2, None) == -1
    assert L.hstu_hip_jagged_write_tail(None, 32, None, 1, None, 64, 64, 3, 2, None) == -5


def _args(backend, **over):
    a = backend.HstuFwdArgs()
    a.q = a.k = a.v = a.out = 0x1000
    a.seq_offsets = 0x2000
    for s in ("q", "k", "v", "o"):
        setattr(a, f"{s}_row_stride", 4 * 128)
        setattr(a, f"{s}_head_stride", 128)
    a.batch, a.heads, a.dqk, a.dv = 2, 4, 128, 128
    a.total_q = a.total_kv = 100
    a.max_seq_len = 64
    a.alpha = 0.1
    a.seq_offsets_i64 = 1
    for key, val in over.items():
        setattr(a, key, val)
    return a


def test_check_args_status_codes(backend):
    chk = lambda **o: backend.lib().hstu_hip_check_args(ctypes.byref(_args(backend, **o)))  # noqa: E731
    assert chk() == 0
    assert backend.lib().hstu_hip_check_args(None) == -1
    assert chk(q=None) == -1
    assert chk(seq_offsets=None) == -1
    assert chk(dtype=7) == -2
    assert chk(dtype=3) == 0  # fp32: rounded to fp16 inside the library
    assert chk(dtype=3, tile_config=3) == -6
    assert chk(dtype=3, q_row_stride=4 * 128 + 4) == 0 and chk(dtype=3, q_row_stride=4 * 128 + 2) == -4
    assert chk(dqk=48, dv=48) == -3
    assert chk(dqk=64, dv=128) == 0  # unequal dims run on tile config 1 ...
    assert chk(dqk=64, dv=128, tile_config=2) == -6  # ... only
    assert chk(dqk=16, dv=16, v_row_stride=4 * 16, v_head_stride=16) == 0
    assert chk(dqk=16, dv=16, dtype=2) == -3  # 8-bit rows are at least 32 wide
    assert chk(q=0x1008) == -4
    assert chk(k_row_stride=4 * 128 + 4) == -4
    assert chk(max_seq_len=0) == -5
    assert chk(total_q=99) == -5
    assert chk(delta_size=8, total_q=17) == -5
    assert chk(delta_size=8, total_q=16) == 0
    assert chk(tile_config=99) == -5
    assert chk(total_q=0, total_kv=0, q=None) == 0  # empty input: nothing is dereferenced
    # fp8 rows are 16-byte aligned at multiples of 16 elements; bf16 at multiples of 8
    assert chk(dtype=2) == 0
    assert chk(dtype=2, k_row_stride=4 * 128 + 8) == -4
    assert chk(dtype=0, k_row_stride=4 * 128 + 8) == 0
    assert chk(workspace=0x1002, workspace_bytes=64) == -4
    # workspace of the persistent kernels (tile configs 2 and 3): 8 work-item counters 64 bytes apart and 8 list
    # lengths (576 bytes); for batches that are not all of length max_seq_len the work lists (a 32-byte record per possible
    # item and XCD, + 32 to align them); for sort_by_length one int per sequence
    need = lambda **o: backend.lib().hstu_hip_workspace_bytes(ctypes.byref(_args(backend, **o)))  # noqa: E731
    assert need() == 576 + (1 * 1 * 256 + 32)
    assert need(total_q=128, total_kv=128) == 576  # 2 sequences of exactly max_seq_len = 64
    assert need(tile_config=1) == 0
    assert need(sort_by_length=1, batch=64) == 576 + 256 + (32 * 1 * 256 + 32)
    assert need(sort_by_length=1, batch=1) == 576 + (1 * 1 * 256 + 32)
    assert need(sort_by_length=1, batch=64, tile_config=1) == 256
    for rc in range(-10, 1):
        assert backend.lib().hstu_hip_status_string(rc)
    with pytest.raises(RuntimeError):
        backend.raise_for_status(-3)
    with pytest.raises(ValueError):
        backend.raise_for_status(-5)


def test_backward_rejects_attn_scale(backend):
    """The backward kernels scale by 1 / max_seq_len; a call that carries the forward's attn_scale is refused before
    anything touches the device (the caller scales dout instead)."""
    a = _args(backend, attn_scale=0x3000)
    g = backend.HstuBwdGrads()
    g.dout = g.dq = g.dk = g.dv = 0x4000
    for s in ("do", "dq", "dk", "dv"):
        setattr(g, f"{s}_row_stride", 4 * 128)
        setattr(g, f"{s}_head_stride", 128)
    assert backend.lib().hstu_hip_mha_bwd(ctypes.byref(a), ctypes.byref(g), None) == -6
    assert backend.lib().hstu_hip_version() >= 101  # HstuFwdArgs ends with attn_scale, attn_scale_per_row


def test_python_mirror_keeps_reference_assertions(pkg):
    q = torch.zeros(10, 2, 32, dtype=torch.bfloat16)
    offs = torch.tensor([0, 10])
    with pytest.raises(AssertionError, match="max_seq_len must be larger than 0"):
        pkg.hstu_mha(0, 0.1, q, q, q, offs)
    with pytest.raises(AssertionError, match="q must be 3-D"):
        pkg.hstu_mha(16, 0.1, q[0], q[0], q, offs)
    with pytest.raises(AssertionError, match="k must be the same shape as q"):
        pkg.hstu_mha(16, 0.1, q, q[:5], q, offs)
    with pytest.raises(AssertionError, match="only support causal attention"):
        pkg.hstu_mha(16, 0.1, q, q, q, offs, causal=False)
    # CPU tensors are refused: there is no fallback path
    with pytest.raises(AssertionError, match="q must be CUDA tensor"):
        pkg.hstu_mha(16, 0.1, q, q, q, offs)
    with pytest.raises(AssertionError, match="delta_q must be padded"):
        pkg.delta_hstu_mha(16, 0.1, q[:9], q, q, torch.tensor([0, 4, 10]))
    with pytest.raises(AssertionError, match="wrong k shape"):
        pkg.delta_hstu_mha(16, 0.1, q[:8], q[:, :1], q, torch.tensor([0, 4, 10]))


def test_package_does_not_import_the_oracle():
    pkg_dir = os.path.join(ROOT, "generative-recommenders_amd")
    for dirpath, _, files in os.walk(pkg_dir):
        for fn in files:
            if fn.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, fn)).read()
                assert "oracle" not in text, os.path.join(dirpath, fn)


def test_valid_pair_counts_match_brute_force():
    from generative_recommenders_amd import workloads

    rng = np.random.default_rng(3)
    checked = 0
    for _ in range(400):
        n = int(rng.integers(1, 80))
        c = int(rng.choice([0, 0, 1, 6]))
        t = int(rng.integers(0, max(1, n - c) + 1)) if rng.random() < 0.7 else 0
        if n - t < c:
            continue
        w = int(rng.choice([0, 1, 7, 30, 200]))
        f = int(rng.choice([0, 0, 3]))
        rows = workloads.valid_pairs_per_row(n, t, w, c, f)
        m = c_ref.mask(n, c, t, w, f)
        assert (rows == m.sum(1)).all(), (n, c, t, w, f)
        d = int(rng.integers(1, n + 1))
        assert rows[n - d :].sum() == c_ref.count_pairs(n, c, t, w, f, d)
        checked += 1
    assert checked > 300


def test_workload_definitions():
    from generative_recommenders_amd import workloads

    h = workloads.make_workload("headline")
    assert (h.batch, h.heads, h.dqk, h.max_seq_len) == (64, 4, 128, 8192)
    pairs = workloads.count_valid_pairs(h)
    assert pairs == 64 * (8192 * 8193 // 2)
    assert workloads.algorithmic_flops(h) == 2 * 256 * 4 * pairs
    # the reference bench's n^2/2 convention agrees with the exact count to 1/n for plain causal
    assert abs(workloads.reference_convention_flops(h) / workloads.algorithmic_flops(h) - 1) < 2e-4
    c3 = workloads.make_workload("cfg3")
    assert c3.lengths.min() >= 256 and c3.lengths.max() <= 8192
    assert (c3.num_targets >= 1).all() and (c3.lengths - c3.num_targets >= 7).all()
    c4 = workloads.make_workload("cfg4")
    assert c4.total_q == 32 * 256 and c4.max_seq_len == 4352
    for name in workloads.WORKLOADS:
        wl = workloads.make_workload(name)
        assert wl.lengths.max() <= wl.max_seq_len
        assert workloads.algorithmic_bytes(wl) > 0


def test_native_operator_schemas_are_the_references():
    """torch.ops.hstu.hstu_mha / hstu_mha_fwd carry the schemas of ops/cpp/hstu_attention/flash_api_cpu.cpp:142-235 of
    the reference (argument names, order, types and defaults), so that its forwarder (ops/hstu_attention.py:50-98,
    27 positional arguments) binds."""
    import torch

    import __graft_entry__

    __graft_entry__.load_package()
    got = str(torch.ops.hstu.hstu_mha.default._schema)
    want = (
        "hstu::hstu_mha(SymInt max_seq_len, float alpha, Tensor q, Tensor k, Tensor v, Tensor? seq_offsets, bool causal, "
        "Tensor? num_targets, Tensor? attn_scale, int max_attn_len, int min_full_attn_seq_len, int contextual_seq_len, "
        "Tensor? q_descale, Tensor? k_descale, Tensor? v_descale, bool sort_by_length, bool deterministic, int sm_margin=0, "
        "SymInt max_q_len=0, Tensor? seq_offsets_q=None, int num_softmax_heads=0, bool training=True, "
        "Tensor? max_seq_len_tensor=None, Tensor? contextual_seq_len_tensor=None, Tensor? max_attn_len_tensor=None, "
        "Tensor? min_full_attn_seq_len_tensor=None, int num_groups=1, bool use_bf16_dq_accum=False) -> Tensor"
    )
    assert got == want
    fwd = str(torch.ops.hstu.hstu_mha_fwd.default._schema)
    assert fwd.startswith("hstu::hstu_mha_fwd(SymInt max_seq_len, float alpha, Tensor q, Tensor k, Tensor v, Tensor? seq_offsets, bool causal, ")
    assert fwd.endswith("int num_groups=1) -> (Tensor, Tensor?)") and "sort_by_length" not in fwd
    # no kernel for host tensors: the dispatcher says so (there is no CPU fallback)
    z = torch.zeros(4, 1, 32)
    import pytest

    with pytest.raises(NotImplementedError):
        torch.ops.hstu.hstu_mha(8, 0.1, z, z, z, torch.tensor([0, 4]), True, None, None, 0, 0, 0, None, None, None, False, False)
