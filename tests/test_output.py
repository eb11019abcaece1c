"""hstu_compute_output: the oracle against independent statements on the CPU, the HIP / hipBLASLt path against the
oracle on the GPU.  Inputs are uniform in [-0.1, 0.1] as in the reference's own test
(ops/tests/hstu_compute_test.py:119-170).  Tolerance for bf16 / fp16 results (rounded once at the end, fp32
accumulation): relative Frobenius error <= 1e-2 and max-abs error <= 2e-2 * max|ref| against the fp32 oracle; the
concatenated operand's copied blocks are bit-exact."""

import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import output_oracle as O
from oracle import uqvk_oracle as U


def _inputs(seed, N, H, linear_dim, D, blocks, group_norm, dtype):
    g = torch.Generator().manual_seed(seed)
    L = H * linear_dim

    def uni(*shape):
        return (torch.rand(shape, generator=g) * 0.2 - 0.1).to(dtype)

    attn, u, x = uni(N, L), uni(N, L), uni(N, D)
    nw, nb = uni(H if group_norm else L), uni(H if group_norm else L)
    w = uni(blocks * L, D)
    return attn, u, x, nw, nb, w


def _blocks(concat_u, concat_x, group_norm):
    if group_norm:
        return 3 if (concat_u and concat_x) else 1
    return 1 + int(concat_u) + int(concat_x)


# ---------------------------------------------------------------- oracle, CPU


def test_oracle_group_norm_matches_the_formula_written_out():
    attn, u, _, nw, nb, _ = _inputs(1, 19, 3, 16, 8, 1, True, torch.float32)
    got = O.norm_mul(attn, u, nw, nb, 1e-6, group_norm=True, num_heads=3, linear_dim=16).double()
    assert torch.allclose(got, u.double() * O.group_norm_by_hand(attn, 3, 16, nw, nb, 1e-6), atol=1e-5)
    # one head: a group norm with a scalar weight is the layer norm with that scalar in every column
    got1 = O.norm_mul(attn, u, nw[:1], nb[:1], 1e-6, group_norm=True, num_heads=1, linear_dim=48).double()
    ln = U.layer_norm_by_hand(attn, nw[:1].expand(48), nb[:1].expand(48), 1e-6)
    assert torch.allclose(got1, u.double() * ln, atol=1e-5)


@pytest.mark.parametrize("act", ["none", "sigmoid", "silu"])
def test_oracle_layer_norm_mode_and_blocks(act):
    attn, u, _, nw, nb, _ = _inputs(2, 11, 2, 16, 8, 1, False, torch.float32)
    ud = u.double()
    mul = {"none": ud, "sigmoid": 1 / (1 + torch.exp(-ud)), "silu": ud / (1 + torch.exp(-ud))}[act]
    y = mul * U.layer_norm_by_hand(attn, nw, nb, 1e-6)
    for cu, cx, silu_u in itertools.product((False, True), (False, True), (False, True)):
        got = O.norm_mul(attn, u, nw, nb, 1e-6, silu_u=silu_u, concat_u=cu, concat_x=cx, mul_u_activation_type=act).double()
        want = ([ud / (1 + torch.exp(-ud)) if silu_u else ud] if cu else []) + ([attn.double()] if cx else []) + [y]
        assert got.shape[1] == 32 * len(want)
        assert torch.allclose(got, torch.cat(want, dim=1), atol=1e-5), (cu, cx, silu_u)


def test_oracle_group_norm_concatenates_only_with_both_flags():
    attn, u, _, nw, nb, _ = _inputs(3, 7, 2, 8, 8, 1, True, torch.float32)
    y = O.norm_mul(attn, u, nw, nb, 1e-6, group_norm=True, num_heads=2, linear_dim=8)
    for cu, cx in ((True, False), (False, True)):
        assert torch.equal(O.norm_mul(attn, u, nw, nb, 1e-6, concat_u=cu, concat_x=cx, group_norm=True, num_heads=2, linear_dim=8), y)
    both = O.norm_mul(attn, u, nw, nb, 1e-6, concat_u=True, concat_x=True, group_norm=True, num_heads=2, linear_dim=8)
    assert torch.equal(both, torch.cat([u, attn, y], dim=1))
    silu = O.norm_mul(attn, u, nw, nb, 1e-6, silu_u=True, concat_u=True, concat_x=True, group_norm=True, num_heads=2, linear_dim=8)
    assert torch.allclose(silu[:, :16], F.silu(u)) and torch.allclose(silu[:, 32:], F.silu(u) * (y / u), atol=1e-5)


def test_oracle_output_with_a_selecting_weight():
    """A one-hot output_weight picks single columns of the concatenated operand, so each block's place shows."""
    N, H, ld, D = 9, 2, 8, 8
    attn, u, x, nw, nb, _ = _inputs(4, N, H, ld, D, 3, False, torch.float32)
    L = H * ld
    w = torch.zeros((3 * L, D))
    picks = [0, L - 1, L, 2 * L - 1, 2 * L, 3 * L - 1, 5, L + 5]
    for col, row in enumerate(picks):
        w[row, col] = 1.0
    out = O.compute_output(attn, u, x, nw, nb, w, 1e-6, concat_u=True, concat_x=True)
    y = (u.double() * U.layer_norm_by_hand(attn, nw, nb, 1e-6)).float()
    joined = torch.cat([u, attn, y], dim=1)
    assert torch.allclose(out, x + joined[:, picks], atol=1e-5)


# ---------------------------------------------------------------- GPU


def test_oracle_philox_known_answers():
    """The known-answer vectors of the generator's authors (Random123, kat_vectors, philox4x32 with 10 rounds)."""
    import numpy as np

    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
        ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
        ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0], [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
    ]
    for ctr, key, want in kat:
        assert O.philox4x32_10(np.array([ctr], dtype=np.uint32), np.array(key, dtype=np.uint32))[0].tolist() == want
    # rows of a batch are independent of each other
    both = O.philox4x32_10(np.array([kat[0][0], kat[2][0]], dtype=np.uint32), np.array([kat[0][1], kat[2][1]], dtype=np.uint32))
    assert both[0].tolist() == kat[0][2] and both[1].tolist() == kat[2][2]


@pytest.mark.parametrize("p", [0.1, 0.5])
def test_oracle_dropout_rate_scale_and_position(p):
    """Keep rate within three standard deviations; survivors are the fp32 values times 1 / (1 - p), the rest zero; the mask
    depends on seed, offset and position only (a wider matrix re-deals it, another offset gives another mask)."""
    rows, width = 512, 256
    keep = O.dropout_keep(p, 1234, 8, rows, width)
    n = rows * width
    assert abs(int(keep.sum()) - n * (1 - p)) <= 3 * (n * p * (1 - p)) ** 0.5
    y = torch.rand((rows, width), generator=torch.Generator().manual_seed(1)) + 0.5
    d = O.dropout(y, p, 1234, 8)
    k = torch.from_numpy(keep)
    assert torch.equal(d[~k], torch.zeros_like(d[~k]))
    scale = torch.tensor(1.0, dtype=torch.float32) / (torch.tensor(1.0, dtype=torch.float32) - torch.tensor(p, dtype=torch.float32))
    assert torch.equal(d[k], y[k] * scale)
    assert (O.dropout_keep(p, 1234, 12, rows, width) != keep).any() and (O.dropout_keep(p, 1235, 8, rows, width) != keep).any()
    assert (O.dropout_keep(p, 1234, 8, rows // 2, width * 2).reshape(rows, width) == keep).all()  # element index = r * width + c



@pytest.fixture(scope="module")
def pkg():
    import __graft_entry__

    __graft_entry__.load_package()
    from generative_recommenders_amd.ops import hstu_compute

    return hstu_compute


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


def _close(got, ref, what):
    got, ref = got.float().cpu(), ref.float()
    assert got.shape == ref.shape, f"{what}: {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), what
    rel = float((got - ref).norm() / ref.norm())
    worst = float((got - ref).abs().max()) / float(ref.abs().max())
    assert rel <= 1e-2 and worst <= 2e-2, f"{what}: relative {rel:.3e}, max-abs / max|ref| {worst:.3e}"


NORM_MUL_CASES = [
    # N, H, linear_dim, group_norm
    (1000, 4, 128, False), (1000, 4, 128, True), (1, 1, 8, False), (3, 2, 8, True), (65, 3, 64, True), (130, 5, 24, False),
    (37, 2, 512, True), (9, 8, 512, False), (21, 4, 256, False), (300, 16, 16, True),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,H,ld,group_norm", NORM_MUL_CASES)
def test_norm_mul_kernel(pkg, dev, N, H, ld, group_norm, dtype):
    L = H * ld
    attn, u, _, nw, nb, _ = _inputs(N + L, N, H, ld, 8, 1, group_norm, dtype)
    for cu, cx, silu_u, act in [(True, True, False, "none"), (False, False, False, "silu"), (True, False, True, "sigmoid"), (False, True, False, "none")]:
        print(f"[case] norm_mul {N} {H} {ld} group={group_norm} {dtype} {cu} {cx} {silu_u} {act}", flush=True)
        got = pkg.norm_mul_dropout(attn.to(dev), u.to(dev), nw.to(dev), nb.to(dev), 1e-6, 0.0, False, silu_u, cu, cx, act, group_norm, H, ld)
        torch.cuda.synchronize()
        ref = O.norm_mul(attn, u, nw, nb, 1e-6, silu_u, cu, cx, act, group_norm, H, ld)
        _close(got, ref, "joined")
        blocks = _blocks(cu, cx, group_norm)
        assert got.shape == (N, blocks * L)
        got = got.cpu()
        if blocks == 3 or (not group_norm and cx):  # the attn block is a copy
            off = L if (blocks == 3 or cu) else 0
            assert torch.equal(got[:, off : off + L], attn)
        if (blocks == 3 or (not group_norm and cu)) and not silu_u:
            assert torch.equal(got[:, :L], u)


OUTPUT_CASES = [
    # N, H, linear_dim, D, concat_u, concat_x, act, group_norm      (first rows: the reference test's shapes)
    (1000, 4, 128, 128, True, True, "none", False),
    (1000, 4, 128, 128, False, True, "silu", False),
    (1000, 4, 128, 128, True, False, "sigmoid", False),
    (1000, 4, 128, 128, False, False, "none", False),
    (1000, 4, 128, 128, True, True, "none", True),
    (1000, 4, 128, 128, True, False, "none", True),
    (4099, 4, 128, 512, True, True, "none", False),
    (1, 2, 8, 8, True, True, "none", False),
    (77, 2, 64, 72, False, True, "none", True),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,H,ld,D,cu,cx,act,group_norm", OUTPUT_CASES)
def test_compute_output(pkg, dev, N, H, ld, D, cu, cx, act, group_norm, dtype):
    print(f"[case] output {N} {H} {ld} {D} {cu} {cx} {act} group={group_norm} {dtype}", flush=True)
    blocks = _blocks(cu, cx, group_norm)
    attn, u, x, nw, nb, w = _inputs(N + D, N, H, ld, D, blocks, group_norm, dtype)
    got = pkg.hstu_compute_output(attn.to(dev), u.to(dev), x.to(dev), nw.to(dev), nb.to(dev), 1e-6, w.to(dev), H, ld, 0.0, False,
                                  cu, cx, act, group_norm, False)
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == (N, D)
    kw = dict(concat_u=cu, concat_x=cx, mul_u_activation_type=act, group_norm=group_norm, num_heads=H, linear_dim=ld)
    _close(got, O.compute_output(attn, u, x, nw, nb, w, 1e-6, **kw), "out vs fp32 oracle")
    _close(got, O.compute_output(attn, u, x, nw, nb, w, 1e-6, round_joined_to=dtype, **kw), "out vs oracle with the operand rounded")
    # the residual alone: a zero weight returns x bit for bit
    zero = pkg.hstu_compute_output(attn.to(dev), u.to(dev), x.to(dev), nw.to(dev), nb.to(dev), 1e-6, torch.zeros_like(w).to(dev), H, ld,
                                   0.3, False, cu, cx, act, group_norm, True)
    assert torch.equal(zero.cpu(), x)


FUSED_CASES = [
    # N, H, linear_dim, concat_u, concat_x, act, group_norm; d_model is 512, the width the concatenating GEMM kernel is built for
    (4099, 4, 128, True, True, "none", False),
    (1000, 4, 128, False, True, "silu", False),
    (1000, 4, 128, True, False, "sigmoid", False),
    (1000, 4, 128, False, False, "none", False),
    (1000, 4, 128, True, True, "none", True),
    (333, 8, 64, True, True, "none", True),
    (129, 2, 32, True, True, "silu", False),
    (1, 8, 128, True, True, "none", False),
    (300, 2, 32, False, False, "none", False),  # one block of 64 columns: two tiles, fewer than the rings hold
    (70000, 2, 64, True, True, "none", False),  # more row blocks than one pass over the XCDs
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,H,ld,cu,cx,act,group_norm", FUSED_CASES)
def test_compute_output_fused_kernel(pkg, dev, N, H, ld, cu, cx, act, group_norm, dtype):
    """``path=2``: the norm-multiply kernel writes y alone, a hand-written GEMM reads u and attn where they are; same bar
    as the library path, and the two paths agree with each other."""
    D = 512
    print(f"[case] fused output {N} {H} {ld} {cu} {cx} {act} group={group_norm} {dtype}", flush=True)
    blocks = _blocks(cu, cx, group_norm)
    attn, u, x, nw, nb, w = _inputs(N + H, N, H, ld, D, blocks, group_norm, dtype)
    args = (attn.to(dev), u.to(dev), x.to(dev), nw.to(dev), nb.to(dev), 1e-6, w.to(dev), H, ld, 0.0, False, cu, cx, act, group_norm, False)
    got = pkg.hstu_compute_output(*args, path=2)
    lib = pkg.hstu_compute_output(*args, path=1)
    torch.cuda.synchronize()
    assert got.dtype == dtype and got.shape == (N, D)
    kw = dict(concat_u=cu, concat_x=cx, mul_u_activation_type=act, group_norm=group_norm, num_heads=H, linear_dim=ld)
    _close(got, O.compute_output(attn, u, x, nw, nb, w, 1e-6, **kw), "fused out vs fp32 oracle")
    _close(got, lib.float().cpu(), "fused out vs library path")


@pytest.mark.gpu
@pytest.mark.parametrize("N", [33000, 257])
def test_compute_output_concat_gemm_on_views_of_wider_buffers(pkg, dev, N):
    """u as the column slice of a [N, 4 * 512] buffer (what the producer leaves), attn as a slice of a padded one: the
    GEMM kernel reads them through their row strides.  N = 33000 also takes this path when none is asked for."""
    print(f"[case] concat-gemm output on strided views N={N}", flush=True)
    H, ld, D = 4, 128, 512
    attn, u, x, nw, nb, w = _inputs(77 + N, N, H, ld, D, 3, False, torch.bfloat16)
    uvqk = torch.zeros(N, 4 * H * ld, dtype=torch.bfloat16, device=dev)
    uvqk[:, : H * ld] = u.to(dev)
    padded = torch.zeros(N, H * ld + 64, dtype=torch.bfloat16, device=dev)
    padded[:, 32 : 32 + H * ld] = attn.to(dev)
    u_view, attn_view = uvqk[:, : H * ld], padded[:, 32 : 32 + H * ld]
    args = (attn_view, u_view, x.to(dev), nw.to(dev), nb.to(dev), 1e-6, w.to(dev), H, ld, 0.0, False, True, True, "none", False, False)
    got = pkg.hstu_compute_output(*args, path=2)
    auto = pkg.hstu_compute_output(*args)
    lib = pkg.hstu_compute_output(*args, path=1)
    torch.cuda.synchronize()
    _close(got, O.compute_output(attn, u, x, nw, nb, w, 1e-6, concat_u=True, concat_x=True), "views: out vs fp32 oracle")
    _close(got, lib.float().cpu(), "views: out vs library path")
    assert torch.equal(auto, got if N >= 32768 else lib)


@pytest.mark.gpu
@pytest.mark.parametrize("D", [256, 768, 1024])
def test_compute_output_concat_gemm_other_widths(pkg, dev, D):
    """d_model = 256, 768, 1024: one, three and four column blocks per row block."""
    print(f"[case] concat-gemm output d_model={D}", flush=True)
    N, H, ld = 2000, 2, 64
    attn, u, x, nw, nb, w = _inputs(500 + D, N, H, ld, D, 3, False, torch.bfloat16)
    args = (attn.to(dev), u.to(dev), x.to(dev), nw.to(dev), nb.to(dev), 1e-6, w.to(dev), H, ld, 0.0, False, True, True, "silu", False, False)
    got = pkg.hstu_compute_output(*args, path=2)
    lib = pkg.hstu_compute_output(*args, path=1)
    torch.cuda.synchronize()
    kw = dict(concat_u=True, concat_x=True, mul_u_activation_type="silu")
    _close(got, O.compute_output(attn, u, x, nw, nb, w, 1e-6, **kw), "other widths: out vs fp32 oracle")
    _close(got, lib.float().cpu(), "other widths: out vs library path")


@pytest.mark.gpu
def test_compute_output_at_the_benchmark_size(pkg, dev):
    """524288 rows, 3 x 512 -> 512 (the size of `bench.py --workload output`): the automatic choice is the concatenating
    GEMM and it agrees with the library path everywhere; a zero weight returns the residual bit for bit (every row block
    and both column halves are stored, none twice with different values); rows picked across the whole range, the last
    one included, against the fp32 oracle."""
    print("[case] output at 524288 rows", flush=True)
    N, H, ld, D = 524288, 4, 128, 512
    g = torch.Generator(device=dev).manual_seed(99)

    def uni(*shape):
        return (torch.rand(shape, generator=g, device=dev) * 0.2 - 0.1).to(torch.bfloat16)

    attn, u, x, nw, nb, w = uni(N, H * ld), uni(N, H * ld), uni(N, D), uni(H * ld), uni(H * ld), uni(3 * H * ld, D)
    args = (attn, u, x, nw, nb, 1e-6, w, H, ld, 0.0, False, True, True, "none", False, False)
    auto = pkg.hstu_compute_output(*args)
    got = pkg.hstu_compute_output(*args, path=2)
    lib = pkg.hstu_compute_output(*args, path=1)
    zero = pkg.hstu_compute_output(attn, u, x, nw, nb, 1e-6, torch.zeros_like(w), H, ld, 0.0, False, True, True, "none", False, False, path=2)
    torch.cuda.synchronize()
    assert torch.equal(auto, got) and torch.equal(zero, x)
    diff = (got.float() - lib.float())
    assert float(diff.norm() / lib.float().norm()) <= 1e-2 and float(diff.abs().max()) <= 2e-2 * float(lib.float().abs().max())
    rows = torch.tensor([0, 1, 255, 256, 257, 70001, 262143, 262144, 400000, N - 257, N - 2, N - 1], device=dev)
    ref = O.compute_output(attn[rows].cpu(), u[rows].cpu(), x[rows].cpu(), nw.cpu(), nb.cpu(), w.cpu(), 1e-6, concat_u=True, concat_x=True)
    _close(got[rows], ref, "benchmark size: sampled rows vs fp32 oracle")


@pytest.mark.gpu
@pytest.mark.parametrize("path", [1, 2])
def test_output_forward_with_silu_on_the_copied_u(dev, path):
    """The C entry point with ``silu_u`` (the Python operator never sets it for the projection): layer norm, all three
    blocks, SiLU(u) as the first of them -- on the concatenating path it is written beside y as a matrix of its own."""
    import ctypes

    from generative_recommenders_amd.ops import hstu_compute as hc

    print(f"[case] hstu_output_forward silu_u path={path}", flush=True)
    N, H, ld, D = 700, 4, 64, 512
    attn, u, x, nw, nb, w = _inputs(4321, N, H, ld, D, 3, False, torch.bfloat16)
    dv = [t.to(dev) for t in (attn, u, x, nw, nb, w)]
    a, keep, blocks = hc._output_args(dv[0], dv[1], dv[3], dv[4], 1e-6, H, ld, True, True, "none", False, True)
    out = torch.empty((N, D), dtype=torch.bfloat16, device=dev)
    a.x, a.x_row_stride, a.output_weight, a.out, a.d_out, a.path = dv[2].data_ptr(), D, dv[5].data_ptr(), out.data_ptr(), D, path
    need = hc.lib().hstu_output_workspace_bytes(ctypes.byref(a))
    ws = torch.empty(need + 256, dtype=torch.uint8, device=dev)
    a.workspace, a.workspace_bytes = (ws.data_ptr() + 255) & ~255, need
    rc = hc.lib().hstu_output_forward(ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    torch.cuda.synchronize()
    assert rc == 0, hc.lib().hstu_linear_last_error()
    _close(out, O.compute_output(attn, u, x, nw, nb, w, 1e-6, silu_u=True, concat_u=True, concat_x=True), "silu_u: out vs fp32 oracle")


@pytest.mark.gpu
def test_fused_output_kernel_refuses_other_widths(pkg, dev):
    attn, u, x, nw, nb, w = _inputs(3, 100, 4, 128, 128, 3, False, torch.bfloat16)
    with pytest.raises(NotImplementedError):
        pkg.hstu_compute_output(attn.to(dev), u.to(dev), x.to(dev), nw.to(dev), nb.to(dev), 1e-6, w.to(dev), 4, 128, 0.0, False, True, True,
                                "none", False, False, path=2)


@pytest.mark.gpu
def test_output_with_the_library_proposals_timed(pkg, dev, monkeypatch):
    """HSTU_LINEAR_TUNING=1: the first call of a new shape runs every proposal of the GEMM library; the result is the same
    product, and later calls (one of them with the switch off again) reproduce it bit for bit."""
    print("[case] output with HSTU_LINEAR_TUNING", flush=True)
    N, H, ld, D = 2304, 2, 64, 192  # a shape no other test uses, so the plan is made here
    attn, u, x, nw, nb, w = _inputs(4242, N, H, ld, D, 3, False, torch.bfloat16)
    args = [t.to(dev) for t in (attn, u, x, nw, nb)] + [1e-6, w.to(dev), H, ld, 0.0, False, True, True, "silu", False, False]
    monkeypatch.setenv("HSTU_LINEAR_TUNING", "1")
    first = pkg.hstu_compute_output(*args)
    again = pkg.hstu_compute_output(*args)
    monkeypatch.delenv("HSTU_LINEAR_TUNING")
    later = pkg.hstu_compute_output(*args)
    torch.cuda.synchronize()
    kw = dict(concat_u=True, concat_x=True, mul_u_activation_type="silu", group_norm=False, num_heads=H, linear_dim=ld)
    _close(first, O.compute_output(attn, u, x, nw, nb, w, 1e-6, **kw), "tuned out vs fp32 oracle")
    assert torch.equal(first, again) and torch.equal(first, later)


@pytest.mark.gpu
def test_output_takes_strided_views_and_rejects_what_it_cannot_do(pkg, dev):
    N, H, ld, D = 50, 2, 64, 64
    attn, u, x, nw, nb, w = [t.to(dev) for t in _inputs(5, N, H, ld, D, 3, False, torch.bfloat16)]
    want = pkg.hstu_compute_output(attn, u, x, nw, nb, 1e-6, w, H, ld, 0.0, False, True, True, "none", False, False)
    wide = torch.cat([u, attn, u], dim=1)  # u and attn as column slices of a wider buffer
    got = pkg.hstu_compute_output(wide[:, H * ld : 2 * H * ld], wide[:, : H * ld], torch.cat([x, x], dim=1)[:, :D], nw, nb, 1e-6, w, H,
                                  ld, 0.0, False, True, True, "none", False, False)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    with pytest.raises(AssertionError):  # a ratio of 1 would drop everything and scale by infinity
        pkg.hstu_compute_output(attn, u, x, nw, nb, 1e-6, w, H, ld, 1.0, True, True, True, "none", False, False)
    with pytest.raises(AssertionError):
        pkg.hstu_compute_output(attn, u, x, nw, nb, 1e-6, w[:-8], H, ld, 0.0, False, True, True, "none", False, False)
    with pytest.raises(AssertionError):
        pkg.hstu_compute_output(attn, u, x, nw, nb, 1e-6, w, H, ld, 0.0, False, True, True, "tanh", False, False)
    with pytest.raises(NotImplementedError):  # group norm over 3 chunks per head
        pkg.norm_mul_dropout(attn[:, :48], u[:, :48], nw[:2], nb[:2], 1e-6, 0.0, False, group_norm=True, num_heads=2, linear_dim=24)
    empty = pkg.hstu_compute_output(attn[:0], u[:0], x[:0], nw, nb, 1e-6, w, H, ld, 0.0, False, True, True, "none", False, False)
    assert empty.shape == (0, D)


@pytest.mark.gpu
def test_preprocess_and_attention_then_output(pkg, dev):
    """One STU layer's forward strung together (modules/stu.py:286-356 of the reference) against the oracles."""
    import numpy as np

    from oracle import hstu_oracle

    H, Dh, d_model, B, N = 2, 64, 128, 5, 200
    rng = np.random.default_rng(11)
    lengths = rng.integers(20, N + 1, size=B)
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int64)
    L = int(offsets[-1])
    g = torch.Generator().manual_seed(12)
    dt = torch.bfloat16
    x = torch.randn((L, d_model), generator=g).to(dt)
    nw, nb = (1 + 0.1 * torch.randn(d_model, generator=g)).to(dt), (0.1 * torch.randn(d_model, generator=g)).to(dt)
    wq = (torch.randn((d_model, 4 * Dh * H), generator=g) / d_model**0.5).to(dt)
    bq = (0.1 * torch.randn(4 * Dh * H, generator=g)).to(dt)
    ow, ob = (1 + 0.1 * torch.randn(Dh * H, generator=g)).to(dt), (0.1 * torch.randn(Dh * H, generator=g)).to(dt)
    wo = (torch.randn((3 * Dh * H, d_model), generator=g) / (3 * Dh * H) ** 0.5).to(dt)
    alpha = 1.0 / Dh**0.5
    print("[case] preprocess_and_attention + output", flush=True)
    u, attn, k, v = pkg.hstu_preprocess_and_attention(
        x.to(dev), nw.to(dev), nb.to(dev), 1e-6, H, Dh, Dh, wq.to(dev), bq.to(dev), N, offsets.to(dev), alpha, True, None, 0, 0,
        False, False, False,
    )
    out = pkg.hstu_compute_output(attn, u, x.to(dev), ow.to(dev), ob.to(dev), 1e-6, wo.to(dev), H, Dh, 0.0, False, True, True, "none", False, False)
    torch.cuda.synchronize()
    assert attn.shape == (L, H * Dh) and k.shape == (L, H, Dh) and v.shape == (L, H, Dh)
    ru, rq, rk, rv = U.compute_uqvk(x, nw, nb, 1e-6, H, Dh, Dh, wq, bq)
    rattn = hstu_oracle.pytorch_hstu_mha(N, alpha, rq, rk, rv, offsets).reshape(L, H * Dh)
    _close(attn, rattn, "attention output")
    _close(out, O.compute_output(rattn, ru, x, ow, ob, wo, 1e-6, concat_u=True, concat_x=True, num_heads=H, linear_dim=Dh), "layer output")


def _grad_close(got, ref, what):
    """2e-2 for the gradients of matrices; 1e-1 for the short parameter vectors, each entry of which is a sum of ~1e4
    signed terms that carry the bf16 roundings of the recomputation (cancellation makes the relative error of such a
    sum several times that of its terms)."""
    got, ref = got.float().cpu(), ref.float()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    rel = float((got - ref).norm() / ref.norm())
    bar = 2e-2 if ref.dim() > 1 else 1e-1
    assert rel <= bar, f"{what}: relative {rel:.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("N,H,ld,D,cu,cx,act,group_norm", [
    (300, 4, 32, 128, True, True, "none", False), (300, 4, 32, 128, False, True, "silu", False),
    (300, 4, 32, 128, True, False, "sigmoid", False), (300, 2, 64, 96, True, True, "none", True), (77, 2, 64, 72, False, True, "none", True),
])
def test_compute_output_gradients(pkg, dev, N, H, ld, D, cu, cx, act, group_norm):
    """Forward on the kernels, gradients by recomputation: against autograd through the fp32 oracle, for every input."""
    print(f"[case] output gradients {N} {H} {ld} {D} {cu} {cx} {act} group={group_norm}", flush=True)
    blocks = _blocks(cu, cx, group_norm)
    ins = _inputs(700 + N + D, N, H, ld, D, blocks, group_norm, torch.bfloat16)
    kw = dict(concat_u=cu, concat_x=cx, mul_u_activation_type=act, group_norm=group_norm, num_heads=H, linear_dim=ld)
    ref_in = [t.float().requires_grad_() for t in ins]
    attn, u, x, nw, nb, w = ref_in
    ref = O.compute_output(attn, u, x, nw, nb, w, 1e-6, **kw)
    d_out = torch.randn(ref.shape, generator=torch.Generator().manual_seed(9))
    ref.backward(d_out)
    hip_in = [t.to(dev).requires_grad_() for t in ins]
    attn_h, u_h, x_h, nw_h, nb_h, w_h = hip_in
    out = pkg.hstu_compute_output(attn_h, u_h, x_h, nw_h, nb_h, 1e-6, w_h, H, ld, 0.0, False, cu, cx, act, group_norm, True)
    out.backward(d_out.to(dev).to(out.dtype))
    torch.cuda.synchronize()
    _close(out.detach(), ref.detach(), "out")
    for name, h, r in zip(("attn", "u", "x", "norm_weight", "norm_bias", "output_weight"), hip_in, ref_in):
        _grad_close(h.grad, r.grad, f"d/d{name}")


@pytest.mark.gpu
def test_one_layer_training_step(pkg, dev):
    """uqvk -> attention -> output, forward and backward through the package, against autograd through the three oracles
    (the layer of modules/stu.py:286-356 of the reference): the gradient reaches x and every parameter."""
    import numpy as np

    from oracle import hstu_oracle

    H, Dh, d_model, B, N = 2, 64, 128, 4, 160
    rng = np.random.default_rng(21)
    lengths = rng.integers(20, N + 1, size=B)
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int64)
    L = int(offsets[-1])
    g = torch.Generator().manual_seed(22)
    dt = torch.bfloat16
    x = torch.randn((L, d_model), generator=g).to(dt)
    nw, nb = (1 + 0.1 * torch.randn(d_model, generator=g)).to(dt), (0.1 * torch.randn(d_model, generator=g)).to(dt)
    wq = (torch.randn((d_model, 4 * Dh * H), generator=g) / d_model**0.5).to(dt)
    bq = (0.1 * torch.randn(4 * Dh * H, generator=g)).to(dt)
    ow, ob = (1 + 0.1 * torch.randn(Dh * H, generator=g)).to(dt), (0.1 * torch.randn(Dh * H, generator=g)).to(dt)
    wo = (torch.randn((3 * Dh * H, d_model), generator=g) / (3 * Dh * H) ** 0.5).to(dt)
    alpha = 1.0 / Dh**0.5
    d_out = torch.randn((L, d_model), generator=g)
    print("[case] one layer, forward and backward", flush=True)
    params = (x, nw, nb, wq, bq, ow, ob, wo)
    ref_in = [t.float().requires_grad_() for t in params]
    rx, rnw, rnb, rwq, rbq, row, rob, rwo = ref_in
    ru, rq, rk, rv = U.compute_uqvk(rx, rnw, rnb, 1e-6, H, Dh, Dh, rwq, rbq)
    rattn = hstu_oracle.pytorch_hstu_mha(N, alpha, rq, rk, rv, offsets).reshape(L, H * Dh)
    rout = O.compute_output(rattn, ru, rx, row, rob, rwo, 1e-6, concat_u=True, concat_x=True, num_heads=H, linear_dim=Dh)
    rout.backward(d_out)
    hip_in = [t.to(dev).requires_grad_() for t in params]
    hx, hnw, hnb, hwq, hbq, how, hob, hwo = hip_in
    u, attn, k, v = pkg.hstu_preprocess_and_attention(hx, hnw, hnb, 1e-6, H, Dh, Dh, hwq, hbq, N, offsets.to(dev), alpha, True, None, 0, 0,
                                                      True, True, False)
    out = pkg.hstu_compute_output(attn, u, hx, how, hob, 1e-6, hwo, H, Dh, 0.0, False, True, True, "none", False, True)
    out.backward(d_out.to(dev).to(dt))
    torch.cuda.synchronize()
    _close(out.detach(), rout.detach(), "layer output")
    names = ("x", "norm_weight", "norm_bias", "uvqk_weight", "uvqk_bias", "output_norm_weight", "output_norm_bias", "output_weight")
    for name, h, r in zip(names, hip_in, ref_in):
        assert h.grad is not None, name
        got, want = h.grad.float().cpu(), r.grad
        rel = float((got - want).norm() / want.norm())
        assert rel <= 3e-2, f"d/d{name}: relative {rel:.3e}"


# ---------------------------------------------------------------- dropout


@pytest.mark.gpu
@pytest.mark.parametrize("p", [0.1, 0.5])
@pytest.mark.parametrize("group_norm", [False, True])
def test_norm_mul_dropout_mask_scale_and_inference(pkg, dev, p, group_norm):
    """training=False is bit-identical to no dropout.  training=True: the device's mask equals the oracle's bit for bit,
    dropped elements are zero, the survivors of the copied blocks are the inputs times 1 / (1 - p) rounded once
    (bit-exact), those of y agree with the fp32 oracle, the keep rate is within three standard deviations."""
    from generative_recommenders_amd.ops import hstu_compute as HC

    N, H, ld = 700, 4, 64
    L = H * ld
    attn, u, _, nw, nb, _ = _inputs(31, N, H, ld, 8, 3, group_norm, torch.bfloat16)
    args = (attn.to(dev), u.to(dev), nw.to(dev), nb.to(dev), 1e-6)
    flags = (False, True, True, "none", group_norm, H, ld)
    print(f"[case] norm_mul dropout p={p} group={group_norm}", flush=True)
    plain = pkg.norm_mul_dropout(*args, 0.0, True, *flags)
    off = pkg.norm_mul_dropout(*args, p, False, *flags)
    assert torch.equal(plain, off)
    seed = (20240607, 16)
    got = pkg.norm_mul_dropout(*args, p, True, *flags, seed=seed)
    again = pkg.norm_mul_dropout(*args, p, True, *flags, seed=seed)
    torch.cuda.synchronize()
    assert torch.equal(got, again)
    keep_dev = HC.dropout_keep_mask((p,) + seed, N, 3 * L, dev).cpu().bool()
    keep = torch.from_numpy(O.dropout_keep(p, seed[0], seed[1], N, 3 * L))
    assert torch.equal(keep_dev, keep)
    n = keep.numel()
    assert abs(int(keep.sum()) - n * (1 - p)) <= 3 * (n * p * (1 - p)) ** 0.5
    got = got.cpu()
    assert torch.equal(got[~keep], torch.zeros_like(got[~keep]))
    ref = O.dropout(O.norm_mul(attn, u, nw, nb, 1e-6, *flags), p, *seed)
    copied = torch.zeros_like(keep)
    copied[:, : 2 * L] = True
    assert torch.equal(got[keep & copied], ref[keep & copied].to(torch.bfloat16))
    _close(got, ref, "joined with dropout")
    if p == 0.5:  # the factor is 2: exact in the rounded type as well
        assert torch.equal(got[keep], (plain.cpu() * 2)[keep])


@pytest.mark.gpu
@pytest.mark.parametrize("p", [0.1, 0.5])
def test_compute_output_dropout_forward_and_backward_share_the_mask(pkg, dev, p):
    """Forward against the oracle with the same mask; gradients against autograd through the oracle with that mask (a
    different mask in the backward would miss by far more than the tolerance); path 2 refuses; the default generator
    gives a fresh mask per call and the same one after re-seeding."""
    N, H, ld, D = 300, 4, 32, 128
    cu, cx, act, group_norm = True, True, "none", False
    ins = _inputs(900 + int(p * 10), N, H, ld, D, 3, group_norm, torch.bfloat16)
    kw = dict(concat_u=cu, concat_x=cx, mul_u_activation_type=act, group_norm=group_norm, num_heads=H, linear_dim=ld)
    seed = (77, 4096)
    print(f"[case] output dropout p={p}", flush=True)
    ref_in = [t.float().requires_grad_() for t in ins]
    attn, u, x, nw, nb, w = ref_in
    ref = O.compute_output(attn, u, x, nw, nb, w, 1e-6, dropout_state=(p,) + seed, **kw)
    d_out = torch.randn(ref.shape, generator=torch.Generator().manual_seed(9))
    ref.backward(d_out)
    hip_in = [t.to(dev).requires_grad_() for t in ins]
    attn_h, u_h, x_h, nw_h, nb_h, w_h = hip_in
    out = pkg.hstu_compute_output(attn_h, u_h, x_h, nw_h, nb_h, 1e-6, w_h, H, ld, p, True, cu, cx, act, group_norm, True, seed=seed)
    out.backward(d_out.to(dev).to(out.dtype))
    torch.cuda.synchronize()
    _close(out.detach(), ref.detach(), "out")
    for name, h, r in zip(("attn", "u", "x", "norm_weight", "norm_bias", "output_weight"), hip_in, ref_in):
        _grad_close(h.grad, r.grad, f"d/d{name}")
    # without gradients, and the same call with training=False
    plain_in = [t.to(dev) for t in ins]
    a2, u2, x2, nw2, nb2, w2 = plain_in
    again = pkg.hstu_compute_output(a2, u2, x2, nw2, nb2, 1e-6, w2, H, ld, p, True, cu, cx, act, group_norm, True, seed=seed)
    assert torch.equal(again, out.detach())
    off = pkg.hstu_compute_output(a2, u2, x2, nw2, nb2, 1e-6, w2, H, ld, p, False, cu, cx, act, group_norm, True)
    assert torch.equal(off, pkg.hstu_compute_output(a2, u2, x2, nw2, nb2, 1e-6, w2, H, ld, 0.0, True, cu, cx, act, group_norm, True))
    with pytest.raises(NotImplementedError):
        pkg.hstu_compute_output(a2, u2, x2, nw2, nb2, 1e-6, w2, H, ld, p, True, cu, cx, act, group_norm, True, path=2)
    # the device's default generator: advanced by every call, reproducible from its seed
    torch.manual_seed(5)
    first = pkg.hstu_compute_output(a2, u2, x2, nw2, nb2, 1e-6, w2, H, ld, p, True, cu, cx, act, group_norm, True)
    second = pkg.hstu_compute_output(a2, u2, x2, nw2, nb2, 1e-6, w2, H, ld, p, True, cu, cx, act, group_norm, True)
    torch.manual_seed(5)
    third = pkg.hstu_compute_output(a2, u2, x2, nw2, nb2, 1e-6, w2, H, ld, p, True, cu, cx, act, group_norm, True)
    assert not torch.equal(first, second) and torch.equal(first, third)
