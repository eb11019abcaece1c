"""Backward of hstu_mha: the two CPU statements of the gradients against each other and against finite differences,
then the HIP kernels against the closed form on the GPU.  Tolerance for bf16 / fp16 gradients (P and dS are rounded
to the operand type before their products, as in the reference's kernel; fp32 accumulation): relative Frobenius
error <= 1e-2 and max-abs error <= 2e-2 * max|ref| per gradient, against the fp32 closed form on the same (rounded)
inputs."""

import itertools

import numpy as np
import pytest
import torch

from oracle import bwd_oracle as G
from oracle import hstu_oracle as O


def _inputs(seed, lengths, H, dqk, dv, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int64)
    L = int(offsets[-1])
    q = (torch.randn((L, H, dqk), generator=g) * scale).to(dtype)
    k = (torch.randn((L, H, dqk), generator=g) * scale).to(dtype)
    v = (torch.randn((L, H, dv), generator=g) * scale).to(dtype)
    dout = (torch.randn((L, H, dv), generator=g) * scale).to(dtype)
    return q, k, v, dout, offsets


MASKS = [
    dict(),
    dict(max_attn_len=5),
    dict(contextual_seq_len=3),
    dict(num_targets=True),
    dict(num_targets=True, max_attn_len=4, contextual_seq_len=2),
    dict(num_targets=True, max_attn_len=3, contextual_seq_len=2, min_full_attn_seq_len=4),
]


def _mask_kwargs(mask, lengths, seed):
    kw = dict(mask)
    if kw.pop("num_targets", False):
        rng = np.random.default_rng(seed)
        c = kw.get("contextual_seq_len", 0)
        kw["num_targets"] = torch.tensor([int(rng.integers(0, max(1, n - c))) if n > c else 0 for n in lengths], dtype=torch.int64)
    return kw


# ---------------------------------------------------------------- CPU


@pytest.mark.parametrize("mi", range(len(MASKS)))
def test_closed_form_matches_autograd(mi):
    lengths = [17, 0, 24, 9, 1]
    q, k, v, dout, offsets = _inputs(mi, lengths, 2, 8, 16, torch.float64)
    kw = _mask_kwargs(MASKS[mi], lengths, mi)
    a = G.autograd_grads(24, 0.3, q, k, v, offsets, dout, **kw)
    c = G.closed_form_grads(24, 0.3, q, k, v, offsets, dout, dtype=torch.float64, row_chunk=7, **kw)
    for name, x, y in zip(("dq", "dk", "dv"), a, c):
        assert torch.allclose(x, y, atol=1e-12), name


def test_forward_oracle_passes_finite_differences():
    lengths = [5, 3]
    q, k, v, _, offsets = _inputs(7, lengths, 1, 4, 4, torch.float64)
    tg = torch.tensor([1, 0])

    def f(q_, k_, v_):
        return O.pytorch_hstu_mha(6, 0.7, q_, k_, v_, offsets, num_targets=tg, max_attn_len=3, contextual_seq_len=1)

    assert torch.autograd.gradcheck(f, tuple(t.requires_grad_() for t in (q, k, v)), eps=1e-6, atol=1e-6)


def test_silu_slope():
    x = torch.tensor([0.0, 40.0, -40.0, 1.3, -0.7], dtype=torch.float64)
    s = G.silu_slope(x)
    assert float(s[0]) == 0.5 and abs(float(s[1]) - 1) < 1e-12 and abs(float(s[2])) < 1e-12
    h = 1e-6
    fd = (torch.nn.functional.silu(x + h) - torch.nn.functional.silu(x - h)) / (2 * h)
    assert torch.allclose(s, fd, atol=1e-8)


def test_gradients_are_linear_in_dout():
    lengths = [12, 7]
    q, k, v, dout, offsets = _inputs(3, lengths, 2, 8, 8, torch.float64)
    a = G.closed_form_grads(12, 0.5, q, k, v, offsets, dout, dtype=torch.float64)
    b = G.closed_form_grads(12, 0.5, q, k, v, offsets, -2.5 * dout, dtype=torch.float64)
    for x, y in zip(a, b):
        assert torch.allclose(-2.5 * x, y, atol=1e-12)


# ---------------------------------------------------------------- GPU


@pytest.fixture(scope="module")
def pkg():
    import __graft_entry__

    return __graft_entry__.load_package()


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


def _close(got, ref, what):
    got, ref = got.float().cpu(), ref.float()
    assert got.shape == ref.shape, what
    assert torch.isfinite(got).all(), what
    denom = float(ref.norm())
    if denom == 0.0:
        assert float(got.abs().max()) == 0.0, what
        return
    rel = float((got - ref).norm()) / denom
    worst = float((got - ref).abs().max()) / float(ref.abs().max())
    assert rel <= 1e-2 and worst <= 2e-2, f"{what}: relative {rel:.3e}, max-abs / max|ref| {worst:.3e}"


def _run_bwd(pkg, dev, N, alpha, q, k, v, dout, offsets, offsets_dtype=torch.int64, **kw):
    dkw = {a: (b.to(dev) if torch.is_tensor(b) else b) for a, b in kw.items()}
    qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
    out = pkg.hstu_mha(N, alpha, qd, kd, vd, offsets.to(offsets_dtype).to(dev), **dkw)
    out.backward(dout.to(dev))
    torch.cuda.synchronize()
    return out.detach(), qd.grad, kd.grad, vd.grad


def _direct(dev, N, alpha, q, k, v, dout, offsets, kw, **how):
    """The backend's entry point without autograd; gradients pre-filled with a sentinel."""
    from generative_recommenders_amd.ops import hip_backend

    qd, kd, vd, dd, od = (t.to(dev) for t in (q, k, v, dout, offsets))
    tg = kw.get("num_targets")
    tg = None if tg is None else tg.to(dev)
    dq, dk, dv = torch.full_like(qd, 7.0), torch.full_like(kd, 7.0), torch.full_like(vd, 7.0)
    hip_backend.mha_bwd(dd, qd, kd, vd, dq, dk, dv, od, tg, N, alpha, kw.get("max_attn_len", 0), kw.get("contextual_seq_len", 0),
                        kw.get("min_full_attn_seq_len", 0), **how)
    torch.cuda.synchronize()
    return dq, dk, dv


def _poisoned_workspace(dev, q, offsets, N):
    """Scratch for the stored-dS form with every 16-bit word a NaN: a block read without having been written shows."""
    from generative_recommenders_amd.ops import hip_backend

    need = hip_backend.mha_bwd_workspace_bytes(q.shape[0], offsets.numel() - 1, q.shape[1], N)
    return torch.full((need,), 0xFF, dtype=torch.uint8, device=dev)


def _check(pkg, dev, N, alpha, q, k, v, dout, offsets, what, **kw):
    """Both forms of the backward against the closed form: scores recomputed (through autograd, whose default it is, and
    through the entry point) and dS stored (through the entry point on NaN-filled scratch); dk and dv do not depend on
    the form."""
    out, dq, dk, dv = _run_bwd(pkg, dev, N, alpha, q, k, v, dout, offsets, **kw)
    rq, rk, rv = G.closed_form_grads(N, alpha, q, k, v, offsets, dout, **kw)
    _close(dq, rq, what + " dq")
    _close(dk, rk, what + " dk")
    _close(dv, rv, what + " dv")
    if q.shape[0] > 0:
        cq, ck, cv = _direct(dev, N, alpha, q, k, v, dout, offsets, kw)
        assert torch.equal(cq, dq) and torch.equal(ck, dk) and torch.equal(cv, dv), what + ": autograd runs the recomputed form"
        sq, sk, sv = _direct(dev, N, alpha, q, k, v, dout, offsets, kw, workspace=_poisoned_workspace(dev, q, offsets, N))
        _close(sq, rq, what + " dq from stored dS on poisoned scratch")
        assert torch.equal(sk, dk) and torch.equal(sv, dv), what + ": dk, dv of the two forms"
    return dq, dk, dv


GRID = [
    # B, N, H, dqk, dv, mask index
    (4, 200, 2, 64, 64, 0), (3, 300, 1, 128, 128, 0), (5, 130, 2, 32, 32, 1), (4, 257, 2, 128, 128, 4), (3, 200, 4, 64, 128, 3),
    (2, 150, 2, 16, 16, 0), (3, 180, 1, 128, 32, 5), (4, 100, 3, 16, 64, 2), (2, 520, 2, 128, 128, 1), (6, 64, 2, 32, 128, 4),
    # longer walks of the key-stationary kernel: the tile slots wrap several times, windows end inside the walk
    (2, 900, 2, 128, 128, 5), (2, 1100, 1, 64, 32, 4), (3, 700, 2, 32, 64, 1), (2, 1300, 1, 128, 64, 2),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,N,H,dqk,dv,mi", GRID)
def test_backward_grid(pkg, dev, B, N, H, dqk, dv, mi, dtype):
    print(f"[case] bwd grid {B} {N} {H} {dqk} {dv} mask={mi} {dtype}", flush=True)
    rng = np.random.default_rng(B * 1000 + N)
    lengths = [int(x) for x in rng.integers(1, N + 1, size=B)]
    lengths[0] = N
    q, k, v, dout, offsets = _inputs(N + dqk, lengths, H, dqk, dv, dtype)
    scale = {0: 1.0, 5: 4.0}.get(mi, 20.0)  # windows and targets in proportion to these lengths
    mask = {a: (int(b * scale) if isinstance(b, int) and not isinstance(b, bool) else b) for a, b in MASKS[mi].items()}
    kw = _mask_kwargs(mask, lengths, N)
    _check(pkg, dev, N, 1.0 / dqk**0.5, q, k, v, dout, offsets, "grid", **kw)


EDGE = [
    ([1], {}), ([2, 1, 3], {}), ([128], {}), ([129], {}), ([127, 64, 65, 63], {}), ([0, 40, 0], {}), ([256, 255, 257], {}),
    ([300], dict(max_attn_len=1)), ([300], dict(max_attn_len=64)), ([300], dict(max_attn_len=1000)),
    ([200, 90], dict(contextual_seq_len=70)), ([200, 140], dict(contextual_seq_len=130, max_attn_len=10)),
    ([150, 150], dict(num_targets=torch.tensor([150, 0]))), ([150, 150], dict(num_targets=torch.tensor([149, 1]), max_attn_len=20)),
    ([400], dict(num_targets=torch.tensor([100]), max_attn_len=50, contextual_seq_len=10, min_full_attn_seq_len=30)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("ei", range(len(EDGE)))
def test_backward_edges(pkg, dev, ei):
    lengths, kw = EDGE[ei]
    print(f"[case] bwd edge {ei} {lengths}", flush=True)
    q, k, v, dout, offsets = _inputs(ei, lengths, 2, 64, 64, torch.bfloat16)
    _check(pkg, dev, max(lengths) + 3, 0.125, q, k, v, dout, offsets, f"edge {ei}", **kw)


@pytest.mark.gpu
def test_backward_is_deterministic_and_takes_views(pkg, dev):
    print("[case] bwd determinism / strided views", flush=True)
    lengths = [500, 300, 77]
    q, k, v, dout, offsets = _inputs(21, lengths, 2, 128, 128, torch.bfloat16)
    a = _run_bwd(pkg, dev, 512, 0.09, q, k, v, dout, offsets, offsets_dtype=torch.int32)
    b = _run_bwd(pkg, dev, 512, 0.09, q, k, v, dout, offsets)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    # q, k, v as column slices of one buffer (the layout hstu_compute_uqvk returns); gradients identical
    fused = torch.cat([q, k, v], dim=2).to(dev)
    qs, ks, vs = (fused[:, :, i * 128 : (i + 1) * 128].detach().requires_grad_() for i in range(3))
    out = pkg.hstu_mha(512, 0.09, qs, ks, vs, offsets.to(dev))
    out.backward(dout.to(dev))
    torch.cuda.synchronize()
    for x, y in zip((qs.grad, ks.grad, vs.grad), b[1:]):
        assert torch.equal(x, y)
    assert torch.equal(out.detach(), b[0])


VARIANT_CASES = [
    # lengths, H, dqk, dv, mask kwargs
    ([700, 300, 1, 513], 2, 128, 128, {}),
    ([256, 255, 257, 0, 64], 2, 64, 64, {}),
    ([1000], 1, 128, 128, dict(max_attn_len=100)),
    ([640, 200], 2, 32, 64, dict(contextual_seq_len=150)),
    ([900, 450], 2, 128, 128, dict(num_targets=torch.tensor([200, 449]), max_attn_len=64, contextual_seq_len=5)),
    ([300, 300], 1, 16, 16, dict(num_targets=torch.tensor([300, 0]))),
    ([2048 + 17], 1, 128, 128, dict(num_targets=torch.tensor([33]), max_attn_len=700, min_full_attn_seq_len=50)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("store_ds", [False, True])
@pytest.mark.parametrize("ci", range(len(VARIANT_CASES)))
def test_backward_through_the_backend_entry_point(pkg, dev, ci, store_ds):
    """The backend's direct entry point (no autograd), gradients pre-filled with a sentinel: every row of every sequence
    must be overwritten; both forms (scores recomputed for dq, or dS stored in NaN-filled scratch)."""
    lengths, H, dqk, dv, kw = VARIANT_CASES[ci]
    print(f"[case] bwd direct {ci} {lengths} store_ds={store_ds}", flush=True)
    q, k, v, dout, offsets = _inputs(100 + ci, lengths, H, dqk, dv, torch.bfloat16)
    N, alpha = max(lengths) + 1, 1.0 / dqk**0.5
    ref = G.closed_form_grads(N, alpha, q, k, v, offsets, dout, **kw)
    how = dict(workspace=_poisoned_workspace(dev, q, offsets, N)) if store_ds else dict(store_ds=False)
    got = _direct(dev, N, alpha, q, k, v, dout, offsets, kw, **how)
    for name, x, r in zip(("dq", "dk", "dv"), got, ref):
        _close(x, r, name)


@pytest.mark.gpu
def test_autograd_backward_form_is_the_callers_choice(pkg, dev):
    """Without a workspace the backward recomputes the scores and allocates nothing that grows with max_seq_len; with the
    caller's workspace it stores dS there (the NaN filling is overwritten).  Same gradients to the kernels' rounding."""
    from generative_recommenders_amd.ops import hip_backend

    print("[case] bwd autograd workspace", flush=True)
    lengths = [700, 300, 513]
    q, k, v, dout, offsets = _inputs(77, lengths, 2, 64, 64, torch.bfloat16)
    N = 1024
    need = hip_backend.mha_bwd_workspace_bytes(q.shape[0], len(lengths), 2, N)
    grads = {}
    for form in ("recomputed", "stored"):
        ws = None
        if form == "stored":
            ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=dev)
        qd, kd, vd = (t.to(dev).detach().requires_grad_() for t in (q, k, v))
        out = pkg.hstu_mha(N, 0.125, qd, kd, vd, offsets.to(dev), bwd_workspace=ws)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats(dev)
        before = torch.cuda.memory_allocated(dev)
        out.backward(dout.to(dev))
        torch.cuda.synchronize()
        grown = torch.cuda.max_memory_allocated(dev) - before
        # three gradients, a bf16 copy of dout and the sort's 4 bytes per sequence; never the dS scratch
        assert grown < need // 4, (form, grown, need)
        if ws is not None:
            assert int((ws != 0xFF).sum()) > need // 8  # dS was written into the caller's memory
        grads[form] = (qd.grad.float().cpu(), kd.grad.float().cpu(), vd.grad.float().cpu())
    for name, a, b in zip(("dq", "dk", "dv"), grads["recomputed"], grads["stored"]):
        _close(a, b, name)


@pytest.mark.gpu
def test_backward_of_a_long_sequence(pkg, dev):
    """4096 rows: 32 key blocks x 64 query tiles per pair, the shape the bench workload has per sequence."""
    print("[case] bwd long", flush=True)
    lengths = [4096, 1000]
    q, k, v, dout, offsets = _inputs(5, lengths, 1, 128, 128, torch.bfloat16, scale=0.5)
    _check(pkg, dev, 4096, 1.0 / 128**0.5, q, k, v, dout, offsets, "long")
    kw = dict(num_targets=torch.tensor([300, 10]), max_attn_len=512, contextual_seq_len=6)
    _check(pkg, dev, 4096, 1.0 / 128**0.5, q, k, v, dout, offsets, "long masked", **kw)


@pytest.mark.gpu
@pytest.mark.parametrize("store_ds", [False, True])
def test_backward_at_the_size_of_the_ragged_benchmark(pkg, dev, store_ds):
    """The third benchmark configuration (64 sequences up to 8192, window 2048, contextual prefix, targets): the
    longest and four other sequences against the closed form."""
    from generative_recommenders_amd import workloads
    from generative_recommenders_amd.ops import hip_backend

    print(f"[case] bwd cfg3 full size store_ds={store_ds}", flush=True)
    wl = workloads.make_workload("cfg3")
    inp = workloads.make_inputs(wl, dev)
    q, k, v, offs, tg = inp["q"], inp["k"], inp["v"], inp["seq_offsets"], inp["num_targets"]
    g = torch.Generator(device=dev).manual_seed(77)
    dout = (torch.randn(v.shape, device=dev, generator=g) * 0.1).to(v.dtype)
    dq, dk, dv = torch.full_like(q, 7.0), torch.full_like(k, 7.0), torch.full_like(v, 7.0)
    hip_backend.mha_bwd(dout, q, k, v, dq, dk, dv, offs, tg, wl.max_seq_len, wl.alpha, wl.max_attn_len, wl.contextual_seq_len,
                        wl.min_full_attn_seq_len, store_ds=store_ds)
    torch.cuda.synchronize()
    order = sorted(range(wl.batch), key=lambda b: -int(wl.lengths[b]))
    picks = [order[0], order[7], order[20], order[40], order[63]]
    ref = G.closed_form_grads(wl.max_seq_len, wl.alpha, q.cpu(), k.cpu(), v.cpu(), offs.cpu(), dout.cpu(), num_targets=tg.cpu(),
                              max_attn_len=wl.max_attn_len, contextual_seq_len=wl.contextual_seq_len, sequences=picks)
    oc = offs.cpu()
    for b in picks:
        s0, s1 = int(oc[b]), int(oc[b + 1])
        for name, got, r in zip(("dq", "dk", "dv"), (dq, dk, dv), ref):
            _close(got[s0:s1], r[s0:s1], f"cfg3 sequence {b} (n = {s1 - s0}) {name}")
    assert torch.isfinite(dq.float()).all() and torch.isfinite(dk.float()).all() and torch.isfinite(dv.float()).all()


@pytest.mark.gpu
def test_backward_forms_agree_at_the_size_of_the_headline_benchmark(pkg, dev):
    """64 sequences of 8192 rows, 4 heads of 128: the dS scratch is 34.5 GB, so its addresses need all of their 64 bits.
    dk and dv of the two forms are the same bits; dq differs only by the rounding of the pre-scaled operand; one
    sequence is also checked against the closed form."""
    from generative_recommenders_amd import workloads
    from generative_recommenders_amd.ops import hip_backend

    print("[case] bwd headline size, both forms", flush=True)
    wl = workloads.make_workload("headline")
    inp = workloads.make_inputs(wl, dev)
    q, k, v, offs = inp["q"], inp["k"], inp["v"], inp["seq_offsets"]
    g = torch.Generator(device=dev).manual_seed(78)
    dout = (torch.randn(v.shape, device=dev, generator=g) * 0.1).to(v.dtype)
    need = hip_backend.mha_bwd_workspace_bytes(q.shape[0], wl.batch, wl.heads, wl.max_seq_len)
    if 2 * need > torch.cuda.mem_get_info(dev)[0]:
        pytest.skip("not enough free device memory for the scratch")
    got = {}
    for form in ("stored", "recompute"):
        dq, dk, dv = torch.full_like(q, 7.0), torch.full_like(k, 7.0), torch.full_like(v, 7.0)
        scratch = torch.full((need,), 0xFF, dtype=torch.uint8, device=dev) if form == "stored" else None
        hip_backend.mha_bwd(dout, q, k, v, dq, dk, dv, offs, None, wl.max_seq_len, wl.alpha, 0, 0, 0, store_ds=False, workspace=scratch)
        torch.cuda.synchronize()
        del scratch
        got[form] = (dq, dk, dv)
    assert torch.equal(got["stored"][1], got["recompute"][1]) and torch.equal(got["stored"][2], got["recompute"][2])
    a, b = got["stored"][0].float(), got["recompute"][0].float()
    assert torch.isfinite(a).all()
    assert float((a - b).norm() / b.norm()) <= 5e-3
    last = wl.batch - 1  # the sequence whose blocks lie at the far end of the scratch
    ref = G.closed_form_grads(wl.max_seq_len, wl.alpha, q.cpu(), k.cpu(), v.cpu(), offs.cpu(), dout.cpu(), sequences=[last])
    s0, s1 = int(offs[last]), int(offs[last + 1])
    for name, x, r in zip(("dq", "dk", "dv"), got["stored"], ref):
        _close(x[s0:s1], r[s0:s1], f"headline size, last sequence, {name}")


@pytest.mark.gpu
@pytest.mark.parametrize("store_ds", [False, True])
def test_backward_and_fused_producer_in_a_hip_graph(pkg, dev, store_ds):
    """hstu_compute_uqvk (fused kernel) -> hstu_mha forward -> backward kernels captured into one HIP graph: every
    replay, with eager work and a synchronisation in between, reproduces the eager results bit for bit."""
    from generative_recommenders_amd.ops import hip_backend, hstu_compute

    print(f"[case] bwd + fused producer in a hip graph store_ds={store_ds}", flush=True)
    H, Dh, d_model = 2, 64, 256
    lengths = [700, 130, 1, 420]
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int64).to(dev)
    L, N = sum(lengths), 700
    g = torch.Generator().manual_seed(5)
    x = torch.randn((L, d_model), generator=g).bfloat16().to(dev)
    nw, nb = torch.ones(d_model).bfloat16().to(dev), torch.zeros(d_model).bfloat16().to(dev)
    w = (torch.randn((d_model, 4 * Dh * H), generator=g) / d_model**0.5).bfloat16().to(dev)
    bias = (0.1 * torch.randn(4 * Dh * H, generator=g)).bfloat16().to(dev)
    dout = (0.1 * torch.randn((L, H, Dh), generator=g)).bfloat16().to(dev)

    def step():
        u, q, k, v = hstu_compute.hstu_compute_uqvk(x, nw, nb, 1e-6, H, Dh, Dh, w, bias, path=2)
        out = pkg.hstu_mha(N, 0.125, q, k, v, offsets)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)  # views' shapes, dense storage
        hip_backend.mha_bwd(dout, q, k, v, dq, dk, dv, offsets, None, N, 0.125, 0, 0, 0, sort_by_length=False, store_ds=store_ds)
        return out, dq, dk, dv

    with torch.no_grad():
        eager = step()
        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            step()
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            captured = step()
        for i in range(3):
            for t in captured:
                t.zero_()
            (x * 1.0).sum().item()
            graph.replay()
            torch.cuda.synchronize()
            for name, a_, b_ in zip(("out", "dq", "dk", "dv"), captured, eager):
                assert torch.equal(a_, b_), f"replay {i}: {name}"


@pytest.mark.gpu
@pytest.mark.parametrize("mi", [0, 4])
def test_backward_of_fp32_inputs(pkg, dev, mi):
    """fp32 is the second dtype of the reference's own test grid (hstu_attention_test.py:271-275).  The kernels take
    16-bit operands: the forward runs on fp16 copies, the backward on bf16 copies (dout can be tiny), both accumulate in
    fp32 and return fp32.  Bar: the bf16 one (relative Frobenius <= 1e-2, max-abs <= 2e-2 max|ref|) against the closed
    form evaluated on the fp32 inputs themselves."""
    print(f"[case] bwd fp32 inputs mask={mi}", flush=True)
    lengths = [300, 129, 1, 64]
    q, k, v, dout, offsets = _inputs(31 + mi, lengths, 2, 64, 64, torch.float32)
    mask = {a: (int(b * 20) if isinstance(b, int) and not isinstance(b, bool) else b) for a, b in MASKS[mi].items()}
    kw = _mask_kwargs(mask, lengths, 7)
    out, dq, dk, dv = _run_bwd(pkg, dev, 320, 0.125, q, k, v, dout * 1e-4, offsets, **kw)  # small upstream gradients
    assert out.dtype == torch.float32 and dq.dtype == torch.float32 and dk.dtype == torch.float32 and dv.dtype == torch.float32
    rq, rk, rv = G.closed_form_grads(320, 0.125, q, k, v, offsets, dout * 1e-4, **kw)
    _close(dq, rq, "fp32 dq")
    _close(dk, rk, "fp32 dk")
    _close(dv, rv, "fp32 dv")


@pytest.mark.gpu
def test_backward_rejections(pkg, dev):
    q, k, v, dout, offsets = _inputs(1, [40, 24], 2, 32, 32, torch.float32)
    with pytest.raises(NotImplementedError):  # fp8 inputs have no backward
        pkg.hstu_mha(64, 0.2, q.to(torch.float8_e4m3fn).to(dev).requires_grad_(), k.to(torch.float8_e4m3fn).to(dev),
                     v.to(torch.float8_e4m3fn).to(dev), offsets.to(dev))
    with pytest.raises(NotImplementedError):
        pkg.delta_hstu_mha(64, 0.2, q.bfloat16()[:16].to(dev).requires_grad_(), k.bfloat16().to(dev), v.bfloat16().to(dev), offsets.to(dev))
    # no gradient asked for: the plain forward path, no graph
    out = pkg.hstu_mha(64, 0.2, q.bfloat16().to(dev), k.bfloat16().to(dev), v.bfloat16().to(dev), offsets.to(dev))
    assert not out.requires_grad
    # only v requires grad: dq and dk are still produced and simply dropped by autograd
    vd = v.bfloat16().to(dev).requires_grad_()
    out = pkg.hstu_mha(64, 0.2, q.bfloat16().to(dev), k.bfloat16().to(dev), vd, offsets.to(dev))
    out.sum().backward()
    assert vd.grad is not None and torch.isfinite(vd.grad).all()
    empty = pkg.hstu_mha(64, 0.2, q.bfloat16()[:0].to(dev).requires_grad_(), k.bfloat16()[:0].to(dev), v.bfloat16()[:0].to(dev),
                         torch.zeros(1, dtype=torch.int64, device=dev))
    assert empty.shape == (0, 2, 32)


@pytest.mark.gpu
@pytest.mark.parametrize("per_row", [False, True])
def test_gradients_with_attn_scale(pkg, dev, per_row):
    """hstu_mha(..., attn_scale=a).backward(): the gradients of q, k, v against autograd (fp64) through the restated
    forward with the same attn_scale (pt_hstu_attention.py:152-165)."""
    print("[case] backward with attn_scale, per_row", per_row, flush=True)
    lengths = [70, 0, 33, 129]
    q, k, v, dout, offsets = _inputs(31, lengths, 2, 32, 32, torch.bfloat16, scale=0.5)
    N, alpha = 160, 0.2
    tg = torch.tensor([5, 0, 33, 0])
    a = (torch.rand(q.shape[0], generator=torch.Generator().manual_seed(9)) + 0.5) / N if per_row else torch.tensor(1.3 / N)
    ref = G.autograd_grads(N, alpha, q, k, v, offsets, dout, num_targets=tg, max_attn_len=40, contextual_seq_len=2, attn_scale=a)
    qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
    out = pkg.hstu_mha(N, alpha, qd, kd, vd, offsets.to(dev), num_targets=tg.to(dev), max_attn_len=40, contextual_seq_len=2,
                       attn_scale=a.to(dev))
    out.backward(dout.to(dev))
    torch.cuda.synchronize()
    for name, got, want in zip(("dq", "dk", "dv"), (qd.grad, kd.grad, vd.grad), ref):
        got, want = got.float().cpu(), want.float()
        rel = float((got - want).norm() / want.norm())
        assert rel <= 1e-2, f"{name}: relative error {rel:.3e}"
        assert float((got - want).abs().max()) <= 2e-2 * float(want.abs().max()), name
