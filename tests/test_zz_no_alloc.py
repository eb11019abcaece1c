"""The entry point that allocates nothing (``hstu_hip_mha_fwd_noalloc``: scratch in a fixed area inside the library)
against ``hstu_hip_mha_fwd`` with a caller-owned workspace: same kernels and schedule, so the outputs must be
bit-identical -- on two calls in a row, the second with a smaller input, for a ragged batch that uses the counters, the
ranking and the work lists, and for a delta call whose kv range is split (partial sums in the area)."""

import numpy as np
import pytest
import torch

from util import make_case

pytestmark = pytest.mark.gpu


def _fwd(pkg, dev, q, k, v, offs, t, N, alpha, noalloc, delta=0, **kw):
    from generative_recommenders_amd.ops import hip_backend

    out = torch.full((q.shape[0], q.shape[1], v.shape[2]), float("nan"), dtype=q.dtype, device=dev)
    hip_backend.mha_fwd(
        q, k, v, out, offs, t, max_seq_len=N, alpha=alpha, delta_size=delta, max_attn_len=kw.pop("w", 0),
        contextual_seq_len=kw.pop("c", 0), min_full_attn_seq_len=0, noalloc=noalloc, **kw,
    )
    torch.cuda.synchronize()
    return out


def test_noalloc_entry_point_matches_the_workspace_one(pkg, dev):
    print("[case] noalloc: ragged full form, then a smaller one, then delta with a kv-split, then a smaller one", flush=True)
    rng = np.random.default_rng(77)
    big = rng.integers(1, 1500, size=90)
    big[3], big[40] = 5000, 0
    small = rng.integers(1, 700, size=21)
    for lengths, N, cfg in ((big, 5000, 0), (small, 700, 0), (big, 5000, 3), (small, 700, 2)):
        tg = np.minimum(lengths, rng.integers(0, 30, size=len(lengths)))
        q, k, v, offs, t = [x.to(dev) for x in make_case(int(lengths.sum()), lengths, 2, 128, targets=tg)]
        kw = dict(w=300, c=3, sort_by_length=True, tile_config=cfg)
        # the plan of this call does use the scratch area: counters + ranking + work lists
        a = _fwd(pkg, dev, q, k, v, offs, t, N, 0.08, True, **dict(kw))
        b = _fwd(pkg, dev, q, k, v, offs, t, N, 0.08, False, **dict(kw))
        assert torch.isfinite(a.float()).all()
        assert torch.equal(a, b), f"full form, {len(lengths)} sequences, tile config {cfg}"
    for B, hist_hi, delta in ((12, 3000, 256), (5, 900, 64)):
        hist = rng.integers(200, hist_hi, size=B)
        lengths = hist + delta
        N = hist_hi + delta
        q, k, v, offs, t = make_case(B, lengths, 4, 128, targets=[delta] * B, delta_size=delta)
        q, k, v, offs, t = [x.to(dev) for x in (q, k, v, offs, t)]
        for splits in (0, 3):
            a = _fwd(pkg, dev, q, k, v, offs, t, N, 0.08, True, delta=delta, kv_splits=splits)
            b = _fwd(pkg, dev, q, k, v, offs, t, N, 0.08, False, delta=delta, kv_splits=splits)
            assert torch.isfinite(a.float()).all()
            assert torch.equal(a, b), f"delta form, {B} users, kv_splits {splits}"


def test_noalloc_entry_point_allocates_nothing_and_refuses_overlap(pkg, dev):
    """What the entry point is for: after the first call on the device (which looks the area up) a call changes neither
    the framework's allocated bytes nor the device's free memory, and takes no workspace from the caller.  And the
    misuse it can detect: a call on another stream while the last one is still running is refused, not raced."""
    from generative_recommenders_amd.ops import hip_backend

    print("[case] noalloc: memory before / after, then a call on a second stream while the first is running", flush=True)
    rng = np.random.default_rng(78)
    lengths = rng.integers(1, 900, size=40)
    q, k, v, offs, t = [x.to(dev) for x in make_case(int(lengths.sum()), lengths, 2, 128, targets=np.zeros(40, dtype=np.int64))]
    out = torch.empty((q.shape[0], 2, 128), dtype=q.dtype, device=dev)
    kw = dict(max_seq_len=900, alpha=0.08, delta_size=0, max_attn_len=0, contextual_seq_len=0, min_full_attn_seq_len=0,
              sort_by_length=True, noalloc=True, workspace_bytes=0)  # workspace_bytes=0: args.workspace stays NULL
    hip_backend.mha_fwd(q, k, v, out, offs, t, **kw)
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev), torch.cuda.mem_get_info(dev)[0])
    hip_backend.mha_fwd(q, k, v, out, offs, t, **kw)
    torch.cuda.synchronize()
    after = (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev), torch.cuda.mem_get_info(dev)[0])
    assert before == after, (before, after)

    # a long call (64 sequences of 4096: about a millisecond) on one stream, then at once a small one on another
    big = np.full(64, 4096)
    qb, kb, vb, ob, tb = [x.to(dev) for x in make_case(5, big, 4, 128, targets=np.zeros(64, dtype=np.int64))]
    outb = torch.empty((qb.shape[0], 4, 128), dtype=qb.dtype, device=dev)
    kwb = dict(kw, max_seq_len=4096)
    s1, s2 = torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        hip_backend.mha_fwd(qb, kb, vb, outb, ob, tb, **kwb)
    with torch.cuda.stream(s2):
        with pytest.raises(RuntimeError, match="in use"):
            hip_backend.mha_fwd(q, k, v, out, offs, t, **kw)
    torch.cuda.synchronize()
    with torch.cuda.stream(s2):  # once the first has finished, the other stream may use the area
        hip_backend.mha_fwd(q, k, v, out, offs, t, **kw)
    torch.cuda.synchronize()
    ref = torch.empty_like(out)
    hip_backend.mha_fwd(q, k, v, ref, offs, t, **dict(kw, noalloc=False, workspace_bytes=None))
    torch.cuda.synchronize()
    assert torch.equal(out, ref)


def test_noalloc_entry_point_rejects_what_does_not_fit(pkg, dev):
    """A kv-split whose partial sums exceed the fixed area is refused with its own status, and nothing is written."""
    from generative_recommenders_amd.ops import hip_backend

    B, delta, H, D = 64, 512, 4, 128  # 8 runs x 32768 rows x 4 heads x 128 x 4 bytes = 512 MB of partial sums
    lengths = np.full(B, 600)
    q, k, v, offs, t = make_case(5, lengths, H, D, targets=[delta] * B, delta_size=delta)
    q, k, v, offs, t = [x.to(dev) for x in (q, k, v, offs, t)]
    out = torch.full((q.shape[0], H, D), 7.0, dtype=q.dtype, device=dev)
    with pytest.raises(RuntimeError, match="scratch"):
        hip_backend.mha_fwd(q, k, v, out, offs, t, max_seq_len=600, alpha=0.1, delta_size=delta, max_attn_len=0,
                            contextual_seq_len=0, min_full_attn_seq_len=0, kv_splits=8, noalloc=True)
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())
