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
