"""CPU tests that pin the oracle (no GPU, no HIP library calls)."""

import itertools
import os

import numpy as np
import pytest
import torch

from oracle import c_ref, hstu_oracle as O

from util import make_case

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small_cases.npz")


# ---------------------------------------------------------------- pad / unpad (stand-ins for the fbgemm ops)
def test_pad_matches_explicit_loop_and_round_trips():
    g = torch.Generator().manual_seed(1)
    lengths = [3, 0, 7, 5, 1]
    offs = torch.tensor([0] + list(np.cumsum(lengths)))
    x = torch.randn((sum(lengths), 6), generator=g)
    N = 7
    dense = O.jagged_to_padded_dense(x, offs, N)
    expect = torch.zeros(len(lengths), N, 6)
    for b, n in enumerate(lengths):
        for i in range(n):
            expect[b, i] = x[int(offs[b]) + i]
    assert torch.equal(dense, expect)
    assert torch.equal(O.dense_to_jagged(dense, offs, x.shape[0]), x)


def test_pad_truncates_rows_past_max_len():
    offs = torch.tensor([0, 5, 8])
    x = torch.arange(8, dtype=torch.float32).view(8, 1)
    dense = O.jagged_to_padded_dense(x, offs, 4)
    assert dense[0, :, 0].tolist() == [0, 1, 2, 3]
    assert dense[1, :, 0].tolist() == [5, 6, 7, 0]


# ---------------------------------------------------------------- mask
def _oracle_mask(n, c, t, w, f, pad=2):
    N = n + pad
    m = O.get_valid_attn_mask(
        True, N, torch.tensor([n]), None if t is None else torch.tensor([t]), w, c, f
    )
    return m[0].numpy()


def test_mask_matches_position_class_formulation_exhaustively():
    """id-formula mask (reference lines 32-84) vs. the per-class column ranges of hstu_ref.c."""
    checked = 0
    for n, c, t, w, f in itertools.product(range(1, 25), (0, 1, 3), (None, 0, 1, 5), (0, 1, 4), (0, 2)):
        if n - (t or 0) < c:
            continue  # caller contract: the history holds the contextual prefix
        m = _oracle_mask(n, c, t, w, f)
        assert (m[:n, :n] == c_ref.mask(n, c, t, w, f)).all(), (n, c, t, w, f)
        # padded key columns are never visible to real rows
        assert not m[:n, n:].any(), (n, c, t, w, f)
        checked += 1
    assert checked > 1500


def test_mask_closed_form_special_cases():
    n = 13
    tril = np.tril(np.ones((n, n), dtype=bool))
    assert (_oracle_mask(n, 0, None, 0, 0, pad=0) == tril).all()  # plain causal
    assert (_oracle_mask(n, 0, None, n + 5, 0, pad=0) == tril).all()  # window wider than the sequence
    assert (_oracle_mask(n, 0, n, 0, 0, pad=0) == np.eye(n, dtype=bool)).all()  # all targets: self only
    assert _oracle_mask(n, n, None, 0, 0, pad=0).all()  # all contextual: everything
    w = 3
    band = tril & ~np.tril(np.ones((n, n), dtype=bool), -(w + 1))
    assert (_oracle_mask(n, 0, None, w, 0, pad=0) == band).all()  # sliding window keeps w past keys + self


def test_mask_target_rows_see_history_and_self_only():
    n, t = 20, 6
    m = _oracle_mask(n, 0, t, 0, 0, pad=0)
    u = n - t
    for r in range(u, n):
        expect = np.zeros(n, dtype=bool)
        expect[:u] = True
        expect[r] = True
        assert (m[r] == expect).all()


def test_rows_helper_matches_batched_mask():
    for n, c, t, w, f in [(30, 3, 4, 5, 2), (17, 0, None, 0, 0), (25, 2, 0, 3, 0), (9, 0, 9, 2, 0)]:
        full = _oracle_mask(n, c, t, w, f, pad=0)
        rows = O._seq_mask_rows(n, 4, min(n, 15), t, w, c, f).numpy()
        assert (rows == full[4 : min(n, 15)]).all()


# ---------------------------------------------------------------- whole op
CASES = [
    # lengths, H, D, N, targets, w, c, f
    ([16, 128, 57, 1, 0, 90], 2, 32, 128, None, 0, 0, 0),
    ([70, 9, 41, 130], 2, 16, 140, [5, 2, 20, 1], 11, 3, 0),
    ([50, 64, 33], 1, 24, 70, [10, 0, 3], 7, 2, 4),
    ([33, 12], 3, 8, 40, [33, 0], 0, 0, 0),
    ([20, 31], 1, 8, 31, None, 5, 4, 0),
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_dense_oracle_matches_scalar_c(case):
    lengths, H, D, N, targets, w, c, f = case
    q, k, v, offs, t = make_case(7, lengths, H, D, targets=targets, dtype=torch.float32)
    alpha = 1.0 / D**0.5
    dense = O.pytorch_hstu_mha(
        N, alpha, q, k, v, offs, num_targets=t, max_attn_len=w, contextual_seq_len=c, min_full_attn_seq_len=f
    )
    ref = c_ref.fwd(N, alpha, q, k, v, offs, t, w, c, f)
    torch.testing.assert_close(dense, ref, atol=1e-7, rtol=1e-4)
    per_seq = O.hstu_mha_per_sequence(
        N, alpha, q, k, v, offs, num_targets=t, max_attn_len=w, contextual_seq_len=c, min_full_attn_seq_len=f,
        row_chunk=17,
    )
    torch.testing.assert_close(per_seq, ref, atol=1e-7, rtol=1e-4)
    # restricted to some query rows: those rows as in the scalar checker's result, every other row untouched
    spans = [(0, 3), (7, 19), (28, 1000)]
    some = O.hstu_mha_per_sequence(
        N, alpha, q, k, v, offs, num_targets=t, max_attn_len=w, contextual_seq_len=c, min_full_attn_seq_len=f,
        row_chunk=5, row_ranges=spans,
    )
    keep = torch.zeros(q.shape[0], dtype=torch.bool)
    for b in range(len(lengths)):
        for a, z in spans:
            keep[int(offs[b]) + a : min(int(offs[b]) + z, int(offs[b + 1]))] = True
    torch.testing.assert_close(some[keep], ref[keep], atol=1e-7, rtol=1e-4)
    assert not some[~keep].any()


@pytest.mark.parametrize("delta,w,c", [(8, 0, 0), (5, 6, 2), (1, 0, 3)])
def test_cached_oracle_matches_scalar_c_and_tail_of_full(delta, w, c):
    lengths, H, D, N = [40, 12, 25, 31], 2, 16, 48
    q, k, v, offs, t = make_case(11, lengths, H, D, targets=[delta] * 4, dtype=torch.float32)
    alpha = 0.3
    # delta queries = the last `delta` rows of the full q (hstu_attention_test.py:382-488 of the reference)
    idx = torch.cat([torch.arange(int(offs[b + 1]) - delta, int(offs[b + 1])) for b in range(4)])
    dq = q[idx]
    got = O.pytorch_cached_hstu_mha(N, alpha, dq, k, v, offs, t, w, c)
    ref = c_ref.fwd(N, alpha, dq, k, v, offs, t, w, c, 0, delta)
    torch.testing.assert_close(got, ref, atol=1e-7, rtol=1e-4)
    full = O.pytorch_hstu_mha(N, alpha, q, k, v, offs, num_targets=t, max_attn_len=w, contextual_seq_len=c)
    torch.testing.assert_close(got, full[idx], atol=1e-7, rtol=1e-5)
    per_seq = O.cached_hstu_mha_per_sequence(N, alpha, dq, k, v, offs, t, w, c)
    torch.testing.assert_close(per_seq, ref, atol=1e-7, rtol=1e-4)


def test_textbook_reduction_for_plain_causal():
    """With a lower-triangular mask the op is tril(silu(alpha QK^T)) / N @ V, computed here in float64."""
    n, H, D, N = 37, 2, 16, 64
    q, k, v, offs, _ = make_case(3, [n], H, D, dtype=torch.float32)
    alpha = 0.25
    got = O.pytorch_hstu_mha(N, alpha, q, k, v, offs)
    for h in range(H):
        s = (q[:, h].double() @ k[:, h].double().T) * alpha
        p = torch.tril(s * torch.sigmoid(s)) / N
        torch.testing.assert_close(got[:, h].double(), p @ v[:, h].double(), atol=1e-8, rtol=1e-5)


def test_invariants_scale_batch_head_and_target_permutation():
    lengths, H, D = [30, 18, 25], 2, 16
    q, k, v, offs, t = make_case(5, lengths, H, D, targets=[6, 3, 0], dtype=torch.float32)
    kw = dict(num_targets=t, max_attn_len=9, contextual_seq_len=2)
    a = O.pytorch_hstu_mha(32, 0.2, q, k, v, offs, **kw)
    # 1/N scale: N is the argument, not the sequence's own length
    b = O.pytorch_hstu_mha(64, 0.2, q, k, v, offs, **kw)
    torch.testing.assert_close(a, b * 2.0, atol=0, rtol=1e-6)
    # batch independence: sequence 1 alone
    s0, s1 = int(offs[1]), int(offs[2])
    alone = O.pytorch_hstu_mha(
        32, 0.2, q[s0:s1], k[s0:s1], v[s0:s1], torch.tensor([0, s1 - s0]), num_targets=t[1:2],
        max_attn_len=9, contextual_seq_len=2,
    )
    torch.testing.assert_close(alone, a[s0:s1], atol=1e-8, rtol=1e-6)
    # head independence
    h1 = O.pytorch_hstu_mha(32, 0.2, q[:, 1:], k[:, 1:], v[:, 1:], offs, **kw)
    torch.testing.assert_close(h1, a[:, 1:], atol=1e-8, rtol=1e-6)
    # swapping two targets of sequence 0 swaps their outputs and changes nothing else
    # (modules/tests/stu_test.py:180-321 of the reference, at operator level)
    n0 = lengths[0]
    perm = torch.arange(q.shape[0])
    perm[n0 - 1], perm[n0 - 4] = n0 - 4, n0 - 1
    c = O.pytorch_hstu_mha(32, 0.2, q[perm], k[perm], v[perm], offs, **kw)
    torch.testing.assert_close(c, a[perm], atol=1e-8, rtol=1e-6)


def test_attn_scale_is_a_factor_per_query_row_in_place_of_one_over_n():
    """PT:152-165: with attn_scale the result is attn_scale[row] * N times the plain one -- per QUERY row (a factor per
    key would not commute with the sum over keys), for every head alike; a 0-dim tensor scales all rows."""
    lengths, H, D, N = [19, 0, 33, 7], 2, 16, 40
    q, k, v, offs, t = make_case(21, lengths, H, D, targets=[3, 0, 9, 1], dtype=torch.float32)
    kw = dict(num_targets=t, max_attn_len=11, contextual_seq_len=2)
    plain = O.pytorch_hstu_mha(N, 0.3, q, k, v, offs, **kw)
    a = torch.rand(q.shape[0], generator=torch.Generator().manual_seed(3)) + 0.5
    scaled = O.pytorch_hstu_mha(N, 0.3, q, k, v, offs, attn_scale=a, **kw)
    torch.testing.assert_close(scaled, plain * (a * N).view(-1, 1, 1), atol=1e-9, rtol=1e-5)
    one = O.pytorch_hstu_mha(N, 0.3, q, k, v, offs, attn_scale=torch.tensor(0.125), **kw)
    torch.testing.assert_close(one, plain * (0.125 * N), atol=1e-9, rtol=1e-5)
    per_seq = O.hstu_mha_per_sequence(N, 0.3, q, k, v, offs, attn_scale=a, row_chunk=5, **kw)
    torch.testing.assert_close(per_seq, scaled, atol=1e-8, rtol=1e-5)
    per_seq1 = O.hstu_mha_per_sequence(N, 0.3, q, k, v, offs, attn_scale=torch.tensor(0.125), **kw)
    torch.testing.assert_close(per_seq1, one, atol=1e-8, rtol=1e-5)


def test_silu_special_values():
    # one key, one query: out = silu(alpha q k) / N * v
    for x, expect in [(0.0, 0.0), (30.0, 30.0), (-30.0, -30.0 / (1 + np.exp(30.0))), (-1.2785, -0.27846)]:
        q = torch.tensor([[[x]]])
        k = torch.tensor([[[1.0]]])
        v = torch.tensor([[[1.0]]])
        got = O.pytorch_hstu_mha(1, 1.0, q, k, v, torch.tensor([0, 1]))
        assert abs(float(got) - expect) < 1e-4 * max(1.0, abs(expect))


def test_golden_fixture_matches_oracle_and_checker():
    z = np.load(GOLDEN)
    names = sorted({key.split(".")[0] for key in z.files})
    assert len(names) >= 5
    for name in names:
        q = torch.from_numpy(z[f"{name}.q"]).view(torch.bfloat16).float()
        k = torch.from_numpy(z[f"{name}.k"]).view(torch.bfloat16).float()
        v = torch.from_numpy(z[f"{name}.v"]).view(torch.bfloat16).float()
        offs = torch.from_numpy(z[f"{name}.offsets"])
        t = torch.from_numpy(z[f"{name}.targets"])
        t = None if int(t[0]) < 0 else t
        N, w, c, f, delta = [int(x) for x in z[f"{name}.params"]]
        alpha = float(z[f"{name}.alpha"][0])
        want = torch.from_numpy(z[f"{name}.out"])
        got = O.hstu_mha_per_sequence(
            N, alpha, q, k, v, offs, num_targets=t, max_attn_len=w, contextual_seq_len=c,
            min_full_attn_seq_len=f, delta_size=delta,
        )
        torch.testing.assert_close(got, want, atol=1e-7, rtol=1e-4)
        torch.testing.assert_close(c_ref.fwd(N, alpha, q, k, v, offs, t, w, c, f, delta), want, atol=0, rtol=0)
