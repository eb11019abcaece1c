"""concat_2D_jagged / split_2D_jagged / write_kv_tail: the oracle against itself on the CPU, the HIP kernels against
the oracle on the GPU (bit-exact: these ops only move bytes)."""

import numpy as np
import pytest
import torch

from oracle import jagged_oracle as J


def _case(seed, B, max_a, max_b, D, dense_a, dense_b, dtype, empty=True):
    """The shapes of the reference's own tests (jagged_tensors_test.py:40-53, 166-179): B 2..8, max_len 20..100,
    D 10..30, each side dense or jagged."""
    rng = np.random.default_rng(seed)
    la = np.full(B, max_a) if dense_a else rng.integers(0 if empty else 1, max_a + 1, size=B)
    lb = np.full(B, max_b) if dense_b else rng.integers(0 if empty else 1, max_b + 1, size=B)
    oa = torch.tensor(np.concatenate([[0], np.cumsum(la)]), dtype=torch.int64)
    ob = torch.tensor(np.concatenate([[0], np.cumsum(lb)]), dtype=torch.int64)
    g = torch.Generator().manual_seed(seed)
    va = torch.randn((int(oa[-1]), D), generator=g).to(dtype)
    vb = torch.randn((int(ob[-1]), D), generator=g).to(dtype)
    return va, vb, oa, ob


def _bits(x):
    return x.contiguous().view(torch.uint8)


GRID = [
    (seed, B, ma, mb, D, da, db, dt)
    for seed, (B, ma, mb, D) in enumerate([(2, 20, 100, 10), (8, 100, 20, 30), (5, 37, 64, 16), (3, 1, 90, 25), (7, 64, 64, 128)])
    for da in (False, True)
    for db in (False, True)
    for dt in (torch.bfloat16, torch.float32)
]


# ---------------------------------------------------------------- oracle, CPU


@pytest.mark.parametrize("seed,B,ma,mb,D,da,db,dt", GRID)
def test_oracle_forms_agree(seed, B, ma, mb, D, da, db, dt):
    va, vb, oa, ob = _case(seed, B, ma, mb, D, da, db, dt)
    want = J.concat_by_batch(va, vb, oa, ob)
    got = J.concat_padded(va, vb, ma, mb, None if da else oa, None if db else ob)
    assert torch.equal(_bits(got), _bits(want))
    # the step-by-step form also takes max_len=None (derived from the offsets)
    if not da and not db:
        assert torch.equal(_bits(J.concat_padded(va, vb, None, None, oa, ob)), _bits(want))
    if not (da and db):  # the split needs offsets on at least one side (pt_jagged_tensors.py:152-166)
        left, right = J.split_padded(ma + mb, want, ma, mb, None if da else oa, None if db else ob)
        assert torch.equal(_bits(left), _bits(va)) and torch.equal(_bits(right), _bits(vb))
    l2, r2 = J.split_by_batch(want, oa, ob)
    assert torch.equal(_bits(l2), _bits(va)) and torch.equal(_bits(r2), _bits(vb))


def test_oracle_long_sequences_are_outside_the_contract():
    """A sequence longer than max_len_left is not simply truncated by the reference: its padding cuts the tail, but
    its mask `pos < len_left` then reaches into the right side's rows.  The step-by-step form reproduces exactly
    that (row count included), which is why callers must keep lengths <= max_len."""
    va = torch.arange(1, 7, dtype=torch.float32).view(6, 1)      # one batch, 6 left rows
    vb = torch.arange(101, 103, dtype=torch.float32).view(2, 1)  # 2 right rows
    oa, ob = torch.tensor([0, 6]), torch.tensor([0, 2])
    got = J.concat_padded(va, vb, 4, 3, oa, ob)  # max_len_left = 4 < 6
    # dense = [1 2 3 4 | 101 102 0]; mask = pos < 6 or 4 <= pos < 6  ->  positions 0..5
    assert got.view(-1).tolist() == [1.0, 2.0, 3.0, 4.0, 101.0, 102.0]


def test_oracle_special_cases():
    va, vb, oa, ob = _case(3, 4, 9, 7, 5, False, False, torch.float32)
    zero = torch.zeros_like(ob)
    # an empty right side leaves the left side unchanged, and vice versa
    assert torch.equal(J.concat_padded(va, vb[:0], 9, 7, oa, zero), va)
    assert torch.equal(J.concat_padded(va[:0], vb, 9, 7, torch.zeros_like(oa), ob), vb)
    # one batch: plain concatenation
    assert torch.equal(J.concat_padded(va[:6], vb[:4], 6, 4, None, None), torch.cat([va[:6], vb[:4]]))


# ---------------------------------------------------------------- HIP, GPU


@pytest.fixture(scope="module")
def pkg():
    import __graft_entry__

    return __graft_entry__.load_package()


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("seed,B,ma,mb,D,da,db,dt", GRID)
def test_hip_concat_and_split_bit_exact(pkg, dev, seed, B, ma, mb, D, da, db, dt):
    print(f"[case] jagged {seed} {B} {ma} {mb} {D} {da} {db} {dt}", flush=True)
    va, vb, oa, ob = _case(seed, B, ma, mb, D, da, db, dt)
    want = J.concat_by_batch(va, vb, oa, ob)
    kw = dict(max_len_left=ma, max_len_right=mb, offsets_left=None if da else oa.to(dev), offsets_right=None if db else ob.to(dev))
    got = pkg.concat_2D_jagged(ma + mb, va.to(dev), vb.to(dev), **kw)
    torch.cuda.synchronize()
    assert got.shape == want.shape and got.dtype == want.dtype
    assert torch.equal(_bits(got.cpu()), _bits(want))
    if da and db:
        return  # split needs at least one jagged side (jagged_tensors.py:127-130 of the reference)
    left, right = pkg.split_2D_jagged(ma + mb, want.to(dev), **kw)
    torch.cuda.synchronize()
    assert torch.equal(_bits(left.cpu()), _bits(va)) and torch.equal(_bits(right.cpu()), _bits(vb))
    # int32 offsets, derived max_len (host sync, as in the reference), explicit totals
    if not da and not db:
        kw32 = dict(offsets_left=oa.to(torch.int32).to(dev), offsets_right=ob.to(torch.int32).to(dev))
        assert torch.equal(_bits(pkg.concat_2D_jagged(ma + mb, va.to(dev), vb.to(dev), **kw32).cpu()), _bits(want))
        l3, r3 = pkg.split_2D_jagged(ma + mb, want.to(dev), total_len_left=va.shape[0], total_len_right=vb.shape[0], **kw32)
        assert torch.equal(_bits(l3.cpu()), _bits(va)) and torch.equal(_bits(r3.cpu()), _bits(vb))


@pytest.mark.gpu
def test_hip_concat_odd_widths_and_strided_views(pkg, dev):
    """Row widths that are not multiples of 16 bytes fall back to narrower accesses; column slices of a wider
    buffer (stride(0) != width) are read in place."""
    print("[case] jagged odd widths", flush=True)
    for D, dt in [(1, torch.int8), (3, torch.int8), (5, torch.bfloat16), (7, torch.float32), (24, torch.bfloat16)]:
        rng = np.random.default_rng(D)
        la, lb = rng.integers(0, 40, size=6), rng.integers(0, 9, size=6)
        oa = torch.tensor(np.concatenate([[0], np.cumsum(la)]), dtype=torch.int64)
        ob = torch.tensor(np.concatenate([[0], np.cumsum(lb)]), dtype=torch.int64)
        wide_a = torch.randint(-100, 100, (int(oa[-1]), 2 * D + 3)).to(dt)
        wide_b = torch.randint(-100, 100, (int(ob[-1]), D + 1)).to(dt)
        va, vb = wide_a[:, 2 : 2 + D], wide_b[:, 1:]
        want = J.concat_by_batch(va, vb, oa, ob)
        got = pkg.concat_2D_jagged(48, wide_a.to(dev)[:, 2 : 2 + D], wide_b.to(dev)[:, 1:], 40, 8, oa.to(dev), ob.to(dev))
        torch.cuda.synchronize()
        assert torch.equal(_bits(got.cpu()), _bits(want)), (D, dt)


@pytest.mark.gpu
def test_hip_concat_large_tensor(pkg, dev):
    """More than 2^31 bytes per tensor (the reference's large-tensor case, jagged_tensors_test.py:196-214, scaled
    to B=70): 64-bit addressing throughout.  Spot-checked rows instead of a full host copy."""
    print("[case] jagged large", flush=True)
    B, ma, mb, D = 70, 32768, 10, 512
    g = torch.Generator(device=dev).manual_seed(5)
    va = torch.randint(-30000, 30000, (B * ma, D), dtype=torch.int16, device=dev, generator=g)
    lb = torch.randint(0, mb + 1, (B,), generator=torch.Generator().manual_seed(6))
    ob = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(lb, 0)])
    vb = torch.randint(-30000, 30000, (int(ob[-1]), D), dtype=torch.int16, device=dev, generator=g)
    assert va.numel() * 2 > 2**31
    out = pkg.concat_2D_jagged(ma + mb, va, vb, ma, mb, None, ob.to(dev))
    torch.cuda.synchronize()
    assert out.shape[0] == va.shape[0] + vb.shape[0]
    for b in (0, 1, B // 2, B - 1):
        start = b * ma + int(ob[b])
        for r in (0, 1, ma // 2, ma - 1):
            assert torch.equal(out[start + r], va[b * ma + r])
        n = int(lb[b])
        if n:
            assert torch.equal(out[start + ma : start + ma + n], vb[int(ob[b]) : int(ob[b]) + n])
    # checksum of the whole tensor: the concatenation only permutes rows
    assert int(out.to(torch.int64).sum()) == int(va.to(torch.int64).sum()) + int(vb.to(torch.int64).sum())


@pytest.mark.gpu
def test_write_kv_tail_equals_concat_and_feeds_delta_attention(pkg, dev):
    """The in-place cache layout: history rows + delta_size spare rows per sequence.  Writing the new rows into the
    spare rows gives the tensor `_construct_full_kv` (modules/stu.py:133-173 of the reference) builds by
    concatenation, bit for bit, and `delta_hstu_mha` on it gives the same output; a second micro-batch only
    overwrites the spare rows."""
    print("[case] write_kv_tail", flush=True)
    B, H, D, delta = 5, 2, 64, 16
    rng = np.random.default_rng(9)
    hist = rng.integers(0, 300, size=B)
    hist[2] = 0
    oc = torch.tensor(np.concatenate([[0], np.cumsum(hist)]), dtype=torch.int64)
    g = torch.Generator().manual_seed(10)
    cache_k = (torch.randn((int(oc[-1]), H * D), generator=g) * 0.1).to(torch.bfloat16)
    cache_v = (torch.randn((int(oc[-1]), H * D), generator=g) * 0.1).to(torch.bfloat16)
    full_offsets = oc + delta * torch.arange(B + 1)
    N = int(hist.max()) + delta
    # one-time set-up: the padded cache (history in place, spare rows arbitrary)
    spare = torch.full((B * delta, H * D), 7.0, dtype=torch.bfloat16)
    full_k = pkg.concat_2D_jagged(N, cache_k.to(dev), spare.to(dev), int(hist.max()), delta, oc.to(dev), None)
    full_v = pkg.concat_2D_jagged(N, cache_v.to(dev), spare.to(dev), int(hist.max()), delta, oc.to(dev), None)
    t = torch.full((B,), delta, dtype=torch.int64)
    for micro_batch in range(2):
        dk = (torch.randn((B * delta, H * D), generator=g) * 0.1).to(torch.bfloat16)
        dv = (torch.randn((B * delta, H * D), generator=g) * 0.1).to(torch.bfloat16)
        dq = (torch.randn((B * delta, H, D), generator=g) * 0.1).to(torch.bfloat16)
        want_k = J.concat_by_batch(cache_k, dk, oc, delta * torch.arange(B + 1))
        want_v = J.concat_by_batch(cache_v, dv, oc, delta * torch.arange(B + 1))
        pkg.write_kv_tail(full_k, full_offsets.to(dev), dk.to(dev))
        pkg.write_kv_tail(full_v, full_offsets.to(dev), dv.to(dev))
        torch.cuda.synchronize()
        assert torch.equal(_bits(full_k.cpu()), _bits(want_k)) and torch.equal(_bits(full_v.cpu()), _bits(want_v))
        out_inplace = pkg.delta_hstu_mha(
            N, 0.125, dq.to(dev), full_k.view(-1, H, D), full_v.view(-1, H, D), full_offsets.to(dev), num_targets=t.to(dev)
        )
        out_concat = pkg.delta_hstu_mha(
            N, 0.125, dq.to(dev), want_k.to(dev).view(-1, H, D), want_v.to(dev).view(-1, H, D), full_offsets.to(dev),
            num_targets=t.to(dev),
        )
        torch.cuda.synchronize()
        assert torch.equal(out_inplace, out_concat)


@pytest.mark.gpu
def test_jagged_wrapper_rejections(pkg, dev):
    a = torch.zeros((4, 8), device=dev)
    with pytest.raises(AssertionError, match="values_left must be 2D"):
        pkg.concat_2D_jagged(8, a.view(2, 2, 8), a, 2, 2)
    with pytest.raises(AssertionError, match="must be equal to values_right shape"):
        pkg.concat_2D_jagged(8, a, a[:, :4], 2, 2)
    with pytest.raises(AssertionError, match="cannot be None at the same time"):
        pkg.split_2D_jagged(8, a, max_len_left=1, max_len_right=1)


@pytest.mark.gpu
@pytest.mark.parametrize("seed,B,ma,mb,D,da,db", [(11, 4, 20, 100, 10, False, False), (12, 8, 100, 20, 30, True, False),
                                                   (13, 5, 37, 64, 16, False, True), (14, 3, 64, 64, 128, False, False)])
def test_hip_concat_and_split_gradients(pkg, dev, seed, B, ma, mb, D, da, db):
    """The gradient of a row copy is the inverse row copy: checked bit for bit against the gradients autograd derives
    for the oracle's per-batch ``torch.cat`` (the reference's test does the same with its two backends,
    jagged_tensors_test.py:92-112)."""
    print(f"[case] jagged gradients {seed} {B} {ma} {mb} {D} {da} {db}", flush=True)
    va, vb, oa, ob = _case(seed, B, ma, mb, D, da, db, torch.float32)
    kw = dict(max_len_left=ma, max_len_right=mb, offsets_left=None if da else oa.to(dev), offsets_right=None if db else ob.to(dev))
    a_ref, b_ref = va.clone().requires_grad_(), vb.clone().requires_grad_()
    want = J.concat_by_batch(a_ref, b_ref, oa, ob)
    g = torch.Generator().manual_seed(seed + 100)
    d_out = torch.randn(want.shape, generator=g)
    want.backward(d_out)
    a_hip, b_hip = va.to(dev).requires_grad_(), vb.to(dev).requires_grad_()
    got = pkg.concat_2D_jagged(ma + mb, a_hip, b_hip, **kw)
    got.backward(d_out.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(got.detach().cpu(), want.detach())
    assert torch.equal(a_hip.grad.cpu(), a_ref.grad) and torch.equal(b_hip.grad.cpu(), b_ref.grad)
    # and the split: its gradient is the concatenation of the two incoming gradients
    joined = want.detach().to(dev).requires_grad_()
    left, right = pkg.split_2D_jagged(ma + mb, joined, **kw)
    d_left, d_right = torch.randn(va.shape, generator=g), torch.randn(vb.shape, generator=g)
    (left * d_left.to(dev)).sum().backward(retain_graph=True)
    (right * d_right.to(dev)).sum().backward()
    torch.cuda.synchronize()
    assert torch.equal(joined.grad.cpu(), J.concat_by_batch(d_left, d_right, oa, ob))
