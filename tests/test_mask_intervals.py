"""The kernels evaluate the mask of a masked tile per query row as a union of two intervals of key POSITIONS and a
point (RowMask::valid_bits in csrc/hstu_common.h).  This test restates that form in Python and checks it against the
reference's id formula (oracle.get_valid_attn_mask, ops/pytorch/pt_hstu_attention.py:32-84) by brute force over every
small setting: sequence length, number of targets, window, contextual prefix, min_full_attn_seq_len."""

import itertools

import torch

from oracle import hstu_oracle


def _interval_mask(n, targets, w, c, f):
    """valid[row, key] from the per-row constants the kernel keeps: klo, khi, cend, pos."""
    shift = c - 1 if c > 0 else 0
    max_id = n - (targets or 0) - shift

    def ident(pos):  # ids are clamped to max_id only when targets are given
        x = max(pos - shift, 0)
        return x if targets is None else min(x, max_id)

    valid = torch.zeros((n, n), dtype=torch.bool)
    for row in range(n):
        idr = ident(row)
        wr = 0x7FFFFFFF if (w == 0 or (f > 0 and idr >= max_id - f)) else w
        lo = idr - wr
        ctx = c > 0 and idr == 0
        klo = lo + shift if lo > 0 else 0
        khi = idr - 1 + shift if idr >= 1 else -1
        cend = max_id + shift if (ctx and max_id > 0) else 0
        for key in range(n):
            valid[row, key] = (key == row) or (klo <= key <= khi) or (key < cend)
    return valid


def _column_interval_mask(n, targets, w, c, f):
    """The same matrix from the per-KEY constants of the backward (KeyMask in csrc/hstu_bwd_kernel.h): the rows that see
    key k are [rlo, rhi], [r2lo, n) (rows whose window is lifted by min_full_attn_seq_len), [0, crows) (contextual
    rows) and k itself."""
    big = 1 << 30
    shift = c - 1 if c > 0 else 0
    max_id = n - (targets or 0) - shift

    def ident(pos):
        x = max(pos - shift, 0)
        return x if targets is None else min(x, max_id)

    valid = torch.zeros((n, n), dtype=torch.bool)
    for key in range(n):
        ids = ident(key)
        clamped = targets is not None
        rlo = big if (clamped and ids + 1 > max_id) else ids + 1 + shift
        if w == 0:
            rhi = big
        else:
            rhi = big if (clamped and ids + w >= max_id) else ids + w + shift
        r2lo = big
        if w > 0 and f > 0:
            first_full = max_id - f
            r2lo = max(rlo, 0 if first_full <= 0 else first_full + shift)
        crows = shift + 1 if (c > 0 and ids < max_id) else 0
        for row in range(n):
            valid[row, key] = (row == key) or (rlo <= row <= rhi) or (row >= r2lo) or (row < crows)
    return valid


def test_position_intervals_equal_the_id_formula():
    checked = 0
    for n, c, w, f in itertools.product([1, 2, 5, 9, 14], [0, 1, 3, 6], [0, 1, 2, 4, 20], [0, 2, 5]):
        if f > 0 and w == 0:
            continue
        for targets in [None] + list(range(0, n + 1)):
            # sequences shorter than the contextual prefix (max_id <= 0) included: the formula still has an answer
            lengths = torch.tensor([n])
            want = hstu_oracle.get_valid_attn_mask(True, n, lengths, None if targets is None else torch.tensor([targets]), w, c, f)[0]
            got = _interval_mask(n, targets, w, c, f)
            assert torch.equal(got, want), (n, targets, w, c, f)
            assert torch.equal(_column_interval_mask(n, targets, w, c, f), want), ("per key", n, targets, w, c, f)
            checked += 1
    assert checked > 1000


_HARNESS = r"""
#include <cstdio>
#define __device__
#define __forceinline__ inline
%s
int main() {
    long bad = 0, total = 0;
    for (int n = 1; n <= 46; n += 3) for (int c = 0; c <= 7; c += (c < 2 ? 1 : 5)) for (int w = 0; w <= 40; w = (w == 0 ? 1 : w * 3))
    for (int f = 0; f <= 6; f += 3) for (int tg = -1; tg <= n; tg += (tg < 1 ? 1 : 7)) {
        if (f > 0 && w == 0) continue;
        const int t = tg < 0 ? 0 : tg;
        SeqMask M; M.n = n; M.w = w; M.c = c; M.f = f; M.shift = c > 0 ? c - 1 : 0;
        M.max_id = n - t - M.shift; M.idclamp = tg >= 0 ? M.max_id : 0x7fffffff;
        for (int r = 0; r < n; ++r) {
            RowMask R; R.init(M, r);
            for (int p0 = 0; p0 < n + 40; ++p0) {
                const unsigned bits = R.valid_bits(p0);
                for (int d = 0; d < 32; ++d, ++total) bad += ((bits >> d) & 1) != (p0 + d < n ? R.valid(M, p0 + d) : false);
            }
        }
        for (int k = 0; k < n; ++k) {
            KeyMask K; K.init(M, k);
            for (int p0 = 0; p0 < n + 40; ++p0) {
                const unsigned bits = K.valid_bits(p0, n);
                for (int d = 0; d < 32; ++d, ++total) bad += ((bits >> d) & 1) != (p0 + d < n ? K.valid(M, p0 + d) : false);
            }
        }
    }
    printf("%%ld %%ld\n", total, bad);
    return 0;
}
"""


def test_kernel_source_bits_equal_the_kernel_source_predicate(tmp_path):
    """The structs themselves, cut out of the kernel headers and compiled for the host: valid_bits() against valid() for
    every row / key, block start and small mask setting, sequences shorter than the contextual prefix included."""
    import os
    import shutil
    import subprocess

    import pytest

    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("needs g++")
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "generative-recommenders_amd", "csrc")
    common = open(os.path.join(csrc, "hstu_common.h")).read()
    bwd = open(os.path.join(csrc, "hstu_bwd_kernel.h")).read()

    def cut(text, begin, end):
        return text[text.index(begin) : text.index(end)]

    structs = (cut(common, "// Per-sequence mask state", "// Chunk swizzles.")
               + cut(common, "// Per-lane constants of the mask predicate for one query row.", "// P^T for one 32x32 block.")
               + cut(bwd, "// Per-lane constants of the mask predicate for one key.", "// Order in which two chains"))
    src = tmp_path / "bits.cpp"
    src.write_text(_HARNESS % structs)
    exe = tmp_path / "bits"
    subprocess.run([gxx, "-O1", "-std=c++17", str(src), "-o", str(exe)], check=True)
    total, bad = (int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split())
    assert total > 100_000_000 and bad == 0
