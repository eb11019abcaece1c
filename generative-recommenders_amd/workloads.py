"""Synthetic jagged workloads and exact work counts for benchmarking the attention path.

The shapes follow the benchmark recipe of the reference
(``generative_recommenders/ops/benchmarks/hstu_attention_bench.py:217-271``): host-seeded length draws,
``seq_offsets = [0] + cumsum(lengths)``, q/k/v as column slices of one ``[L, H, 2*Dqk+Dv]`` buffer or dense,
and its FLOP convention (``_flops``, lines 38-62) next to the exact count of mask-valid pairs.
"""

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np
import torch


@dataclass
class Workload:
    name: str
    batch: int
    heads: int
    dqk: int
    dv: int
    max_seq_len: int
    lengths: np.ndarray  # [B] total length of each sequence (contextual + history + targets)
    num_targets: Optional[np.ndarray] = None
    max_attn_len: int = 0
    contextual_seq_len: int = 0
    min_full_attn_seq_len: int = 0
    delta_size: int = 0
    dtype: str = "bf16"
    alpha: float = 0.0
    seed: int = 0
    notes: str = ""
    extra: Dict[str, float] = field(default_factory=dict)

    def __post_init__(self) -> None:
        if self.alpha == 0.0:
            self.alpha = 1.0 / float(np.sqrt(self.dqk))

    @property
    def total_kv(self) -> int:
        return int(self.lengths.sum())

    @property
    def total_q(self) -> int:
        return self.batch * self.delta_size if self.delta_size > 0 else self.total_kv


def valid_pairs_per_row(
    n: int, t: int = 0, max_attn_len: int = 0, contextual_seq_len: int = 0, min_full_attn_seq_len: int = 0
) -> np.ndarray:
    """Number of key positions each query position of one sequence attends to (closed form, O(n)).

    Derived from the mask of ``pt_hstu_attention.py:32-84``; ``t`` is the number of targets (0 if none given).
    """
    c, w, f = contextual_seq_len, max_attn_len, min_full_attn_seq_len
    u = n - t
    i = np.arange(n, dtype=np.int64)
    big = np.int64(1) << 40
    wrow = np.full(n, w if w > 0 else big, dtype=np.int64)
    if w > 0 and f > 0:
        wrow[i >= u - f] = big
    out = np.zeros(n, dtype=np.int64)
    hist = (i >= c) & (i < u)
    tgt = i >= u
    if c == 0:
        out[hist] = np.minimum(i[hist], wrow[hist]) + 1
        out[tgt] = np.minimum(u, wrow[tgt]) + 1
    else:
        out[i < min(c, n)] = u
        idh = i - c + 1
        out[hist] = np.minimum(wrow[hist], idh[hist] - 1) + np.where(idh[hist] <= wrow[hist], c, 0) + 1
        out[tgt] = np.minimum(wrow[tgt], u - c) + np.where(u - c + 1 <= wrow[tgt], c, 0) + 1
    return out


def count_valid_pairs(wl: Workload) -> int:
    """Exact number of mask-valid (query, key) pairs of a workload, summed over sequences (not heads)."""
    total = 0
    for b in range(wl.batch):
        n = int(wl.lengths[b])
        if n == 0:
            continue
        t = 0 if wl.num_targets is None else int(wl.num_targets[b])
        rows = valid_pairs_per_row(n, t, wl.max_attn_len, wl.contextual_seq_len, wl.min_full_attn_seq_len)
        if wl.delta_size > 0:
            rows = rows[n - wl.delta_size :]
        total += int(rows.sum())
    return total


def algorithmic_flops(wl: Workload) -> float:
    """``2 * (Dqk + Dv) * H * valid pairs``: both matrix products, multiply-add = 2; exp/rcp/mask not counted."""
    return 2.0 * (wl.dqk + wl.dv) * wl.heads * count_valid_pairs(wl)


def reference_convention_flops(wl: Workload) -> float:
    """The reference bench's figure: ``H * (Dqk + Dv) * sum n_b^2`` (``hstu_attention_bench.py:38-62``),
    scaled by ``delta_size / max_seq_len`` in delta mode (lines 387-388)."""
    n2 = float((wl.lengths.astype(np.float64) ** 2).sum())
    fl = wl.heads * (wl.dqk + wl.dv) * n2
    if wl.delta_size > 0:
        fl = fl / wl.max_seq_len * wl.delta_size
    return fl


def algorithmic_bytes(wl: Workload) -> float:
    """Every operand touched once: q, k, v read, out written, plus the index arrays."""
    elt = 1 if wl.dtype == "fp8" else 2
    out_elt = 2
    b = elt * wl.heads * (wl.total_q * wl.dqk + wl.total_kv * (wl.dqk + wl.dv))
    b += out_elt * wl.heads * wl.total_q * wl.dv
    b += 8 * (wl.batch + 1) + (8 * wl.batch if wl.num_targets is not None else 0)
    return float(b)


def make_workload(name: str) -> Workload:
    """The benchmark configurations by name: ``cfg1`` .. ``cfg5``, ``headline``, ``ragged8k``, ``refbench_<N>``, ``refbench_delta_<N>``."""
    if name == "cfg1":
        rng = np.random.default_rng(1001)
        return Workload(name, 8, 2, 32, 32, 128, rng.integers(16, 129, size=8), dtype="fp32", seed=1001)
    if name == "cfg2":
        rng = np.random.default_rng(1002)
        return Workload(name, 256, 4, 128, 128, 1024, rng.integers(64, 1025, size=256), seed=1002)
    if name == "cfg3":
        rng = np.random.default_rng(1003)
        c = 6
        n = np.clip(rng.zipf(1.2, size=64), 256, 8192).astype(np.int64)
        t = np.minimum(rng.integers(1, 513, size=64), n - c - 1)
        return Workload(
            name, 64, 4, 128, 128, 8192, n, num_targets=t, max_attn_len=2048, contextual_seq_len=c, seed=1003
        )
    if name == "headline":
        return Workload(name, 64, 4, 128, 128, 8192, np.full(64, 8192, dtype=np.int64), seed=1000)
    if name == "ragged8k":
        # the headline's shape with unequal lengths (uniform in 1024..8192, plain causal): same kernel, but the work goes
        # through the ranking, the work lists and the per-XCD counters instead of the arithmetic deal of an equal-length batch
        rng = np.random.default_rng(1006)
        return Workload(name, 64, 4, 128, 128, 8192, rng.integers(1024, 8193, size=64).astype(np.int64), seed=1006)
    if name.startswith("ragged_"):
        # ragged_<lo>_<hi>[_<B>]: the headline's shape (H = 4, d = 128, bf16, plain causal) with B (default 64) lengths
        # uniform in lo..hi; for looking at the kernel choice between batch shapes
        parts = [int(x) for x in name.split("_")[1:]]
        lo, hi, batch = parts[0], parts[1], (parts[2] if len(parts) > 2 else 64)
        rng = np.random.default_rng(1007)
        return Workload(name, batch, 4, 128, 128, hi, rng.integers(lo, hi + 1, size=batch).astype(np.int64), seed=1007)
    if name == "cfg4":
        rng = np.random.default_rng(1004)
        hist = rng.integers(1024, 4097, size=32)
        return Workload(
            name,
            32,
            4,
            128,
            128,
            4096 + 256,
            hist + 256,
            num_targets=np.full(32, 256, dtype=np.int64),
            delta_size=256,
            seed=1004,
        )
    if name == "cfg5":
        rng = np.random.default_rng(1005)
        n = rng.integers(4096, 16385, size=16)
        t = rng.integers(64, 257, size=16)
        return Workload(name, 16, 8, 128, 128, 16384, n, num_targets=t, dtype="fp8", seed=1005)
    if name.startswith("refbench_"):
        # the recipe of the reference's own benchmark (ops/benchmarks/hstu_attention_bench.py:65-93, 217-271): B = 512,
        # H = 4, d = 128, lengths from generate_sparse_seq_len(sparsity 0.95) + apply_sampling(alpha 2.0), 1..20 targets
        # per sequence, alpha = 1 / d, inputs uniform in +-0.01, q/k/v column slices of one buffer; refbench_<N> for
        # max_seq_len N (the reference sweeps N = 256 .. 4096 by default)
        from .common import apply_sampling, generate_sparse_seq_len

        # refbench_delta_<N>: its --has-delta-q form (:229-232): every length grows by delta_size = 256, which are the
        # targets and the only query rows; delta_q uniform in +-0.1 as the inputs of that form are (:253-257, where
        # q/k/v keep +-0.01; here one amplitude serves all three, the timing does not depend on it)
        delta = name.startswith("refbench_delta_")
        N = int(name.rsplit("_", 1)[1])
        with torch.random.fork_rng(devices=[]):
            torch.manual_seed(1001)
            lengths = generate_sparse_seq_len(size=512, max_seq_len=N, sparsity=0.95, device=torch.device("cpu"))
            lengths = apply_sampling(lengths, 2.0, max_seq_len=N)
            t = torch.randint(1, 21, (512,), dtype=lengths.dtype)
            t = torch.where(t > lengths, lengths, t)
        if delta:
            return Workload(name, 512, 4, 128, 128, N + 256, lengths.numpy().astype(np.int64) + 256,
                            num_targets=np.full(512, 256, dtype=np.int64), delta_size=256, alpha=1.0 / 128, seed=1001,
                            extra={"uniform": 0.01, "fused_buffer": 1.0})
        return Workload(name, 512, 4, 128, 128, N, lengths.numpy().astype(np.int64), num_targets=t.numpy().astype(np.int64),
                        alpha=1.0 / 128, seed=1001, extra={"uniform": 0.01, "fused_buffer": 1.0})
    raise ValueError(f"unknown workload {name!r}")


WORKLOADS: List[str] = ["cfg1", "cfg2", "cfg3", "headline", "cfg4", "cfg5"]


def make_inputs(wl: Workload, device: torch.device, dtype: Optional[torch.dtype] = None, fused_buffer: bool = False):
    """Random q, k, v ~ N(0, 1) * 0.1 (seeded), int64 ``seq_offsets`` and ``num_targets`` on ``device``.

    With ``fused_buffer`` q/k/v are column slices of one ``[L, H, 2*Dqk+Dv]`` tensor, the layout the
    reference's callers produce (``hstu_compute.py:90-103``); delta mode always draws a dense ``delta_q``.
    Returns a dict; fp8 workloads return bf16 tensors (quantisation is the caller's step).
    """
    if dtype is None:
        dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32, "fp8": torch.bfloat16}[wl.dtype]
    L = wl.total_kv
    fused_buffer = fused_buffer or bool(wl.extra.get("fused_buffer"))
    if L * wl.heads * (2 * wl.dqk + wl.dv) > (1 << 29) and device.type != "cpu":
        gen = torch.Generator(device=device)  # large workloads are drawn on the device
        where = device
    else:
        gen, where = torch.Generator(device="cpu"), torch.device("cpu")
    gen.manual_seed(wl.seed)

    def draw(*shape):
        if "uniform" in wl.extra:
            a = float(wl.extra["uniform"])
            return (torch.rand(shape, generator=gen, device=where) * (2 * a) - a).to(dtype).to(device)
        return (torch.randn(shape, generator=gen, device=where) * 0.1).to(dtype).to(device)

    if fused_buffer:
        x = draw(L, wl.heads, 2 * wl.dqk + wl.dv)
        q, k, v = torch.split(x, [wl.dqk, wl.dqk, wl.dv], dim=-1)
    else:
        q, k, v = draw(L, wl.heads, wl.dqk), draw(L, wl.heads, wl.dqk), draw(L, wl.heads, wl.dv)
    if wl.delta_size > 0:
        q = draw(wl.batch * wl.delta_size, wl.heads, wl.dqk)
    offsets = torch.zeros(wl.batch + 1, dtype=torch.int64)
    offsets[1:] = torch.from_numpy(np.cumsum(wl.lengths.astype(np.int64)))
    nt = None if wl.num_targets is None else torch.from_numpy(wl.num_targets.astype(np.int64)).to(device)
    return {"q": q, "k": k, "v": v, "seq_offsets": offsets.to(device), "num_targets": nt}
