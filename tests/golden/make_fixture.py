"""Regenerates ``small_cases.npz`` from the scalar C checker (``oracle/hstu_ref.c``).

Run from the repository root: ``python tests/golden/make_fixture.py``.  Inputs are stored as bfloat16 bit
patterns (int16), so the same bytes feed the fp32 oracle (after widening) and the bf16 kernels.
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import c_ref  # noqa: E402

CASES = [
    # name, lengths, H, D, N, targets, w, c, f, delta
    ("causal_d32", [16, 128, 57, 1, 0, 33], 1, 32, 128, None, 0, 0, 0, 0),
    ("targets_window_ctx_d64", [70, 9, 41, 100], 1, 64, 140, [5, 2, 20, 1], 11, 3, 0, 0),
    ("min_full_d128", [66, 33], 1, 128, 160, [10, 3], 7, 2, 4, 0),
    ("delta_d128", [70, 40], 1, 128, 128, [8, 8], 0, 0, 0, 8),
    ("delta_window_ctx_d32", [90, 36, 64], 1, 32, 96, [12, 12, 12], 9, 4, 0, 12),
]


def main() -> None:
    out = {}
    for i, (name, lengths, H, D, N, targets, w, c, f, delta) in enumerate(CASES):
        g = torch.Generator().manual_seed(4000 + i)
        lengths_t = torch.tensor(lengths, dtype=torch.int64)
        offs = torch.zeros(len(lengths) + 1, dtype=torch.int64)
        offs[1:] = torch.cumsum(lengths_t, 0)
        L = int(offs[-1])
        Lq = len(lengths) * delta if delta > 0 else L
        q = (torch.randn((Lq, H, D), generator=g) * 0.1).to(torch.bfloat16).float()
        k = (torch.randn((L, H, D), generator=g) * 0.1).to(torch.bfloat16).float()
        v = (torch.randn((L, H, D), generator=g) * 0.1).to(torch.bfloat16).float()
        t = None if targets is None else torch.tensor(targets, dtype=torch.int64)
        alpha = 1.0 / D**0.5
        ref = c_ref.fwd(N, alpha, q, k, v, offs, t, w, c, f, delta)
        out[f"{name}.q"] = q.to(torch.bfloat16).view(torch.int16).numpy()
        out[f"{name}.k"] = k.to(torch.bfloat16).view(torch.int16).numpy()
        out[f"{name}.v"] = v.to(torch.bfloat16).view(torch.int16).numpy()
        out[f"{name}.offsets"] = offs.numpy()
        out[f"{name}.targets"] = np.array([-1]) if t is None else t.numpy()
        out[f"{name}.params"] = np.array([N, w, c, f, delta], dtype=np.int64)
        out[f"{name}.alpha"] = np.array([alpha], dtype=np.float64)
        out[f"{name}.out"] = ref.numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "small_cases.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
