"""Regenerates ``side_cases.npz``: small frozen cases for the rows either side of the attention forward -- the
backward, ``hstu_compute_uqvk`` and ``hstu_compute_output`` -- from the fp64 statements under ``oracle/``.

Run from the repository root: ``python tests/golden/make_side_fixture.py``.  Inputs are stored as bfloat16 bit patterns
(int16), so the same bytes feed the oracles (after widening) and the bf16 kernels; expected outputs are float32 roundings of fp64 results.
The gradients come from autograd through the dense restatement of the forward (``bwd_oracle.autograd_grads``), the
independent statement, so that the closed form used elsewhere in the tests is checked against frozen numbers too.
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import bwd_oracle, output_oracle, uqvk_oracle  # noqa: E402


def bits(x: torch.Tensor) -> np.ndarray:
    return x.to(torch.bfloat16).view(torch.int16).numpy()


def main() -> None:
    out = {}
    # ---- backward: two mask settings
    for i, (lengths, H, dqk, dv, N, targets, w, c) in enumerate(
        [([37, 1, 64, 20], 2, 32, 16, 64, None, 0, 0), ([50, 33, 70], 1, 64, 64, 72, [4, 30, 9], 9, 3)]
    ):
        g = torch.Generator().manual_seed(7000 + i)
        offs = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int64)
        L = int(offs[-1])
        q, k = [(torch.randn((L, H, dqk), generator=g) * 0.5).to(torch.bfloat16) for _ in range(2)]
        v, dout = [(torch.randn((L, H, dv), generator=g) * 0.5).to(torch.bfloat16) for _ in range(2)]
        t = None if targets is None else torch.tensor(targets, dtype=torch.int64)
        alpha = 1.0 / dqk**0.5
        dq, dk, dvv = bwd_oracle.autograd_grads(N, alpha, q, k, v, offs, dout, num_targets=t, max_attn_len=w, contextual_seq_len=c)
        p = f"bwd{i}_"
        out.update({p + "q": bits(q), p + "k": bits(k), p + "v": bits(v), p + "dout": bits(dout), p + "offsets": offs.numpy(),
                    p + "targets": np.zeros(0, dtype=np.int64) if t is None else t.numpy(),
                    p + "params": np.array([N, w, c], dtype=np.int64), p + "alpha": np.array([alpha]),
                    p + "dq": dq.float().numpy(), p + "dk": dk.float().numpy(), p + "dv": dvv.float().numpy()})
    # ---- uqvk and output: one case each (the output case with the flags the reference's STU layer passes)
    g = torch.Generator().manual_seed(7100)
    L, d_model, H, attn, hidden = 45, 128, 2, 32, 32
    n_out = (2 * hidden + 2 * attn) * H
    x = (torch.randn((L, d_model), generator=g) * 1.5 + 0.3).to(torch.bfloat16)
    nw, nb = (1 + 0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16), (0.1 * torch.randn(d_model, generator=g)).to(torch.bfloat16)
    w_, b_ = (torch.randn((d_model, n_out), generator=g) / d_model**0.5).to(torch.bfloat16), (0.1 * torch.randn(n_out, generator=g)).to(torch.bfloat16)
    u, q, k, v = uqvk_oracle.compute_uqvk(x.double(), nw.double(), nb.double(), 1e-6, H, attn, hidden, w_.double(), b_.double())
    out.update({"uqvk_x": bits(x), "uqvk_nw": bits(nw), "uqvk_nb": bits(nb), "uqvk_w": bits(w_), "uqvk_b": bits(b_),
                "uqvk_dims": np.array([H, attn, hidden], dtype=np.int64), "uqvk_u": u.float().numpy(), "uqvk_q": q.float().numpy(),
                "uqvk_k": k.float().numpy(), "uqvk_v": v.float().numpy()})
    D = H * hidden
    attn_t, u_t = [(torch.rand((L, D), generator=g) * 0.2 - 0.1).to(torch.bfloat16) for _ in range(2)]
    x2 = (torch.rand((L, d_model), generator=g) * 0.2 - 0.1).to(torch.bfloat16)
    ow, ob = [(torch.rand(D, generator=g) * 0.2 - 0.1).to(torch.bfloat16) for _ in range(2)]
    wo = (torch.rand((3 * D, d_model), generator=g) * 0.2 - 0.1).to(torch.bfloat16)
    res = output_oracle.compute_output(attn_t.double(), u_t.double(), x2.double(), ow.double(), ob.double(), wo.double(), 1e-6,
                                       concat_u=True, concat_x=True, num_heads=H, linear_dim=hidden).double()
    out.update({"out_attn": bits(attn_t), "out_u": bits(u_t), "out_x": bits(x2), "out_nw": bits(ow), "out_nb": bits(ob), "out_w": bits(wo),
                "out_dims": np.array([H, hidden], dtype=np.int64), "out_result": res.float().numpy()})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "side_cases.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
