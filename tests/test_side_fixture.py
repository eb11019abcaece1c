"""Frozen cases for the backward, hstu_compute_uqvk and hstu_compute_output (tests/golden/side_cases.npz): the fp32
oracles and the closed-form gradients against the stored fp64 results on the CPU, the HIP kernels against them on the
GPU.  Tolerances: oracles 1e-4 relative Frobenius (fp32 against fp64); kernels as in the parity tests (relative
Frobenius <= 1e-2, max-abs <= 2e-2 * max|ref|)."""

import os

import numpy as np
import pytest
import torch

from oracle import bwd_oracle, output_oracle, uqvk_oracle

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "side_cases.npz")


def _bf16(a):
    return torch.from_numpy(a.copy()).view(torch.bfloat16)


def _rel(got, ref):
    got, ref = got.double(), torch.as_tensor(ref).double()
    return float((got - ref).norm() / ref.norm()), float((got - ref).abs().max() / ref.abs().max())


def _bwd_case(z, i):
    p = f"bwd{i}_"
    N, w, c = (int(x) for x in z[p + "params"])
    t = z[p + "targets"]
    kw = dict(num_targets=None if t.size == 0 else torch.from_numpy(t.copy()), max_attn_len=w, contextual_seq_len=c)
    tensors = [_bf16(z[p + n]) for n in ("q", "k", "v", "dout")]
    return N, float(z[p + "alpha"][0]), tensors, torch.from_numpy(z[p + "offsets"].copy()), kw, [z[p + n] for n in ("dq", "dk", "dv")]


def test_oracles_reproduce_the_fixture():
    z = np.load(FIXTURE)
    for i in range(2):
        N, alpha, (q, k, v, dout), offs, kw, want = _bwd_case(z, i)
        got = bwd_oracle.closed_form_grads(N, alpha, q, k, v, offs, dout, **kw)
        for g_, w_ in zip(got, want):
            assert _rel(g_, w_)[0] <= 1e-4
    H, attn, hidden = (int(x) for x in z["uqvk_dims"])
    got = uqvk_oracle.compute_uqvk(_bf16(z["uqvk_x"]), _bf16(z["uqvk_nw"]), _bf16(z["uqvk_nb"]), 1e-6, H, attn, hidden, _bf16(z["uqvk_w"]),
                                   _bf16(z["uqvk_b"]))
    for g_, name in zip(got, ("uqvk_u", "uqvk_q", "uqvk_k", "uqvk_v")):
        assert _rel(g_, z[name])[0] <= 1e-4, name
    H, ld = (int(x) for x in z["out_dims"])
    got = output_oracle.compute_output(_bf16(z["out_attn"]), _bf16(z["out_u"]), _bf16(z["out_x"]), _bf16(z["out_nw"]), _bf16(z["out_nb"]),
                                       _bf16(z["out_w"]), 1e-6, concat_u=True, concat_x=True, num_heads=H, linear_dim=ld)
    assert _rel(got, z["out_result"])[0] <= 1e-4


@pytest.mark.gpu
def test_kernels_reproduce_the_fixture():
    import __graft_entry__

    pkg = __graft_entry__.load_package()
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    dev = torch.device("cuda:0")
    z = np.load(FIXTURE)
    for i in range(2):
        print(f"[case] side fixture bwd{i}", flush=True)
        N, alpha, (q, k, v, dout), offs, kw, want = _bwd_case(z, i)
        qd, kd, vd = (t.to(dev).requires_grad_() for t in (q, k, v))
        dkw = {a: (b.to(dev) if torch.is_tensor(b) else b) for a, b in kw.items()}
        pkg.hstu_mha(N, alpha, qd, kd, vd, offs.to(dev), **dkw).backward(dout.to(dev))
        torch.cuda.synchronize()
        for g_, w_ in zip((qd.grad, kd.grad, vd.grad), want):
            rel, worst = _rel(g_.cpu(), w_)
            assert rel <= 1e-2 and worst <= 2e-2, (i, rel, worst)
    print("[case] side fixture uqvk / output", flush=True)
    H, attn, hidden = (int(x) for x in z["uqvk_dims"])
    got = pkg.hstu_compute_uqvk(*(_bf16(z[n]).to(dev) for n in ("uqvk_x", "uqvk_nw", "uqvk_nb")), 1e-6, H, attn, hidden,
                                _bf16(z["uqvk_w"]).to(dev), _bf16(z["uqvk_b"]).to(dev))
    for g_, name in zip(got, ("uqvk_u", "uqvk_q", "uqvk_k", "uqvk_v")):
        rel, worst = _rel(g_.cpu(), z[name])
        assert rel <= 1e-2 and worst <= 2e-2, (name, rel, worst)
    H, ld = (int(x) for x in z["out_dims"])
    got = pkg.hstu_compute_output(*(_bf16(z[n]).to(dev) for n in ("out_attn", "out_u", "out_x", "out_nw", "out_nb")), 1e-6,
                                  _bf16(z["out_w"]).to(dev), H, ld, 0.0, False, True, True, "none", False, False)
    rel, worst = _rel(got.cpu(), z["out_result"])
    assert rel <= 1e-2 and worst <= 2e-2, (rel, worst)
