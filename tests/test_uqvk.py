"""hstu_compute_uqvk: the oracle against independent statements on the CPU, the HIP / hipBLASLt path against the
oracle on the GPU.  Tolerance for bf16 / fp16 results (rounded once at the end, fp32 accumulation): relative
Frobenius error <= 1e-2 and max-abs error <= 2e-2 * max|ref| against the fp32 oracle."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import uqvk_oracle as U

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _inputs(seed, L, d_model, H, attn, hidden, dtype):
    g = torch.Generator().manual_seed(seed)
    n_out = (2 * hidden + 2 * attn) * H
    x = (torch.randn((L, d_model), generator=g) * 1.5 + 0.3).to(dtype)
    nw = (1.0 + 0.1 * torch.randn(d_model, generator=g)).to(dtype)
    nb = (0.1 * torch.randn(d_model, generator=g)).to(dtype)
    w = (torch.randn((d_model, n_out), generator=g) / d_model**0.5).to(dtype)
    b = (0.1 * torch.randn(n_out, generator=g)).to(dtype)
    return x, nw, nb, w, b


# ---------------------------------------------------------------- oracle, CPU


def test_oracle_layer_norm_matches_the_formula_written_out():
    x, nw, nb, _, _ = _inputs(1, 37, 96, 2, 8, 8, torch.float32)
    got = U.layer_norm(x, nw, nb, 1e-6).double()
    assert torch.allclose(got, U.layer_norm_by_hand(x, nw, nb, 1e-6), atol=1e-5)
    # a layer norm does not see a positive rescaling or a shift of its input
    assert torch.allclose(U.layer_norm(3.0 * x + 7.0, nw, nb, 1e-9).double(), got, atol=1e-4)


def test_oracle_uqvk_against_pieces_written_by_hand():
    L, d, H, attn, hidden = 21, 64, 3, 8, 16
    x, nw, nb, w, b = _inputs(2, L, d, H, attn, hidden, torch.float32)
    u, q, k, v = U.compute_uqvk(x, nw, nb, 1e-6, H, attn, hidden, w, b)
    full = U.layer_norm_by_hand(x, nw, nb, 1e-6) @ w.double() + b.double()
    hu, ha = hidden * H, attn * H
    zu = full[:, :hu]
    assert torch.allclose(u.double(), zu / (1 + torch.exp(-zu)), atol=1e-4)
    assert torch.allclose(v.double(), full[:, hu : 2 * hu].reshape(L, H, hidden), atol=1e-4)
    assert torch.allclose(q.double(), full[:, 2 * hu : 2 * hu + ha].reshape(L, H, attn), atol=1e-4)
    assert torch.allclose(k.double(), full[:, 2 * hu + ha :].reshape(L, H, attn), atol=1e-4)
    assert float(F.silu(torch.tensor(0.0))) == 0.0 and abs(float(F.silu(torch.tensor(30.0))) - 30.0) < 1e-6


def test_uqvk_library_exports_and_struct_mirror():
    import __graft_entry__

    __graft_entry__.load_package()
    from generative_recommenders_amd.ops import hstu_compute as hc

    header = open(os.path.join(ROOT, "include", "hstu_linear.h")).read()
    declared = set(re.findall(r"\b(hstu_(?:uqvk|output|linear)_\w+)\s*\(", re.sub(r"/\*.*?\*/", "", header, flags=re.S)))
    assert declared == set(hc.EXPORTS)
    L = hc.lib()
    for name in hc.EXPORTS:
        assert hasattr(L, name)
    for struct, mirror in (("HstuUqvkArgs", hc.HstuUqvkArgs), ("HstuOutputArgs", hc.HstuOutputArgs)):
        body = header[header.index("typedef struct %s {" % struct) : header.index("} %s;" % struct)]
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S).replace("typedef struct %s {" % struct, "")
        names = []
        for decl in body.split(";"):
            decl = decl.strip()
            if decl:
                parts = decl.split(",")
                names.append(re.findall(r"(\w+)\s*$", parts[0].strip())[0])
                names += [p.strip() for p in parts[1:]]
        assert names == [f[0] for f in mirror._fields_], struct
    # validation happens before anything touches the device
    assert L.hstu_uqvk_forward(None, None) == -1
    a = hc.HstuUqvkArgs()
    a.rows, a.d_model, a.heads, a.attn_dim, a.hidden_dim = 4, 64, 2, 8, 8
    assert L.hstu_uqvk_forward(ctypes.byref(a), None) == -1  # pointers missing
    a.heads = 0
    assert L.hstu_uqvk_forward(ctypes.byref(a), None) == -5
    assert L.hstu_uqvk_layer_norm(None, 64, None, None, 1e-5, None, 64, 4, 60, 0, None) == -5  # d_model not a multiple of 8
    assert L.hstu_uqvk_layer_norm(None, 64, None, None, 1e-5, None, 64, 0, 64, 0, None) == 0
    assert L.hstu_output_forward(None, None) == -1
    o = hc.HstuOutputArgs()
    o.rows, o.d_out, o.heads, o.linear_dim = 4, 64, 2, 32
    assert L.hstu_output_forward(ctypes.byref(o), None) == -5  # residual row stride below d_out
    o.x_row_stride = 64
    assert L.hstu_output_forward(ctypes.byref(o), None) == -1  # pointers missing
    o.attn_row_stride = o.u_row_stride = 64
    o.group_norm, o.linear_dim = 1, 24  # 3 chunks per head: not a power of two
    assert L.hstu_output_norm_mul(ctypes.byref(o), None, 48, None) == -6
    o.group_norm, o.linear_dim, o.rows = 0, 32, 0
    assert L.hstu_output_norm_mul(ctypes.byref(o), None, 64, None) == 0
    assert L.hstu_output_workspace_bytes(ctypes.byref(o)) == 0
    o.rows, o.concat_u, o.concat_x = 4, 1, 1
    assert L.hstu_output_workspace_bytes(ctypes.byref(o)) == 4 * 3 * 64 * 2 + (64 << 20)
    src = open(os.path.join(ROOT, "generative-recommenders_amd", "ops", "hstu_compute.py")).read()
    assert "oracle" not in src


# ---------------------------------------------------------------- GPU


@pytest.fixture(scope="module")
def pkg():
    import __graft_entry__

    __graft_entry__.load_package()
    from generative_recommenders_amd.ops import hstu_compute

    return hstu_compute


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


def _close(got, ref, what):
    got, ref = got.float().cpu(), ref.float()
    assert got.shape == ref.shape, f"{what}: {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), what
    rel = float((got - ref).norm() / ref.norm())
    worst = float((got - ref).abs().max()) / float(ref.abs().max())
    assert rel <= 1e-2 and worst <= 2e-2, f"{what}: relative {rel:.3e}, max-abs / max|ref| {worst:.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,d_model", [(1, 64), (130, 512), (1000, 128), (77, 1024), (5, 4096), (64, 8)])
def test_layer_norm_kernel(pkg, dev, L, d_model, dtype):
    print(f"[case] layer norm {L} {d_model} {dtype}", flush=True)
    x, nw, nb, _, _ = _inputs(L + d_model, L, d_model, 1, 8, 8, dtype)
    got = pkg.layer_norm(x.to(dev), nw.to(dev), nb.to(dev), 1e-6)
    torch.cuda.synchronize()
    _close(got, U.layer_norm_by_hand(x, nw, nb, 1e-6), "layer norm")
    wide = torch.cat([x, x], dim=1).to(dev)  # a column slice: row stride != width
    got2 = pkg.layer_norm(wide[:, :d_model], nw.to(dev), nb.to(dev), 1e-6)
    torch.cuda.synchronize()
    assert torch.equal(got2, got)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("path", [0, 1])
@pytest.mark.parametrize(
    "L,d_model,H,attn,hidden",
    # the first five shapes qualify for the fused kernel (d_model in 128..512 by 128, hidden * H and n_out multiples of 128)
    [(300, 512, 4, 128, 128), (1000, 128, 2, 32, 64), (257, 256, 4, 64, 32), (1, 384, 1, 64, 128), (2049, 512, 2, 64, 64),
     (1, 64, 1, 16, 16), (130, 512, 3, 16, 32), (77, 192, 2, 64, 64)],
)
def test_compute_uqvk(pkg, dev, L, d_model, H, attn, hidden, dtype, path):
    """Against the fp32 oracle, and tightly against the oracle with the reference's one intermediate rounding (the
    normalised x in the input type); `path` 0 lets the library choose (fused kernel where the shape allows), 1 forces
    the layer-norm kernel + hipBLASLt."""
    print(f"[case] uqvk {L} {d_model} {H} {attn} {hidden} {dtype} path={path}", flush=True)
    x, nw, nb, w, b = _inputs(L + d_model + attn, L, d_model, H, attn, hidden, dtype)
    fused_shape = d_model in (128, 256, 384, 512) and (hidden * H) % 128 == 0 and ((2 * hidden + 2 * attn) * H) % 128 == 0
    if path == 0 and fused_shape:
        path = 2  # the automatic choice must be the fused kernel here: asking for it explicitly may not fail
    if path == 0 and not fused_shape:
        with pytest.raises(NotImplementedError):
            pkg.hstu_compute_uqvk(x.to(dev), nw.to(dev), nb.to(dev), 1e-6, H, attn, hidden, w.to(dev), b.to(dev), path=2)
    u, q, k, v = pkg.hstu_compute_uqvk(x.to(dev), nw.to(dev), nb.to(dev), 1e-6, H, attn, hidden, w.to(dev), b.to(dev), path=path)
    torch.cuda.synchronize()
    assert u.shape == (L, hidden * H) and q.shape == (L, H, attn) and k.shape == (L, H, attn) and v.shape == (L, H, hidden)
    assert u.dtype == dtype and q.stride(2) == 1 and (L == 1 or q.stride(0) == (2 * hidden + 2 * attn) * H)
    for name, got, ref in zip("uqkv", (u, q, k, v), U.compute_uqvk(x, nw, nb, 1e-6, H, attn, hidden, w, b)):
        _close(got, ref, name)
    for name, got, ref in zip("uqkv", (u, q, k, v), U.compute_uqvk(x, nw, nb, 1e-6, H, attn, hidden, w, b, round_normed_to=dtype)):
        got, ref = got.float().cpu(), ref.float()
        assert float((got - ref).norm() / ref.norm()) <= 4e-3, name


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "L,d_model,H,attn,hidden",
    [(700, 1024, 4, 128, 128), (1, 64, 2, 128, 128), (300, 512, 4, 128, 128), (5000, 768, 2, 128, 128), (1025, 1024, 8, 64, 64)],
)
def test_compute_uqvk_hand_written_gemm(pkg, dev, L, d_model, H, attn, hidden, dtype):
    """``path=3``: the layer-norm kernel, then the GEMM kernel of the output projection in its bias / SiLU form (the bias
    as the start of the sums, SiLU on the u columns in the epilogue), on request only.  Same bar as the other paths."""
    print(f"[case] uqvk gemm {L} {d_model} {H} {attn} {hidden} {dtype}", flush=True)
    x, nw, nb, w, b = _inputs(L + d_model + 3, L, d_model, H, attn, hidden, dtype)
    dv = [t.to(dev) for t in (x, nw, nb, w, b)]
    got = pkg.hstu_compute_uqvk(dv[0], dv[1], dv[2], 1e-6, H, attn, hidden, dv[3], dv[4], path=3)
    lib = pkg.hstu_compute_uqvk(dv[0], dv[1], dv[2], 1e-6, H, attn, hidden, dv[3], dv[4], path=1)
    torch.cuda.synchronize()
    for name, g_, l_, ref in zip("uqkv", got, lib, U.compute_uqvk(x, nw, nb, 1e-6, H, attn, hidden, w, b)):
        _close(g_, ref, name + " vs fp32 oracle")
        _close(g_, l_.float().cpu(), name + " vs library path")


@pytest.mark.gpu
def test_uqvk_with_a_total_length_that_changes_from_batch_to_batch(pkg, dev):
    """The hipBLASLt path keeps one plan per size class of the row count, not per row count: lengths of one class
    (1100, 1101, 1279), of others (640, 5000), and the first again, each against the oracle."""
    d_model, H, attn, hidden = 192, 2, 64, 64  # no fused kernel for this d_model: layer-norm kernel + hipBLASLt
    for L in (1100, 1101, 1279, 640, 5000, 1100, 1):
        print(f"[case] uqvk changing rows {L}", flush=True)
        x, nw, nb, w, b = _inputs(L, L, d_model, H, attn, hidden, torch.bfloat16)
        got = pkg.hstu_compute_uqvk(x.to(dev), nw.to(dev), nb.to(dev), 1e-6, H, attn, hidden, w.to(dev), b.to(dev), path=1)
        torch.cuda.synchronize()
        for name, g_, ref in zip("uqkv", got, U.compute_uqvk(x, nw, nb, 1e-6, H, attn, hidden, w, b)):
            _close(g_, ref, f"{name} at {L} rows")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("L,d_model,H,attn,hidden", [(300, 512, 4, 128, 128), (1000, 128, 2, 32, 64), (2049, 512, 2, 64, 64), (1, 384, 1, 64, 128)])
def test_uqvk_fp8_epilogue(pkg, dev, L, d_model, H, attn, hidden, dtype):
    """The fused kernel's e4m3 copy of v | q | k: byte-equal to e4m3(rounded value * (1 / scale)) clamped to +-448 (scales
    from this batch's own maxima, and a quarter of them so that the clamp is exercised); the maxima it reports are exact;
    u and the 16-bit q, k, v are what the plain call returns; the bytes feed the fp8 attention in place."""
    import __graft_entry__

    top = __graft_entry__.load_package()
    print(f"[case] uqvk fp8 epilogue {L} {d_model} {H} {attn} {hidden} {dtype}", flush=True)
    x, nw, nb, w, b = _inputs(L + d_model + attn + 5, L, d_model, H, attn, hidden, dtype)
    dv = [t.to(dev) for t in (x, nw, nb, w, b)]
    u, q, k, v = pkg.hstu_compute_uqvk(dv[0], dv[1], dv[2], 1e-6, H, attn, hidden, dv[3], dv[4])
    want_max = torch.stack([v.float().abs().max(), q.float().abs().max(), k.float().abs().max()])
    for shrink in (1.0, 0.25):
        vs, qs, ks = (float(m) / 448.0 * shrink for m in want_max)
        u8, q8, k8, v8, absmax = pkg.hstu_compute_uqvk_fp8(dv[0], dv[1], dv[2], 1e-6, H, attn, hidden, dv[3], dv[4], qs, ks, vs)
        torch.cuda.synchronize()
        assert torch.equal(u8, u)
        assert torch.equal(absmax, want_max), (absmax, want_max)
        for name, got, src, scale in (("q", q8, q, qs), ("k", k8, k, ks), ("v", v8, v, vs)):
            assert got.dtype == torch.float8_e4m3fn and got.shape == src.shape
            inv = float(np.float32(1.0) / np.float32(scale))
            ref = (src.float().cpu() * inv).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
            assert torch.equal(got.cpu().view(torch.uint8), ref.view(torch.uint8)), f"{name} at shrink {shrink}"
    if L >= 300:  # the bytes where they are, as the attention's operands
        n = L // 3
        offs = torch.tensor([0, n, n, L], dtype=torch.int64, device=dev)
        vs, qs, ks = (float(m) / 448.0 for m in want_max)
        u8, q8, k8, v8, _ = pkg.hstu_compute_uqvk_fp8(dv[0], dv[1], dv[2], 1e-6, H, attn, hidden, dv[3], dv[4], qs, ks, vs)
        out8 = top.hstu_mha(L, 1.0 / attn**0.5, q8, k8, v8, offs, q_scale=qs, k_scale=ks, v_scale=vs)
        out16 = top.hstu_mha(L, 1.0 / attn**0.5, q, k, v, offs)
        torch.cuda.synchronize()
        a, c = out8.float().flatten(), out16.float().flatten()
        assert float(torch.dot(a, c) / (a.norm() * c.norm())) >= 0.995


@pytest.mark.gpu
def test_uqvk_fp8_epilogue_needs_the_fused_kernel(pkg, dev):
    x, nw, nb, w, b = _inputs(3, 77, 192, 2, 64, 64, torch.bfloat16)
    with pytest.raises(NotImplementedError):
        pkg.hstu_compute_uqvk_fp8(x.to(dev), nw.to(dev), nb.to(dev), 1e-6, 2, 64, 64, w.to(dev), b.to(dev), 1.0, 1.0, 1.0)


@pytest.mark.gpu
def test_uqvk_feeds_attention_in_place(pkg, dev):
    """q, k, v are column slices of the projection's output; hstu_mha reads them where they are."""
    import __graft_entry__
    from oracle import hstu_oracle as O

    top = __graft_entry__.load_package()
    print("[case] uqvk -> hstu_mha", flush=True)
    lengths = [200, 0, 64, 37]
    offs = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int64)
    L, d_model, H, D = int(offs[-1]), 256, 2, 64
    x, nw, nb, w, b = _inputs(99, L, d_model, H, D, D, torch.bfloat16)
    u, q, k, v = pkg.hstu_compute_uqvk(x.to(dev), nw.to(dev), nb.to(dev), 1e-6, H, D, D, w.to(dev), b.to(dev))
    out = top.hstu_mha(200, 0.125, q, k, v, offs.to(dev))
    torch.cuda.synchronize()
    ref = O.hstu_mha_per_sequence(200, 0.125, q.float().cpu(), k.float().cpu(), v.float().cpu(), offs)
    err = float((out.float().cpu() - ref).norm() / ref.norm())
    assert err <= 1e-2, err


@pytest.mark.gpu
def test_uqvk_takes_parameters_that_are_slices_of_larger_tensors(pkg, dev):
    """Weights that start in the middle of a larger allocation (not 16-byte aligned) and x as a column slice."""
    L, d_model, H, attn, hidden = 200, 256, 2, 64, 64
    x, nw, nb, w, b = _inputs(9, L, d_model, H, attn, hidden, torch.bfloat16)
    want = pkg.hstu_compute_uqvk(x.to(dev), nw.to(dev), nb.to(dev), 1e-6, H, attn, hidden, w.to(dev), b.to(dev))
    pad = torch.zeros(3, dtype=torch.bfloat16)
    nw2, nb2, b2 = (torch.cat([pad, t]).to(dev)[3:] for t in (nw, nb, b))
    x2 = torch.cat([x, x], dim=1).to(dev)[:, d_model:]
    print("[case] uqvk sliced parameters", flush=True)
    got = pkg.hstu_compute_uqvk(x2, nw2, nb2, 1e-6, H, attn, hidden, w.to(dev), b2)
    torch.cuda.synchronize()
    for g_, w_ in zip(got, want):
        assert torch.equal(g_, w_)


@pytest.mark.gpu
def test_uqvk_wrapper_rejections(pkg, dev):
    x, nw, nb, w, b = [t.to(dev) for t in _inputs(5, 16, 64, 2, 8, 8, torch.bfloat16)]
    with pytest.raises(AssertionError, match="uvqk_weight must be"):
        pkg.hstu_compute_uqvk(x, nw, nb, 1e-6, 2, 8, 16, w, b)
    with pytest.raises(RuntimeError):
        pkg.hstu_compute_uqvk(x.float(), nw.float(), nb.float(), 1e-6, 2, 8, 8, w.float(), b.float())
    empty = pkg.hstu_compute_uqvk(x[:0], nw, nb, 1e-6, 2, 8, 8, w, b)
    assert empty[0].shape == (0, 16) and empty[1].shape == (0, 2, 8)


def test_backward_math_of_the_package_is_the_oracle_s():
    """The backward of the dense steps recomputes them with torch operators inside the package (which may not import
    the oracle): pin those restatements against the oracle on the CPU, every flag combination of the consumer included."""
    import __graft_entry__

    __graft_entry__.load_package()
    from generative_recommenders_amd.ops import hstu_compute as hc

    from oracle import output_oracle as O

    x, nw, nb, w, b = _inputs(77, 40, 64, 2, 8, 16, torch.float32)
    want = U.compute_uqvk(x, nw, nb, 1e-6, 2, 8, 16, w, b)
    got = hc._uqvk_math(x, nw, nb, 1e-6, 2 * 16, w, b)
    u, v, q, k = torch.split(got, [32, 32, 16, 16], dim=1)
    for g_, w_ in zip((u, q.reshape(-1, 2, 8), k.reshape(-1, 2, 8), v.reshape(-1, 2, 16)), want):
        assert torch.allclose(g_, w_, rtol=1e-5, atol=1e-6)
    assert torch.allclose(hc._layer_norm_math(x, nw, nb, 1e-6), U.layer_norm(x, nw, nb, 1e-6), rtol=1e-6, atol=1e-6)
    gen = torch.Generator().manual_seed(5)
    H, ld = 2, 32
    attn, uu = torch.randn((30, H * ld), generator=gen), torch.randn((30, H * ld), generator=gen)
    for group in (False, True):
        wn = torch.randn(H if group else H * ld, generator=gen)
        bn = torch.randn(H if group else H * ld, generator=gen)
        for cu in (False, True):
            for cx in (False, True):
                for act in ("none", "sigmoid", "silu"):
                    for su in (False, True):
                        a_ = hc._norm_mul_math(attn, uu, wn, bn, 1e-6, su, cu, cx, act, group, H, ld)
                        b_ = O.norm_mul(attn, uu, wn, bn, 1e-6, su, cu, cx, act, group, H, ld)
                        assert a_.shape == b_.shape and torch.allclose(a_, b_, rtol=1e-5, atol=1e-6), (group, cu, cx, act, su)


def _grad_close(got, ref, what):
    """2e-2 for the gradients of matrices; 1e-1 for the short parameter vectors, each entry of which is a sum of ~1e4
    signed terms that carry the bf16 roundings of the recomputation (cancellation makes the relative error of such a
    sum several times that of its terms)."""
    got, ref = got.float().cpu(), ref.float()
    assert got.shape == ref.shape and torch.isfinite(got).all(), what
    rel = float((got - ref).norm() / ref.norm())
    bar = 2e-2 if ref.dim() > 1 else 1e-1
    assert rel <= bar, f"{what}: relative {rel:.3e}"


@pytest.mark.gpu
@pytest.mark.parametrize("L,d_model,H,attn,hidden", [(300, 128, 2, 64, 64), (77, 192, 2, 32, 64), (1000, 512, 4, 128, 128)])
def test_uqvk_gradients(pkg, dev, L, d_model, H, attn, hidden):
    """Forward on the kernels, gradients by recomputation: against autograd through the fp32 oracle."""
    print(f"[case] uqvk gradients {L} {d_model} {H} {attn} {hidden}", flush=True)
    dt = torch.bfloat16
    x, nw, nb, w, b = _inputs(900 + L, L, d_model, H, attn, hidden, dt)
    ref_in = [t.float().requires_grad_() for t in (x, nw, nb, w, b)]
    ru, rq, rk, rv = U.compute_uqvk(ref_in[0], ref_in[1], ref_in[2], 1e-6, H, attn, hidden, ref_in[3], ref_in[4])
    gen = torch.Generator().manual_seed(3)
    du, dq, dk, dv = [torch.randn(t.shape, generator=gen) for t in (ru, rq, rk, rv)]
    (ru * du).sum().backward(retain_graph=True)
    ((rq * dq).sum() + (rk * dk).sum() + (rv * dv).sum()).backward()
    hip_in = [t.to(dev).requires_grad_() for t in (x, nw, nb, w, b)]
    u, q, k, v = pkg.hstu_compute_uqvk(hip_in[0], hip_in[1], hip_in[2], 1e-6, H, attn, hidden, hip_in[3], hip_in[4])
    loss = (u.float() * du.to(dev)).sum() + (q.float() * dq.to(dev)).sum() + (k.float() * dk.to(dev)).sum() + (v.float() * dv.to(dev)).sum()
    loss.backward()
    torch.cuda.synchronize()
    for name, h, r in zip(("x", "norm_weight", "norm_bias", "uvqk_weight", "uvqk_bias"), hip_in, ref_in):
        _grad_close(h.grad, r.grad, f"d/d{name}")
    # the layer norm alone
    xl = x.to(dev).requires_grad_()
    pkg.layer_norm(xl, nw.to(dev), nb.to(dev), 1e-6).float().pow(2).sum().backward()
    xr = x.float().requires_grad_()
    U.layer_norm(xr, nw.float(), nb.float(), 1e-6).pow(2).sum().backward()
    _grad_close(xl.grad, xr.grad, "layer norm d/dx")
