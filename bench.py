#!/usr/bin/env python3
"""Benchmark of the HSTU attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--tile-config ID] [--no-cpu]

A step is one forward pass (one launch) over one synthetic jagged batch that is already resident in
HBM.  Prints ONE JSON line: the headline metric, the MFMA (or HBM) roofline of the kernel computed
from algorithmic work and HIP-event time, and the CPU oracle timed on a bounded sample of the same
workload on this box's host cores.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0}  # MI355X dense MFMA, published
PEAK_HBM_GBS = 8000.0
HBM_BOUND = {"cfg2", "cfg4"}  # short sequences / cached-KV streaming: priced against HBM bandwidth


def measured_traffic(key):
    """(HBM bytes of one call, the summary they come from), read from profiles/traffic.json -- written by
    `bench.py --profile-summary` from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file, each counter scaled by
    what it reads for a plain 1 GiB copy -- or (None, None) where nothing has been measured."""
    from generative_recommenders_amd import profile_summary

    e = profile_summary.load_traffic().get(key)
    return (e["bytes"], e["profile"]) if e else (None, None)


def traffic_fields(key):
    nbytes, source = measured_traffic(key)
    return {"traffic": nbytes, "traffic_source": source}


def run_gpu(wl, args, pkg, workloads, torch):
    dev = torch.device("cuda:0")
    inp = workloads.make_inputs(wl, dev, fused_buffer=args.fused_buffer)
    q, k, v = inp["q"], inp["k"], inp["v"]
    kw = dict(num_targets=inp["num_targets"], max_attn_len=wl.max_attn_len, contextual_seq_len=wl.contextual_seq_len,
              tile_config=args.tile_config, kv_splits=args.kv_splits)
    sort_kw = dict(sort_by_length=not args.no_sort)  # the reference's bench sets the same hint for its native path
    scales = {}
    if wl.dtype == "fp8":
        qs, ks, vs = [float(x.float().abs().max()) / 448.0 for x in (q, k, v)]
        q = (q.float() / qs).to(torch.float8_e4m3fn)
        k = (k.float() / ks).to(torch.float8_e4m3fn)
        v = (v.float() / vs).to(torch.float8_e4m3fn)
        scales = dict(q_scale=qs, k_scale=ks, v_scale=vs)
    if wl.delta_size > 0:
        def step():
            return pkg.delta_hstu_mha(wl.max_seq_len, wl.alpha, q, k, v, inp["seq_offsets"], **kw, **scales)
    else:
        def step():
            return pkg.hstu_mha(wl.max_seq_len, wl.alpha, q, k, v, inp["seq_offsets"],
                                min_full_attn_seq_len=wl.min_full_attn_seq_len, **kw, **scales, **sort_kw)

    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    del out
    return timed_steps(step, args, torch, flush=wl.name in HBM_BOUND and not args.no_flush)


def timed_steps(step, args, torch, flush):
    """(wall ms per step, timing statistics) over args.steps steps, every step between its own pair of HIP events on the
    stream the kernels are launched on (torch's current stream).  statistics: mean (the figure the line is computed
    from), median, 10th and 90th percentile, number of steps.  With `flush` a 512 MB fill runs between steps, outside
    the timed intervals: the workloads priced against HBM bandwidth have working sets smaller than the 256 MB Infinity
    Cache, and back-to-back repetitions would read them from there."""
    scratch = torch.empty(512 << 20, dtype=torch.uint8, device="cuda:0") if flush else None
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i, (a, b) in enumerate(pairs):
        if flush:
            scratch.fill_(i & 0xFF)
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms = sorted(a.elapsed_time(b) for a, b in pairs)
    n = len(ms)
    stats = {"mean": sum(ms) / n, "median": ms[n // 2] if n % 2 else 0.5 * (ms[n // 2 - 1] + ms[n // 2]),
             "p10": ms[min(n - 1, int(0.1 * n))], "p90": ms[min(n - 1, int(0.9 * n))], "n": n}
    return (stats["mean"] if flush else wall_ms), stats


def timing_fields(stats):
    return {"kernel_ms": round(stats["mean"], 4), "kernel_ms_median": round(stats["median"], 4), "kernel_ms_p10": round(stats["p10"], 4),
            "kernel_ms_p90": round(stats["p90"], 4), "timed_steps": stats["n"]}


def run_cpu_baseline(wl, torch, workloads, budget_s=20.0):
    """The PyTorch oracle (per-sequence form of the reference's pytorch_hstu_mha, fp32) on a bounded sample."""
    import numpy as np

    from oracle import hstu_oracle

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    order = sorted(range(wl.batch), key=lambda b: -int(wl.lengths[b]))
    # sample: the longest sequence first, then every 8th by length, until the time budget is spent
    picks = [order[0]] + order[8::8]
    picks += [b for b in order if b not in picks]
    done, flops, t_used = [], 0.0, 0.0
    for b in picks:
        sub = workloads.Workload(
            "s", 1, wl.heads, wl.dqk, wl.dv, wl.max_seq_len, np.asarray(wl.lengths[b : b + 1]),
            None if wl.num_targets is None else np.asarray(wl.num_targets[b : b + 1]), wl.max_attn_len,
            wl.contextual_seq_len, wl.min_full_attn_seq_len, wl.delta_size, wl.dtype, wl.alpha, wl.seed + b,
        )
        inp = workloads.make_inputs(sub, torch.device("cpu"), dtype=torch.float32)
        t0 = time.perf_counter()
        hstu_oracle.hstu_mha_per_sequence(
            wl.max_seq_len, wl.alpha, inp["q"], inp["k"], inp["v"], inp["seq_offsets"], num_targets=inp["num_targets"],
            max_attn_len=wl.max_attn_len, contextual_seq_len=wl.contextual_seq_len,
            min_full_attn_seq_len=wl.min_full_attn_seq_len, delta_size=wl.delta_size,
        )
        t_used += time.perf_counter() - t0
        flops += workloads.algorithmic_flops(sub)
        done.append(b)
        if t_used > budget_s:
            break
    return {
        "value": round(flops / t_used / 1e12, 5),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{len(done)} of {wl.batch} sequences of workload {wl.name} (lengths "
        f"{[int(wl.lengths[b]) for b in done]}), fp32 PyTorch oracle per sequence, {t_used:.1f} s",
    }


def run_jagged(name, args, pkg, torch):
    """K/V-cache plumbing around delta_hstu_mha at the sizes of cfg4 (32 users, history 1024..4096, 256 new rows, rows of
    H*D = 512 bf16): `kvcat` = concat_2D_jagged(cache, delta) as the reference's _construct_full_kv does per layer and
    micro-batch; `kvtail` = write_kv_tail, the in-place form that copies the new rows only."""
    import numpy as np

    from oracle import jagged_oracle

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1004)
    B, delta, width = 32, 256, 512
    hist = rng.integers(1024, 4097, size=B)
    oc = torch.tensor(np.concatenate([[0], np.cumsum(hist)]), dtype=torch.int64)
    g = torch.Generator().manual_seed(1004)
    cache = (torch.randn((int(oc[-1]), width), generator=g) * 0.1).to(torch.bfloat16)
    new = (torch.randn((B * delta, width), generator=g) * 0.1).to(torch.bfloat16)
    cache_d, new_d, oc_d = cache.to(dev), new.to(dev), oc.to(dev)
    full_offsets = (oc + delta * torch.arange(B + 1)).to(dev)
    max_hist = int(hist.max())
    full = pkg.concat_2D_jagged(max_hist + delta, cache_d, new_d, max_hist, delta, oc_d, None)
    if name == "cfg4_1024":
        # What one layer does for 1024 candidates per user with cfg4's shapes: four micro-batches of 256, each writing its
        # K and V rows behind the cached history (write_kv_tail, twice) and attending from its 256 query rows to history
        # + itself (delta_hstu_mha) -- twelve kernels, the unit M-FALCON's cost is quoted in.
        from generative_recommenders_amd import workloads

        wl = workloads.make_workload("cfg4")
        Hh, D = wl.heads, wl.dqk
        full_k = full
        full_v = full.clone()
        qs = [(torch.randn((B * delta, Hh, D), generator=g) * 0.1).to(torch.bfloat16).to(dev) for _ in range(4)]
        ks = [(torch.randn((B * delta, width), generator=g) * 0.1).to(torch.bfloat16).to(dev) for _ in range(4)]
        vs = [(torch.randn((B * delta, width), generator=g) * 0.1).to(torch.bfloat16).to(dev) for _ in range(4)]
        targets = torch.full((B,), delta, dtype=torch.int64, device=dev)

        def step():
            out = None
            for mb in range(4):
                pkg.write_kv_tail(full_k, full_offsets, ks[mb])
                pkg.write_kv_tail(full_v, full_offsets, vs[mb])
                out = pkg.delta_hstu_mha(wl.max_seq_len, wl.alpha, qs[mb], full_k.view(-1, Hh, D), full_v.view(-1, Hh, D), full_offsets,
                                         num_targets=targets)
            return out

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        wall_ms, st = timed_steps(step, args, torch, flush=not args.no_flush)
        flops = 4 * workloads.algorithmic_flops(wl)
        tf = flops / (st["mean"] * 1e-3) / 1e12
        print(json.dumps({
            "metric": "M-FALCON layer step per 1024 candidates: 4 x (write_kv_tail K, V + delta_hstu_mha), TFLOP/s of the attention's work",
            "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
            "data": "synthetic", "config": {"workload": name, "batch": B, "delta_size": delta, "micro_batches": 4, "heads": Hh, "d": D,
                                            "history_rows": int(oc[-1])},
            "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                         "frac": round(tf / PEAK_TFLOPS["bf16"], 4), "traffic": None,
                         "kernel": "4 x (2 hstu_jagged_write_tail_kernel + hstu_plan/prep + delta attention kernel)", **timing_fields(st),
                         "algorithmic_flops": flops, "us_per_micro_batch": round(st["mean"] * 1e3 / 4, 1)},
        }))
        return
    if name == "kvcat":
        def step():
            return pkg.concat_2D_jagged(max_hist + delta, cache_d, new_d, max_hist, delta, oc_d, None)
        nbytes = 2 * (cache.numel() + new.numel()) * 2
        kernel = "hstu_jagged_copy_kernel"
    else:
        def step():
            return pkg.write_kv_tail(full, full_offsets, new_d)
        nbytes = 2 * new.numel() * 2
        kernel = "hstu_jagged_write_tail_kernel"
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    wall_ms, st = timed_steps(step, args, torch, flush=not args.no_flush)
    ev_ms = st["mean"]
    gbs = nbytes / (ev_ms * 1e-3) / 1e9
    line = {
        "metric": "K/V cache (+) delta rows per call, GB/s moved (cfg4 sizes)", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": name, "batch": B, "delta_size": delta, "row_bytes": width * 2, "history_rows": int(oc[-1])},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4), **traffic_fields(name), "kernel": kernel,
                     **timing_fields(st), "algorithmic_bytes": nbytes},
    }
    if not args.no_cpu:
        torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))))
        reps, t_used = 0, 0.0
        dense_off = delta * torch.arange(B + 1)
        while t_used < 5.0:
            t0 = time.perf_counter()
            jagged_oracle.concat_by_batch(cache, new, oc, dense_off)
            t_used += time.perf_counter() - t0
            reps += 1
        cat_bytes = 2 * (cache.numel() + new.numel()) * 2
        line["cpu_baseline"] = {"value": round(cat_bytes * reps / t_used / 1e9, 2), "unit": "GB/s", "cores": torch.get_num_threads(),
                                "kind": "port", "sample": f"{reps} full concatenations of the same cache and rows (per-batch torch.cat), {t_used:.1f} s"}
    print(json.dumps(line))


def run_linear(name, args, pkg, torch):
    """The dense steps either side of the attention at the headline's token count (524288 rows, d_model 512, H=4,
    attn = hidden = 128): `uqvk` = layer norm + projection + bias + SiLU(u) (hstu_compute_uqvk), `layernorm` = its
    layer-norm kernel alone, `output` = norm * u, concatenation, projection + residual (hstu_compute_output with the
    STU layer's flags), `normmul` = its norm-multiply-concatenate kernel alone."""
    from generative_recommenders_amd.ops import hstu_compute

    from oracle import output_oracle, uqvk_oracle

    dev = torch.device("cuda:0")
    L, d_model, H, D = 64 * 8192, 512, 4, 128
    n_out = 4 * D * H
    g = torch.Generator(device=dev).manual_seed(1000)

    def rnd(*shape, scale=1.0, shift=0.0):
        return (torch.randn(shape, device=dev, generator=g) * scale + shift).to(torch.bfloat16)

    if name == "cfg5_e2e":
        # the fifth baseline configuration end to end: the fused producer writes q, k, v as e4m3 (and the batch's maxima),
        # the fp8 attention reads them where they are -- 16 sequences of 4096 .. 16384, H = 8, d = 128, d_model 512
        from generative_recommenders_amd import workloads

        import __graft_entry__ as ge

        top = ge.load_package()
        wl = workloads.make_workload("cfg5")
        L, H = wl.total_kv, wl.heads
        n_out = 4 * D * H
    x = rnd(L, d_model, scale=1.5, shift=0.3)
    if name == "cfg5_e2e":
        import numpy as np

        offsets = torch.tensor([0] + [int(t) for t in np.cumsum(wl.lengths)], dtype=torch.int64, device=dev)
        targets = torch.tensor([int(t) for t in wl.num_targets], dtype=torch.int64, device=dev)
        nw, nb = rnd(d_model, scale=0.1, shift=1.0), rnd(d_model, scale=0.1)
        w, b = rnd(d_model, n_out, scale=1.0 / d_model**0.5), rnd(n_out, scale=0.1)
        # the scales a serving loop would carry over from the batch before: this batch's own maxima / 448
        _, _, _, _, amax = hstu_compute.hstu_compute_uqvk_fp8(x, nw, nb, 1e-6, H, D, D, w, b, 1.0, 1.0, 1.0)
        vs, qs, ks = (float(m) / 448.0 for m in amax)

        def step():
            u, q8, k8, v8, _ = hstu_compute.hstu_compute_uqvk_fp8(x, nw, nb, 1e-6, H, D, D, w, b, qs, ks, vs)
            return top.hstu_mha(wl.max_seq_len, wl.alpha, q8, k8, v8, offsets, num_targets=targets, q_scale=qs, k_scale=ks,
                                v_scale=vs, sort_by_length=True)

        cpu = None
        flops = 2.0 * L * d_model * n_out + workloads.algorithmic_flops(wl)
        nbytes = 2.0 * (L * d_model + d_model * n_out + L * n_out) + 1.0 * L * 3 * H * D + 2.0 * L * H * D
        kernel = "hstu_uqvk_fused_kernel (e4m3 epilogue) + hstu_fwd_stream_kernel (fp8)"
        metric = "fused q/k/v producer -> fp8 attention, TFLOP/s (cfg5: 16 sequences of 4096..16384, H8 d128, d_model 512)"
    elif name == "layer":
        # one STU layer forward on the headline batch (64 sequences of 8192): hstu_preprocess_and_attention, then
        # hstu_compute_output on its u and attention output -- the three steps of this library back to back
        from generative_recommenders_amd import workloads

        wl = workloads.make_workload("headline")
        offsets = torch.arange(0, L + 1, wl.max_seq_len, dtype=torch.int64, device=dev)
        nw, nb = rnd(d_model, scale=0.1, shift=1.0), rnd(d_model, scale=0.1)
        w, b = rnd(d_model, n_out, scale=1.0 / d_model**0.5), rnd(n_out, scale=0.1)
        onw, onb = rnd(H * D, scale=0.1, shift=1.0), rnd(H * D, scale=0.1)
        ow = rnd(3 * H * D, d_model, scale=1.0 / (3 * H * D) ** 0.5)

        def step():
            u, attn, _, _ = hstu_compute.hstu_preprocess_and_attention(
                x, nw, nb, 1e-6, H, D, D, w, b, wl.max_seq_len, offsets, wl.alpha, True, None, 0, 0, False, False, True)
            return hstu_compute.hstu_compute_output(attn, u, x, onw, onb, 1e-6, ow, H, D, 0.0, False, True, True, "none", False, False)

        cpu = None
        attn_flops = workloads.algorithmic_flops(wl)
        flops = 2.0 * L * d_model * n_out + attn_flops + 2.0 * L * 3 * H * D * d_model
        nbytes = 2.0 * (L * d_model * 3 + d_model * n_out + 3 * H * D * d_model)  # x in (twice: the residual), out
        kernel = "hstu_uqvk_fused_kernel + hstu_fwd_stream_kernel + hstu_norm_mul_kernel + hstu_output_gemm_kernel"
        metric = "STU layer fwd TFLOP/s (uqvk, attention, output; 64 x 8192 tokens, d_model 512, H4 d128)"
    elif name in ("uqvk", "layernorm"):
        nw, nb = rnd(d_model, scale=0.1, shift=1.0), rnd(d_model, scale=0.1)
        w, b = rnd(d_model, n_out, scale=1.0 / d_model**0.5), rnd(n_out, scale=0.1)
        if name == "uqvk":
            step = lambda: hstu_compute.hstu_compute_uqvk(x, nw, nb, 1e-6, H, D, D, w, b, path=args.uqvk_path)  # noqa: E731
            cpu = lambda r: uqvk_oracle.compute_uqvk(x[:r].float().cpu(), nw.float().cpu(), nb.float().cpu(), 1e-6, H, D, D, w.float().cpu(), b.float().cpu())  # noqa: E731
            flops, nbytes = 2.0 * L * d_model * n_out, 2.0 * (L * d_model + d_model * n_out + L * n_out)
            kernel = ("hstu_layer_norm_kernel + 2 hipBLASLt GEMMs (bias, bias + SiLU epilogues)" if args.uqvk_path == 1
                      else "hstu_uqvk_fused_kernel")
            metric = "hstu_compute_uqvk fwd TFLOP/s (524288 tokens, d_model 512 -> 2048)"
        else:
            step = lambda: hstu_compute.layer_norm(x, nw, nb, 1e-6)  # noqa: E731
            cpu = lambda r: uqvk_oracle.layer_norm(x[:r].float().cpu(), nw.float().cpu(), nb.float().cpu(), 1e-6)  # noqa: E731
            flops, nbytes = 0.0, 2.0 * 2 * L * d_model
            kernel, metric = "hstu_layer_norm_kernel", "layer norm GB/s (524288 rows of 512 bf16)"
    else:
        attn, u = rnd(L, H * D, scale=0.1), rnd(L, H * D, scale=0.5)
        nw, nb = rnd(H * D, scale=0.1, shift=1.0), rnd(H * D, scale=0.1)
        w = rnd(3 * H * D, d_model, scale=1.0 / (3 * H * D) ** 0.5)
        if name == "output":
            step = lambda: hstu_compute.hstu_compute_output(attn, u, x, nw, nb, 1e-6, w, H, D, 0.0, False, True, True, "none", False, False, path=args.output_path)  # noqa: E731
            cpu = lambda r: output_oracle.compute_output(attn[:r].float().cpu(), u[:r].float().cpu(), x[:r].float().cpu(), nw.float().cpu(), nb.float().cpu(), w.float().cpu(), 1e-6, concat_u=True, concat_x=True)  # noqa: E731
            flops, nbytes = 2.0 * L * 3 * H * D * d_model, 2.0 * (2 * L * H * D + 2 * L * d_model + 3 * H * D * d_model)
            kernel = ("hstu_norm_mul_kernel + hipBLASLt GEMM (residual as C operand)" if args.output_path == 1
                      else "hstu_norm_mul_kernel (y alone) + hstu_output_gemm_kernel")
            metric = "hstu_compute_output fwd TFLOP/s (524288 tokens, 3 x 512 -> 512)"
        else:
            step = lambda: hstu_compute.norm_mul_dropout(attn, u, nw, nb, 1e-6, 0.0, False, False, True, True, "none")  # noqa: E731
            cpu = lambda r: output_oracle.norm_mul(attn[:r].float().cpu(), u[:r].float().cpu(), nw.float().cpu(), nb.float().cpu(), 1e-6, concat_u=True, concat_x=True)  # noqa: E731
            flops, nbytes = 0.0, 2.0 * (2 + 3) * L * H * D
            kernel, metric = "hstu_norm_mul_kernel", "norm * u + concatenation GB/s (524288 rows, 2 x 512 in, 3 x 512 out, bf16)"
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    wall_ms, st = timed_steps(step, args, torch, flush=False)
    ev_ms = st["mean"]
    tflops = flops / (ev_ms * 1e-3) / 1e12
    gbs = nbytes / (ev_ms * 1e-3) / 1e9
    if flops > 0:
        roof = {"bound": "mfma", "achieved": round(tflops, 1), "peak": PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                "frac": round(tflops / PEAK_TFLOPS["bf16"], 4)}
        value, unit = round(tflops, 2), "TFLOP/s"
    else:
        roof = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)}
        value, unit = round(gbs, 1), "GB/s"
    traffic = traffic_fields(name + "_library" if (name == "uqvk" and args.uqvk_path == 1) or (name == "output" and args.output_path == 1) else name)
    if name == "cfg5_e2e":
        roof["note"] = "both kernels' flops over their summed time, against the bf16 peak (the attention's own peak is fp8's: see workload cfg5)"
    roof.update({**traffic, "kernel": kernel, **timing_fields(st),
                 "algorithmic_flops": flops, "algorithmic_bytes": nbytes, "hbm_gbs_algorithmic": round(gbs, 1)})
    line = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16 producer + fp8 attention" if name == "cfg5_e2e" else "bf16",
            "data": "synthetic", "config": {"workload": name, "rows": L, "d_model": d_model, "heads": H, "attn_dim": D, "hidden_dim": D},
            "roofline": roof}
    if not args.no_cpu and cpu is not None:
        torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))))
        rows = 32768
        reps, t_used = 0, 0.0
        while t_used < 10.0:
            t0 = time.perf_counter()
            cpu(rows)
            t_used += time.perf_counter() - t0
            reps += 1
        frac = rows / L
        cpu_val = (flops * frac * reps / t_used / 1e12) if flops > 0 else (nbytes * frac * reps / t_used / 1e9)
        line["cpu_baseline"] = {"value": round(cpu_val, 4), "unit": unit, "cores": torch.get_num_threads(), "kind": "port",
                                "sample": f"{reps} passes of the fp32 oracle over the first {rows} of {L} rows (conversion to fp32 included), {t_used:.1f} s"}
    print(json.dumps(line))


def run_bwd(name, args, pkg, workloads, torch, emit=True):
    """Backward of hstu_mha (dq, dk, dv from dout) on the headline shape (`bwd`) or on the ragged third baseline
    configuration (`bwd_cfg3`).  A step is one call of the backward entry point: its two kernels.  Algorithmic work:
    five products per mask-valid pair (S, dP, dV, dQ, dK -- the count of the reference's bench,
    ops/benchmarks/hstu_attention_bench.py:51-60), i.e. 2 * (3 * Dqk + 2 * Dv) flops."""
    from generative_recommenders_amd.ops import hip_backend

    from oracle import bwd_oracle

    dev = torch.device("cuda:0")
    wl = workloads.make_workload("headline" if name == "bwd" else "cfg3")
    inp = workloads.make_inputs(wl, dev)
    q, k, v, offsets, targets = inp["q"], inp["k"], inp["v"], inp["seq_offsets"], inp["num_targets"]
    g = torch.Generator(device=dev).manual_seed(wl.seed + 1)
    dout = (torch.randn(v.shape, device=dev, generator=g) * 0.1).to(v.dtype)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    # the dS scratch is the caller's and is allocated once, as a training loop would keep it
    stored = args.bwd_form == "stored"
    scratch = None
    if stored:
        need = hip_backend.mha_bwd_workspace_bytes(q.shape[0], wl.batch, wl.heads, wl.max_seq_len)
        scratch = torch.empty(need, dtype=torch.uint8, device=dev)

    def step():
        hip_backend.mha_bwd(dout, q, k, v, dq, dk, dv, offsets, targets, wl.max_seq_len, wl.alpha, wl.max_attn_len,
                            wl.contextual_seq_len, wl.min_full_attn_seq_len, store_ds=False, workspace=scratch)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    wall_ms, st = timed_steps(step, args, torch, flush=False)
    ev_ms = st["mean"]
    pair_flops = 2.0 * (3 * wl.dqk + 2 * wl.dv)
    flops = workloads.algorithmic_flops(wl) / (2.0 * (wl.dqk + wl.dv)) * pair_flops
    nbytes = 2.0 * wl.total_kv * wl.heads * (4 * wl.dqk + 3 * wl.dv)  # q, k, dq, dk and v, dout, dv once each
    tflops = flops / (ev_ms * 1e-3) / 1e12
    line = {
        "metric": "HSTU attn bwd effective TFLOP/s + % MFMA peak", "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": wl.dtype, "data": "synthetic",
        "config": {"workload": name, "batch": wl.batch, "heads": wl.heads, "dqk": wl.dqk, "dv": wl.dv, "max_seq_len": wl.max_seq_len,
                   "total_tokens": wl.total_kv, "max_attn_len": wl.max_attn_len, "contextual_seq_len": wl.contextual_seq_len,
                   "num_targets": wl.num_targets is not None, "form": args.bwd_form,
                   "scratch_bytes": 0 if scratch is None else scratch.numel()},
        "pct_mfma_peak": round(100.0 * tflops / PEAK_TFLOPS[wl.dtype], 2),
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": PEAK_TFLOPS[wl.dtype], "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_TFLOPS[wl.dtype], 4),
                     **traffic_fields(name + ("_stored" if stored else "")),
                     "kernel": ("hstu_bwd_dkdv_pp_kernel" if min(wl.dqk, wl.dv) >= 32 else "hstu_bwd_dkdv_kernel") + " + " + ("hstu_bwd_dq_stored_kernel" if stored else "hstu_bwd_dq_kernel"),
                     **timing_fields(st),
                     "algorithmic_flops": flops, "algorithmic_bytes": nbytes},
    }
    if not args.no_cpu and emit:
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(cores)
        order = sorted(range(wl.batch), key=lambda b: -int(wl.lengths[b]))
        picks = [order[0]] + order[8::8]
        qc, kc, vc, dc = [t.float().cpu() for t in (q, k, v, dout)]
        oc, tc = offsets.cpu(), None if targets is None else targets.cpu()
        done, cpu_flops, t_used = [], 0.0, 0.0
        import numpy as np
        for b in picks:
            t0 = time.perf_counter()
            bwd_oracle.closed_form_grads(wl.max_seq_len, wl.alpha, qc, kc, vc, oc, dc, num_targets=tc, max_attn_len=wl.max_attn_len,
                                         contextual_seq_len=wl.contextual_seq_len, min_full_attn_seq_len=wl.min_full_attn_seq_len,
                                         sequences=[b])
            t_used += time.perf_counter() - t0
            sub = workloads.Workload("s", 1, wl.heads, wl.dqk, wl.dv, wl.max_seq_len, np.asarray(wl.lengths[b : b + 1]),
                                     None if wl.num_targets is None else np.asarray(wl.num_targets[b : b + 1]), wl.max_attn_len,
                                     wl.contextual_seq_len, wl.min_full_attn_seq_len, 0, wl.dtype, wl.alpha, wl.seed)
            cpu_flops += workloads.algorithmic_flops(sub) / (2.0 * (wl.dqk + wl.dv)) * pair_flops
            done.append(b)
            if t_used > 15.0:
                break
        line["cpu_baseline"] = {"value": round(cpu_flops / t_used / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                                "sample": f"{len(done)} of {wl.batch} sequences (lengths {[int(wl.lengths[b]) for b in done]}), "
                                          f"fp32 closed-form gradients per sequence, {t_used:.1f} s"}
    if emit:
        print(json.dumps(line))
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="headline")
    ap.add_argument("--tile-config", type=int, default=0)
    ap.add_argument("--output-path", type=int, default=0, help="workload output: 0 / 2 = norm-multiply kernel + concatenating GEMM kernel, 1 = norm-multiply kernel + hipBLASLt")
    ap.add_argument("--uqvk-path", type=int, default=0, help="workload uqvk: 0 / 2 = fused kernel, 1 = layer-norm kernel + hipBLASLt")
    ap.add_argument("--bwd-form", choices=["stored", "recompute"], default="stored",
                    help="workloads bwd, bwd_cfg3: dS stored in scratch memory and dq streamed from it, or the scores recomputed for dq")
    ap.add_argument("--kv-splits", type=int, default=0, help="0 = the library's own rule, 1 = off, 2..8 = forced")
    ap.add_argument("--fused-buffer", action="store_true", help="q/k/v as column slices of one [L,H,3D] buffer")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-flush", action="store_true",
                    help="HBM-priced workloads (cfg2, cfg4, kvcat, kvtail): do not flush the caches between steps")
    ap.add_argument("--no-jagged", action="store_true",
                    help="headline only: do not also time the ragged cfg3 batch for the extra `jagged_cfg3` entry")
    ap.add_argument("--no-bwd", action="store_true",
                    help="headline only: do not also time the backward of the same call for the extra `backward` entry")
    ap.add_argument("--no-sort", action="store_true", help="do not pass sort_by_length=True to hstu_mha")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 1 GiB device copy, so that a counter run can scale FETCH_SIZE/WRITE_SIZE")
    ap.add_argument("--profile-summary", metavar="DIR", default=None,
                    help="no GPU work: turn the rocprofv3 csv files under DIR (kt/, fetch/, write/, optionally sq/) into a summary "
                         "under profiles/ and record the measured HBM traffic in profiles/traffic.json")
    ap.add_argument("--profile-out", default=None, help="--profile-summary: file to write (default profiles/<workload>.md)")
    ap.add_argument("--profile-kernels", default="hstu", help="--profile-summary: comma-separated substrings of the kernel names that make up one call")
    ap.add_argument("--profile-extra", default="", help="--profile-summary: the extra bench.py arguments the profiled runs were given")
    ap.add_argument("--profile-key", default=None, help="--profile-summary: key in profiles/traffic.json (default: the workload)")
    args = ap.parse_args()
    if args.profile_summary:
        import __graft_entry__

        __graft_entry__.load_package()
        from generative_recommenders_amd import profile_summary

        out = args.profile_out or os.path.join(ROOT, "profiles", args.workload + ".md")
        total = profile_summary.write_summary(args.profile_summary, args.workload, out, args.profile_kernels, args.profile_extra, args.profile_key)
        print(f"{out}: HBM traffic of one call {total / 1e9:.3f} GB")
        return
    if args.gpus != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus must be 1 "
              "(sequences are independent, so N GPUs would each run the same kernel on a slice)", file=sys.stderr)
        sys.exit(2)

    import torch

    import __graft_entry__

    pkg = __graft_entry__.load_package()
    from generative_recommenders_amd import workloads

    jagged = args.workload in ("kvcat", "kvtail", "cfg4_1024")
    producer = args.workload in ("uqvk", "layernorm", "output", "normmul", "layer", "cfg5_e2e")
    backward = args.workload in ("bwd", "bwd_cfg3")
    wl = None if jagged or producer or backward else workloads.make_workload(args.workload)
    if wl is not None and wl.dtype == "fp32":
        print("bench.py: cfg1 is the CPU correctness case, not a GPU bench workload", file=sys.stderr)
        sys.exit(2)
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    if jagged:
        run_jagged(args.workload, args, pkg, torch)
        return
    if producer:
        run_linear(args.workload, args, pkg, torch)
        return
    if backward:
        run_bwd(args.workload, args, pkg, workloads, torch)
        return
    wall_ms, st = run_gpu(wl, args, pkg, workloads, torch)
    ev_ms = st["mean"]
    flops = workloads.algorithmic_flops(wl)
    ref_flops = workloads.reference_convention_flops(wl)
    nbytes = workloads.algorithmic_bytes(wl)
    tflops = flops / (ev_ms * 1e-3) / 1e12
    if wl.name in HBM_BOUND:
        ach = nbytes / (ev_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(ach / PEAK_HBM_GBS, 4), **traffic_fields(wl.name)}
    else:
        peak = PEAK_TFLOPS[wl.dtype]
        roof = {"bound": "mfma", "achieved": round(tflops, 1), "peak": peak, "unit": "TFLOP/s",
                "frac": round(tflops / peak, 4), **traffic_fields(wl.name)}
    cfg, splits = pkg.ops.hip_backend.plan_for(
        batch=wl.batch, heads=wl.heads, dqk=wl.dqk, dv=wl.dv, total_q=wl.batch * wl.delta_size if wl.delta_size else wl.total_kv,
        total_kv=wl.total_kv, max_seq_len=wl.max_seq_len, delta_size=wl.delta_size, tile_config=args.tile_config,
        kv_splits=args.kv_splits, sort_by_length=wl.delta_size == 0 and not args.no_sort)
    roof["kernel"] = {1: "hstu_fwd_kernel", 2: "hstu_fwd_stream_kernel", 3: "hstu_fwd_pp_kernel<NG=1>"}[cfg]
    roof["kv_splits"] = splits
    roof.update(timing_fields(st))
    roof["algorithmic_flops"] = flops
    roof["algorithmic_bytes"] = nbytes
    line = {
        "metric": "HSTU attn fwd effective TFLOP/s + % MFMA peak, jagged B=64 L<=8192 H4 d128",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": wl.dtype,
        "data": "synthetic",
        "config": {
            "workload": wl.name,
            "batch": wl.batch, "heads": wl.heads, "dqk": wl.dqk, "dv": wl.dv, "max_seq_len": wl.max_seq_len,
            "total_tokens": wl.total_kv, "max_attn_len": wl.max_attn_len, "contextual_seq_len": wl.contextual_seq_len,
            "num_targets": wl.num_targets is not None, "delta_size": wl.delta_size,
            "tile_config": args.tile_config, "kv_splits": args.kv_splits, "fused_buffer": args.fused_buffer,
        },
        "pct_mfma_peak": round(100.0 * tflops / PEAK_TFLOPS[wl.dtype], 2),
        "reference_convention_tflops": round(ref_flops / (ev_ms * 1e-3) / 1e12, 2),
        "hbm_gbs_algorithmic": round(nbytes / (ev_ms * 1e-3) / 1e9, 1),
        "roofline": roof,
    }
    if wl.name == "headline" and not args.no_jagged:
        # the same shape class with the DLRMv3-like ragged batch of the third baseline configuration (Zipf lengths,
        # window, contextual prefix, targets), measured in the same run; a few extra milliseconds
        wl3 = workloads.make_workload("cfg3")
        saved = (args.steps, args.warmup)
        args.steps, args.warmup = max(10, min(args.steps, 50)), 3
        try:
            _, st3 = run_gpu(wl3, args, pkg, workloads, torch)
            ms3 = st3["mean"]
            exact3 = workloads.algorithmic_flops(wl3) / (ms3 * 1e-3) / 1e12
            conv3 = workloads.reference_convention_flops(wl3) / (ms3 * 1e-3) / 1e12
            line["jagged_cfg3"] = {
                "workload": "cfg3", **timing_fields(st3), "exact_tflops": round(exact3, 2),
                "pct_mfma_peak_exact": round(100.0 * exact3 / PEAK_TFLOPS[wl3.dtype], 2),
                "reference_convention_tflops": round(conv3, 2),
                "pct_mfma_peak_reference_convention": round(100.0 * conv3 / PEAK_TFLOPS[wl3.dtype], 2),
                "note": "reference convention = H*(Dqk+Dv)*sum(n^2), the figure the reference's bench prints; it counts pairs "
                        "that max_attn_len masks out",
            }
        except Exception as exc:  # noqa: BLE001  (an extra entry must not cost the line its main figure)
            line["jagged_cfg3"] = {"workload": "cfg3", "error": f"{type(exc).__name__}: {exc}"[:300]}
        args.steps, args.warmup = saved
    if wl.name == "headline" and not args.no_jagged:
        # the headline's own shape with unequal lengths (1024..8192, plain causal): what the same kernel does when the
        # batch is ragged and the work goes through the work lists instead of the arithmetic deal
        wlr = workloads.make_workload("ragged8k")
        saved = (args.steps, args.warmup)
        args.steps, args.warmup = max(10, min(args.steps, 50)), 3
        try:
            _, str_ = run_gpu(wlr, args, pkg, workloads, torch)
            exr = workloads.algorithmic_flops(wlr) / (str_["mean"] * 1e-3) / 1e12
            line["ragged8k"] = {
                "workload": "ragged8k", "lengths": "64 sequences, uniform in 1024..8192, plain causal", **timing_fields(str_),
                "exact_tflops": round(exr, 2), "pct_mfma_peak_exact": round(100.0 * exr / PEAK_TFLOPS[wlr.dtype], 2),
            }
        except Exception as exc:  # noqa: BLE001
            line["ragged8k"] = {"workload": "ragged8k", "error": f"{type(exc).__name__}: {exc}"[:300]}
        args.steps, args.warmup = saved
    if wl.name == "headline" and not args.no_bwd:
        # the backward of the same call (dq, dk, dv from dout), measured in the same run: about half a second
        saved = (args.steps, args.warmup, args.bwd_form)
        args.steps, args.warmup = 10, 3
        try:
            # the stored-dS form wants 34.5 GB of scratch: without that much free memory the other form is measured, and
            # whatever goes wrong here must not cost the line its main figure
            from generative_recommenders_amd.ops import hip_backend

            need = hip_backend.mha_bwd_workspace_bytes(wl.total_kv, wl.batch, wl.heads, wl.max_seq_len)
            if args.bwd_form == "stored" and torch.cuda.mem_get_info(0)[0] < need + (8 << 30):
                args.bwd_form = "recompute"
            b = run_bwd("bwd", args, pkg, workloads, torch, emit=False)
            line["backward"] = {"workload": "bwd", "form": b["config"]["form"], "scratch_bytes": b["config"]["scratch_bytes"],
                                "kernel_ms": b["roofline"]["kernel_ms"], "exact_tflops": b["value"], "pct_mfma_peak": b["pct_mfma_peak"],
                                "kernels": b["roofline"]["kernel"],
                                "note": "2 * (3 * Dqk + 2 * Dv) flops per mask-valid pair, the count of the reference's bench"}
        except Exception as exc:  # noqa: BLE001
            line["backward"] = {"workload": "bwd", "error": f"{type(exc).__name__}: {exc}"[:300]}
        args.steps, args.warmup, args.bwd_form = saved
    if not args.no_cpu:
        line["cpu_baseline"] = run_cpu_baseline(wl, torch, workloads)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
