"""Turns the csv files of three ``rocprofv3`` runs of ``bench.py`` into a short summary under ``profiles/`` and records
the measured HBM traffic of one call in ``profiles/traffic.json``, which ``bench.py`` reads for ``roofline.traffic``.

    python -m generative_recommenders_amd.profile_summary  is not available (the directory name has a hyphen); use
    python bench.py --profile-summary DIR --workload NAME [--profile-kernels hstu] [--profile-extra "..."]

``DIR`` holds what these three commands wrote (run from /tmp with TMPDIR=/tmp; R = repository root):

    rocprofv3 --kernel-trace --stats --output-format csv -d DIR/kt    -o NAME -- python3 R/bench.py --workload NAME --no-cpu EXTRA > DIR/kt_stdout.log
    rocprofv3 --pmc FETCH_SIZE       --output-format csv -d DIR/fetch -o NAME -- python3 R/bench.py --workload NAME --no-cpu --calibrate-copy --steps 3 --warmup 1 EXTRA
    rocprofv3 --pmc WRITE_SIZE       --output-format csv -d DIR/write -o NAME -- python3 R/bench.py --workload NAME --no-cpu --calibrate-copy --steps 3 --warmup 1 EXTRA

and optionally ``DIR/sq`` from ``rocprofv3 --pmc SQ_BUSY_CU_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU_MFMA_MOPS_BF16
GRBM_GUI_ACTIVE`` (any counters; they are tabulated, and the core clock is derived from GRBM_GUI_ACTIVE and the
timestamps of the same dispatches).

The counters FETCH_SIZE / WRITE_SIZE are scaled by what they read for the plain 1 GiB device copy that
``--calibrate-copy`` launches in the same run (1 GiB read, 1 GiB written).
"""

import csv
import glob
import json
import os
from typing import Dict, List, Optional

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
XCDS = 8  # GRBM counters come back summed over the accelerator dies


def load_traffic() -> Dict[str, dict]:
    """``{workload: {"bytes": HBM bytes of one call, "profile": summary file}}`` (empty if the file is missing)."""
    try:
        with open(TRAFFIC_JSON) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def _find(d: str, pattern: str) -> Optional[str]:
    hits = sorted(glob.glob(os.path.join(d, "**", pattern), recursive=True))
    return hits[0] if hits else None


def _counter_table(path: str) -> Dict[str, Dict[str, List[float]]]:
    """kernel name -> counter name -> values per dispatch; the pseudo counter ``_duration_ns`` holds End - Start of the
    same dispatches (one entry per row of the first counter seen for that kernel)"""
    agg: Dict[str, Dict[str, List[float]]] = {}
    with open(path) as f:
        for r in csv.DictReader(f):
            per = agg.setdefault(r["Kernel_Name"], {})
            per.setdefault(r["Counter_Name"], []).append(float(r["Counter_Value"]))
            if "End_Timestamp" in r and next(iter(per)) == r["Counter_Name"]:
                per.setdefault("_duration_ns", []).append(float(r["End_Timestamp"]) - float(r["Start_Timestamp"]))
    return agg


def write_summary(d: str, workload: str, out_path: str, kernels: str = "hstu", extra: str = "", traffic_key: Optional[str] = None) -> float:
    """Writes ``out_path`` and updates ``profiles/traffic.json``; returns the HBM bytes of one call."""
    only = kernels.split(",")
    rel = os.path.relpath(d, ROOT)
    L = [f"# rocprofv3: workload `{workload}`\n"]
    L.append("Commands (run on the MI355X box from /tmp with TMPDIR=/tmp; R = repository root):\n")
    L.append("```")
    x = (" " + extra) if extra else ""
    L.append(f"rocprofv3 --kernel-trace --stats --output-format csv -d $R/{rel}/kt -o {workload} -- python3 $R/bench.py --workload {workload} --no-cpu{x}")
    L.append(f"rocprofv3 --pmc FETCH_SIZE --output-format csv -d $R/{rel}/fetch -o {workload} -- python3 $R/bench.py --workload {workload} --no-cpu --calibrate-copy --steps 3 --warmup 1{x}")
    L.append(f"rocprofv3 --pmc WRITE_SIZE --output-format csv -d $R/{rel}/write -o {workload} -- python3 $R/bench.py --workload {workload} --no-cpu --calibrate-copy --steps 3 --warmup 1{x}")
    L.append(f"python3 $R/bench.py --profile-summary $R/{rel} --workload {workload} --profile-kernels {kernels}" + (f' --profile-extra "{extra}"' if extra else ""))
    L.append("```\n")
    L.append("## Kernel trace (`*_kernel_stats.csv`)\n")
    L.append("| kernel | calls | average ns | min ns | max ns | % |")
    L.append("|---|---|---|---|---|---|")
    avg_ns: Dict[str, float] = {}
    stats = _find(os.path.join(d, "kt"), "*kernel_stats.csv")
    if stats:
        with open(stats) as f:
            for r in csv.DictReader(f):
                avg_ns[r["Name"]] = float(r["AverageNs"])
                L.append(f"| `{r['Name'][:90]}` | {r['Calls']} | {float(r['AverageNs']):.0f} | {r['MinNs']} | {r['MaxNs']} | {float(r['Percentage']):.2f} |")
    log = os.path.join(d, "kt_stdout.log")
    if os.path.exists(log):
        L.append("\nbench.py line of the same run (HIP events around every timed step; its `traffic` field, which bench.py reads from\nprofiles/traffic.json, is left out: the counters below are the measurement and what this summary writes there):\n")
        for line in open(log):
            if line.startswith("{"):
                j = json.loads(line)
                keep = ("value", "unit", "ms_per_step", "pct_mfma_peak", "roofline")
                shown = {k: j[k] for k in keep if k in j}
                if isinstance(shown.get("roofline"), dict):
                    # the line's own `traffic` was read from an earlier summary; the counters below are this run's
                    shown["roofline"] = {k: v for k, v in shown["roofline"].items() if k not in ("traffic", "traffic_source")}
                L.append("```")
                L.append(json.dumps(shown))
                L.append("```")
    L.append("\n## HBM traffic counters (KiB per dispatch)\n")
    res: Dict[str, float] = {}
    for name in ("fetch", "write"):
        path = _find(os.path.join(d, name), "*counter_collection.csv")
        if not path:
            continue
        agg = _counter_table(path)
        L.append(f"`{name.upper()}_SIZE`:\n")
        L.append("| kernel | dispatches | mean KiB | max KiB |")
        L.append("|---|---|---|---|")
        ncalls = 0
        for k, counters in agg.items():
            v = counters.get(f"{name.upper()}_SIZE", [])
            if not v:
                continue
            L.append(f"| `{k[:80]}` | {len(v)} | {sum(v) / len(v):.1f} | {max(v):.1f} |")
            if any(o in k for o in only):
                if only[0] in k and ncalls == 0:
                    ncalls = len(v)
                res[name + "_sum"] = res.get(name + "_sum", 0.0) + sum(v)
            if "copyBuffer" in k:
                res[name + "_copy"] = max(v)
        L.append("")
        if ncalls:
            res[name] = res[name + "_sum"] / ncalls
    total = 0.0
    if all(k in res for k in ("fetch", "write", "fetch_copy", "write_copy")):
        gib = 1048576.0
        ff, wf = gib / res["fetch_copy"], gib / res["write_copy"]
        L.append(f"Calibration: the plain 1 GiB device copy (`__amd_rocclr_copyBuffer`, reads 1048576 KiB and writes 1048576 KiB) reads "
                 f"FETCH_SIZE = {res['fetch_copy']:.0f} and WRITE_SIZE = {res['write_copy']:.0f}, so the scale factors are {ff:.3f} (fetch) and {wf:.3f} (write).\n")
        fb, wb = res["fetch"] * ff * 1024, res["write"] * wf * 1024
        total = fb + wb
        L.append(f"(Per call: the sum over all dispatches of the kernels whose names contain one of `{kernels}`, divided by the number of "
                 "calls, i.e. of dispatches of the first of them.)\n")
        L.append(f"HBM traffic of one call: fetch {fb / 1e9:.3f} GB + write {wb / 1e9:.3f} GB = **{total / 1e9:.3f} GB**.")
    sq = _find(os.path.join(d, "sq"), "*counter_collection.csv")
    if sq:
        L.append("\n## Other counters (mean per dispatch)\n")
        L.append("| kernel | counter | mean |")
        L.append("|---|---|---|")
        for k, counters in _counter_table(sq).items():
            if not any(o in k for o in only):
                continue
            for cname, v in sorted(counters.items()):
                L.append(f"| `{k[:60]}` | {cname.lstrip('_')} | {sum(v) / len(v):.4g} |")
            dur = counters.get("_duration_ns", [])
            if "GRBM_GUI_ACTIVE" in counters and dur and sum(dur) / len(dur) > 1e5:
                # the counter is summed over the 8 XCDs; duration from the timestamps of the same dispatches
                cyc = sum(counters["GRBM_GUI_ACTIVE"]) / len(counters["GRBM_GUI_ACTIVE"]) / XCDS
                L.append(f"| `{k[:60]}` | core clock = GRBM_GUI_ACTIVE / {XCDS} XCDs / duration of the same dispatches | {cyc / (sum(dur) / len(dur)):.3f} GHz |")
    os.makedirs(os.path.dirname(out_path), exist_ok=True)
    with open(out_path, "w") as f:
        f.write("\n".join(L) + "\n")
    if total > 0:
        table = load_traffic()
        table[traffic_key or workload] = {"bytes": round(total), "profile": os.path.relpath(out_path, ROOT)}
        with open(TRAFFIC_JSON, "w") as f:
            json.dump(table, f, indent=1, sort_keys=True)
            f.write("\n")
    return total
