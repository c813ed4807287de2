"""Turns raw rocprofv3 output of the benchmark into the short summaries kept under profiles/.

    python -m nabla_amd.kernel_bench --summarize DIR [--workload llama3-8b]
    (or: python -m nabla_amd.profile_summary DIR)

Expected under DIR, made by these five commands (each from the repository root, after
`cd /tmp && export TMPDIR=/tmp && cd -`; the program follows `--` directly):

    rocprofv3 --kernel-trace --stats -d DIR/kt -o kt --output-format csv -- python3 bench.py --no-cpu-baseline --primary-only --no-ceiling > DIR/kt_bench.json
    rocprofv3 --pmc FETCH_SIZE -d DIR/fetch -o fetch --output-format csv -- python3 bench.py --no-cpu-baseline --primary-only --no-ceiling
    rocprofv3 --pmc WRITE_SIZE -d DIR/write -o write --output-format csv -- python3 bench.py --no-cpu-baseline --primary-only --no-ceiling
    rocprofv3 --pmc FETCH_SIZE -d DIR/cfetch -o cfetch --output-format csv -- python3 bench.py --calibrate-copy 8 --steps 3 > DIR/cfetch.json
    rocprofv3 --pmc WRITE_SIZE -d DIR/cwrite -o cwrite --output-format csv -- python3 bench.py --calibrate-copy 8 --steps 3

(add `--workload NAME` to the three bench.py lines for another workload).  The counters are
scaled by what the same counters read for the library's plain copy kernel over 8 GiB, a
transfer of known size.  Writes profiles/adamw_fused_step_<workload>.md and the workload's entry
of profiles/traffic.json, which bench.py quotes as `roofline.traffic` (naming its source).
"""
from __future__ import annotations

import csv
import datetime
import glob
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
COPY_GIB = 8


def _one(pattern):
    hits = sorted(glob.glob(pattern, recursive=True))
    if not hits:
        raise FileNotFoundError(f"no file matches {pattern}")
    return hits[0]


def _counter(base, sub):
    """{kernel name: [counter value per dispatch]} from DIR/sub/**/*counter_collection.csv*."""
    out = {}
    with open(_one(os.path.join(base, sub, "**", "*counter_collection.csv*"))) as f:
        for r in csv.DictReader(f):
            if r["Kernel_Name"].startswith("nbo_"):
                out.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
    return out


def _last_json(path):
    with open(path) as f:
        lines = [ln for ln in f.read().strip().splitlines() if ln.startswith("{")]
    return json.loads(lines[-1])


def _mean(xs):
    return sum(xs) / len(xs)


KERNEL_SOURCES = ("nabla_amd/csrc/kernels/nbo_kernels.hip", "nabla_amd/csrc/nbo_device_types.h")


def kernel_source_hash() -> str:
    """sha256 over the files the step's kernels are compiled from: what a set of counters was
    collected for.  profiles/traffic.json stores it, bench.py and the tests compare it."""
    import hashlib

    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _commit():
    try:
        return subprocess.run(["git", "rev-parse", "--short", "HEAD"], cwd=ROOT, capture_output=True,
                              text=True, timeout=10).stdout.strip() or "unknown"
    except Exception:
        return "unknown"


def summarize(base: str) -> str:
    with open(_one(os.path.join(base, "kt", "**", "*kernel_stats.csv"))) as f:
        stats = [r for r in csv.DictReader(f) if r["Name"].startswith("nbo_")]
    fetch, write = _counter(base, "fetch"), _counter(base, "write")
    cf, cw = _counter(base, "cfetch")["nbo_copy_f32x4"], _counter(base, "cwrite")["nbo_copy_f32x4"]
    bench = _last_json(os.path.join(base, "kt_bench.json"))
    copy = _last_json(os.path.join(base, "cfetch.json"))
    workload = bench["config"]["workload"]
    n = bench["config"]["params"]
    dom = bench["roofline"]["kernel"]
    fam = dom.split("_")[2]
    norm_k = f"nbo_norm_{fam}"
    flags = "" if workload == "llama3-8b" else f" --workload {workload}"
    copy_kib = COPY_GIB * (1 << 30) / 1024
    # the first copy launch of each calibration run pays for page faults of fresh memory: left out
    f_scale = copy_kib / _mean(cf[1:])  # KiB of real traffic per counter unit
    w_scale = copy_kib / _mean(cw[1:])
    upd_b = bench["roofline"]["algorithmic_bytes_per_launch"] // n
    L = []
    L.append(f"# rocprofv3 summary: fused AdamW step, `{workload}` set (`python bench.py{flags}`), MI355X\n")
    L.append(f"Made by `python -m nabla_amd.kernel_bench --summarize {base}` at commit {_commit()} on "
             f"{datetime.date.today().isoformat()} from the output of (each from the repository root, after "
             "`cd /tmp && export TMPDIR=/tmp && cd -`):\n")
    L.append("```")
    d = base.rstrip("/")
    L.append(f"rocprofv3 --kernel-trace --stats -d {d}/kt -o kt --output-format csv -- python3 bench.py --no-cpu-baseline --primary-only --no-ceiling{flags} > {d}/kt_bench.json")
    L.append(f"rocprofv3 --pmc FETCH_SIZE -d {d}/fetch -o fetch --output-format csv -- python3 bench.py --no-cpu-baseline --primary-only --no-ceiling{flags}")
    L.append(f"rocprofv3 --pmc WRITE_SIZE -d {d}/write -o write --output-format csv -- python3 bench.py --no-cpu-baseline --primary-only --no-ceiling{flags}")
    L.append(f"rocprofv3 --pmc FETCH_SIZE -d {d}/cfetch -o cfetch --output-format csv -- python3 bench.py --calibrate-copy {COPY_GIB} --steps 3 > {d}/cfetch.json")
    L.append(f"rocprofv3 --pmc WRITE_SIZE -d {d}/cwrite -o cwrite --output-format csv -- python3 bench.py --calibrate-copy {COPY_GIB} --steps 3")
    L.append("```\n")
    L.append("## Kernel trace (`--kernel-trace --stats`), this library's kernels only\n")
    L.append("| Kernel | Calls | Avg (ms) | Min (ms) | Max (ms) | StdDev (ms) |")
    L.append("|---|---|---|---|---|---|")
    for r in stats:
        L.append(f"| {r['Name']} | {r['Calls']} | {float(r['AverageNs']) / 1e6:.4f} | {float(r['MinNs']) / 1e6:.4f} | "
                 f"{float(r['MaxNs']) / 1e6:.4f} | {float(r['StdDev']) / 1e6:.4f} |")
    by_name = {r["Name"]: r for r in stats}
    avg_ms = float(by_name[dom]["AverageNs"]) / 1e6
    L.append("")
    L.append("`nbo_probe_rmw2` (region probe of the state placement), `nbo_fill_zero` (fresh state) and `nbo_cast_master` "
             f"run while the optimizer is set up, before the warm-up steps; the step itself is `{norm_k}` -> `nbo_finalize` "
             f"-> `{dom}`.\n")
    L.append(f"`bench.py` in the same run reported `roofline.avg_launch_ms` = {bench['roofline']['avg_launch_ms']} (HIP events "
             f"on the launch stream) against {avg_ms:.4f} ms here; `ms_per_step` = {bench['ms_per_step']}, `value` = "
             f"{bench['value']} GB/s.\n")
    L.append(f"Algorithmic bytes per launch of `{dom}`: {n} params x {upd_b} B = {n * upd_b / 1e9:.2f} GB -> "
             f"{n * upd_b / avg_ms / 1e6:.0f} GB/s = {n * upd_b / avg_ms / 1e6 / 8000 * 100:.1f} % of 8 TB/s.\n")
    L.append("## HBM traffic (`--pmc FETCH_SIZE`, `--pmc WRITE_SIZE`), per dispatch\n")
    L.append(f"Calibration: the library's plain copy kernel over {COPY_GIB} GiB (reads {copy_kib:.0f} KiB, writes "
             f"{copy_kib:.0f} KiB) makes `FETCH_SIZE` read {_mean(cf[1:]):.1f} and `WRITE_SIZE` {_mean(cw[1:]):.1f}; "
             f"scale factors {f_scale:.4f} and {w_scale:.4f} KiB per counter unit.\n")
    L.append("| Kernel | FETCH_SIZE (avg) | fetched GB | WRITE_SIZE (avg) | written GB | algorithmic R / W GB |")
    L.append("|---|---|---|---|---|---|")
    alg = {dom: (n * upd_b / 2 / 1e9, n * upd_b / 2 / 1e9), norm_k: (n * 2 / 1e9, 0.0), "nbo_finalize": (0.0, 0.0)}
    traffic = {}
    for k in (norm_k, "nbo_finalize", dom):
        fv, wv = _mean(fetch[k]), _mean(write[k])
        fg, wg = fv * f_scale * 1024 / 1e9, wv * w_scale * 1024 / 1e9
        L.append(f"| {k} | {fv:.1f} | {fg:.3f} | {wv:.1f} | {wg:.3f} | {alg[k][0]:.3f} / {alg[k][1]:.3f} |")
        traffic[k] = {"fetch_bytes": round(fv * f_scale * 1024), "write_bytes": round(wv * w_scale * 1024)}
    t, tn = traffic[dom], traffic[norm_k]
    upd_bytes = t["fetch_bytes"] + t["write_bytes"]
    L.append("")
    L.append(f"Update kernel: {upd_bytes / 1e9:.2f} GB of HBM traffic per launch against {n * upd_b / 1e9:.2f} GB algorithmic "
             f"(ratio {upd_bytes / (n * upd_b):.4f}).\n")
    norm_ms = float(by_name[norm_k]["AverageNs"]) / 1e6
    fin_ms = float(by_name["nbo_finalize"]["AverageNs"]) / 1e6
    step_bytes = upd_bytes + tn["fetch_bytes"] + tn["write_bytes"]
    L.append(f"Counter-derived HBM throughput: update kernel {upd_bytes / 1e9:.2f} GB / {avg_ms:.4f} ms = "
             f"{upd_bytes / avg_ms / 1e6:.0f} GB/s = {upd_bytes / avg_ms / 1e6 / 80:.1f} % of the 8 TB/s peak; norm pass "
             f"{tn['fetch_bytes'] / 1e9:.2f} GB / {norm_ms:.4f} ms = {tn['fetch_bytes'] / norm_ms / 1e6:.0f} GB/s; the three "
             f"kernels of a step together {step_bytes / 1e9:.2f} GB / {avg_ms + norm_ms + fin_ms:.4f} ms = "
             f"{step_bytes / (avg_ms + norm_ms + fin_ms) / 1e6:.0f} GB/s = "
             f"{step_bytes / (avg_ms + norm_ms + fin_ms) / 1e6 / 80:.1f} % of peak (wall clock per step in the same run: "
             f"{bench['ms_per_step']} ms).\n")
    L.append(f"For scale: the plain copy kernel of the calibration run ({COPY_GIB} GiB in, {COPY_GIB} GiB out, source and "
             f"destination both the caller's allocations) moved {copy['GBps']} GB/s in the same session.\n")
    text = "\n".join(L)
    os.makedirs(os.path.join(ROOT, "profiles"), exist_ok=True)
    md = os.path.join("profiles", f"adamw_fused_step_{workload.replace('1.1b', '1b').replace('-', '_').replace('.', '_')}.md")
    with open(os.path.join(ROOT, md), "w") as f:
        f.write(text)
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    table = {}
    if os.path.exists(tpath):
        with open(tpath) as f:
            table = json.load(f)
    table[f"{workload}:{dom}"] = upd_bytes
    table.setdefault("_detail", {})
    if "workload" in table["_detail"]:  # the single-workload layout of earlier files
        table["_detail"] = {table["_detail"]["workload"]: {k: v for k, v in table["_detail"].items() if k != "workload"}}
    table["_detail"][workload] = {
        "per_launch_bytes": traffic,
        "calibration": {"fetch_KiB_per_unit": f_scale, "write_KiB_per_unit": w_scale},
        "source": md, "commit": _commit(), "date": datetime.date.today().isoformat(),
        "kernel_source_sha256": kernel_source_hash()}
    with open(tpath, "w") as f:
        json.dump(table, f, indent=1)
    return text


def counter_table(base: str, kernels=None) -> str:
    """Markdown table of the per-dispatch averages of every counter of a `rocprofv3 --pmc` run
    under `base`, one column per kernel of this library (or those named)."""
    acc = {}
    with open(_one(os.path.join(base, "**", "*counter_collection.csv*"))) as f:
        for r in csv.DictReader(f):
            k = r["Kernel_Name"]
            if not k.startswith("nbo_") or (kernels and k not in kernels):
                continue
            acc.setdefault(r["Counter_Name"], {}).setdefault(k, []).append(float(r["Counter_Value"]))
    cols = sorted({k for c in acc.values() for k in c})
    lines = ["| Counter | " + " | ".join(f"{k} (avg of {len(next(iter(acc.values()))[k])} dispatches)" for k in cols) + " |",
             "|---|" + "---|" * len(cols)]
    for c in sorted(acc):
        lines.append(f"| {c} | " + " | ".join(f"{_mean(acc[c][k]):,.0f}" if k in acc[c] else "-" for k in cols) + " |")
    return "\n".join(lines)


def main(base: str, kernels=None) -> None:
    if os.path.isdir(os.path.join(base, "kt")):
        print(summarize(base))
    else:  # a single --pmc run: just the table
        print(counter_table(base, kernels))


if __name__ == "__main__":
    if len(sys.argv) < 2:
        sys.exit("usage: python -m nabla_amd.profile_summary DIR [kernel,kernel,...]")
    main(sys.argv[1], sys.argv[2].split(",") if len(sys.argv) > 2 else None)
