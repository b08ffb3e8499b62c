"""Turn the rocprofv3 output of a bench.py workload into the short text summary kept under profiles/
and into that workload's entry of profiles/traffic.json (the HBM bytes bench.py reports as
`roofline.traffic`).  The non-interactive counterpart of the reference's profile sweeps
(test_linear.py:126-130, test_ffn.py:96-109), which print wall-clock times only.

    python -m ffn_kernel_amd.profile_summary OUT --workload cfg4 [--traffic-json profiles/traffic.json] > profiles/<name>.txt

OUT holds one sub-directory per rocprofv3 run of `python3 bench.py --workload W --steps S --warmup U
--cpu-rows 0 [--no-decode]`, each made with `--output-format csv -d OUT/<run> -o t`:
    trace   --kernel-trace --stats
    fetch   --pmc FETCH_SIZE            write   --pmc WRITE_SIZE
    cfetch / cwrite : the same two counters on `--workload copy1g` (a 1 GiB device copy; calibration)
    any other sub-directory with a counter_collection.csv is listed as it is (e.g. sq, tcc).
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import re
import sys
from pathlib import Path

GIB_KIB = 1 << 20


def _counters(run_dir: Path):
    """{kernel: {counter: [values per dispatch]}} of one --pmc run."""
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    for f in glob.glob(str(run_dir / "**" / "*counter_collection.csv"), recursive=True):
        with open(f) as fh:
            for r in csv.DictReader(fh):
                agg[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return agg


def _kernel_stats(run_dir: Path):
    rows = []
    for f in glob.glob(str(run_dir / "**" / "*kernel_stats.csv"), recursive=True):
        with open(f) as fh:
            rows += list(csv.DictReader(fh))
    return rows


def _calibration(out: Path, counter: str, sub: str):
    """true KiB / counter KiB for a plain 1 GiB device copy, or None when the run is absent."""
    best = None
    for kernel, cs in _counters(out / sub).items():
        for c, v in cs.items():
            avg = sum(v) / len(v)
            if c == counter and avg > 5e5:
                best = (kernel, avg, GIB_KIB / avg)
    return best


def _ours(kernel: str) -> bool:
    return "ffnk::" in kernel


# Which kernels make up a workload's roofline entry in bench.py.
def _roofline_kernels(workload: str):
    if workload == "cfg4":  # the up-projection + SwiGLU launches (DUAL template argument)
        return lambda k: re.search(r"RoutedGemmCfg<\d+, \d+, \d+, \d+, true", k) is not None
    return _ours  # decode / linear workloads: every launch of one call


def summarize(out: Path, workload: str, traffic_json: Path | None, min_pct: float = 0.5) -> str:
    lines = [f"workload: {workload}"]
    stats = _kernel_stats(out / "trace")
    # counters are listed for the kernels that matter: at least min_pct of the traced kernel time
    shown = {r["Name"] for r in stats if float(r["Percentage"]) >= min_pct} if stats else None
    if stats:
        lines += ["", "== rocprofv3 --kernel-trace --stats (ns) =="]
        for r in stats:
            if float(r["Percentage"]) > 0.05:
                lines.append(f"{r['Name'][:110]:110s} calls={r['Calls']:>4s} avg={float(r['AverageNs']):11.0f} "
                             f"min={r['MinNs']:>9s} max={r['MaxNs']:>9s} pct={r['Percentage']}")
    lines += ["", "== rocprofv3 --pmc (average per dispatch) =="]
    per_kernel = {}
    for sub in sorted(p.name for p in out.iterdir() if p.is_dir() and p.name not in ("trace", "cfetch", "cwrite")):
        for kernel, cs in sorted(_counters(out / sub).items()):
            if not _ours(kernel) and "Cijk" not in kernel:
                continue
            if shown is not None and kernel not in shown:
                continue
            for c, v in sorted(cs.items()):
                lines.append(f"{kernel[:100]:100s} {c:30s} n={len(v):3d} avg={sum(v) / len(v):.5g}")
                per_kernel[(kernel, c)] = v
    # What the counters say about each listed kernel, as far as the runs at hand allow: the clock the part held
    # (GRBM_GUI_ACTIVE is summed over the 8 XCDs; per XCD it is the launch's duration in shader cycles, taken in another
    # run than the traced duration), and the share of the 1024 SIMD-cycles per chip cycle in which an MFMA executed.
    avg_ns = {r["Name"]: float(r["AverageNs"]) for r in stats} if stats else {}
    derived = []
    for kernel in sorted({k for (k, _) in per_kernel}):
        def mean(c):
            v = per_kernel.get((kernel, c))
            return sum(v) / len(v) if v else None
        gui, mfma = mean("GRBM_GUI_ACTIVE"), mean("SQ_VALU_MFMA_BUSY_CYCLES")
        parts = []
        if gui and avg_ns.get(kernel, 0.0) >= 2e5:  # shorter launches: the counter's window is mostly idle time around the kernel
            parts.append(f"cycles per XCD {gui / 8:.4g}, i.e. {gui / 8 / avg_ns[kernel]:.2f} GHz over the traced {avg_ns[kernel] / 1e3:.1f} us")
        if gui and mfma and avg_ns.get(kernel, 0.0) >= 2e5:
            parts.append(f"MFMA busy {100 * mfma / (gui / 8 * 1024):.1f} % of SIMD-cycles")
        if parts:
            derived.append(f"{kernel[:100]:100s} " + "; ".join(parts))
    if derived:
        lines += ["", "== derived per kernel =="] + derived
    cal = {}
    lines += ["", "== calibration: plain 1 GiB device copy (reads 1 GiB, writes 1 GiB per dispatch) =="]
    for counter, sub in (("FETCH_SIZE", "cfetch"), ("WRITE_SIZE", "cwrite")):
        got = _calibration(out, counter, sub)
        if got:
            lines.append(f"{got[0][:90]:90s} {counter:12s} avg={got[1]:.5g} KiB -> factor (true KiB / counter) = {got[2]:.4f}")
            cal[counter] = got[2]
    if "FETCH_SIZE" in cal and "WRITE_SIZE" in cal:
        pick = _roofline_kernels(workload)
        names = sorted({k for (k, c) in per_kernel if c == "FETCH_SIZE" and pick(k)})
        if names:
            # calls of the workload in the run = dispatches of its most frequent kernel (a row partition shared
            # between calls is launched once per run and weighs in with that share)
            n_calls = max(len(per_kernel[(k, "FETCH_SIZE")]) for k in names)
            fetch = sum(sum(per_kernel[(k, "FETCH_SIZE")]) for k in names) / n_calls
            write = sum(sum(per_kernel.get((k, "WRITE_SIZE"), [0.0])) for k in names) / n_calls
            nbytes = (fetch * cal["FETCH_SIZE"] + write * cal["WRITE_SIZE"]) * 1024
            lines += ["", "== HBM traffic of the roofline kernel(s), per call ==",
                      f"kernels: {len(names)} ({n_calls} calls in the run)"]
            lines += [f"  {k[:120]}" for k in names]
            lines.append(f"FETCH_SIZE {fetch:.5g} KiB x {cal['FETCH_SIZE']:.3f} + WRITE_SIZE {write:.5g} KiB x "
                         f"{cal['WRITE_SIZE']:.3f} = {nbytes / 1e6:.1f} MB")
            dur = sum(avg_ns.get(k, 0.0) for k in names)
            if dur > 0:
                lines.append(f"over the traced {dur / 1e3:.1f} us of these kernels: {nbytes / dur:.0f} GB/s of HBM traffic")
            if traffic_json is not None:
                table = json.loads(traffic_json.read_text()) if traffic_json.exists() else {}
                table[workload] = {"bytes": round(nbytes), "fetch_kib": round(fetch, 1), "write_kib": round(write, 1),
                                   "fetch_factor": round(cal["FETCH_SIZE"], 4), "write_factor": round(cal["WRITE_SIZE"], 4)}
                traffic_json.write_text(json.dumps(table, indent=1, sort_keys=True) + "\n")
    return "\n".join(lines) + "\n"


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("out", type=Path)
    ap.add_argument("--workload", required=True)
    ap.add_argument("--traffic-json", type=Path, default=None)
    ap.add_argument("--min-pct", type=float, default=0.5, help="list counters of kernels with at least this share of the time")
    args = ap.parse_args()
    sys.stdout.write(summarize(args.out, args.workload, args.traffic_json, args.min_pct))
    return 0


if __name__ == "__main__":
    sys.exit(main())
