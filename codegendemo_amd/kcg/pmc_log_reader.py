"""Reads profiler output and sets the engine's kernels beside the library's: the role of the
reference's pmc_log_reader.py (pmc_log_reader.py:1-31), which scrapes a `hipprof --pmc` text log for the
"performance" lines that follow kernel names containing "GEMM_MNK" (generated kernels) or "Cij"
(the Tensile kernels behind torch.matmul) and prints the two lists `eps_torch` / `eps_kcg`.

On MI355X the profiler is rocprofv3 and its output is CSV:

    rocprofv3 --kernel-trace --stats --output-format csv -d out/trace -o run -- python3 bench.py
    rocprofv3 --pmc SQ_INSTS_MFMA SQ_LDS_BANK_CONFLICT --output-format csv -d out/pmc -o run -- python3 bench.py
    python -m codegendemo_amd.kcg.pmc_log_reader out [--mnk 4096x4096x4096] [--markdown]

* `*_kernel_trace.csv` (one row per dispatch): duration = End_Timestamp - Start_Timestamp; Gflops per
  dispatch = 2*M*N*K / duration, M, N, K read from the generated kernel's own name
  (`GEMM_MNK<M>x<N>x<K>_...`, main.cc:119-145); a library kernel has no shape in its name and is priced with
  `--mnk`, or with the shape of the generated kernels when those all share one.
* `*_counter_collection.csv` (one row per dispatch and counter): mean counter value per dispatch and kernel.
"""
import argparse
import csv
import glob
import json
import os
import re
import sys
from collections import OrderedDict, defaultdict

KEY_KCG = "GEMM_MNK"      # pmc_log_reader.py:5
KEY_TORCH = "Cij"         # pmc_log_reader.py:6
_NAME_MNK = re.compile(r"GEMM_MNK(\d+)x(\d+)x(\d+)_")


def kernel_family(name: str):
    """'kcg' for a generated kernel, 'torch' for a Tensile/hipBLASLt kernel, None for anything else."""
    if KEY_KCG in name:
        return "kcg"
    if name.startswith(KEY_TORCH) or (" " + KEY_TORCH) in name:
        return "torch"
    return None


def flops_from_name(name: str):
    """2*M*N*K of a generated kernel, from its name; None when the name carries no shape."""
    m = _NAME_MNK.search(name)
    if not m:
        return None
    M, N, K = (int(g) for g in m.groups())
    return 2 * M * N * K


def find_csv(paths, suffix):
    out = []
    for p in paths:
        if os.path.isdir(p):
            out += sorted(glob.glob(os.path.join(p, "**", "*" + suffix), recursive=True))
        elif p.endswith(suffix):
            out.append(p)
    return out


def read_kernel_trace(files):
    """{kernel name: [duration_ns, ...]} in dispatch order, generated and library kernels only."""
    out = OrderedDict()
    for f in files:
        with open(f, newline="") as fh:
            for row in csv.DictReader(fh):
                name = row["Kernel_Name"]
                if kernel_family(name) is None:
                    continue
                out.setdefault(name, []).append(int(row["End_Timestamp"]) - int(row["Start_Timestamp"]))
    return out


def read_counters(files):
    """{kernel name: {counter: mean value per dispatch}}; rows of one dispatch and counter (one per
    XCD or shader engine for some counters) are summed first."""
    per_dispatch = defaultdict(lambda: defaultdict(float))
    names = {}
    for f in files:
        with open(f, newline="") as fh:
            for row in csv.DictReader(fh):
                name = row["Kernel_Name"]
                if kernel_family(name) is None:
                    continue
                key = (f, row["Dispatch_Id"])
                names[key] = name
                per_dispatch[key][row["Counter_Name"]] += float(row["Counter_Value"])
    sums = defaultdict(lambda: defaultdict(list))
    for key, ctrs in per_dispatch.items():
        for c, v in ctrs.items():
            sums[names[key]][c].append(v)
    return {n: {c: sum(v) / len(v) for c, v in d.items()} for n, d in sums.items()}


def price(trace, mnk=None):
    """Per kernel: family, calls, mean/min/max ns, Gflops per dispatch.  `mnk` prices library kernels."""
    kcg_flops = {flops_from_name(n) for n in trace if kernel_family(n) == "kcg"} - {None}
    lib_flops = None
    if mnk:
        M, N, K = (int(x) for x in mnk.lower().split("x"))
        lib_flops = 2 * M * N * K
    elif len(kcg_flops) == 1:
        lib_flops = next(iter(kcg_flops))
    rows = []
    for name, d in trace.items():
        fam = kernel_family(name)
        fl = flops_from_name(name) if fam == "kcg" else lib_flops
        rows.append({
            "family": fam, "name": name, "calls": len(d), "mean_ns": sum(d) / len(d), "min_ns": min(d), "max_ns": max(d),
            "gflops": [fl / ns for ns in d] if fl else None,       # flop per ns == Gflop/s
        })
    return rows


def _fmt_eps(rows, fam):
    vals = []
    for r in rows:
        if r["family"] == fam and r["gflops"]:
            vals += ["%f(Gflops)" % g for g in r["gflops"]]
    return vals


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("paths", nargs="+", help="rocprofv3 output directories or CSV files")
    ap.add_argument("--mnk", help="MxNxK of the library GEMM dispatches, e.g. 4096x4096x4096")
    ap.add_argument("--markdown", action="store_true", help="tables instead of the reference's two lists")
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args(argv)
    trace = read_kernel_trace(find_csv(args.paths, "kernel_trace.csv"))
    counters = read_counters(find_csv(args.paths, "counter_collection.csv"))
    rows = price(trace, args.mnk)
    if args.json:
        print(json.dumps({"kernels": [{k: v for k, v in r.items() if k != "gflops"} |
                                      {"mean_gflops": (sum(r["gflops"]) / len(r["gflops"]) if r["gflops"] else None)}
                                      for r in rows], "counters": counters}))
        return 0
    if args.markdown:
        print("| kernel | family | calls | mean ns | min ns | max ns | mean TFLOP/s |\n|---|---|---|---|---|---|---|")
        for r in rows:
            tf = "%.1f" % (sum(r["gflops"]) / len(r["gflops"]) / 1e3) if r["gflops"] else "-"
            print("| `%s` | %s | %d | %.0f | %d | %d | %s |" % (r["name"][:120], r["family"], r["calls"], r["mean_ns"],
                                                                r["min_ns"], r["max_ns"], tf))
        if counters:
            ctr_names = sorted({c for d in counters.values() for c in d})
            kernels = list(counters)
            print("\n| counter (mean per dispatch) | " + " | ".join("`%s`" % k[:60] for k in kernels) + " |")
            print("|---|" + "---|" * len(kernels))
            for c in ctr_names:
                print("| %s | " % c + " | ".join("%.0f" % counters[k][c] if c in counters[k] else "-" for k in kernels) + " |")
        return 0
    print("eps_torch : ", _fmt_eps(rows, "torch"))     # pmc_log_reader.py:30-31
    print("eps_kcg : ", _fmt_eps(rows, "kcg"))
    for r in rows:
        tf = " %.1f TFLOP/s" % (sum(r["gflops"]) / len(r["gflops"]) / 1e3) if r["gflops"] else ""
        print("%-5s %5d calls  mean %.1f us  min %.1f us%s  %s" % (r["family"], r["calls"], r["mean_ns"] / 1e3,
                                                                   r["min_ns"] / 1e3, tf, r["name"][:100]))
    for k, d in counters.items():
        print("counters of", k[:100])
        for c in sorted(d):
            print("    %-32s %.6g" % (c, d[c]))
    return 0


if __name__ == "__main__":
    sys.exit(main())
