"""rocprofv3 profiles of bench.py's workloads, and the short text summaries / counter table made from them.

    python snntc-2023_amd/snntc_amd/profile_tables.py collect [--workloads cfg2 cfg3 ...] [--raw DIR] [--out DIR]

runs, once per workload and from the repository root,

    rocprofv3 --kernel-trace --stats          -- python3 bench.py --workload W --steps 20 --warmup 5 --no-cpu-baseline
    rocprofv3 --pmc FETCH_SIZE                -- python3 bench.py --workload W --steps 3 --warmup 1 --no-cpu-baseline --no-graph --calibration-copies 3
    rocprofv3 --pmc WRITE_SIZE                -- (the same command)
    rocprofv3 --pmc SQ_ACTIVE_INST_VALU SQ_INSTS_VALU SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAVES GRBM_GUI_ACTIVE
                                              -- (the same command without --calibration-copies)

each pass a run of its own under a time limit (counters and traces are never combined), keeps the raw
output under --raw DIR and writes into --out (default profiles/):

    <W>_step_kernel_trace.txt     top kernels by total time, with the bench line of the traced run
    <W>_hbm_traffic_pmc.txt       FETCH_SIZE / WRITE_SIZE per launch, scaled by what the plain 256 MiB device
                                  copies of the same run read on those counters
    <W>_valu_utilisation_pmc.txt  vector instructions and the share of clocks in which one issues
    counters.json                 per workload and bench kernel name: HBM bytes per launch and VALU busy,
                                  averaged over the launches of a step, with the commit they were taken at
                                  (bench.py reads this table for the roofline.traffic field)

`summarise` redoes the text files and the table from raw output that is already there (kept with --keep-raw).
"""
import argparse
import tempfile
import collections
import json
import os
import re
import sqlite3
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

TRACE_ARGS = ["--steps", "20", "--warmup", "5", "--no-cpu-baseline"]
PMC_ARGS = ["--steps", "3", "--warmup", "1", "--no-cpu-baseline", "--no-graph"]
VALU_COUNTERS = ["SQ_ACTIVE_INST_VALU", "SQ_INSTS_VALU", "SQ_BUSY_CYCLES", "SQ_WAVE_CYCLES", "SQ_WAVES", "GRBM_GUI_ACTIVE"]
COPY_KIB = 256 * 1024                 # one calibration copy reads and writes this many KiB
N_COPIES = 3
N_SIMDS = 1024                        # 256 CUs x 4
N_XCDS = 8

# kernel symbol -> the name bench.py's per-kernel timing uses
BENCH_NAMES = [
    (r"scan_(filter|lds|lds_split)_kernel|(^|[^_])scan_kernel", "scan"),
    (r"merge_patches_kernel", "merge_patches"),
    (r"sort_segments_kernel", "sort_segments"),
    (r"cv_grad_input_chan_kernel|fc_grad_input_kernel<true>", "cv_grad_input"),
    (r"fc_grad_input_kernel", "fc_grad_input"),
    (r"cv_grad_weight_|grad_weight_dense_kernel|grad_weight_kernel", "grad_weight"),
    (r"fc_backward_narrow_kernel", "fc_backward_narrow"),
    (r"backward_prologue_kernel", "prep_upstream"),
    (r"reduce_partials_kernel", "reduce_partials"),
    (r"min_pool_forward_kernel", "min_pool"),
    (r"min_pool_backward_kernel", "min_pool_grad"),
    (r"pad_time_kernel", "pad_time"),
    (r"crop_time_kernel", "crop_time"),
    (r"cv_col2im_kernel", "cv_col2im"),
    (r"softmax_time_loss_kernel", "softmax_time_loss"),
    (r"sgd_update_kernel", "sgd_update"),
]


def short(name):
    return name.replace("snntc::(anonymous namespace)::", "").replace("void ", "").split("(")[0]


def bench_name(kernel):
    for pat, name in BENCH_NAMES:
        if re.search(pat, kernel):
            return name
    return None


def emits_causal_sets(kernel):
    """Scan instantiations whose last template argument is `true` also write causal-set sizes: they belong
    to bench.py's accounting forward, not to the timed step."""
    return bench_name(kernel) == "scan" and re.search(r"true>$", kernel) is not None


def find_db(directory):
    hits = []
    for base, _dirs, files in os.walk(directory):
        hits += [os.path.join(base, f) for f in files if f.endswith(".db")]
    if not hits:
        raise FileNotFoundError(f"no rocprofv3 database under {directory}")
    return sorted(hits)[-1]


def run_pass(raw, tag, rocprof_args, bench_args, limit):
    out_dir = os.path.join(raw, tag)
    subprocess.run(["rm", "-rf", out_dir], check=True)
    cmd = ["rocprofv3"] + rocprof_args + ["-d", out_dir, "-o", tag, "--", "python3", "bench.py"] + bench_args
    shown = " ".join(["rocprofv3"] + rocprof_args + ["--", "python3", "bench.py"] + bench_args)
    print("+", shown, flush=True)
    env = dict(os.environ, TMPDIR="/tmp")
    with open(os.path.join(raw, tag + ".json"), "w") as so, open(os.path.join(raw, tag + ".err"), "w") as se:
        r = subprocess.run(["timeout", "-s", "KILL", str(limit)] + cmd, cwd=ROOT, stdout=so, stderr=se, env=env)
    if r.returncode != 0:
        raise RuntimeError(f"{shown}: exit status {r.returncode} (see {raw}/{tag}.err)")
    with open(os.path.join(raw, tag + ".cmd"), "w") as f:
        f.write(shown + "\n")


def collect(workloads, raw):
    os.makedirs(raw, exist_ok=True)
    for w in workloads:
        run_pass(raw, f"{w}_trace", ["--kernel-trace", "--stats"], ["--workload", w] + TRACE_ARGS, 300)
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            run_pass(raw, f"{w}_{counter}", ["--pmc", counter],
                     ["--workload", w] + PMC_ARGS + ["--calibration-copies", str(N_COPIES)], 180)
        run_pass(raw, f"{w}_valu", ["--pmc"] + VALU_COUNTERS, ["--workload", w] + PMC_ARGS, 180)


def counters_by_kernel(db):
    """{kernel symbol: {counter: (sum over dispatches, dispatches)}}"""
    con = sqlite3.connect(db)
    rows = con.execute("select kernel_name, counter_name, sum(value), count(*) from counters_collection "
                       "group by kernel_name, counter_name").fetchall()
    out = collections.OrderedDict()
    for kernel, counter, total, n in rows:
        out.setdefault(short(kernel), {})[counter] = (float(total), int(n))
    return out


def read_cmd(raw, tag):
    with open(os.path.join(raw, tag + ".cmd")) as f:
        return f.read().strip()


def git_commit():
    r = subprocess.run(["git", "rev-parse", "--short", "HEAD"], cwd=ROOT, capture_output=True, text=True)
    return r.stdout.strip() or "unknown"


def summarise(workloads, raw, out, commit=None):
    os.makedirs(out, exist_ok=True)
    table = {"commit": commit or git_commit(),
             "note": "rocprofv3 --pmc readings per launch, averaged over the launches of a kernel in one step of the "
                     "workload (scan instantiations that also write causal-set sizes excluded: they belong to the "
                     "accounting forward): hbm_bytes_per_launch = FETCH_SIZE * f + WRITE_SIZE * g KiB with the "
                     "scale factors f, g of the calibration copies of the same run; valu_busy = SQ_ACTIVE_INST_VALU "
                     "* 4 / 1024 SIMDs / (GRBM_GUI_ACTIVE / 8).  Written by snntc_amd/profile_tables.py.",
             "workloads": {}}
    for w in workloads:
        # ---- kernel trace
        line = open(os.path.join(raw, f"{w}_trace.json")).read().strip().splitlines()[-1]
        d = json.loads(line)
        r = d["roofline"]
        con = sqlite3.connect(find_db(os.path.join(raw, f"{w}_trace")))
        rows = list(con.execute("select name,total_calls,total_duration,average,percentage from top_kernels"))
        text = [f"# rocprofv3 kernel-trace summary: bench.py --workload {w} (MI355X, gfx950)",
                f"# command: {read_cmd(raw, w + '_trace')}",
                "# The run covers graph warm-up and capture, the timed pass (HIP-graph replays), an eager pass, the event-timed",
                "# pass and the accounting forward (scan instantiations whose last template argument is true belong to the latter).",
                f"# bench.py line of the same run (under the profiler): value={d['value']:.0f} samples/s, ms_per_step={d['ms_per_step']:.4f};",
                f"# dominant kernel {r['kernel']}: avg_launch_us={r['avg_launch_us']:.1f} (HIP events in bench.py), roofline.frac={r['frac']:.4f}",
                "# Kernel names: snntc:: prefixes and argument lists dropped; at::native::* and __amd_rocclr_* are PyTorch's kernels.",
                "", "%-72s %8s %14s %12s %7s" % ("kernel", "calls", "total_us", "avg_us", "%")]
        for name, calls, tot, avg, pct in rows[:24]:
            text.append("%-72s %8d %14.1f %12.2f %7.2f" % (short(name)[:72], calls, tot, avg, pct))
        open(os.path.join(out, f"{w}_step_kernel_trace.txt"), "w").write("\n".join(text) + "\n")

        # ---- HBM traffic
        fetch = counters_by_kernel(find_db(os.path.join(raw, f"{w}_FETCH_SIZE")))
        write = counters_by_kernel(find_db(os.path.join(raw, f"{w}_WRITE_SIZE")))
        copy = next(k for k in fetch if "copyBuffer" in k)
        sf = COPY_KIB / (fetch[copy]["FETCH_SIZE"][0] / N_COPIES)
        sw = COPY_KIB / (write[copy]["WRITE_SIZE"][0] / N_COPIES)
        text = [f"# HBM traffic of the library's kernels, bench.py --workload {w} (MI355X, gfx950): KiB per dispatch",
                f"# command (FETCH_SIZE): {read_cmd(raw, w + '_FETCH_SIZE')}",
                f"# command (WRITE_SIZE): {read_cmd(raw, w + '_WRITE_SIZE')}",
                f"# calibration: the {N_COPIES} plain device copies of 256 MiB at the start of each run ({COPY_KIB} KiB read and written each):",
                f"# FETCH_SIZE reads {fetch[copy]['FETCH_SIZE'][0] / N_COPIES:.1f} per copy -> scale {sf:.3f}; WRITE_SIZE reads "
                f"{write[copy]['WRITE_SIZE'][0] / N_COPIES:.1f} -> scale {sw:.3f} (small copies of the run included: < 0.1 %)",
                "", "%-48s %9s %16s %16s %14s" % ("kernel", "launches", "FETCH KiB/launch", "WRITE KiB/launch", "HBM MB/launch")]
        per_name = collections.defaultdict(lambda: [0.0, 0])
        for k, c in fetch.items():
            if bench_name(k) is None or "FETCH_SIZE" not in c or k not in write:
                continue
            n = c["FETCH_SIZE"][1]
            fv, wv = c["FETCH_SIZE"][0] / n, write[k]["WRITE_SIZE"][0] / write[k]["WRITE_SIZE"][1]
            mb = (fv * sf + wv * sw) * 1024 / 1e6
            text.append("%-48s %9d %16.1f %16.1f %14.1f" % (k[:48], n, fv, wv, mb))
            if not emits_causal_sets(k):
                per_name[bench_name(k)][0] += mb * 1e6 * n
                per_name[bench_name(k)][1] += n
        open(os.path.join(out, f"{w}_hbm_traffic_pmc.txt"), "w").write("\n".join(text) + "\n")

        # ---- VALU utilisation
        valu = counters_by_kernel(find_db(os.path.join(raw, f"{w}_valu")))
        text = [f"# VALU utilisation of the library's kernels, bench.py --workload {w} (MI355X, gfx950): per dispatch",
                f"# command: {read_cmd(raw, w + '_valu')}",
                "# GRBM_GUI_ACTIVE is summed over the 8 XCDs: clocks of a dispatch = GRBM_GUI_ACTIVE / 8.",
                "# VALU busy = SQ_ACTIVE_INST_VALU * 4 / (1024 SIMDs) / clocks  (a wave64 instruction occupies a SIMD for 4 clocks)",
                "# wave-instr = SQ_INSTS_VALU per dispatch (vector instructions issued, per wavefront)",
                "", "%-48s %9s %12s %10s %16s %10s" % ("kernel", "launches", "clocks", "us@2.3GHz", "VALU wave-instr", "VALU busy")]
        busy_by_name = collections.defaultdict(lambda: [0.0, 0.0])
        for k, c in valu.items():
            if bench_name(k) is None or "GRBM_GUI_ACTIVE" not in c:
                continue
            n = c["GRBM_GUI_ACTIVE"][1]
            clk = c["GRBM_GUI_ACTIVE"][0] / n / N_XCDS
            act = c["SQ_ACTIVE_INST_VALU"][0] / n
            text.append("%-48s %9d %12.0f %10.1f %16.0f %10.3f" % (k[:48], n, clk, clk / 2300, c["SQ_INSTS_VALU"][0] / n,
                                                                   act * 4 / N_SIMDS / clk))
            if not emits_causal_sets(k):
                busy_by_name[bench_name(k)][0] += act * 4 / N_SIMDS * n
                busy_by_name[bench_name(k)][1] += clk * n
        open(os.path.join(out, f"{w}_valu_utilisation_pmc.txt"), "w").write("\n".join(text) + "\n")

        entry = {}
        for name, (total, n) in per_name.items():
            entry.setdefault(name, {})["hbm_bytes_per_launch"] = total / n
        for name, (act, clk) in busy_by_name.items():
            entry.setdefault(name, {})["valu_busy"] = act / clk
        table["workloads"][w] = entry
    # workloads summarised earlier stay in the table
    path = os.path.join(out, "counters.json")
    if os.path.exists(path):
        try:
            old = json.load(open(path))
            for w, e in old.get("workloads", {}).items():
                table["workloads"].setdefault(w, dict(e, carried_from_commit=old.get("commit")))
        except ValueError:
            pass
    json.dump(table, open(path, "w"), indent=1, sort_keys=True)
    print(f"wrote {len(workloads)} workload(s) into {out}")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("action", choices=["collect", "summarise"])
    ap.add_argument("--workloads", nargs="+", default=["cfg2", "cfg3", "cfg4", "cfg5"])
    ap.add_argument("--raw", default=None, help="folder for the raw rocprofv3 output (collect: a temporary one by default)")
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles"))
    ap.add_argument("--keep-raw", action="store_true", help="keep the rocprofv3 databases after summarising")
    ap.add_argument("--commit", default=None, help="commit the measured tree is at (default: git rev-parse HEAD here)")
    args = ap.parse_args()
    if args.raw is None:
        if args.action == "summarise":
            ap.error("summarise needs --raw (the folder a collect run with --keep-raw left)")
        args.raw = tempfile.mkdtemp(prefix="snntc_profiles_")
    if args.action == "collect":
        collect(args.workloads, args.raw)
    summarise(args.workloads, args.raw, args.out, args.commit)
    if args.action == "collect" and not args.keep_raw:
        for w in args.workloads:
            for tag in ("trace", "FETCH_SIZE", "WRITE_SIZE", "valu"):
                subprocess.run(["rm", "-rf", os.path.join(args.raw, f"{w}_{tag}")], check=True)


if __name__ == "__main__":
    sys.exit(main())
