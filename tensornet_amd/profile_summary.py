"""Turns the rocprofv3 output of three runs of bench.py into the two files under profiles/ that the
benchmark's roofline figures rest on:

    profiles/cfg3_adagrad_dim16_pull_push.md   kernel durations (kernel trace) and HBM traffic per launch
    profiles/cfg3_traffic.json                 {kernel: HBM bytes per launch}, which bench.py reads

The runs (MI355X box, from the repository root, with TMPDIR=/tmp):

    rocprofv3 --kernel-trace --stats -d prof_out/prof_trace -o t -- python3 bench.py --steps 5 --warmup 2 --no-cpu --no-others --no-traffic
    rocprofv3 --pmc FETCH_SIZE -d prof_out/prof_fetch -o f -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-others --no-traffic
    rocprofv3 --pmc WRITE_SIZE -d prof_out/prof_write -o w -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-others --no-traffic
    python3 bench.py --no-traffic > prof_out/bench_full.json
    python3 -m tensornet_amd.profile_summary --trace prof_out/prof_trace --fetch prof_out/prof_fetch \\
        --write prof_out/prof_write --bench prof_out/bench_full.json --commit <commit of the profiled tree>

With --trace and --title only (no counter runs) it writes a table of kernel durations, e.g. for the small
configurations, whose steps are a handful of short kernels (one run per configuration):

    rocprofv3 --kernel-trace --stats -d prof_out/prof_cfg1 -o t -- python3 bench.py --config cfg1 --steps 50 --warmup 5 \
        --no-cpu --no-dense --no-combiner --no-decay --no-fallback --no-traffic
    python3 -m tensornet_amd.profile_summary --trace prof_out/prof_cfg1 --title "cfg1 ..." --out profiles/<name>.md [--append]

With --counters (one or more directories of `rocprofv3 --pmc <SQ counters>` runs of the same command, at most 8 SQ
counters a run) and --title it writes the per-dispatch averages of those counters for the step's kernels and a few
ratios of them (what share of its wavefronts' time a kernel waits, and on what):

    rocprofv3 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_ANY SQ_WAIT_INST_ANY SQ_WAIT_INST_LDS SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT \
        -d prof_out/pmc_a -o p -- python3 bench.py --steps 3 --warmup 1 --no-cpu --no-dense --no-combiner --no-decay --no-fallback --no-others --no-traffic
    rocprofv3 --pmc SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_LDS SQ_INSTS_VMEM_RD SQ_INSTS_VMEM_WR SQ_ACTIVE_INST_VMEM SQ_ACTIVE_INST_VALU SQ_INST_LEVEL_VMEM \
        -d prof_out/pmc_b -o p -- python3 bench.py --steps 3 --warmup 1 --no-cpu --no-dense --no-combiner --no-decay --no-fallback --no-others --no-traffic
    python3 -m tensornet_amd.profile_summary --counters prof_out/pmc_a prof_out/pmc_b --title "..." --out profiles/<name>.md

FETCH_SIZE / WRITE_SIZE count in KiB per dispatch in units that are not bytes on every ASIC: both are
scaled by the factor that makes the same counter reproduce the known traffic of the dense Adam stream of
the same run (k_dense_adam_v4 on 2e8 parameters reads 16 B and writes 16 B per parameter).
"""
import argparse
import glob
import json
import os
import sqlite3
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DENSE_PARAMS = 2 * 10 ** 8


def short(name):
    name = name.replace("void ", "").replace("(anonymous namespace)::", "").replace("tn::", "")
    return name[:name.index("(")] if "(" in name else name


def _db(directory):
    found = glob.glob(os.path.join(directory, "**", "*_results.db"), recursive=True)
    if not found:
        raise SystemExit("no rocprofv3 result database under " + directory)
    return sqlite3.connect(found[0]).cursor()


def read_trace(directory):
    cur = _db(directory)
    rows = cur.execute("select name, count(*), avg(end-start), min(end-start), max(end-start), sum(end-start) "
                       "from kernels group by name order by 6 desc")
    return [dict(name=short(r[0]), calls=r[1], avg_ns=r[2], min_ns=r[3], max_ns=r[4]) for r in rows if "tn::" in r[0]]


def read_counter(directory):
    cur = _db(directory)
    rows = cur.execute("select kernel_name, count(*), avg(value) from counters_collection group by kernel_name")
    return {short(r[0]): r[2] for r in rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--trace")
    ap.add_argument("--counters", nargs="+", help="directories of --pmc runs: a table of their counters per kernel")
    ap.add_argument("--fetch")
    ap.add_argument("--write")
    ap.add_argument("--bench", help="file holding the JSON line of a full bench.py run")
    ap.add_argument("--title", help="durations only: heading of the table")
    ap.add_argument("--note", default="", help="durations only: a line under the heading (the command, the step time)")
    ap.add_argument("--append", action="store_true", help="durations only: add to --out instead of replacing it")
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles", "cfg3_adagrad_dim16_pull_push.md"))
    ap.add_argument("--traffic", default=os.path.join(ROOT, "profiles", "cfg3_traffic.json"))
    ap.add_argument("--commit", default=None, help="commit of the profiled tree (default: git rev-parse HEAD here)")
    args = ap.parse_args()
    if args.counters:
        if not args.title:
            raise SystemExit("--counters needs --title")
        table, names = {}, []
        for d in args.counters:
            cur = _db(d)
            for k, c, n, v in cur.execute("select kernel_name, counter_name, count(*), avg(value) from counters_collection "
                                          "where kernel_name like '%tn::%' group by kernel_name, counter_name"):
                table.setdefault(short(k), {})[c] = v
                table[short(k)]["_n"] = n
                if c not in names:
                    names.append(c)
        skip = ("k_load_rows", "k_probe<true>", "k_finish_insert", "k_reset_status")
        rows = sorted(((k, v) for k, v in table.items() if not k.startswith(skip)),
                      key=lambda kv: -kv[1].get("SQ_BUSY_CYCLES", 0))
        out = ["# %s\n" % args.title, args.note, "",
               "Per-dispatch averages (summed over the device's shader engines / XCDs as rocprofv3 reports them).\n",
               "| kernel | " + " | ".join(n.replace("SQ_", "") for n in names) + " |", "|---|" + "---|" * len(names)]
        for k, v in rows:
            out.append("| %s | " % k + " | ".join("%.3g" % v.get(n, 0) for n in names) + " |")

        def ratio(v, a, b):
            return "%.2f" % (v[a] / v[b]) if v.get(a) is not None and v.get(b) else "-"

        out += ["", "Ratios: share of its wavefronts' cycles a kernel waits for anything / for an instruction to come back / "
                    "for LDS; LDS bank-conflict cycles per cycle the LDS is busy with the kernel's instructions; vector "
                    "memory instructions in flight per wavefront cycle (of 1).\n",
                "| kernel | WAIT_ANY / WAVE_CYCLES | WAIT_INST_ANY / WAVE_CYCLES | WAIT_INST_LDS / WAVE_CYCLES | "
                "LDS_BANK_CONFLICT / ACTIVE_INST_LDS | INST_LEVEL_VMEM / WAVE_CYCLES |", "|---|---|---|---|---|---|"]
        for k, v in rows:
            out.append("| %s | %s | %s | %s | %s | %s |" % (
                k, ratio(v, "SQ_WAIT_ANY", "SQ_WAVE_CYCLES"), ratio(v, "SQ_WAIT_INST_ANY", "SQ_WAVE_CYCLES"),
                ratio(v, "SQ_WAIT_INST_LDS", "SQ_WAVE_CYCLES"), ratio(v, "SQ_LDS_BANK_CONFLICT", "SQ_ACTIVE_INST_LDS"),
                ratio(v, "SQ_INST_LEVEL_VMEM", "SQ_WAVE_CYCLES")))
        with open(args.out, "w") as f:
            f.write("\n".join(out) + "\n")
        print("wrote %s (%d kernels, %d counters)" % (args.out, len(rows), len(names)))
        return
    if not args.trace:
        raise SystemExit("--trace is needed (or --counters)")
    if not (args.fetch and args.write and args.bench):
        if not args.title:
            raise SystemExit("either --fetch, --write and --bench (the cfg3 profile) or --title (durations only)")
        trace = read_trace(args.trace)
        out = ["## %s\n" % args.title, args.note, "",
               "| kernel | launches | avg us | min us | max us |", "|---|---|---|---|---|"]
        out += ["| %s | %d | %.1f | %.1f | %.1f |" % (r["name"], r["calls"], r["avg_ns"] / 1e3, r["min_ns"] / 1e3, r["max_ns"] / 1e3)
                for r in trace]
        with open(args.out, "a" if args.append else "w") as f:
            f.write("\n".join(out) + "\n\n")
        print("wrote %s (%d kernels)" % (args.out, len(trace)))
        return
    sys.path.insert(0, ROOT)
    import bench

    line = json.loads(open(args.bench).read().strip().split("\n")[-1])
    trace = read_trace(args.trace)
    fetch, write = read_counter(args.fetch), read_counter(args.write)
    dense = [k for k in fetch if k.startswith("k_dense_adam_v4")]
    if not dense:
        raise SystemExit("the counter runs hold no k_dense_adam_v4 dispatch to scale by (run bench.py with its dense leg)")
    dense_kib = 16.0 * DENSE_PARAMS / 1024
    ff, wf = dense_kib / fetch[dense[0]], dense_kib / write[dense[0]]
    shape = line["batch_shape"]
    opt, dim = line["config"]["optimizer"], line["config"]["dim"]
    commit = args.commit or subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True,
                                           text=True).stdout.strip()
    if not commit:
        raise SystemExit("no commit to record: pass --commit (the GPU box has no .git)")

    traffic = {}
    out = ["# cfg3 pull+push (dim-16 AdaGrad, 16384 x 100 slots, 5e8 resident keys): rocprofv3 kernel trace and HBM traffic\n",
           "Written at commit `%s` by (MI355X box, from the repository root, with TMPDIR=/tmp):\n" % commit,
           "```\n"
           "rocprofv3 --kernel-trace --stats -d prof_out/prof_trace -o t -- python3 bench.py --steps 5 --warmup 2 --no-cpu --no-others --no-traffic\n"
           "rocprofv3 --pmc FETCH_SIZE -d prof_out/prof_fetch -o f -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-others --no-traffic\n"
           "rocprofv3 --pmc WRITE_SIZE -d prof_out/prof_write -o w -- python3 bench.py --steps 2 --warmup 1 --no-cpu --no-others --no-traffic\n"
           "python3 bench.py --no-traffic > prof_out/bench_full.json\n"
           "python3 -m tensornet_amd.profile_summary --trace prof_out/prof_trace --fetch prof_out/prof_fetch --write prof_out/prof_write "
           "--bench prof_out/bench_full.json --commit %s\n"
           "```\n" % commit,
           "Durations: per-dispatch `end - start` of the kernel trace, library kernels only. Traffic: FETCH_SIZE / WRITE_SIZE per "
           "dispatch, scaled by the factor the same counter shows for `k_dense_adam_v4` on 2e8 parameters (16 B read and 16 B "
           "written per parameter): FETCH x %.3f, WRITE x %.3f. `alg MB` = algorithmic bytes per launch "
           "(`bench.kernel_algorithmic_bytes`, mean batch shape of the run).\n" % (ff, wf),
           "| kernel | launches | avg us | min us | max us | read MB/launch | written MB/launch | alg MB/launch |",
           "|---|---|---|---|---|---|---|---|"]
    for r in trace:
        n = r["name"]
        rd = fetch.get(n, 0.0) * ff * 1024 / 1e6
        wr = write.get(n, 0.0) * wf * 1024 / 1e6
        alg = bench.kernel_algorithmic_bytes(n, opt, dim, shape) / 1e6
        if rd + wr > 0:
            traffic[n.split("<")[0]] = int((rd + wr) * 1e6)
        out.append("| %s | %d | %.1f | %.1f | %.1f | %.1f | %.1f | %s |" % (
            n, r["calls"], r["avg_ns"] / 1e3, r["min_ns"] / 1e3, r["max_ns"] / 1e3, rd, wr, ("%.1f" % alg) if alg else "-"))
    roof = line["roofline"]
    out += ["",
            "bench.py's own line of the same workload (%d timed steps on batches of their own, %.0f new keys per step, HIP-event pairs around "
            "every launch): %.3f ms/step, %.3e lookups/s, step algorithmic bytes / time = %.1f GB/s = %.2f %% of 8 TB/s; "
            "dominant critical-path kernel %s at %.1f us per launch (%.0f GB/s by algorithmic bytes = %.1f %% of peak)."
            % (line["steps"], line["config"].get("new_keys_per_step", 0), line["ms_per_step"], line["value"],
               line["step_algorithmic_GBps"], 100 * line["step_frac_of_hbm_peak"], roof["kernel"], roof["avg_launch_us"],
               roof["achieved"], 100 * roof["frac"]),
            "",
            "Per-step kernel time from the HIP events (ms): " + ", ".join(
                "%s %.3f" % kv for kv in sorted(line["kernels_ms_per_step"].items(), key=lambda kv: -kv[1])),
            "",
            "Fraction of 8 TB/s by algorithmic bytes: " + ", ".join(
                "%s %.3f" % kv for kv in sorted(line["kernels_frac_of_hbm_peak"].items(), key=lambda kv: -kv[1])),
            ""]
    with open(args.out, "w") as f:
        f.write("\n".join(out))
    with open(args.traffic, "w") as f:
        json.dump({"commit": commit, "fetch_factor": round(ff, 4), "write_factor": round(wf, 4),
                   "workload": line["config"]["workload"], "bytes_per_launch": traffic}, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote %s and %s (%d kernels)" % (args.out, args.traffic, len(traffic)))


if __name__ == "__main__":
    main()
