"""Turn the CSV output of rocprofv3 passes over bench.py into a short summary.

    python3 -m openfish_amd.profile_report OUT_DIR --title "..." --bench-args "..." \
        [--md profiles/NAME.md] [--traffic-key hac_n512_c4 --traffic-json profiles/traffic.json]

OUT_DIR holds one sub-directory per pass, each written by one rocprofv3 run of the same
`python3 bench.py <bench-args>` command (a pass that is missing is left out of the summary):

    trace/   rocprofv3 --kernel-trace --stats --output-format csv -d OUT_DIR/trace -o t -- python3 bench.py ...
    fetch/   rocprofv3 --pmc FETCH_SIZE       --output-format csv -d OUT_DIR/fetch -o f -- python3 bench.py ...
    write/   rocprofv3 --pmc WRITE_SIZE       --output-format csv -d OUT_DIR/write -o w -- python3 bench.py ...
    sq/      rocprofv3 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_LDS SQ_WAIT_INST_LDS
                       SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_VALU --output-format csv -d OUT_DIR/sq -o s -- ...
    sq2/     rocprofv3 --pmc SQ_WAVE_CYCLES SQ_WAIT_ANY SQ_ACTIVE_INST_ANY SQ_ACTIVE_INST_LDS SQ_INSTS_VALU_FMA_F64
                       SQ_INSTS_VALU_TRANS_F32 SQ_INSTS_BRANCH SQ_WAIT_INST_ANY --output-format csv -d OUT_DIR/sq2 -o s -- ...

FETCH_SIZE and WRITE_SIZE are scaled by what the same counters read for the library's plain copy
kernel, which bench.py launches once when given --calibrate-copy MIB (MIB read, MIB written).
With --traffic-key the scaled HBM bytes per launch of every decode kernel are also stored in the
JSON table bench.py takes `roofline.traffic` from.
"""
import argparse
import collections
import csv
import glob
import json
import os
import re

SQ_COUNTERS = ["SQ_WAVES", "SQ_BUSY_CYCLES", "SQ_INSTS_VALU", "SQ_INSTS_SALU", "SQ_INSTS_LDS", "SQ_WAIT_INST_LDS",
               "SQ_LDS_BANK_CONFLICT", "SQ_ACTIVE_INST_VALU"]
SQ2_COUNTERS = ["SQ_WAVE_CYCLES", "SQ_WAIT_ANY", "SQ_ACTIVE_INST_ANY", "SQ_ACTIVE_INST_LDS", "SQ_INSTS_VALU_FMA_F64",
                "SQ_INSTS_VALU_TRANS_F32", "SQ_INSTS_BRANCH", "SQ_WAIT_INST_ANY"]
SCAN_MODES = {"0": "two_tier", "1": "precise", "2": "fast"}
# kernel function -> the stage name bench.py uses
STAGE_OF = {"scan_post_kernel": "scan", "bwd_scan_kernel": "bwd", "fwd_post_kernel": "fwd_post", "fwd_post_roles_kernel": "fwd_post",
            "beam_kernel": "beam", "sequence_kernel": "sequence", "path_sums_kernel": "path_sums"}


def template_ints(name):
    """integer template arguments of a kernel name, mangled (ILi64ELi1E...) or demangled (<64, 1, ...>)"""
    m = re.search(r"I((?:Li\d+E)+)", name)
    if m:
        return re.findall(r"Li(\d+)E", m.group(1))
    m = re.search(r"<([0-9, ]+)>", name)
    return [x.strip() for x in m.group(1).split(",")] if m else []


def short(name):
    for fn in ("scan_post_kernel", "bwd_scan_kernel", "fwd_post_roles_kernel", "fwd_post_kernel", "beam_kernel",
               "sequence_kernel", "path_sums_kernel", "copy_kernel", "rotary_vec8_kernel", "rotary_kernel"):
        if fn in name:
            a = template_ints(name)
            if fn == "fwd_post_roles_kernel" and len(a) >= 3:
                return "%s<S=%s,SPL=%s,DEPTH=%s>" % (fn, a[0], a[1], a[2])
            if fn in ("scan_post_kernel", "bwd_scan_kernel", "fwd_post_kernel") and len(a) >= 4:
                return "%s<S=%s,SPL=%s,DEPTH=%s,%s>" % (fn, a[0], a[1], a[2], SCAN_MODES.get(a[3], a[3]))
            if fn == "beam_kernel" and len(a) >= 3:
                return "beam_kernel<S=%s,chunks/group=%s,columns=%s>" % (a[0], a[1], a[2])
            return "%s<%s>" % (fn, ",".join(a)) if a else fn
    return name[:60]


def stage_of(short_name):
    return STAGE_OF.get(short_name.split("<")[0])


def first(pattern):
    hits = sorted(glob.glob(pattern, recursive=True))
    return hits[0] if hits else None


def counters(path):
    """{kernel: {counter: mean per dispatch}}"""
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    with open(path) as fh:
        for r in csv.DictReader(fh):
            agg[short(r["Kernel_Name"])][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return {k: {c: sum(v) / len(v) for c, v in d.items()} for k, d in agg.items()}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("out_dir")
    ap.add_argument("--title", required=True)
    ap.add_argument("--bench-args", required=True, help="the arguments bench.py was given in every pass")
    ap.add_argument("--md", help="file to write (default: stdout)")
    ap.add_argument("--traffic-key", help="entry of the traffic table to (re)write, e.g. hac_n512_c4")
    ap.add_argument("--traffic-json", default=os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                                                           "profiles", "traffic.json"))
    ap.add_argument("--updates", type=float, default=0,
                    help="state updates of one scan sweep per launch (N * T * S): adds VALU instructions per update")
    ap.add_argument("--steps-per-wave", type=float, default=0,
                    help="time steps T every scan wave takes: adds fp64 FMA per wave and time step")
    a = ap.parse_args()

    base, args = a.out_dir, a.bench_args
    out = ["# %s\n" % a.title,
           "Commands (on the GPU box, from the repository root, one rocprofv3 run per pass; `A` = `%s`):\n" % args,
           "```",
           "rocprofv3 --kernel-trace --stats --output-format csv -d OUT/trace -o t -- python3 bench.py A",
           "rocprofv3 --pmc FETCH_SIZE --output-format csv -d OUT/fetch -o f -- python3 bench.py A",
           "rocprofv3 --pmc WRITE_SIZE --output-format csv -d OUT/write -o w -- python3 bench.py A",
           "rocprofv3 --pmc %s --output-format csv -d OUT/sq -o s -- python3 bench.py A" % " ".join(SQ_COUNTERS),
           "rocprofv3 --pmc %s --output-format csv -d OUT/sq2 -o s -- python3 bench.py A" % " ".join(SQ2_COUNTERS),
           "python3 -m openfish_amd.profile_report OUT --title ... --bench-args \"A\" --md <this file>",
           "```\n"]

    stats = first(os.path.join(base, "trace", "**", "*kernel_stats.csv"))
    if stats:
        out.append("## Kernel durations (`--kernel-trace --stats`)\n")
        out.append("| kernel | calls | mean us | min us | max us | % of GPU time |\n|---|---|---|---|---|---|")
        with open(stats) as fh:
            for r in csv.DictReader(fh):
                out.append("| %s | %s | %.1f | %.1f | %.1f | %.1f |" % (
                    short(r["Name"]), r["Calls"], float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3,
                    float(r["MaxNs"]) / 1e3, float(r["Percentage"])))

    fetch = first(os.path.join(base, "fetch", "**", "*counter_collection.csv"))
    write = first(os.path.join(base, "write", "**", "*counter_collection.csv"))
    if fetch and write:
        f = {k: d.get("FETCH_SIZE", 0.0) for k, d in counters(fetch).items()}
        w = {k: d.get("WRITE_SIZE", 0.0) for k, d in counters(write).items()}
        out.append("\n## HBM traffic per launch (`--pmc FETCH_SIZE`, `--pmc WRITE_SIZE`; KiB as reported)\n")
        m = re.search(r"--calibrate-copy (\d+)", args)
        copy = [k for k in f if k.startswith("copy_kernel")]
        ff = wf = 1.0
        if m and copy and f[copy[0]] > 0 and w.get(copy[0], 0) > 0:
            kib = int(m.group(1)) * 1024
            ff, wf = kib / f[copy[0]], kib / w[copy[0]]
            out.append("Calibration: the plain copy kernel reads and writes %s MiB; the counters report FETCH_SIZE = "
                       "%.1f KiB and WRITE_SIZE = %.1f KiB for it, so they are scaled by %.4f (fetch) and %.4f "
                       "(write).\n" % (m.group(1), f[copy[0]], w[copy[0]], ff, wf))
        else:
            out.append("No copy kernel in this run: counters unscaled.\n")
        out.append("| kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | read GB | written GB | total GB |\n|---|---|---|---|---|---|")
        table = {}
        for k in f:
            if k.startswith("__amd"):
                continue
            rd, wr = f[k] * ff * 1024, w.get(k, 0.0) * wf * 1024
            out.append("| %s | %.1f | %.1f | %.3f | %.3f | %.3f |" % (k, f[k], w.get(k, 0.0), rd / 1e9, wr / 1e9, (rd + wr) / 1e9))
            if stage_of(k):
                table[stage_of(k)] = {"kernel": k, "read_bytes": round(rd), "write_bytes": round(wr), "hbm_bytes": round(rd + wr)}
        if a.traffic_key:
            try:
                with open(a.traffic_json) as fh:
                    whole = json.load(fh)
            except (OSError, ValueError):
                whole = {}
            table["bench_args"] = args
            merged = whole.get(a.traffic_key, {})  # runs of both scan arrangements fill one entry
            merged.update(table)
            whole[a.traffic_key] = merged
            with open(a.traffic_json, "w") as fh:
                json.dump(whole, fh, indent=1, sort_keys=True)
                fh.write("\n")

    sq = first(os.path.join(base, "sq", "**", "*counter_collection.csv"))
    if sq:
        c = counters(sq)
        out.append("\n## SQ counters per launch (`--pmc %s`)\n" % " ".join(SQ_COUNTERS))
        head = [n.replace("SQ_", "") for n in SQ_COUNTERS] + (["VALU per state update"] if a.updates else [])
        out.append("| kernel | " + " | ".join(head) + " |\n|---|" + "---|" * len(head))
        for k, d in c.items():
            if k.startswith("__amd"):
                continue
            cells = [("%.3g" % d[n]) if n in d else "-" for n in SQ_COUNTERS]
            if a.updates:
                sweeps = {"scan": 2, "bwd": 1, "fwd_post": 1}.get(stage_of(k))
                cells.append("%.1f" % (d.get("SQ_INSTS_VALU", 0.0) * 64 / (sweeps * a.updates)) if sweeps else "-")
            out.append("| %s | " % k + " | ".join(cells) + " |")
        if a.updates:
            out.append("\nVALU per state update = SQ_INSTS_VALU (wave instructions) x 64 lanes / (sweeps x N x T x S state "
                       "updates): the vector instructions one lane issues for one update of one state, everything "
                       "around the update (loads, posterior, exchange through LDS) included.")

    sq2 = first(os.path.join(base, "sq2", "**", "*counter_collection.csv"))
    if sq and sq2:
        c1, c2 = counters(sq), counters(sq2)
        out.append("\n## Where the waves' time goes (`--pmc %s`, with the table above)\n" % " ".join(SQ2_COUNTERS))
        out.append("Per launch. The SQ's time counters tick once per four clocks; WAVE_CYCLES adds up the lifetimes of all "
                   "waves, ACTIVE_INST_VALU the time their vector instructions occupy a SIMD's ALU. `VALU share of wave "
                   "time` x `waves per SIMD` is the fraction of time a SIMD's vector ALU is busy (1024 SIMDs; the waves of "
                   "these kernels are all resident at once).\n")
        out.append("| kernel | WAVE_CYCLES | WAIT_ANY | ACTIVE_INST_ANY | ACTIVE_INST_LDS | INSTS_VALU_FMA_F64 | INSTS_VALU_TRANS_F32 | "
                   "INSTS_BRANCH | VALU share of wave time | waves per SIMD | SIMD vector ALU busy | fp64 FMA per wave and time step |"
                   "\n|---|---|---|---|---|---|---|---|---|---|---|---|")
        for k, d in c2.items():
            if k.startswith("__amd") or k not in c1:
                continue
            wc, act, waves = d.get("SQ_WAVE_CYCLES", 0.0), c1[k].get("SQ_ACTIVE_INST_VALU", 0.0), c1[k].get("SQ_WAVES", 0.0)
            share = act / wc if wc else 0.0
            per_simd = waves / 1024.0
            steps = a.steps_per_wave
            out.append("| %s | %.3g | %.3g | %.3g | %.3g | %.3g | %.3g | %.3g | %.3f | %.2f | %.2f | %s |" % (
                k, wc, d.get("SQ_WAIT_ANY", 0.0), d.get("SQ_ACTIVE_INST_ANY", 0.0), d.get("SQ_ACTIVE_INST_LDS", 0.0),
                d.get("SQ_INSTS_VALU_FMA_F64", 0.0), d.get("SQ_INSTS_VALU_TRANS_F32", 0.0), d.get("SQ_INSTS_BRANCH", 0.0),
                share, per_simd, min(1.0, share * per_simd),
                ("%.2f" % (d.get("SQ_INSTS_VALU_FMA_F64", 0.0) / (waves * steps))) if (steps and waves and stage_of(k) in ("scan", "bwd", "fwd_post")) else "-"))
        if a.steps_per_wave:
            out.append("\nfp64 FMA per wave and time step = SQ_INSTS_VALU_FMA_F64 / (waves x T): the second tier of the default "
                       "arithmetic is the only user of fp64 in the scans besides the 32 warm-up steps of either sweep (70 fp64 "
                       "FMA per wave and step there); one trip through it is 23 fp64 FMA, so the figure, less the warm-up's "
                       "share, over 23 is the number of trips per wave-level update.")

    log = first(os.path.join(base, "trace.log"))
    if log:
        with open(log) as fh:
            js = [line.strip() for line in fh if line.startswith("{")]
        if js:
            out.append("\n## bench.py line of the traced run (timings include the tracer's overhead)\n\n```\n%s\n```" % js[-1])

    text = "\n".join(out) + "\n"
    if a.md:
        with open(a.md, "w") as fh:
            fh.write(text)
    else:
        print(text)


if __name__ == "__main__":
    main()
