"""Summarises rocprofv3 output of bench.py runs: kernel durations, HBM-side traffic, shader counters.

    python -m tracea_amd.profile_summary <dir> [--write-inputs]

<dir> holds one sub-directory per run, each made by one of the commands below (run from the
repository root; one counter group per run, never combined with a trace):

    trace/            rocprofv3 --kernel-trace --stats --output-format csv -d <dir>/trace -o t -- python3 bench.py
    fetch_<w>/        rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir>/fetch_<w> -o p -- \\
                          python3 bench.py --no-extras --workload <w> --steps 5 --warmup 2
    write_<w>/        the same with --pmc WRITE_SIZE
    sq_<w>/           the same with --pmc SQ_BUSY_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_MFMA \\
                          SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_WAVE_CYCLES SQ_WAIT_INST_LDS SQ_WAIT_INST_ANY
    <run>/bench.json  the line bench.py printed in that run (its stdout), for the variant that ran

<w> is gemm, conv, attention, attention_causal or copy (copy: the calibration workload of known size).
Prints the tables of profiles/bench_kernels_mi355x.md and, with --write-inputs, rewrites
profiles/roofline_inputs.json, the table bench.py's roofline blocks read.
"""
import collections
import csv
import glob
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# dominant kernel of a workload: the first of these name fragments that occurs in the run
KERNELS = {"gemm": ["contraction_kernel"], "conv": ["conv_wave16_kernel", "conv_resident_kernel", "conv_patch_kernel", "contraction_kernel"],
           "attention": ["fa2_fwd"], "attention_causal": ["fa2_fwd"], "copy": ["copyBuffer", "copy"]}
ALGORITHMIC_BYTES = {"gemm": 2.0 * 3 * 4096 * 4096, "conv": 2.0 * (2 * 32 * 56 * 56 * 64 + 64 * 576),
                     "attention": 2.0 * 4 * 4 * 32 * 4096 * 128, "attention_causal": 2.0 * 4 * 4 * 32 * 4096 * 128}
COPY_KIB = 262144.0          # the calibration copy reads and writes 256 MiB
SHADER_ENGINES = 32          # SQ_BUSY_CYCLES is summed over the shader engines of the device
SIMDS = 1024                 # SQ_VALU_MFMA_BUSY_CYCLES over its SIMDs


def _rows(pattern):
    for f in sorted(glob.glob(pattern)):
        with open(f, newline="") as fh:
            for row in csv.DictReader(fh):
                yield row


def kernel_stats(run_dir):
    """[(name, calls, avg_ns, min_ns, max_ns, total_ns)] of a --kernel-trace --stats run."""
    out = []
    for row in _rows(os.path.join(run_dir, "*", "*kernel_stats.csv")):
        out.append((row["Name"], int(row["Calls"]), float(row["AverageNs"]), float(row["MinNs"]), float(row["MaxNs"]),
                    float(row["TotalDurationNs"]) if "TotalDurationNs" in row else float(row["AverageNs"]) * int(row["Calls"])))
    if not out:
        for row in _rows(os.path.join(run_dir, "*kernel_stats.csv")):
            out.append((row["Name"], int(row["Calls"]), float(row["AverageNs"]), float(row["MinNs"]), float(row["MaxNs"]),
                        float(row["AverageNs"]) * int(row["Calls"])))
    return out


def launch_runs(run_dir, least=20):
    """Runs of consecutive dispatches of one kernel at one grid size, in time order: bench.py's legs
    launch one kernel back to back (warm-up, then the timed steps), so each leg of a single-kernel workload
    is one run.  [(name, workgroups, launches, avg_ns, median_ns, min_ns)] for runs of at least `least`."""
    rows = list(_rows(os.path.join(run_dir, "*kernel_trace.csv"))) + list(_rows(os.path.join(run_dir, "*", "*kernel_trace.csv")))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    runs, cur = [], None
    for r in rows:
        wg = int(r["Workgroup_Size_X"]) * int(r["Workgroup_Size_Y"]) * int(r["Workgroup_Size_Z"])
        key = (r["Kernel_Name"], int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"]) // max(1, wg))
        d = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        if cur and cur[0] == key:
            cur[1].append(d)
        else:
            cur = [key, [d]]
            runs.append(cur)
    out = []
    for (name, groups), ds in runs:
        if len(ds) >= least and "tracea_amd" in name:
            ds = sorted(ds)
            out.append((name, groups, len(ds), sum(ds) / len(ds), ds[len(ds) // 2], ds[0]))
    return out


def counters(run_dir, workload):
    """{counter: mean per dispatch} and mean duration (ns, or None) of the workload's dominant kernel in a --pmc run."""
    per = collections.defaultdict(lambda: collections.defaultdict(list))
    dur = collections.defaultdict(list)
    for row in list(_rows(os.path.join(run_dir, "*", "*counter_collection.csv"))) + list(_rows(os.path.join(run_dir, "*counter_collection.csv"))):
        name = row["Kernel_Name"]
        per[name][row["Counter_Name"]].append(float(row["Counter_Value"]))
        if row.get("Start_Timestamp") and row.get("End_Timestamp"):
            dur[name].append(float(row["End_Timestamp"]) - float(row["Start_Timestamp"]))
    for frag in KERNELS[workload]:
        names = [n for n in per if frag in n]
        if names:
            name = max(names, key=lambda n: sum(len(v) for v in per[n].values()))
            d = dur.get(name)
            return name, {k: sum(v) / len(v) for k, v in per[name].items()}, (sum(d) / len(d) if d else None)
    return None, {}, None


def variant_of(run_dir, workload):
    try:
        with open(os.path.join(run_dir, "bench.json")) as f:
            for line in f:
                line = line.strip()
                if line.startswith("{"):
                    j = json.loads(line)
                    if j.get("config", {}).get("variant"):
                        return j["config"]["variant"]
    except (OSError, ValueError):
        pass
    return None


def short(name, n=110):
    return name if len(name) <= n else name[: n - 3] + "..."


def main(argv):
    if not argv or argv[0].startswith("-"):
        raise SystemExit(__doc__)
    base = argv[0]
    write = "--write-inputs" in argv
    print("## Kernel durations (trace/: one default bench.py run, every leg)\n")
    print("| kernel | calls | avg ns | min ns | max ns |\n|---|---|---|---|---|")
    stats = kernel_stats(os.path.join(base, "trace"))
    for name, calls, avg, mn, mx, tot in sorted(stats, key=lambda r: -r[5])[:24]:
        print("| `%s` | %d | %.0f | %.0f | %.0f |" % (short(name), calls, avg, mn, mx))
    print("\n## The same run by leg: runs of back-to-back launches of one kernel, in time order (single-kernel legs only)\n")
    print("| kernel | workgroups | launches | avg ns | median ns | min ns |\n|---|---|---|---|---|---|")
    for name, groups, n, avg, med, mn in launch_runs(os.path.join(base, "trace")):
        print("| `%s` | %d | %d | %.0f | %.0f | %.0f |" % (short(name.replace("void tracea_amd::", "").replace("(tracea_amd::ContractionArgs)", "").replace("(tracea_amd::AttentionArgs)", ""), 80), groups, n, avg, med, mn))
    _, cf, _ = counters(os.path.join(base, "fetch_copy"), "copy")
    _, cw, _ = counters(os.path.join(base, "write_copy"), "copy")
    fscale = COPY_KIB / cf["FETCH_SIZE"] if cf.get("FETCH_SIZE") else None
    wscale = COPY_KIB / cw["WRITE_SIZE"] if cw.get("WRITE_SIZE") else None
    print("\n## Traffic counters (KiB per dispatch as reported; copy of 256 MiB: FETCH_SIZE %s, WRITE_SIZE %s -> scale %s / %s)\n"
          % (cf.get("FETCH_SIZE"), cw.get("WRITE_SIZE"), fscale and round(fscale, 3), wscale and round(wscale, 3)))
    print("| workload | kernel | FETCH_SIZE | WRITE_SIZE | fetched MB | written MB | total MB | algorithmic MB |\n|---|---|---|---|---|---|---|---|")
    table = {}
    for w in ("gemm", "conv", "attention", "attention_causal"):
        name, f, _ = counters(os.path.join(base, "fetch_" + w), w)
        _, wr, _ = counters(os.path.join(base, "write_" + w), w)
        row = {"kernel": name, "variant": variant_of(os.path.join(base, "fetch_" + w), w)}
        if f.get("FETCH_SIZE") is not None and wr.get("WRITE_SIZE") is not None and fscale and wscale:
            fb, wb = f["FETCH_SIZE"] * fscale * 1024.0, wr["WRITE_SIZE"] * wscale * 1024.0
            row.update(fetch_kib=round(f["FETCH_SIZE"], 1), write_kib=round(wr["WRITE_SIZE"], 1), fetch_scale=round(fscale, 4),
                       write_scale=round(wscale, 4), traffic_bytes=round(fb + wb), algorithmic_bytes=ALGORITHMIC_BYTES[w])
            print("| %s | `%s` | %.1f | %.1f | %.1f | %.1f | %.1f | %.1f |" % (w, short(name or "?", 60), f["FETCH_SIZE"], wr["WRITE_SIZE"],
                                                                         fb / 1e6, wb / 1e6, (fb + wb) / 1e6, ALGORITHMIC_BYTES[w] / 1e6))
        table[w] = row
    print("\n## Shader counters (sums over the device, mean per dispatch)\n")
    print("| workload | SQ_INSTS_MFMA | SQ_VALU_MFMA_BUSY_CYCLES | SQ_BUSY_CYCLES | cycles per launch | ns per launch | clock GHz | matrix-pipe utilisation | LDS bank conflicts / LDS active |\n|---|---|---|---|---|---|---|---|---|")
    for w in ("gemm", "conv", "attention", "attention_causal"):
        name, c, d = counters(os.path.join(base, "sq_" + w), w)
        if not c:
            continue
        cyc = c.get("SQ_BUSY_CYCLES", 0.0) / SHADER_ENGINES
        util = c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) / (cyc * SIMDS) if cyc else None
        clock = cyc / d if d else None
        conf = c.get("SQ_LDS_BANK_CONFLICT", 0.0) / c["SQ_LDS_IDX_ACTIVE"] if c.get("SQ_LDS_IDX_ACTIVE") else None
        print("| %s | %.6g | %.6g | %.6g | %.0f | %s | %s | %s | %s |" % (
            w, c.get("SQ_INSTS_MFMA", 0), c.get("SQ_VALU_MFMA_BUSY_CYCLES", 0), c.get("SQ_BUSY_CYCLES", 0), cyc,
            "%.0f" % d if d else "n/a", "%.3f" % clock if clock else "n/a", "%.3f" % util if util else "n/a",
            "%.3f" % conf if conf is not None else "n/a"))
        table[w].update(cycles_per_launch=round(cyc), mfma_utilisation=util and round(util, 4),
                        lds_conflict_share=conf is not None and round(conf, 4) or None)
        if clock:
            table[w]["clock_ghz"] = round(clock, 3)
            table[w]["ns_per_launch_under_counters"] = round(d)
    if write:
        out = {"comment": "written by `python -m tracea_amd.profile_summary <dir> --write-inputs` from rocprofv3 counter runs of "
                          "bench.py (commands: profiles/bench_kernels_mi355x.md); traffic_bytes = FETCH_SIZE and WRITE_SIZE per "
                          "dispatch, each scaled by what the same counter reads for a 256 MiB copy; clock_ghz = SQ_BUSY_CYCLES / "
                          "32 shader engines / kernel duration in the counter run",
               "workloads": table}
        with open(os.path.join(ROOT, "profiles", "roofline_inputs.json"), "w") as f:
            json.dump(out, f, indent=1, sort_keys=True)
            f.write("\n")
        print("\nwrote profiles/roofline_inputs.json")


if __name__ == "__main__":
    main(sys.argv[1:])
