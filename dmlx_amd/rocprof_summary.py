#!/usr/bin/env python3
"""Turns rocprofv3 CSV output of a bench.py run into the short text summaries kept under profiles/ and into the
entries of profiles/counters.json that bench.py quotes (so that no figure there is typed by hand).

  python -m dmlx_amd.rocprof_summary trace  <dir> --title "..." --command "..." > profiles/<name>_kernel_trace.txt
      <dir> holds kt_kernel_trace.csv (rocprofv3 --kernel-trace --stats -o kt --output-format csv): one line per
      kernel of libdmoe and launch grid with calls, average / minimum / maximum duration and share of the total.

  python -m dmlx_amd.rocprof_summary counters <dir> [<dir> ...] --title "..." --command "..." [--command "..."]
      <dir>s hold pmc_counter_collection.csv (rocprofv3 --pmc ... -o pmc --output-format csv), one run per
      directory: per kernel of libdmoe (and per plain device copy, the known-size kernel that scales FETCH_SIZE /
      WRITE_SIZE) the average, minimum and maximum of every counter over the kernel's dispatches.

  python -m dmlx_amd.rocprof_summary json <config> <stage> --kernel <substring> [--grid-y-min N] <dir> [<dir> ...]
        --source "profiles/a.txt, profiles/b.txt"
      reads the same counter directories and writes entry c<config>.<stage> of profiles/counters.json:
        traffic_bytes  = FETCH_SIZE x (copy bytes / FETCH_SIZE of a copy) + WRITE_SIZE x (copy bytes / WRITE_SIZE of a
                         copy), in bytes per dispatch (both counters are KiB); needs the --copy-probe copies in the runs
        mfma_busy      = SQ_VALU_MFMA_BUSY_CYCLES / (1024 SIMDs x GRBM_GUI_ACTIVE / 8 XCDs)
        valu_per_mfma  = (SQ_INSTS_VALU - SQ_INSTS_MFMA) / SQ_INSTS_MFMA
        wait_share     = SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES
      Only the quantities whose counters are present are written.
"""
import argparse
import collections
import csv
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
COPY_BYTES = 256 << 20      # bench.py --copy-probe: bytes read (and written) by each calibration copy
N_SIMD = 1024               # 256 compute units x 4
N_XCD = 8


def short(name):
    return name.replace("dmoe::", "").replace("void ", "").split("(")[0]


def trace(args):
    agg = collections.OrderedDict()
    with open(os.path.join(args.dirs[0], "kt_kernel_trace.csv")) as f:
        for r in csv.DictReader(f):
            if "dmoe::" not in r["Kernel_Name"]:
                continue
            wg = (int(r["Workgroup_Size_X"]), int(r["Workgroup_Size_Y"]))
            grid = (int(r["Grid_Size_X"]) // wg[0], int(r["Grid_Size_Y"]) // wg[1])
            key = (short(r["Kernel_Name"]), grid, int(r["VGPR_Count"]), int(r["Accum_VGPR_Count"]), int(r["LDS_Block_Size"]))
            agg.setdefault(key, []).append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    total = sum(sum(v) for v in agg.values())
    out = [f"# {args.title}", "", "command (one MI355X):", ""] + [f"    {c}" for c in args.command] + [
        "", "Source: the kernel trace of that run, kernels of libdmoe only, grouped by kernel and launch grid (workgroups",
        "x, y). The rest of the trace is the one-time synthetic weight generation in torch. Durations in microseconds.", "",
        f"{'kernel':62s} {'grid':>12s} {'vgpr':>5s} {'agpr':>5s} {'lds':>7s} {'calls':>6s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s} {'share':>7s}"]
    for (name, grid, v, a, lds), ds in sorted(agg.items(), key=lambda kv: -sum(kv[1])):
        out.append(f"{name[:60]:62s} {str(grid[0]) + 'x' + str(grid[1]):>12s} {v:5d} {a:5d} {lds:7d} {len(ds):6d} "
                   f"{sum(ds) / len(ds):9.2f} {min(ds):9.2f} {max(ds):9.2f} {100 * sum(ds) / total:6.1f}%")
    print("\n".join(out))


def read_counters(dirs):
    """{(kernel, workgroups, counter): [values per dispatch]} over all runs; the runtime's device copies under 'COPY'."""
    agg = collections.defaultdict(list)
    for d in dirs:
        per_dispatch = collections.defaultdict(float)
        meta = {}
        with open(os.path.join(d, "pmc_counter_collection.csv")) as f:
            for r in csv.DictReader(f):
                name = r["Kernel_Name"]
                if "dmoe::" in name:
                    k = short(name)
                elif "copyBuffer" in name:      # the runtime's device-to-device copy kernel (torch's dst.copy_(src))
                    k = "COPY"
                else:
                    continue
                key = (d, r["Dispatch_Id"], r["Counter_Name"])
                per_dispatch[key] += float(r["Counter_Value"])     # a counter may be split over several rows
                meta[key] = (k, int(r["Grid_Size"]) // max(1, int(r["Workgroup_Size"])))
        for key, v in per_dispatch.items():
            k, wgs = meta[key]
            agg[(k, wgs, key[2])].append(v)
    return agg


def derived(agg, kernel, min_workgroups=0):
    """The figures bench.py quotes for one kernel, from the counters that are present."""

    def avg(counter, copy=False):
        vals = []
        for (k, wgs, c), v in agg.items():
            if c != counter:
                continue
            if copy:
                if k == "COPY":
                    vals += v
            elif kernel in k and wgs >= min_workgroups:
                vals += v
        if copy and vals:   # the --copy-probe copies are the largest device copies of a run: those within 2 % of the top
            vals = [x for x in vals if x >= 0.98 * max(vals)]
        return sum(vals) / len(vals) if vals else None

    rec = {}
    fetch, write = avg("FETCH_SIZE"), avg("WRITE_SIZE")
    if fetch is not None and write is not None:
        cf, cw = avg("FETCH_SIZE", copy=True), avg("WRITE_SIZE", copy=True)
        if cf and cw:
            f_scale, w_scale = COPY_BYTES / cf, COPY_BYTES / cw     # bytes per counter unit
            rec["traffic_bytes"] = int(round(fetch * f_scale + write * w_scale))
            rec["fetch_scale"] = round(f_scale / 1024, 3)           # in KiB: 2.0 = the counter reads half the bytes
            rec["write_scale"] = round(w_scale / 1024, 3)
    busy, gui = avg("SQ_VALU_MFMA_BUSY_CYCLES"), avg("GRBM_GUI_ACTIVE")
    if busy is not None and gui:
        rec["mfma_busy"] = round(busy / (N_SIMD * gui / N_XCD), 3)
    valu, mfma = avg("SQ_INSTS_VALU"), avg("SQ_INSTS_MFMA")
    if valu is not None and mfma:
        rec["valu_per_mfma"] = round((valu - mfma) / mfma, 2)
    wait, wave = avg("SQ_WAIT_INST_ANY"), avg("SQ_WAVE_CYCLES")
    if wait is not None and wave:
        rec["wait_share"] = round(wait / wave, 3)
    return rec


def counters(args):
    agg = read_counters(args.dirs)
    out = [f"# {args.title}", "", "commands (one MI355X, one rocprofv3 run each):", ""] + [f"    {c}" for c in args.command] + [
        "", "Per dispatch, over all dispatches of the kernel in the runs (pre-run, warm-up, timed and stage-timed windows); kernels",
        f"whose name contains '{args.kernels}'. FETCH_SIZE / WRITE_SIZE are KiB; COPY = the runtime's device-copy kernel, whose",
        "largest dispatches are the 256 MiB copies of --copy-probe (the scale of those two counters); SQ_ACTIVE_* / SQ_WAIT_* /",
        "SQ_WAVE_CYCLES count units of four cycles; GRBM_GUI_ACTIVE is summed over the 8 XCDs.", "",
        f"{'kernel':52s} {'workgroups':>10s} {'counter':30s} {'n':>5s} {'avg':>16s} {'min':>16s} {'max':>16s}"]
    names = []
    for (k, wgs, c), v in sorted(agg.items()):
        if args.kernels not in k and not (k == "COPY" and max(v) >= 1024 and c in ("FETCH_SIZE", "WRITE_SIZE")):
            continue
        out.append(f"{k[:50]:52s} {wgs:10d} {c:30s} {len(v):5d} {sum(v) / len(v):16.1f} {min(v):16.1f} {max(v):16.1f}")
        if k != "COPY" and (k, wgs) not in names:
            names.append((k, wgs))
    out += ["", "Derived per kernel and launch size (what profiles/counters.json holds): traffic_bytes = FETCH_SIZE x fetch_scale +",
            "WRITE_SIZE x write_scale (scales = bytes of a --copy-probe copy / its counter reading, in KiB); mfma_busy =",
            "SQ_VALU_MFMA_BUSY_CYCLES / (1024 SIMDs x GRBM_GUI_ACTIVE / 8); valu_per_mfma = (SQ_INSTS_VALU - SQ_INSTS_MFMA) /",
            "SQ_INSTS_MFMA; wait_share = SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES.", ""]
    for k, wgs in names:
        sub = {key: v for key, v in agg.items() if key[0] == "COPY" or (key[0] == k and key[1] == wgs)}
        out.append(f"{k[:50]:52s} {wgs:10d} {json.dumps(derived(sub, k))}")
    print("\n".join(out))


def to_json(args):
    agg = read_counters(args.dirs)
    rec = derived(agg, args.kernel, args.min_workgroups)
    if not rec:
        sys.exit(f"no counters of a kernel matching {args.kernel!r} in {args.dirs}")
    rec["source"] = args.source
    path = os.path.join(ROOT, "profiles", "counters.json")
    try:
        with open(path) as f:
            data = json.load(f)
    except OSError:
        data = {}
    data["_comment"] = ("Counter readings per dispatch of the dominant GEMM kernels, written by dmlx_amd/rocprof_summary.py from "
                        "the rocprofv3 --pmc output behind the summaries in this folder; bench.py reports them next to its "
                        "live timings.")
    entry = data.setdefault(f"c{args.config}", {}).setdefault(args.stage, {})
    entry.update(rec)
    with open(path, "w") as f:
        json.dump(data, f, indent=2)
        f.write("\n")
    print(json.dumps({f"c{args.config}": {args.stage: entry}}, indent=2))


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="mode", required=True)
    for name in ("trace", "counters"):
        p = sub.add_parser(name)
        p.add_argument("dirs", nargs="+")
        p.add_argument("--title", required=True)
        p.add_argument("--command", action="append", default=[])
        p.add_argument("--kernels", default="gemm", help="counters: list only kernels whose name contains this")
    p = sub.add_parser("json")
    p.add_argument("config", type=int)
    p.add_argument("stage")
    p.add_argument("dirs", nargs="+")
    p.add_argument("--kernel", required=True, help="substring of the kernel's name, e.g. 'qgemm_wide_kernel<FmtAffine4, true>' (namespace prefixes dropped)")
    p.add_argument("--min-workgroups", type=int, default=0, help="ignore launches of fewer workgroups (the shared expert's)")
    p.add_argument("--source", required=True)
    args = ap.parse_args()
    {"trace": trace, "counters": counters, "json": to_json}[args.mode](args)


if __name__ == "__main__":
    main()
