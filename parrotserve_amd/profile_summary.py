"""Summaries of rocprofv3 runs over bench.py, written to profiles/ (text) and profiles/counters.json.

Usage, after the collection runs below have put their CSV output under one directory:

    python -m parrotserve_amd.profile_summary <dir>

Collection (on the GPU box, from /tmp with TMPDIR=/tmp; one rocprofv3 run per line, `-d <dir>/<name> -o r
--output-format csv` on each; counter runs never carry a trace option):

    trace_c2   rocprofv3 --kernel-trace --stats -- python3 bench.py --no-cpu --no-extras
    trace_all  rocprofv3 --kernel-trace --stats -- python3 bench.py --no-cpu
    trace_e2e  rocprofv3 --kernel-trace --stats -- python3 bench.py --e2e-only
    fetch      rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --no-cpu --no-extras --steps 24 --warmup 8
    write      rocprofv3 --pmc WRITE_SIZE -- python3 bench.py --no-cpu --no-extras --steps 24 --warmup 8
    cal_fetch  rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --copy-calibration
    cal_write  rocprofv3 --pmc WRITE_SIZE -- python3 bench.py --copy-calibration
    sq1        rocprofv3 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_ANY SQ_WAIT_INST_ANY SQ_ACTIVE_INST_ANY
                              SQ_INSTS_VALU SQ_INSTS_MFMA -- python3 bench.py --no-cpu --no-extras --steps 24 --warmup 8
    sq2        rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_WAIT_INST_LDS SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS
                              SQ_ACTIVE_INST_VMEM SQ_INSTS_VMEM_RD SQ_INSTS_LDS SQ_INSTS_SALU -- (same command)
    grbm       rocprofv3 --pmc GRBM_GUI_ACTIVE GRBM_COUNT -- (same command)
    pf1        rocprofv3 --pmc SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_MFMA SQ_INSTS_VALU
                              SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS SQ_WAIT_INST_LDS -- python3 bench.py --prefill-only
    pf2        rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_LDS SQ_INSTS_VALU_TRANS_F32
                              SQ_INSTS_VMEM_RD SQ_INSTS_SALU SQ_WAIT_ANY SQ_WAVES -- python3 bench.py --prefill-only
    pf3        rocprofv3 --pmc GRBM_GUI_ACTIVE GRBM_COUNT -- python3 bench.py --prefill-only
    timeline.json   python3 bench.py --timeline > <dir>/timeline.json   (no profiler; fused decode and prefill kernels)

A missing run only leaves its summary out.  The profiler sums SQ / GRBM counters over the chip's 8 XCDs;
FETCH_SIZE / WRITE_SIZE are KiB per dispatch and are scaled by what the same counters read for a plain copy of known
size (cal_fetch / cal_write).
"""
from __future__ import annotations

import collections
import csv
import glob
import json
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROFILES = os.path.join(ROOT, "profiles")
XCDS, SIMDS = 8, 1024  # MI355X: 8 XCDs, 256 CUs x 4 SIMDs
MFMA_PEAK = 2.5e15
PRE = "rocprofv3 %s --output-format csv -d <out> -o r -- python3 bench.py %s"


def _csv(d, name, kind):
    hits = glob.glob(os.path.join(d, name, "**", "*" + kind + ".csv"), recursive=True)
    return hits[0] if hits else None


def _short(n):
    return re.sub(r"\(.*", "", n).replace("void ", "")[:64]


def _commit():
    try:
        h = subprocess.run(["git", "rev-parse", "--short", "HEAD"], cwd=ROOT, capture_output=True, text=True).stdout.strip()
        dirty = subprocess.run(["git", "status", "--porcelain", "--", "parrotserve_amd/csrc", "bench.py"], cwd=ROOT,
                               capture_output=True, text=True).stdout.strip()
        return h + ("+uncommitted changes" if dirty else "")
    except OSError:
        return "unknown"


def counters_of(path, patterns):
    """{(pattern, counter): mean per dispatch}, the first quarter of each kernel's dispatches (warm-up) left out."""
    acc = collections.defaultdict(list)
    if path is None:
        return {}
    for row in csv.DictReader(open(path)):
        for p in patterns:
            if p in row["Kernel_Name"]:
                acc[(p, row["Counter_Name"])].append(float(row["Counter_Value"]))
    return {k: sum(v[len(v) // 4:]) / len(v[len(v) // 4:]) for k, v in acc.items()}


def trace_table(path, min_calls=5):
    grp = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        if "ph::" not in r["Kernel_Name"]:
            continue
        wgs = "%sx%sx%s" % (int(r["Grid_Size_X"]) // max(1, int(r["Workgroup_Size_X"])), r["Grid_Size_Y"], r["Grid_Size_Z"])
        grp[(_short(r["Kernel_Name"]), wgs)].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    lines = [f"{'kernel':64s} {'workgroups':>14s} {'calls':>6s} {'avg_us':>9s} {'median':>9s} {'min_us':>9s} {'max_us':>9s}"]
    for (k, g), v in sorted(grp.items(), key=lambda kv: -sum(kv[1])):
        if len(v) < min_calls:
            continue
        v = sorted(v)
        lines.append(f"{k:64s} {g:>14s} {len(v):6d} {sum(v) / len(v):9.2f} {v[len(v) // 2]:9.2f} {v[0]:9.2f} {v[-1]:9.2f}")
    return "\n".join(lines)


def _write(name, text):
    os.makedirs(PROFILES, exist_ok=True)
    with open(os.path.join(PROFILES, name), "w") as f:
        f.write(text.rstrip() + "\n")
    print("wrote profiles/" + name)


def main(d):
    commit = _commit()
    out = {"commit": commit, "hbm_traffic_bytes": {}}
    head = f"(taken at commit {commit}; summary by python -m parrotserve_amd.profile_summary)\n"

    # ---- kernel traces -------------------------------------------------------------------------------------------
    for name, args, title, fname in (
            ("trace_c2", "--no-cpu --no-extras", "headline benchmark (config 2: fp16, B 64, one 4096-token prefix, "
             "suffix U[16,512], 32x128, 8 KV sets)", "bench_config2_kernel_trace.txt"),
            ("trace_all", "--no-cpu", "bench.py with the other configurations' workloads (its `extras`)",
             "bench_all_workloads_kernel_trace.txt"),
            ("trace_e2e", "--e2e-only", "the 13B-shape decode experiment (batch 64, shared 8192, diverged 10; fused "
             "per-layer ops) -- the library's kernels only; the GEMMs are library code", "e2e_decode_13b_kernel_trace.txt")):
        p = _csv(d, name, "kernel_trace")
        if p:
            _write(fname, "rocprofv3 kernel trace of " + title + "\n" + head + "command (on the GPU box, from /tmp):\n  " +
                   PRE % ("--kernel-trace --stats", args) + "\nthe library's kernels, one row per (kernel, workgroups); "
                   "durations in microseconds from the trace's start / end timestamps\n\n" + trace_table(p))

    # ---- HBM traffic ---------------------------------------------------------------------------------------------
    pats = ["decode_fused_kernel", "decode_items_kernel", "merge_kernel", "prefix_mfma8_kernel"]
    cf = counters_of(_csv(d, "cal_fetch", "counter_collection"), ["move_rows"]).get(("move_rows", "FETCH_SIZE"))
    cw = counters_of(_csv(d, "cal_write", "counter_collection"), ["move_rows"]).get(("move_rows", "WRITE_SIZE"))
    fe = counters_of(_csv(d, "fetch", "counter_collection"), pats)
    wr = counters_of(_csv(d, "write", "counter_collection"), pats)
    if cf and cw and fe and wr:
        known = 131072 * 8192 / 1024.0  # KiB read and written by one launch of the calibration copy
        ff, fw = known / cf, known / cw
        out["fetch_size_scale"], out["write_size_scale"] = ff, fw
        t = ["HBM traffic per launch of the headline benchmark's kernels (rocprofv3 --pmc, KiB per dispatch, mean over the "
             "timed launches)", head + "commands (on the GPU box, from /tmp; one counter per run):",
             "  " + PRE % ("--pmc FETCH_SIZE", "--no-cpu --no-extras --steps 24 --warmup 8"),
             "  " + PRE % ("--pmc WRITE_SIZE", "--no-cpu --no-extras --steps 24 --warmup 8"),
             "calibration (the library's move kernel as a plain copy of 131072 rows x 8 KiB: 1 GiB read, 1 GiB written per launch):",
             "  " + PRE % ("--pmc FETCH_SIZE", "--copy-calibration"), "  " + PRE % ("--pmc WRITE_SIZE", "--copy-calibration"),
             f"  FETCH_SIZE reads {cf:.1f} KiB for {known:.0f} KiB read  -> scale x{ff:.3f}",
             f"  WRITE_SIZE reads {cw:.1f} KiB for {known:.0f} KiB written -> scale x{fw:.3f}", "",
             f"{'kernel':24s} {'FETCH_SIZE':>12s} {'WRITE_SIZE':>12s} {'read MB':>10s} {'write MB':>10s} {'total MB':>10s}"]
        for k in pats:
            if (k, "FETCH_SIZE") not in fe or (k, "WRITE_SIZE") not in wr:
                continue
            f_, w_ = fe[(k, "FETCH_SIZE")], wr[(k, "WRITE_SIZE")]
            rb, wb = f_ * ff * 1024, w_ * fw * 1024
            out["hbm_traffic_bytes"][k] = rb + wb
            t.append(f"{k:24s} {f_:12.1f} {w_:12.1f} {rb / 1e6:10.1f} {wb / 1e6:10.1f} {(rb + wb) / 1e6:10.1f}")
        t += ["", "algorithmic bytes per launch at this workload: decode_fused_kernel (prefix + suffix phases) 2 x (4096 + "
              "17389 tokens) x 32 x 128 x 2 B = 352.0 MB of K/V (+ Q per split, partials written); decode_items_kernel (the "
              "batch without its prefix) 284.9 MB; prefix_mfma8_kernel (the batch with empty suffixes) 67.1 MB; merge_kernel "
              "reads the partials (its mean includes the short merges behind the phases run on their own)."]
        _write("bench_config2_hbm_traffic.txt", "\n".join(t))

    # ---- SQ counters of the decode kernels -----------------------------------------------------------------------
    sq = {}
    for n in ("sq1", "sq2", "grbm"):
        sq.update(counters_of(_csv(d, n, "counter_collection"), pats))
    if sq:
        t = ["Counters of the decode kernels at config 2 (rocprofv3 --pmc, mean per launch, summed over the chip's 8 XCDs)",
             head + "commands (on the GPU box, from /tmp; one pass per run, at most 8 SQ counters each):",
             "  " + PRE % ("--pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_ANY SQ_WAIT_INST_ANY SQ_ACTIVE_INST_ANY "
                           "SQ_INSTS_VALU SQ_INSTS_MFMA", "--no-cpu --no-extras --steps 24 --warmup 8"),
             "  " + PRE % ("--pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_WAIT_INST_LDS SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS "
                           "SQ_ACTIVE_INST_VMEM SQ_INSTS_VMEM_RD SQ_INSTS_LDS SQ_INSTS_SALU",
                           "--no-cpu --no-extras --steps 24 --warmup 8"),
             "  " + PRE % ("--pmc GRBM_GUI_ACTIVE GRBM_COUNT", "--no-cpu --no-extras --steps 24 --warmup 8"), ""]
        names = sorted({c for (_, c) in sq})
        t.append(f"{'counter':28s}" + "".join(f"{k.replace('_kernel', ''):>18s}" for k in pats))
        for c in names:
            t.append(f"{c:28s}" + "".join(f"{sq.get((k, c), float('nan')):18.0f}" for k in pats))
        t.append("")
        durations = {}  # average dispatch time per kernel from the kernel trace of the same command, microseconds
        tp = _csv(d, "trace_c2", "kernel_trace")
        if tp:
            acc = collections.defaultdict(list)
            for r in csv.DictReader(open(tp)):
                for k in pats:
                    if k in r["Kernel_Name"]:
                        acc[k].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
            durations = {k: sum(v) / len(v) for k, v in acc.items()}
        for k in pats:
            busy, act, n_mfma = sq.get((k, "SQ_VALU_MFMA_BUSY_CYCLES")), sq.get((k, "GRBM_GUI_ACTIVE")), sq.get((k, "SQ_INSTS_MFMA"))
            if not busy or not act:
                continue
            util = busy / (act / XCDS * SIMDS)
            out.setdefault(k, {})["mfma_pipe_utilisation"] = util
            if k in durations:
                # under --pmc every dispatch is serialised and GRBM_GUI_ACTIVE spans its set-up as well, which for a
                # kernel of some tens of microseconds overstates the denominator: the same busy cycles against the
                # kernel trace's own duration, at the 2.4 GHz the peak figures are quoted at
                by_time = busy / SIMDS / (durations[k] * 2400.0)
                out[k]["mfma_pipe_utilisation_by_trace_duration"] = by_time
                out[k]["trace_duration_us"] = durations[k]
            wait = sq.get((k, "SQ_WAIT_ANY"), 0) / max(1.0, sq.get((k, "SQ_WAVE_CYCLES", ), 1.0))
            out[k]["wait_fraction_of_wave_cycles"] = wait
            t.append(f"{k}: matrix-pipe utilisation = SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / {XCDS} XCDs x {SIMDS} "
                     f"SIMDs) = {busy:.0f} / {act / XCDS * SIMDS:.0f} = {util * 100:.1f} %  ({busy / max(1, n_mfma or 1):.0f} "
                     f"cycles per v_mfma_f32_32x32x16, {n_mfma or 0:.0f} of them); waves wait (SQ_WAIT_ANY / "
                     f"SQ_WAVE_CYCLES) {wait * 100:.0f} % of their cycles")
            if k in durations:
                t.append(f"    against the kernel trace's duration ({durations[k]:.2f} us, not serialised by the counter pass): "
                         f"{busy / SIMDS:.0f} busy cycles per SIMD / ({durations[k]:.2f} us x 2.4 GHz) = "
                         f"{out[k]['mfma_pipe_utilisation_by_trace_duration'] * 100:.1f} %")
        t += ["", "The prefix phase is a dense contraction with exactly B = 64 FLOP per K/V byte: from HBM the matrix pipe cannot "
              "be busy more than min(1, 64 x 8 TB/s / 2.5 PFLOP/s) = 20 % of the time, and the kernel is a chain of dependent "
              "steps per workgroup (slot window, ring fill, four tile steps, fold), not a steady stream -- see "
              "decode_fused_config2_timeline.txt for where the time goes."]
        _write("prefix_config2_mfma_counters.txt", "\n".join(t))

    # ---- prefill counters ----------------------------------------------------------------------------------------
    pf = {}
    for n in ("pf1", "pf2", "pf3"):
        pf.update(counters_of(_csv(d, n, "counter_collection"), ["prefill_mfma8_kernel"]))
    if pf:
        g = lambda c: pf.get(("prefill_mfma8_kernel", c), float("nan"))
        t = ["Counters of prefill_mfma8_kernel<bf16, 256-query tiles, 64-token steps> on config 4 (16 chunks, 9,404 new tokens over "
             "2048-token parents, 40 x 128, bf16), mean per launch, rocprofv3 --pmc, summed over the chip's 8 XCDs.",
             head + "commands (on the GPU box, from /tmp; one pass per run):",
             "  " + PRE % ("--pmc SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_MFMA SQ_INSTS_VALU "
                           "SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS SQ_WAIT_INST_LDS", "--prefill-only"),
             "  " + PRE % ("--pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_LDS SQ_INSTS_VALU_TRANS_F32 SQ_INSTS_VMEM_RD "
                           "SQ_INSTS_SALU SQ_WAIT_ANY SQ_WAVES", "--prefill-only"),
             "  " + PRE % ("--pmc GRBM_GUI_ACTIVE GRBM_COUNT", "--prefill-only"), "", f"{'counter':28s} {'per launch':>16s}"]
        for c in sorted({c for (_, c) in pf}):
            t.append(f"{c:28s} {g(c):16.0f}")
        mf, va, tr = g("SQ_INSTS_MFMA"), g("SQ_INSTS_VALU"), g("SQ_INSTS_VALU_TRANS_F32")
        util = g("SQ_VALU_MFMA_BUSY_CYCLES") / (g("GRBM_GUI_ACTIVE") / XCDS * SIMDS)
        out["prefill_mfma8_kernel"] = {"mfma_pipe_utilisation": util, "valu_per_mfma": va / mf, "trans_per_mfma": tr / mf}
        t += ["", f"matrix-pipe utilisation = SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / {XCDS} x {SIMDS} SIMDs) = {util * 100:.1f} %",
              f"vector-ALU instructions per matrix instruction {va / mf:.2f}, of which exponentials (quarter rate) {tr / mf:.2f}; "
              f"LDS reads per matrix instruction {g('SQ_INSTS_LDS') / mf:.2f}; bank conflicts {g('SQ_LDS_BANK_CONFLICT'):.0f}; "
              f"waves wait {g('SQ_WAIT_ANY') / g('SQ_WAVE_CYCLES') * 100:.0f} % of their cycles",
              f"matrix work issued: {mf:.0f} x 32,768 FLOP = {mf * 32768 / 1e9:.1f} GFLOP per launch"]
        _write("prefill_config4_mfma_counters.txt", "\n".join(t))

    # ---- timeline of the fused decode kernel ---------------------------------------------------------------------
    tl = os.path.join(d, "timeline.json")
    if os.path.exists(tl):
        j = pj = None
        for line in open(tl):
            if line.startswith("{"):
                both = json.loads(line)
                j = both["fused_kernel_timeline"]
                pj = both.get("prefill_kernel_timeline")
        if pj:
            m = pj["marks"]
            t = ["Where the waves of prefill_mfma8_kernel<bf16, 256-query tiles, 64-token steps> spend a launch: one 256-query chunk "
                 f"over a 2048-token parent, 40 heads = 40 workgroups resident at once, {pj['steps']} steps each (per-wave timestamps at "
                 "marks inside the kernel, profiling variant of the library; microseconds from the first wave's entry; median over 6 "
                 "launches per wave, then the spread over the launch's 320 waves)",
                 head + "command (on the GPU box; no profiler):\n  python3 bench.py --timeline", "",
                 f"{'mark':50s} {'min':>7s} {'p10':>7s} {'p50':>7s} {'p90':>7s} {'max':>7s}"]
            for k, v in m.items():
                t.append(f"{k:50s} {v['min']:7.2f} {v['p10']:7.2f} {v['p50']:7.2f} {v['p90']:7.2f} {v['max']:7.2f}")
            first = m["step 0 (tile landed, workgroup barrier passed)"]["p50"]
            done, end = m["tile loop done"]["p50"], m["kernel exit"]["p50"]
            t += ["", f"median wave: prologue (entry to step 0) {first - m['kernel entry']['p50']:.1f} us, tile loop {done - first:.1f} us = "
                  f"{(done - first) / pj['steps']:.2f} us per step, epilogue (loop done to exit) {end - done:.1f} us"]
            out["prefill_kernel_timeline"] = m
            _write("prefill_tile_timeline.txt", "\n".join(t))
        if j:
            t = ["Where the waves of decode_fused_kernel spend a launch at config 2 (per-wave timestamps at marks inside the kernel, "
                 "profiling variant of the library; microseconds from the first wave's entry; median over 8 launches per wave, then "
                 "the spread over the launch's 2048 waves)", head + "command (on the GPU box; no profiler):\n  python3 bench.py --timeline", "",
                 f"{'mark':62s} {'min':>7s} {'p10':>7s} {'p50':>7s} {'p90':>7s} {'max':>7s}"]
            for k, v in j["marks"].items():
                t.append(f"{k:62s} {v['min']:7.2f} {v['p10']:7.2f} {v['p50']:7.2f} {v['p90']:7.2f} {v['max']:7.2f}")
            t += ["", f"spread of 'suffix stream done' inside a workgroup (its slowest wave gates the prefix steps), median: "
                  f"{j['suffix_done_spread_inside_workgroup_p50']} us",
                  "kernel exit of the slowest wave of a workgroup, median per XCD (workgroup id mod 8): " +
                  ", ".join(str(x) for x in j["exit_by_xcd_p50"])]
            out["decode_fused_kernel_timeline"] = j["marks"]
            _write("decode_fused_config2_timeline.txt", "\n".join(t))

    with open(os.path.join(PROFILES, "counters.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote profiles/counters.json")


if __name__ == "__main__":
    if len(sys.argv) != 2:
        sys.exit(__doc__)
    main(sys.argv[1])
