"""
rocprofv3 output -> the short text summaries kept under ``profiles/``.

``bench.py --trace-pass hot|cold`` and ``bench.py --counter-pass`` are the
programs that get profiled; each prints one JSON line (its *table*) saying
which kernel ran for which configuration, with how many warm-up and measured
launches and how many algorithmic bytes.  The functions here join such a table
with the CSV files rocprofv3 wrote and produce a summary whose last line,
``json: {...}``, is keyed by KERNEL NAME -- ``bench.py`` looks figures up by
the name of the kernel it has just timed, so a summary that was not refreshed
after the generator changed yields nothing instead of a stale number.

    python -m neon_amd.profile_summary durations --csv K.csv --log pass.log --out profiles/X.txt --command "..."
    python -m neon_amd.profile_summary traffic --fetch F.csv --write W.csv --log pass.log --out ... --command "..." --command "..."
    python -m neon_amd.profile_summary issue --csv S1.csv --csv S2.csv --log pass.log --out ... --command "..."
    python -m neon_amd.profile_summary lds --csv L.csv --log pass.log --out ... --command "..."

The metric for durations is the one the kernels are judged by: rocprofv3
kernel duration (end - start timestamp of the dispatch), median over the
measured launches after the warm-up launches have been dropped.
"""
import argparse
import collections
import csv
import json
import statistics
import sys


def read_table(log_path):
    """the table a profiled bench.py pass printed (its only JSON line with a ``pass`` key)"""
    with open(log_path) as f:
        for line in f:
            line = line.strip()
            if line.startswith("{") and '"pass"' in line:
                return json.loads(line)
    raise ValueError("no pass table in %s" % log_path)


def lookup(summary_path, kernel_name):
    """the record of ``kernel_name`` in a summary's json line, or None"""
    try:
        with open(summary_path) as f:
            lines = [l for l in f if l.startswith("json: ")]
        return json.loads(lines[-1][6:]).get(kernel_name)
    except (IOError, OSError, IndexError, ValueError):
        return None


def lookup_part(summary_path, part):
    """as ``lookup`` for a prebuilt kernel, whose name is the compiler's: the first record
    whose kernel name contains ``part``, or None"""
    try:
        with open(summary_path) as f:
            lines = [l for l in f if l.startswith("json: ")]
        for name, rec in json.loads(lines[-1][6:]).items():
            if part in name:
                return rec
    except (IOError, OSError, IndexError, ValueError):
        pass
    return None


def _dispatches(csv_path):
    """kernel name -> list of durations in ns, in dispatch order"""
    rows = []
    with open(csv_path) as f:
        for r in csv.DictReader(f):
            rows.append((int(r["Dispatch_Id"]), r["Kernel_Name"], int(r["End_Timestamp"]) - int(r["Start_Timestamp"])))
    rows.sort()
    out = collections.defaultdict(list)
    for _, name, ns in rows:
        out[name].append(ns)
    return out


def durations(csv_path, table, out_path, commands):
    per_kernel = _dispatches(csv_path)
    _resolve(table["rows"], list(per_kernel))
    taken = collections.defaultdict(int)       # launches of a kernel already assigned to earlier rows
    lines, js = [], {}
    mode = table["pass"]
    lines.append("rocprofv3 kernel durations of the benchmark op-trees, %s, one MI355X (gfx950)" % table["what"])
    lines.append("")
    lines.append("command%s (from the repository root on the GPU box; TMPDIR=/tmp):" % ("s" if len(commands) > 1 else ""))
    for c in commands:
        lines.append("  " + c)
    lines.append("")
    lines.append("Per kernel: duration = End_Timestamp - Start_Timestamp of each dispatch in the kernel trace; the first")
    lines.append("`warm` launches are dropped, the statistics are over the `calls` launches that follow.  frac = algorithmic")
    lines.append("bytes / median duration / 8 TB/s.  %s" % table["note"])
    lines.append("")
    lines.append("%-52s %5s %5s %9s %9s %9s %7s  %s" % ("configuration", "warm", "calls", "median us", "min us", "max us",
                                                  "frac", "kernel"))
    for row in table["rows"]:
        name, warm, n = row["kernel"], row["warmup"], row["launches"]
        seq = per_kernel.get(name, [])[taken[name]:taken[name] + warm + n]
        taken[name] += warm + n
        meas = seq[warm:]
        if len(meas) < n:
            lines.append("%-52s  (only %d of %d launches found in the trace)" % (row["label"][:52], len(seq), warm + n))
            continue
        med = statistics.median(meas) / 1e3
        frac = row["algorithmic_bytes"] / (med * 1e-6) / 8e12
        lines.append("%-52s %5d %5d %9.2f %9.2f %9.2f %7.3f  %s" % (row["label"][:52], warm, len(meas), med,
                                                                  min(meas) / 1e3, max(meas) / 1e3, frac, name[:100]))
        rec = {"label": row["label"], "median_us": round(med, 3), "min_us": round(min(meas) / 1e3, 3),
               "max_us": round(max(meas) / 1e3, 3), "calls": len(meas), "algorithmic_bytes": row["algorithmic_bytes"],
               "frac": round(frac, 4), "pass": mode}
        js.setdefault(name, rec)
    lines.append("")
    lines.append("json: " + json.dumps(js))
    with open(out_path, "w") as f:
        f.write("\n".join(lines) + "\n")
    return js


def _counters(csv_path):
    """kernel name -> counter name -> values in dispatch order"""
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    with open(csv_path) as f:
        for r in csv.DictReader(f):
            agg[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return agg


def _resolve(rows, names):
    """rows of prebuilt kernels name a part of the compiler's kernel name: fill in the full one"""
    for r in rows:
        if not r.get("kernel") and r.get("kernel_contains"):
            found = [n for n in names if r["kernel_contains"] in n]
            r["kernel"] = found[0] if found else r["kernel_contains"]
    return rows


def traffic(fetch_csv, write_csv, table, out_path, commands):
    """FETCH_SIZE / WRITE_SIZE (KiB per dispatch), each scaled by what the same
    counter reads for the pass's plain copy kernel of known size"""
    fetch, write = _counters(fetch_csv), _counters(write_csv)
    rows = _resolve(table["rows"], list(fetch))
    cal = rows[0]
    assert cal["label"].startswith("copy"), "the first row of a counter pass is the calibration copy"
    kib = cal["algorithmic_bytes"] / 2 / 1024.0
    f_cal, w_cal = fetch[cal["kernel"]]["FETCH_SIZE"][-1], write[cal["kernel"]]["WRITE_SIZE"][-1]
    fs, ws = kib / f_cal, kib / w_cal
    out, js = [], {}
    out.append("HBM traffic per launch from rocprofv3 hardware counters, one MI355X (gfx950)")
    out.append("")
    out.append("commands (two separate passes, from the repository root on the GPU box; TMPDIR=/tmp):")
    for c in commands:
        out.append("  " + c)
    out.append("")
    out.append("`bench.py --counter-pass` launches, three times each, a plain copy kernel of known size (out = x * 1.0 over")
    out.append("25,000,000 fp32: 100,000,000 B read and as many written = %.0f KiB each way) and the kernel behind every" % kib)
    out.append("benchmark configuration and the batch-norm pair.  Counter values are KiB per dispatch (last dispatch shown).")
    out.append("")
    out.append("calibration (copy kernel %s):" % cal["kernel"])
    out.append("  FETCH_SIZE  %9.0f KiB reported for %.0f KiB read     -> scale factor %.4f" % (f_cal, kib, fs))
    out.append("  WRITE_SIZE  %9.0f KiB reported for %.0f KiB written  -> scale factor %.4f" % (w_cal, kib, ws))
    out.append("")
    out.append("%-30s %12s %12s %12s %12s %7s  %s" % ("configuration", "FETCH KiB", "WRITE KiB", "HBM bytes", "algorithmic",
                                               "ratio", "kernel"))
    for r in rows[1:]:
        try:
            f, w = fetch[r["kernel"]]["FETCH_SIZE"][-1], write[r["kernel"]]["WRITE_SIZE"][-1]
        except IndexError:
            out.append("%-24s  (kernel %s not in the counter files)" % (r["label"], r["kernel"]))
            continue
        total = (f * fs + w * ws) * 1024.0
        out.append("%-30s %12.0f %12.0f %12.0f %12d %7.3f  %s" % (r["label"][:30], f, w, total, r["algorithmic_bytes"],
                                                                 total / r["algorithmic_bytes"], r["kernel"][:90]))
        js[r["kernel"]] = {"label": r["label"], "traffic_bytes": round(total), "algorithmic_bytes": r["algorithmic_bytes"],
                           "ratio": round(total / r["algorithmic_bytes"], 4)}
    out.append("")
    out.append("FETCH_SIZE counts what reaches the L2s from the memory side (the 256 MB memory-side cache included), so")
    out.append("kernels re-run on tensors that cache holds still show their read traffic; the totals of the split column")
    out.append("reductions include the partials their workgroups hand over (written through and read back once).")
    out.append("")
    out.append("json: " + json.dumps(js))
    with open(out_path, "w") as f:
        f.write("\n".join(out) + "\n")
    return js


def issue(csv_paths, table, out_path, commands, cu_count=256, clock_ghz=2.4):
    """instruction counts per wave and the issue time they imply"""
    agg = collections.defaultdict(dict)
    for p in csv_paths:
        for name, per in _counters(p).items():
            for cname, vals in per.items():
                agg[name][cname] = sum(vals) / len(vals)
    _resolve(table["rows"], list(agg))
    out, js = [], {}
    out.append("Issue-side counters of the benchmark kernels, rocprofv3 on one MI355X (gfx950)")
    out.append("")
    out.append("commands (one pass each; from the repository root on the GPU box; TMPDIR=/tmp):")
    for c in commands:
        out.append("  " + c)
    out.append("")
    out.append("Per dispatch (mean over the pass's launches).  waves = SQ_WAVES; X/wave = SQ_INSTS_X / waves; `VALU issue us`")
    out.append("= VALU/wave x waves per SIMD x 4 cycles / %.1f GHz: the time a SIMD needs just to issue the kernel's vector" % clock_ghz)
    out.append("instructions (a wave64 instruction occupies a 16-lane SIMD for 4 cycles); waves/SIMD = waves / (%d CUs x 4)." % cu_count)
    out.append("")
    out.append("%-24s %8s %10s %8s %8s %10s %10s %10s %13s  %s" % ("configuration", "waves", "VALU/wave", "SALU/w", "LDS/w",
                                                              "VMEM rd/w", "VMEM wr/w", "waves/SIMD", "VALU issue us", "kernel"))
    for r in table["rows"]:
        c = agg.get(r["kernel"])
        if not c or not c.get("SQ_WAVES"):
            continue
        waves = c["SQ_WAVES"]
        per = lambda k: c.get(k, 0.0) / waves
        wps = waves / (cu_count * 4.0)
        issue_us = per("SQ_INSTS_VALU") * wps * 4 / (clock_ghz * 1e3)
        out.append("%-24s %8d %10.1f %8.1f %8.1f %10.1f %10.1f %10.1f %13.2f  %s" % (
            r["label"][:24], waves, per("SQ_INSTS_VALU"), per("SQ_INSTS_SALU"), per("SQ_INSTS_LDS"),
            per("SQ_INSTS_VMEM_RD"), per("SQ_INSTS_VMEM_WR"), wps, issue_us, r["kernel"]))
        js[r["kernel"]] = {"label": r["label"], "waves": waves, "valu_per_wave": round(per("SQ_INSTS_VALU"), 1),
                           "valu_issue_us": round(issue_us, 3)}
    out.append("")
    out.append("json: " + json.dumps(js))
    with open(out_path, "w") as f:
        f.write("\n".join(out) + "\n")
    return js


def lds(csv_paths, table, out_path, commands):
    """LDS instruction and conflict counters of the kernels that stage data in LDS"""
    agg = collections.defaultdict(dict)
    for p in csv_paths:
        for name, per in _counters(p).items():
            for cname, vals in per.items():
                agg[name][cname] = sum(vals) / len(vals)
    _resolve(table["rows"], list(agg))
    out, js = [], {}
    out.append("LDS counters, rocprofv3 on one MI355X (gfx950)")
    out.append("")
    out.append("command (from the repository root on the GPU box; TMPDIR=/tmp):")
    for c in commands:
        out.append("  " + c)
    out.append("")
    out.append("Per dispatch (mean over the pass's launches).  LDS/wave = SQ_INSTS_LDS / SQ_WAVES; conflict = the share of")
    out.append("the cycles the LDS was addressing (SQ_LDS_IDX_ACTIVE) that went to bank conflicts (SQ_LDS_BANK_CONFLICT).")
    out.append("")
    out.append("%-32s %8s %9s %14s %14s %9s  %s" % ("operation", "waves", "LDS/wave", "idx active cyc", "conflict cyc", "conflict",
                                             "kernel"))
    for r in table["rows"]:
        c = agg.get(r["kernel"])
        if not c or not c.get("SQ_WAVES") or not c.get("SQ_INSTS_LDS"):
            continue
        act, conf = c.get("SQ_LDS_IDX_ACTIVE", 0.0), c.get("SQ_LDS_BANK_CONFLICT", 0.0)
        out.append("%-32s %8d %9.1f %14.0f %14.0f %8.1f%%  %s" % (r["label"][:32], c["SQ_WAVES"], c["SQ_INSTS_LDS"] / c["SQ_WAVES"],
                                                              act, conf, 100.0 * conf / act if act else 0.0, r["kernel"][:80]))
        js[r["kernel"]] = {"label": r["label"], "lds_per_wave": round(c["SQ_INSTS_LDS"] / c["SQ_WAVES"], 1),
                           "bank_conflict_share": round(conf / act, 4) if act else None}
    out.append("")
    out.append("json: " + json.dumps(js))
    with open(out_path, "w") as f:
        f.write("\n".join(out) + "\n")
    return js


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("kind", choices=("durations", "traffic", "issue", "lds"))
    ap.add_argument("--csv", action="append", default=[])
    ap.add_argument("--fetch")
    ap.add_argument("--write")
    ap.add_argument("--log", required=True, help="stdout of the profiled bench.py pass (holds its table)")
    ap.add_argument("--out", required=True)
    ap.add_argument("--command", action="append", default=[], help="the rocprofv3 command line(s), quoted in the summary")
    args = ap.parse_args(argv)
    table = read_table(args.log)
    if args.kind == "durations":
        js = durations(args.csv[0], table, args.out, args.command)
    elif args.kind == "traffic":
        js = traffic(args.fetch, args.write, table, args.out, args.command)
    elif args.kind == "lds":
        js = lds(args.csv, table, args.out, args.command)
    else:
        js = issue(args.csv, table, args.out, args.command)
    print("%s: %d kernels -> %s" % (args.kind, len(js), args.out))


if __name__ == "__main__":
    sys.exit(main())
