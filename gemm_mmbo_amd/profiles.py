"""rocprofv3 evidence for this library's kernels: capture the passes, then turn their CSV files into a short text summary.

    python -m gemm_mmbo_amd.report capture CASE --out DIR [--summary FILE]     # needs a GPU; runs rocprofv3 once per pass
    python -m gemm_mmbo_amd.report summarise CASE DIR [--summary FILE]         # pure CPU: reads what `capture` left in DIR
    python -m gemm_mmbo_amd.report cases                                       # lists the cases

The reference has one sweep script over its benchmark binary and reads the numbers off the terminal
(src/gemm/run.sh:1-5 over src/gemm/benchmark.cc:89-109); this is the same loop with the profiler in it and a file at
the end.

A case is a program (bench.py with one leg, or this package's report driver over a list of shapes) and the rocprofv3
passes to run it under.  Every pass is a run of its own, `rocprofv3 <flags> -d DIR/<pass> -o <pass> --output-format csv --
python3 <program>`, with the program's stdout kept in DIR/<pass>.stdout: the program prints JSON lines that say how
many launches it timed, what its own HIP-event timing of them was, and what a register-only MFMA loop sustained in the
same session on the same box (mmbo_probe_mfma_ceiling) -- so that a summary taken on one box can be compared with a
benchmark line from another through `kernel / ceiling`, which is independent of the box's clocks.

What the summary reports, and how it is computed from the CSV files:
  * kernel time     = MEDIAN over the TIMED dispatches of End_Timestamp - Start_Timestamp in <pass>_kernel_trace.csv.  The
                      timed dispatches are the last N of the kernel in the run, N taken from the program's JSON (warm-up and
                      settle launches come first and run on a chip that has not reached its steady clock yet).
  * TFLOP/s         = algorithmic flop per launch (2 m n k batch) / kernel time; fraction of the published matrix peak.
  * gap             = median of (next Start - this End) over the timed dispatches: 0 when launches run back to back; when the
                      profiler makes every dispatch wait for the previous one's completion signal it is a few microseconds.
  * shader clock    = GRBM_GUI_ACTIVE / 8 XCDs / kernel duration   (long kernels only: the counter also ticks around a short one)
  * MFMA busy       = SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 * 1024 SIMDs); for short kernels
                      SQ_VALU_MFMA_BUSY_CYCLES / 1024 / (duration * 2.4 GHz) instead
  * LDS conflicts   = SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE
  * L2 hit rate     = TCC_HIT_sum / (TCC_HIT_sum + TCC_MISS_sum)
  * fetched/written = FETCH_SIZE / WRITE_SIZE (KiB per dispatch) * 1024 * factor, factor = known bytes of a plain copy-like
                      kernel in the same run / what the counter read for it (bench.py makes one elementwise pass over A for
                      this; on MI355X FETCH_SIZE reads half the true bytes, WRITE_SIZE all of them)
"""
import csv
import glob
import json
import os
import re
import statistics
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PEAK_TFLOPS = {"h": 2500.0, "s": 157.3, "d": 78.6}
ESZ = {"h": 2, "s": 4, "d": 8}
LIB_KERNEL = re.compile(r"mmbo(::|\d+)?.*(gemm_x16_kernel|gemm_ring_kernel|gemm_staged_kernel|dgemm_kernel|splitk_reduce_kernel)")
LONG_KERNEL_NS = 200e3          # below this GRBM_GUI_ACTIVE is not a clock measurement

SQ_COUNTERS = ["SQ_VALU_MFMA_BUSY_CYCLES", "SQ_BUSY_CYCLES", "SQ_WAVE_CYCLES", "SQ_INSTS_VALU_MFMA_MOPS_F16",
               "SQ_INSTS_VALU_MFMA_MOPS_F32", "SQ_LDS_BANK_CONFLICT", "SQ_LDS_IDX_ACTIVE", "SQ_WAIT_INST_ANY", "GRBM_GUI_ACTIVE"]
TCC_COUNTERS = ["TCC_HIT_sum", "TCC_MISS_sum", "TCC_EA0_RDREQ_sum", "TCC_REQ_sum"]
PASSES = {
    "trace": ["--kernel-trace", "--stats"],
    "sq": ["--pmc"] + SQ_COUNTERS + ["--kernel-trace"],
    "tcc": ["--pmc"] + TCC_COUNTERS + ["--kernel-trace"],
    "fetch": ["--pmc", "FETCH_SIZE", "--kernel-trace"],
    "write": ["--pmc", "WRITE_SIZE", "--kernel-trace"],
}

SKINNY = ["h,N,N,4096,128,4096", "s,N,N,4096,128,4096", "h,N,N,128,4096,8192", "s,N,N,128,4096,8192",
          "h,N,N,1023,777,513", "s,N,N,1023,777,513"]
CONFIGS = ["s,N,N,1024,1024,1024", "s,N,T,4096,4096,4096,1,1.5,0.5", "s,T,N,4096,4096,4096,1,1.5,0.5",
           "h,T,N,512,512,512,64,1,1", "d,N,T,44160,2048,384,1,-1,1,44160"]
MIDSIZE = ["h,N,N,2048,2048,2048", "h,N,N,3000,3000,3000", "h,N,N,4096,4096,4096"]

CASES = {
    "gemm_x16_f16_8192": {
        "title": "HGEMM NN 8192^3 (fp16 in/out, fp32 accumulate), the benchmark's headline leg",
        "program": ["bench.py", "--no-cpu", "--only", "f16"], "short": ["--steps", "5", "--warmup", "2"],
        "passes": ["trace", "sq", "tcc", "fetch", "write"], "dtype": "h", "shape": (8192, 8192, 8192, 1, 0.0)},
    "gemm_x16_f32_8192": {
        "title": "SGEMM NN 8192^3, the benchmark's fp32 leg",
        "program": ["bench.py", "--no-cpu", "--only", "f32"], "short": ["--steps", "10", "--warmup", "2"],
        "passes": ["trace", "sq", "tcc", "fetch", "write"], "dtype": "s", "shape": (8192, 8192, 8192, 1, 0.0)},
    "skinny_cfg4": {
        "title": "Skinny and irregular GEMMs (benchmark configuration 4), NN, alpha = 1, beta = 0, automatic pick",
        "program": ["-m", "gemm_mmbo_amd.report", "shapes"] + SKINNY + ["--no-check", "--reps", "10", "--ceilings"],
        "passes": ["trace", "sq", "fetch", "write"], "specs": SKINNY},
    "cfg1_cfg2_cfg5_hpl": {
        "title": "Benchmark configurations 1, 2, 5 and the reference's fp64 HPL shape (src/gemm/run.sh:2-5), automatic pick",
        "program": ["-m", "gemm_mmbo_amd.report", "shapes"] + CONFIGS + ["--no-check", "--reps", "10", "--ceilings"],
        "passes": ["trace", "sq"], "specs": CONFIGS},
    "midsize_fp16": {
        "title": "HGEMM NN at sizes whose tile counts do not fill a whole number of rounds of 256 CUs, automatic pick",
        "program": ["-m", "gemm_mmbo_amd.report", "shapes"] + MIDSIZE + ["--no-check", "--reps", "10", "--ceilings"],
        "passes": ["trace", "sq"], "specs": MIDSIZE},
}


# ---------------------------------------------------------------------------------------------- reading rocprofv3's files
def _find(outdir, suffix):
    hits = sorted(glob.glob(os.path.join(outdir, "**", "*" + suffix), recursive=True))
    return hits[0] if hits else None


def read_trace(passdir):
    """Dispatches of <passdir>/*_kernel_trace.csv in dispatch order: [{'name', 'start', 'end', 'id'}]."""
    path = _find(passdir, "_kernel_trace.csv")
    if not path:
        return []
    rows = []
    for r in csv.DictReader(open(path, newline="")):
        rows.append({"name": r["Kernel_Name"], "start": int(r["Start_Timestamp"]), "end": int(r["End_Timestamp"]),
                     "id": int(r.get("Dispatch_Id") or len(rows))})
    rows.sort(key=lambda d: (d["start"], d["id"]))
    return rows


def read_counters(passdir):
    """{dispatch id: {'name', counter: value}} from <passdir>/*_counter_collection.csv (one row per dispatch and counter;
    a counter that rocprofv3 reports per XCD or per instance in several rows is summed)."""
    path = _find(passdir, "_counter_collection.csv")
    out = {}
    if not path:
        return out
    for r in csv.DictReader(open(path, newline="")):
        d = out.setdefault(int(r["Dispatch_Id"]), {"name": r["Kernel_Name"]})
        d[r["Counter_Name"]] = d.get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    return out


def read_json_lines(path):
    out = []
    if path and os.path.exists(path):
        for line in open(path):
            line = line.strip()
            if line.startswith("{"):
                try:
                    out.append(json.loads(line))
                except ValueError:
                    pass
    return out


def median(xs):
    return statistics.median(xs) if xs else float("nan")


def short_name(name, width=112):
    name = name.replace("void ", "")
    return name if len(name) <= width else name[:width - 3] + "..."


# ---------------------------------------------------------------------------------------------- what belongs to which GEMM
def split_by_shape(dispatches, records):
    """The library's dispatches of a `report shapes` run, cut into one list per shape record.  A GEMM call launches one
    main kernel, followed by the reduction kernel when it ran with split-K; a record says how many calls the driver made
    for its shape (`calls_total`, of which the last `calls_timed` are the timed ones).  Returns
    [(record, all dispatches of the shape, its timed dispatches)]; raises if the calls do not add up to what the trace holds."""
    calls = []
    for d in dispatches:
        if not LIB_KERNEL.search(d["name"]):
            continue
        if "splitk_reduce" in d["name"]:
            if not calls:
                raise ValueError("the trace starts with a reduction kernel")
            calls[-1].append(d)
        else:
            calls.append([d])
    want = sum(r["calls_total"] for r in records)
    if want != len(calls):
        raise ValueError(f"the trace holds {len(calls)} GEMM calls of this library, the program's records account for {want}")
    out, at = [], 0
    for r in records:
        mine = calls[at:at + r["calls_total"]]
        at += r["calls_total"]
        timed = mine[len(mine) - r["calls_timed"]:]
        out.append((r, [d for c in mine for d in c], [d for c in timed for d in c]))
    return out


def per_kernel(dispatches):
    """{kernel name: [durations in ns]} in first-seen order."""
    out = {}
    for d in dispatches:
        out.setdefault(d["name"], []).append(d["end"] - d["start"])
    return out


def gaps(dispatches):
    return [b["start"] - a["end"] for a, b in zip(dispatches, dispatches[1:])]


def counter_means(counters, ids):
    """Mean of every counter over the dispatches `ids`."""
    acc = {}
    for i in ids:
        for k, v in counters.get(i, {}).items():
            if k != "name":
                acc.setdefault(k, []).append(v)
    return {k: sum(v) / len(v) for k, v in acc.items()}


def derived_lines(c, dur_ns, flops=None):
    """Text lines of the derived figures (module docstring) from per-dispatch counter means `c` and the duration."""
    L = []
    if "GRBM_GUI_ACTIVE" in c and "SQ_VALU_MFMA_BUSY_CYCLES" in c:
        if dur_ns >= LONG_KERNEL_NS:
            clk = c["GRBM_GUI_ACTIVE"] / 8 / dur_ns
            busy = c["SQ_VALU_MFMA_BUSY_CYCLES"] / (c["GRBM_GUI_ACTIVE"] / 8 * 1024)
            L.append(f"shader clock = GRBM_GUI_ACTIVE / 8 XCDs / duration = {clk:.2f} GHz")
            L.append(f"MFMA busy = SQ_VALU_MFMA_BUSY_CYCLES / (GRBM_GUI_ACTIVE / 8 * 1024 SIMDs) = {busy * 100:.1f} %"
                     f"   (busy x clock / 2.4 GHz = {busy * clk / 2.4:.3f} of the matrix peak)")
        else:
            busy = c["SQ_VALU_MFMA_BUSY_CYCLES"] / 1024 / (dur_ns * 2.4)
            L.append(f"MFMA busy cycles = {busy * 100:.1f} % of the kernel's duration at 2.4 GHz (too short a kernel for a clock figure)")
    for key, per in (("SQ_INSTS_VALU_MFMA_MOPS_F16", 512), ("SQ_INSTS_VALU_MFMA_MOPS_F32", 512)):
        if flops and c.get(key, 0) > 0:
            L.append(f"{key} * {per} = {c[key] * per:.4e} flop (algorithmic {flops:.4e})")
    if c.get("SQ_LDS_IDX_ACTIVE", 0) > 0:
        L.append(f"LDS bank-conflict cycles / LDS active cycles = {c.get('SQ_LDS_BANK_CONFLICT', 0.0) / c['SQ_LDS_IDX_ACTIVE'] * 100:.1f} %")
    if c.get("TCC_HIT_sum", 0) + c.get("TCC_MISS_sum", 0) > 0:
        L.append(f"L2 hit rate = TCC_HIT / (TCC_HIT + TCC_MISS) = {c['TCC_HIT_sum'] / (c['TCC_HIT_sum'] + c['TCC_MISS_sum']) * 100:.1f} %")
    return L


def command_line(case, pass_name, short=False):
    c = CASES[case]
    prog = c["program"] + (c.get("short", []) if short else [])
    prog = [("<repo>/" + p if p == "bench.py" else p) for p in prog]
    return ("cd /tmp && export TMPDIR=/tmp PYTHONPATH=<repo> && rocprofv3 " + " ".join(PASSES[pass_name]) +
            f" -d <out>/{pass_name} -o {pass_name} --output-format csv -- python3 " + " ".join(prog))


# ---------------------------------------------------------------------------------------------- the summaries
CALIBRATION = re.compile(r"elementwise_kernel|CUDAFunctor_add|vectorized")


def calibration_factor(passdir, counter, true_bytes):
    """bytes per KiB-unit of `counter` for a plain elementwise pass of `true_bytes` read and written: the first dispatch
    in the pass that looks like torch's elementwise kernel and is preceded by the operand fills."""
    cnt = read_counters(passdir)
    best = None
    for i in sorted(cnt):
        d = cnt[i]
        if CALIBRATION.search(d["name"]) and counter in d and d[counter] > 0:
            # the calibration pass is the one whose reading is nearest the expected one (other elementwise kernels of the
            # run -- fills, casts -- move different byte counts)
            ratio = true_bytes / (d[counter] * 1024.0)
            score = abs((ratio if ratio >= 1 else 1 / ratio) - (2.0 if counter == "FETCH_SIZE" else 1.0))
            if best is None or score < best[0]:
                best = (score, ratio, d["name"], d[counter])
    return best[1:] if best else None


def summarise_bench(case, outdir):
    c = CASES[case]
    m, n, k, batch, beta = c["shape"]
    d = c["dtype"]
    flops = 2.0 * m * n * k * batch
    alg_read, alg_write = (m * k + k * n) * ESZ[d] * batch, m * n * ESZ[d] * batch
    peak = PEAK_TFLOPS[d]
    L = [c["title"] + "; MI355X", "=" * 120]
    tr = read_trace(os.path.join(outdir, "trace"))
    recs = read_json_lines(os.path.join(outdir, "trace.stdout"))
    bench = recs[-1] if recs else {}
    mine = [x for x in tr if LIB_KERNEL.search(x["name"]) and "splitk" not in x["name"]]
    if not mine:
        raise ValueError(f"{outdir}/trace holds no dispatch of this library's kernels")
    by = per_kernel(mine)
    kernel = max(by, key=lambda kname: sum(by[kname]))
    runs = [x for x in mine if x["name"] == kernel]
    steps = int(bench.get("steps") or 0) or min(50, len(runs))
    timed = runs[-steps:]
    durs = [x["end"] - x["start"] for x in timed]
    med = median(durs)
    tf = flops / med * 1e-3
    L += [f"kernel: {kernel}", f"tile config: {bench.get('config', {}).get('tile_config', '?')}", ""]
    L += ["1. " + " ".join(["rocprofv3"] + PASSES["trace"]), "   command: " + command_line(case, "trace"),
          f"   {len(runs)} dispatches of the kernel in the run (warm-up, settle phase, timed region); the TIMED ones are the last {len(timed)}:",
          f"   median {med / 1e3:.1f} us   min {min(durs) / 1e3:.1f}   max {max(durs) / 1e3:.1f}   mean {sum(durs) / len(durs) / 1e3:.1f}   "
          f"gap between consecutive dispatches: median {median(gaps(timed)) / 1e3:.1f} us",
          f"   => {tf:.1f} TFLOP/s at {flops:.4e} flop per launch = {tf / peak:.4f} of the {peak} TFLOP/s matrix peak  [frac from the median of the timed dispatches]",
          f"   (all {len(runs)} dispatches: mean {sum(by[kernel]) / len(runs) / 1e3:.1f} us -- includes the launches before the chip has settled; not the figure to compare)"]
    if bench:
        ev = bench.get("ms_per_step") if "ms_per_step" in bench else None
        L.append(f"   bench.py's own HIP-event timing of the same launches inside this profiled run: median {ev * 1e3:.1f} us per launch "
                 f"({bench.get('value')} TFLOP/s, frac {bench.get('roofline', {}).get('frac')})" if ev else "   (no bench.py record in trace.stdout)")
        ceil = bench.get("mfma_issue_ceiling", {})
        key = {"h": "f16", "s": "f32", "d": "f64"}[d]
        for kind in ("random", "ones"):
            cc = ceil.get(f"{key}_{kind}_operands")
            if cc:
                L.append(f"   register-only MFMA loop in the same session, {kind} operands (mmbo_probe_mfma_ceiling): {cc['tflops']} TFLOP/s at "
                         f"{cc['shader_mhz']} MHz = {cc['tflops'] / peak:.3f} of peak;  kernel / ceiling = {tf / cc['tflops']:.4f}")
        L.append("   To compare with a benchmark line from another box: frac differs by the boxes' sustained clocks (a few percent on the"
                 " power-limited fp16 kernel); kernel / ceiling (random operands) = roofline.frac_of_measured_mfma_ceiling does not.")
    L.append("")
    num = 2
    for pname in c["passes"][1:]:
        pdir = os.path.join(outdir, pname)
        ptr = read_trace(pdir)
        cnt = read_counters(pdir)
        if not cnt:
            L += [f"{num}. {pname}: pass not captured", ""]
            num += 1
            continue
        runs_p = [x for x in ptr if x["name"] == kernel]
        runs_p = runs_p[len(runs_p) // 10:]                          # drop the first tenth (cold chip)
        ids = [x["id"] for x in runs_p]
        cm = counter_means(cnt, ids)
        dur_p = sum(x["end"] - x["start"] for x in runs_p) / max(len(runs_p), 1)
        L += [f"{num}. rocprofv3 " + " ".join(PASSES[pname][:-1]), "   command: " + command_line(case, pname, short=True),
              f"   {len(ids)} dispatches (all but the first tenth), mean duration under counter collection {dur_p / 1e3:.1f} us; per-dispatch means:"]
        for name in sorted(cm):
            L.append(f"     {name:32s} {cm[name]:.5g}")
        if pname in ("fetch", "write"):
            counter = "FETCH_SIZE" if pname == "fetch" else "WRITE_SIZE"
            cal_bytes = m * k * ESZ[d]                               # bench.py: one elementwise pass over A
            cal = calibration_factor(pdir, counter, cal_bytes)
            if cal and counter in cm:
                factor, cname, reading = cal
                got = cm[counter] * 1024.0 * factor
                alg = alg_read if pname == "fetch" else alg_write
                L.append(f"   calibration kernel ({short_name(cname, 60)}): one elementwise pass over A, {cal_bytes / 2**20:.0f} MiB read and written; "
                         f"{counter} = {reading:.0f} KiB => factor {factor:.2f}")
                L.append(f"   => {'fetched' if pname == 'fetch' else 'written'} per launch = {got / 1e6:.0f} MB (algorithmic {alg / 1e6:.0f} MB)")
                L.append(f"   {counter.lower()}_bytes={got:.4g}")
            else:
                L.append("   (no calibration kernel found in this pass)")
        else:
            L += ["   derived: " + x for x in derived_lines(cm, dur_p, flops)]
        L.append("")
        num += 1
    fetch = re.search(r"fetch_size_bytes=(\S+)", "\n".join(L))
    write = re.search(r"write_size_bytes=(\S+)", "\n".join(L))
    if fetch and write:
        taken = time.strftime("%Y-%m-%d", time.gmtime(os.path.getmtime(_find(os.path.join(outdir, "trace"), "_kernel_trace.csv"))))
        L.append(f"traffic: fetch_bytes={fetch.group(1)} write_bytes={write.group(1)} tile_config={bench.get('config', {}).get('tile_config', '?')} "
                 f"taken={taken}")
        L.append("(the line above is what bench.py reports as roofline.traffic while this leg still runs this tile config)")
    return "\n".join(L) + "\n"


def summarise_shapes(case, outdir):
    c = CASES[case]
    L = [c["title"] + "; MI355X", "=" * 120, "", "commands (one run per pass, all shapes in one run):"]
    for pname in c["passes"]:
        L.append("  " + command_line(case, pname))
    L += ["Per shape the driver makes a first launch, three to size the groups, one group of warm-up and ten timed groups; the figures",
          "below are MEDIANS over the dispatches of the timed groups.  'per GEMM' sums the kernels one call launches (split-K: GEMM +",
          "reduction).  Where the profiler makes every dispatch wait for the previous one's completion signal ('gap' > 0) a two-launch",
          "GEMM costs more here than back to back in a stream; the driver's own HIP-event time per call, measured inside this same",
          "profiled run, is printed beside it.  Algorithmic bytes count C twice where beta != 0.", ""]
    recs_all = read_json_lines(os.path.join(outdir, "trace.stdout"))
    recs = [r for r in recs_all if "calls_total" in r]
    ceil = next((r["mfma_issue_ceiling"] for r in recs_all if "mfma_issue_ceiling" in r), {})
    if ceil:
        L.append("register-only MFMA loops in the same session (mmbo_probe_mfma_ceiling): " +
                 "; ".join(f"{k}: {v['tflops']} TFLOP/s at {v['shader_mhz']} MHz" for k, v in sorted(ceil.items())))
        L.append("")
    parts = split_by_shape(read_trace(os.path.join(outdir, "trace")), recs)
    extra = {}
    for pname in c["passes"][1:]:
        pdir = os.path.join(outdir, pname)
        precs = [r for r in read_json_lines(os.path.join(outdir, pname + ".stdout")) if "calls_total" in r]
        ptr = read_trace(pdir)
        if precs and ptr:
            extra[pname] = (split_by_shape(ptr, precs), read_counters(pdir))
    for si, (r, _, timed) in enumerate(parts):
        d = r["dtype"]
        flops = 2.0 * r["m"] * r["n"] * r["k"] * r["batch"]
        alg = r["algorithmic_bytes"]
        L.append(f"{r['spec']}:  {dict(h='HGEMM', s='SGEMM', d='DGEMM')[d]} {r['transA']}{r['transB']} {r['m']} x {r['n']} x {r['k']}"
                 + (f" x {r['batch']} (strided batched)" if r["batch"] > 1 else "") + f", alpha = {r['alpha']:g}, beta = {r['beta']:g};  "
                 f"algorithmic {alg / 1e6:.1f} MB, {flops / 1e9:.2f} GFLOP;  config {r['config']}")
        tot = 0.0
        for name, durs in per_kernel(timed).items():
            tot += median(durs)
            L.append(f"   {short_name(name):112s} timed dispatches {len(durs):4d}  median {median(durs) / 1e3:8.1f} us  min {min(durs) / 1e3:8.1f}")
        tf = flops / tot * 1e-3
        bound_tf = min(PEAK_TFLOPS[d], flops / alg * 8.0)
        L.append(f"   per GEMM {tot / 1e3:.1f} us -> {tf:.1f} TFLOP/s = {tf / PEAK_TFLOPS[d]:.4f} of the {PEAK_TFLOPS[d]} TFLOP/s matrix peak; "
                 f"{alg / tot:.0f} GB/s algorithmic = {alg / tot / 8000:.3f} of 8 TB/s; {tf / bound_tf:.3f} of the roofline bound min(peak, intensity x 8 TB/s)")
        L.append(f"   gap between consecutive dispatches: median {median(gaps(timed)) / 1e3:.1f} us;  the driver's HIP-event time per call in this run: "
                 f"{r['gpu_ms_median'] * 1e3:.1f} us ({r['tflops']} TFLOP/s, {r['frac_of_peak']} of peak)")
        key = {"h": "f16", "s": "f32", "d": "f64"}[d] + "_random_operands"
        if key in ceil and r["bound"] == "mfma":
            L.append(f"   kernel / ceiling (random operands) = {tf / ceil[key]['tflops']:.4f}")
        if "sq" in extra:
            sparts, cnt = extra["sq"]
            _, _, stimed = sparts[si]
            main = [x for x in stimed if "splitk" not in x["name"]]
            cm = counter_means(cnt, [x["id"] for x in main])
            dur = sum(x["end"] - x["start"] for x in main) / max(len(main), 1)
            L += [f"   counters (main kernel, {dur / 1e3:.1f} us under collection): " + x for x in derived_lines(cm, dur)]
        moved = []
        for pname, counter, factor, word in (("fetch", "FETCH_SIZE", 2.0, "fetched"), ("write", "WRITE_SIZE", 1.0, "written")):
            if pname in extra:
                sparts, cnt = extra[pname]
                prec, _, stimed = sparts[si]          # (each pass sizes its own groups: its own record says how many calls it timed)
                per_call = sum(cnt.get(x["id"], {}).get(counter, 0.0) for x in stimed) / max(prec["calls_timed"], 1)
                moved.append(f"{word} {per_call * 1024 * factor / 1e6:.1f} MB")
        if moved:
            L.append("   measured per GEMM (all its launches; FETCH_SIZE x 2.0, WRITE_SIZE x 1.0 -- the factors these counters read for a "
                     "plain pass of known size, see gemm_x16_f16_8192.txt): " + ", ".join(moved))
        L.append("")
    return "\n".join(L) + "\n"


def summarise(case, outdir):
    if case not in CASES:
        raise ValueError(f"unknown case '{case}' (have: {', '.join(CASES)})")
    return summarise_shapes(case, outdir) if "specs" in CASES[case] else summarise_bench(case, outdir)


# ---------------------------------------------------------------------------------------------- capture (needs a GPU)
def capture(case, outdir, timeout=420):
    """Runs the case's passes, one rocprofv3 run each, program stdout to <outdir>/<pass>.stdout.  Stops at the first pass
    that fails or runs into its time limit (nothing further is started on the GPU then) and returns its exit status."""
    c = CASES[case]
    os.makedirs(outdir, exist_ok=True)
    env = dict(os.environ, TMPDIR="/tmp", PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    for i, pname in enumerate(c["passes"]):
        prog = list(c["program"]) + (c.get("short", []) if i > 0 else [])
        prog = [os.path.join(ROOT, p) if p == "bench.py" else p for p in prog]
        cmd = ["rocprofv3"] + PASSES[pname] + ["-d", os.path.join(os.path.abspath(outdir), pname), "-o", pname, "--output-format", "csv",
                                               "--", "python3"] + prog
        print(f"[capture {case}] pass {pname}: {' '.join(cmd)}", flush=True)
        with open(os.path.join(outdir, pname + ".stdout"), "w") as so, open(os.path.join(outdir, pname + ".stderr"), "w") as se:
            p = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=so, stderr=se, start_new_session=True)
            try:
                rc = p.wait(timeout=timeout)
            except subprocess.TimeoutExpired:
                import signal
                os.killpg(p.pid, signal.SIGKILL)
                p.wait()
                print(f"[capture {case}] pass {pname} ran into its {timeout} s limit and was killed; stopping", flush=True)
                return 124
        if rc != 0:
            print(f"[capture {case}] pass {pname} exited with {rc}; stopping (see {outdir}/{pname}.stderr)", flush=True)
            return rc
    return 0


def main(argv):
    import argparse
    ap = argparse.ArgumentParser(prog="python -m gemm_mmbo_amd.report")
    ap.add_argument("mode", choices=["capture", "summarise", "cases"])
    ap.add_argument("case", nargs="?")
    ap.add_argument("dir", nargs="?")
    ap.add_argument("--out", default=None, help="capture: directory for rocprofv3's files")
    ap.add_argument("--summary", default=None, help="write the text summary here (default: print it)")
    ap.add_argument("--timeout", type=int, default=420, help="capture: seconds per pass")
    a = ap.parse_args(argv)
    if a.mode == "cases":
        for name, c in CASES.items():
            print(f"{name}: {c['title']}  (passes: {', '.join(c['passes'])})")
        return 0
    if not a.case:
        ap.error("give a CASE")
    outdir = a.out or a.dir
    if not outdir:
        ap.error("give the directory (capture: --out DIR; summarise: CASE DIR)")
    if a.mode == "capture":
        rc = capture(a.case, outdir, a.timeout)
        if rc != 0:
            return rc
    text = summarise(a.case, outdir)
    if a.summary:
        with open(a.summary, "w") as f:
            f.write(text)
        print(f"wrote {a.summary}")
    else:
        sys.stdout.write(text)
    return 0
