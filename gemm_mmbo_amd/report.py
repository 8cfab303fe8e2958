"""Sweep / report driver: one machine-readable record per GEMM shape.

The reference sweeps its benchmark binary over a list of sizes and prints one free-text line per size
(src/gemm/run.sh:1-5 over src/gemm/benchmark.cc:89-109: kernel time, TFLOP/s and "efficiency" against a hard-coded
peak, with rocBLAS's result as the check, :110-117).  This is that driver for this library, with records instead of text:

    python -m gemm_mmbo_amd.report configs                  # the benchmark configurations (fp16/fp32 8192^3 included)
    python -m gemm_mmbo_amd.report hpl [--step 3840]        # the reference's sweep: DGEMM NT M = 44160 down to 384,
                                                            # N = 2048, K = 384, ldc = 44160, alpha = -1, beta = 1
    python -m gemm_mmbo_amd.report shapes SPEC [SPEC ...]   # SPEC = dtype,ta,tb,m,n,k[,batch[,alpha[,beta[,ldc]]]]
                                                            # dtype s|h|d, ta/tb N|T;  e.g.  h,N,N,4096,128,4096
    options:  --json FILE (one JSON object per line)   --csv FILE   --reps R (timed groups, default 10)
              --inner I (launches per group; default: enough for about 2 ms)   --config ID (default: the automatic pick)
              --no-check   --print-profile-commands   --ceilings
    python -m gemm_mmbo_amd.report capture CASE --out DIR [--summary FILE]    # run the case under rocprofv3, pass by pass
    python -m gemm_mmbo_amd.report summarise CASE DIR [--summary FILE]        # rocprofv3's CSV files -> text (no GPU needed)
    python -m gemm_mmbo_amd.report cases                                      # (gemm_mmbo_amd/profiles.py)

Per shape: GPU milliseconds per launch (median, minimum and maximum over the groups, HIP events on the launch stream),
TFLOP/s, fraction of the matrix peak, the roofline bound min(peak, arithmetic intensity x 8 TB/s) and the fraction of it,
algorithmic GB/s, the config that ran, and the largest relative error against the same product computed by this
library's fp64 kernel from the same operands (the reference checks against an fp64 BLAS the same way; fp64 shapes are
checked with a second fp64 config where one exists).  --print-profile-commands prints, per shape, the rocprofv3 command
lines (kernel trace, MFMA / LDS counters, fetched and written bytes) that profile exactly that shape through this module.

A GPU and the built library are required; there is no CPU path.
"""
import argparse
import csv
import json
import math
import sys

PEAK_TFLOPS = {"h": 2500.0, "s": 157.3, "d": 78.6}         # MI355X dense matrix peaks: fp16, fp32, fp64
HBM_TBPS = 8.0
ESZ = {"h": 2, "s": 4, "d": 8}
FIELDS = ["spec", "calls_total", "calls_timed", "dtype", "transA", "transB", "m", "n", "k", "batch", "lda", "ldb", "ldc", "alpha", "beta", "config_id", "config",
          "gpu_ms_median", "gpu_ms_min", "gpu_ms_max", "groups", "launches_per_group", "tflops", "frac_of_peak", "bound",
          "bound_tflops", "frac_of_bound", "algorithmic_bytes", "algorithmic_GBps", "frac_of_hbm_peak", "max_rel_err",
          "checked_against"]

CONFIGS = [
    # dtype ta tb  m     n     k     batch alpha beta
    ("s", "N", "N", 1024, 1024, 1024, 1, 1.0, 0.0, None),
    ("s", "N", "T", 4096, 4096, 4096, 1, 1.5, 0.5, None), ("s", "T", "N", 4096, 4096, 4096, 1, 1.5, 0.5, None),
    ("h", "N", "N", 8192, 8192, 8192, 1, 1.0, 0.0, None), ("s", "N", "N", 8192, 8192, 8192, 1, 1.0, 0.0, None),
    ("s", "N", "N", 1023, 777, 513, 1, 1.0, 0.0, None), ("h", "N", "N", 1023, 777, 513, 1, 1.0, 0.0, None),
    ("s", "N", "N", 4096, 128, 4096, 1, 1.0, 0.0, None), ("h", "N", "N", 4096, 128, 4096, 1, 1.0, 0.0, None),
    ("s", "N", "N", 128, 4096, 8192, 1, 1.0, 0.0, None), ("h", "N", "N", 128, 4096, 8192, 1, 1.0, 0.0, None),
    ("h", "T", "N", 512, 512, 512, 64, 1.0, 1.0, None),
    ("d", "N", "T", 44160, 2048, 384, 1, -1.0, 1.0, None),
]


def parse_spec(spec):
    f = spec.split(",")
    if len(f) < 6 or f[0] not in ESZ or f[1] not in "NT" or f[2] not in "NT":
        raise ValueError(f"bad shape '{spec}': want dtype,ta,tb,m,n,k[,batch[,alpha[,beta[,ldc]]]] with dtype s|h|d, ta/tb N|T")
    m, n, k = int(f[3]), int(f[4]), int(f[5])
    batch = int(f[6]) if len(f) > 6 else 1
    alpha = float(f[7]) if len(f) > 7 else 1.0
    beta = float(f[8]) if len(f) > 8 else 0.0
    ldc = int(f[9]) if len(f) > 9 else None
    return (f[0], f[1], f[2], m, n, k, batch, alpha, beta, ldc)


def spec_of(shape):
    d, ta, tb, m, n, k, batch, alpha, beta, ldc = shape
    s = f"{d},{ta},{tb},{m},{n},{k},{batch},{alpha:g},{beta:g}"
    return s + (f",{ldc}" if ldc else "")


def roofline(d, m, n, k, batch, beta):
    flops = 2.0 * m * n * k * batch
    nbytes = batch * (m * k + k * n + m * n * (2 if beta != 0 else 1)) * ESZ[d]
    hbm_tflops = flops / nbytes * HBM_TBPS if nbytes else float("inf")      # arithmetic intensity x 8 TB/s, in TFLOP/s
    bound = "mfma" if PEAK_TFLOPS[d] <= hbm_tflops else "hbm"
    return flops, nbytes, bound, min(PEAK_TFLOPS[d], hbm_tflops)


def run_shape(G, torch, shape, reps, inner, config, check, seed=1):
    d, ta, tb, m, n, k, batch, alpha, beta, ldc = shape
    dtype = {"s": G.F32, "h": G.F16, "d": G.F64}[d]
    tdt = {"s": torch.float32, "h": torch.float16, "d": torch.float64}[d]
    ita, itb = int(ta == "T"), int(tb == "T")
    lda, ldb, ldc = (k if ita else m), (n if itb else k), (ldc or m)
    if ldc < m:
        raise ValueError("ldc smaller than m")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    scale = 0.1 if d == "h" else 1.0
    A = ((torch.rand(m * k * batch, device="cuda", generator=gen, dtype=torch.float64) * 2 - 1) * scale).to(tdt)
    B = ((torch.rand(k * n * batch, device="cuda", generator=gen, dtype=torch.float64) * 2 - 1) * scale).to(tdt)
    C0 = (torch.rand(ldc * n * batch, device="cuda", generator=gen, dtype=torch.float64) * 2 - 1).to(tdt)
    C = C0.clone()
    stream = torch.cuda.current_stream()
    cid = G.select_config(dtype, ita, itb, m, n, k, batch) if config is None else config
    name = G.config_info(dtype, cid)["name"]

    def launch(dt=dtype, a=A, b=B, c=C, cfg=cid):
        G.gemm_strided_batched(dt, ita, itb, m, n, k, alpha, a, lda, m * k, b, ldb, k * n, beta, c, ldc, ldc * n, batch, cfg,
                               stream)

    calls = [0]                              # GEMM calls made for this shape with the config under test (for trace readers)
    plain_launch = launch

    def launch():
        calls[0] += 1
        plain_launch()

    launch()
    torch.cuda.synchronize()
    rel, against = None, None
    if check:
        rel, against = check_result(G, torch, shape, dtype, (ita, itb, lda, ldb, ldc), A, B, C0, C, cid)
    # timing: `reps` groups of `inner` back-to-back launches; each group between two events on the launch stream
    if inner is None:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(3):
            launch()
        e1.record(stream)
        torch.cuda.synchronize()
        inner = max(1, min(200, int(2.0 / max(e0.elapsed_time(e1) / 3, 1e-3))))
    for _ in range(inner):
        launch()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    torch.cuda.synchronize()
    ev[0].record(stream)
    for g in range(reps):
        for _ in range(inner):
            launch()
        ev[g + 1].record(stream)
    torch.cuda.synchronize()
    per = sorted(ev[g].elapsed_time(ev[g + 1]) / inner for g in range(reps))
    med = per[len(per) // 2] if len(per) % 2 else 0.5 * (per[len(per) // 2 - 1] + per[len(per) // 2])
    flops, nbytes, bound, bound_tf = roofline(d, m, n, k, batch, beta)
    tf = flops / med * 1e-9
    gbps = nbytes / med * 1e-6
    return {"spec": spec_of(shape), "calls_total": calls[0], "calls_timed": reps * inner,
            "dtype": d, "transA": ta, "transB": tb, "m": m, "n": n, "k": k, "batch": batch, "lda": lda, "ldb": ldb, "ldc": ldc,
            "alpha": alpha, "beta": beta, "config_id": cid, "config": name, "gpu_ms_median": round(med, 5),
            "gpu_ms_min": round(per[0], 5), "gpu_ms_max": round(per[-1], 5), "groups": reps, "launches_per_group": inner,
            "tflops": round(tf, 2), "frac_of_peak": round(tf / PEAK_TFLOPS[d], 4), "bound": bound,
            "bound_tflops": round(bound_tf, 1), "frac_of_bound": round(tf / bound_tf, 4), "algorithmic_bytes": nbytes,
            "algorithmic_GBps": round(gbps, 1), "frac_of_hbm_peak": round(gbps / (HBM_TBPS * 1e3), 4),
            "max_rel_err": None if rel is None else float(f"{rel:.3e}"), "checked_against": against}


def check_result(G, torch, shape, dtype, lay, A, B, C0, C, cid):
    """max |C - R| / max(|R|, rms(R)) over the m x n x batch window, R = the same product from this library's fp64 kernel
    on the operands widened to fp64 (exactly representable).  For an fp64 shape R comes from another fp64 config."""
    d, ta, tb, m, n, k, batch, alpha, beta, _ = shape
    ita, itb, lda, ldb, ldc = lay
    if m * n * batch == 0:
        return 0.0, "empty"
    stream = torch.cuda.current_stream()
    if dtype == G.F64:
        others = [c for c in range(G.num_configs(G.F64)) if c != cid]
        if not others:
            return None, None
        rcfg, against = others[0], "fp64 config " + G.config_info(G.F64, others[0])["name"]
        A64, B64 = A, B
    else:
        rcfg, against = G.select_config(G.F64, ita, itb, m, n, k, batch), "this library's fp64 kernel on the widened operands"
        A64, B64 = A.double(), B.double()
    R = C0.double().clone()
    G.gemm_strided_batched(G.F64, ita, itb, m, n, k, alpha, A64, lda, m * k, B64, ldb, k * n, beta, R, ldc, ldc * n, batch, rcfg,
                           stream)
    torch.cuda.synchronize()
    got = C.double().view(batch, n, ldc)[:, :, :m]
    ref = R.view(batch, n, ldc)[:, :, :m]
    rms = float(ref.pow(2).mean().sqrt())
    err = (got - ref).abs() / torch.clamp(ref.abs(), min=max(rms, 1e-300))
    worst = float(err.max())
    if not math.isfinite(worst) or bool(torch.isnan(got).any()):
        worst = float("inf")
    return worst, against


def profile_commands(shape):
    """rocprofv3 command lines that profile exactly this shape through this module (the program comes directly after --)."""
    spec = spec_of(shape)
    prog = f"python3 -m gemm_mmbo_amd.report shapes {spec} --no-check --reps 10"
    pre = "cd /tmp && export TMPDIR=/tmp && export PYTHONPATH=<repository root> && "
    return [
        pre + f"rocprofv3 --kernel-trace --stats -d <out> -o stats --output-format csv -- {prog}",
        pre + "rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE "
              f"GRBM_GUI_ACTIVE --kernel-trace -d <out> -o pmc --output-format csv -- {prog}",
        pre + f"rocprofv3 --pmc FETCH_SIZE --kernel-trace -d <out> -o pmc --output-format csv -- {prog}",
        pre + f"rocprofv3 --pmc WRITE_SIZE --kernel-trace -d <out> -o pmc --output-format csv -- {prog}",
    ]


def main(argv=None):
    argv = sys.argv[1:] if argv is None else list(argv)
    if argv and argv[0] in ("capture", "summarise", "cases"):
        from . import profiles
        return profiles.main(argv)
    ap = argparse.ArgumentParser(prog="python -m gemm_mmbo_amd.report", description=__doc__.split("\n\n")[0])
    ap.add_argument("mode", choices=["configs", "hpl", "shapes"])
    ap.add_argument("specs", nargs="*")
    ap.add_argument("--json", default=None)
    ap.add_argument("--csv", default=None)
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--inner", type=int, default=None)
    ap.add_argument("--config", type=int, default=None)
    ap.add_argument("--step", type=int, default=3840, help="hpl: step of M (the reference's run.sh uses 384)")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--print-profile-commands", action="store_true")
    ap.add_argument("--ceilings", action="store_true",
                    help="finish with one record of what a register-only MFMA loop sustains on this box right now")
    args = ap.parse_args(argv)
    if args.reps < 1:
        ap.error("--reps must be at least 1")
    if args.mode == "configs":
        shapes = list(CONFIGS)
    elif args.mode == "hpl":
        shapes = [("d", "N", "T", M, 2048, 384, 1, -1.0, 1.0, 44160) for M in range(44160, 0, -args.step)]
    else:
        if not args.specs:
            ap.error("shapes: give at least one SPEC")
        try:
            shapes = [parse_spec(s) for s in args.specs]
        except ValueError as e:
            ap.error(str(e))

    import torch
    from . import api as G
    G.lib()
    if not torch.cuda.is_available():
        print("gemm_mmbo_amd.report: no GPU visible", file=sys.stderr)
        return 1
    jf = open(args.json, "w") if args.json else None
    cf = open(args.csv, "w", newline="") if args.csv else None
    cw = csv.DictWriter(cf, fieldnames=FIELDS) if cf else None
    if cw:
        cw.writeheader()
    rc = 0
    for shape in shapes:
        rec = run_shape(G, torch, shape, args.reps, args.inner, args.config, not args.no_check)
        line = json.dumps(rec)
        print(line, flush=True)
        if jf:
            jf.write(line + "\n")
        if cw:
            cw.writerow(rec)
        if args.print_profile_commands:
            for c in profile_commands(shape):
                print("# " + c)
        torch.cuda.empty_cache()
    if args.ceilings:
        ceil = {}
        for name, dt in (("f16", G.F16), ("f32", G.F32), ("f64", G.F64)):
            for rnd in (0, 1):
                tf, mhz = G.probe_mfma_ceiling(dt, bool(rnd))
                ceil[f"{name}_{'random' if rnd else 'ones'}_operands"] = {"tflops": round(tf, 1), "shader_mhz": round(mhz)}
        line = json.dumps({"mfma_issue_ceiling": ceil})
        print(line, flush=True)
        if jf:
            jf.write(line + "\n")
    for f in (jf, cf):
        if f:
            f.close()
    return rc


if __name__ == "__main__":
    sys.exit(main())
