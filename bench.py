"""Headline benchmark: GEMM TFLOP/s at 8192^3 on one MI355X, fp16 (value) and fp32 (in "also"); "also" further
carries the two HBM-bound skinny shapes (achieved algorithmic GB/s), three ragged shapes, the reference's own workload, DGEMM NT
44160 x 2048 x 384 with alpha = -1, beta = 1, and DGEMM at 8192^3.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

A step is one GEMM launch through the C ABI on operands already resident in HBM.  Prints ONE JSON line.
After the W warm-up launches a settle phase keeps launching until the per-launch time has stopped drifting (the chip
needs some tens of milliseconds of load to reach its steady clock and power state; the phase is reported as
"settle_ms" / "settle_launches" and is not part of the timed region).  The timed region then holds exactly K launches
between two stream synchronisations, cut into at least ten groups by HIP events recorded on the launch stream:
"value" and "ms_per_step" are the MEDIAN per-launch time over the groups (the convention of this benchmark set: median
of at least ten repetitions); mean, minimum and maximum over the groups and the wall-clock mean are reported beside it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "GEMM TFLOP/s + % of MFMA peak, fp16 & fp32 at 8192^3, 1 MI355X"
PEAK_TFLOPS = {"f16": 2500.0, "f32": 157.3, "f64": 78.6}      # MI355X published dense matrix peaks
# Bytes per launch that crossed the L2 <-> fabric boundary come from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this
# same command (each scaled by the counter's reading for a plain elementwise pass of known size).  They are not measured
# by this run: they are read from the "traffic:" line of the profile summary below, which names the kernel they were
# taken on, and are reported only while that is still the kernel this run launches.
TRAFFIC_PROFILE = {"f16": "profiles/gemm_x16_f16_8192.txt", "f32": "profiles/gemm_x16_f32_8192.txt"}


def profiled_traffic(head, tile_config):
    """(bytes per launch or None, where the figure comes from) from the profile summary's line
       traffic: fetch_bytes=<float> write_bytes=<float> tile_config=<name> taken=<date>"""
    import re
    path = os.path.join(ROOT, TRAFFIC_PROFILE[head])
    try:
        text = open(path).read()
    except OSError:
        return None, f"{TRAFFIC_PROFILE[head]} missing"
    m = re.search(r"^traffic: fetch_bytes=(\S+) write_bytes=(\S+) tile_config=(\S+) taken=(\S+)", text, flags=re.M)
    if not m:
        return None, f"{TRAFFIC_PROFILE[head]} has no traffic line"
    if m.group(3) != tile_config:
        return None, f"{TRAFFIC_PROFILE[head]} was taken on {m.group(3)}, this run launches {tile_config}"
    return float(m.group(1)) + float(m.group(2)), f"{TRAFFIC_PROFILE[head]} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, taken {m.group(4)})"


def timed_launches(torch, stream, step, steps, warmup, settle=True, groups=None, settle_min_ms=100.0, settle_max_ms=600.0):
    """warm-up, settle phase, then exactly `steps` launches in event-delimited groups (one per launch up to 25 groups).
    Returns a dict: median/mean/min/max per-launch ms over the groups, wall ms per launch, settle figures."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    settle_ms, settle_n = 0.0, 0
    if settle:
        # launch in chunks until >= settle_min_ms (100 ms) have passed and two consecutive chunks agree within 1.5 %
        # (at most settle_max_ms, 600 ms)
        t_begin = time.perf_counter()
        prev = None
        chunk = 4
        while True:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            for _ in range(chunk):
                step()
            b.record(stream)
            torch.cuda.synchronize()
            cur = a.elapsed_time(b) / chunk
            settle_n += chunk
            settle_ms = (time.perf_counter() - t_begin) * 1e3
            stable = prev is not None and abs(cur - prev) <= 0.015 * prev
            if (settle_ms >= settle_min_ms and stable) or settle_ms >= settle_max_ms:
                break
            prev = cur
            if cur * chunk < 10.0:
                chunk = min(chunk * 2, 4096)
    groups = max(1, min(steps, groups or 25))
    bounds = [round(i * steps / groups) for i in range(groups + 1)]
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(groups + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev[0].record(stream)
    for g in range(groups):
        for _ in range(bounds[g + 1] - bounds[g]):
            step()
        ev[g + 1].record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    per = sorted(ev[g].elapsed_time(ev[g + 1]) / (bounds[g + 1] - bounds[g]) for g in range(groups))
    med = per[len(per) // 2] if len(per) % 2 else 0.5 * (per[len(per) // 2 - 1] + per[len(per) // 2])
    return {"median_ms": med, "mean_ms": ev[0].elapsed_time(ev[groups]) / steps, "min_ms": per[0], "max_ms": per[-1],
            "wall_ms": wall_ms, "groups": groups, "settle_ms": settle_ms, "settle_launches": settle_n}


def time_gemm(G, torch, dtype, m, n, k, steps, warmup, seed):
    """Returns (timing dict of timed_launches, config description, device tensors)."""
    tdt = torch.float32 if dtype == G.F32 else torch.float16
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    if dtype == G.F16:      # A, B ~ N(0,1)*0.1 rounded to fp16
        A = (torch.randn(m * k, device="cuda", generator=gen) * 0.1).to(tdt)
        B = (torch.randn(k * n, device="cuda", generator=gen) * 0.1).to(tdt)
    else:                   # A, B ~ U[-1,1]
        A = torch.rand(m * k, device="cuda", generator=gen) * 2 - 1
        B = torch.rand(k * n, device="cuda", generator=gen) * 2 - 1
    C = torch.full((m * n,), float("nan"), device="cuda", dtype=tdt)     # beta = 0: never read
    # one plain elementwise pass over A (reads and writes A.numel()*itemsize bytes), outside the timed region:
    # the copy kernel of known size that rocprofv3's FETCH_SIZE / WRITE_SIZE readings are scaled by
    calib = torch.add(A, 0)
    del calib
    stream = torch.cuda.current_stream()
    cid = G.select_config(dtype, 0, 0, m, n, k, 1)

    def step():
        G.gemm(dtype, G.OP_N, G.OP_N, m, n, k, 1.0, A, m, B, k, 0.0, C, m, cid, stream)

    t = timed_launches(torch, stream, step, steps, warmup)
    return t, G.config_info(dtype, cid), (A, B, C)


def spot_check(G, dtype, m, n, k, A, B, C):
    """A band of 64 rows of C against the fp64 oracle (the full check lives in tests/)."""
    import numpy as np
    from oracle import oracle as O
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import util as U
    hA, hB, hC = A.cpu().numpy(), B.cpu().numpy(), C.cpu().numpy()
    r0 = 4000
    want = O.gemm_f64(dtype, 0, 0, 64, n, k, 1.0, hA[r0:], m, hB, k, 0.0, None, m)
    floor = float(np.sqrt(np.mean(want * want)))
    rel, _ = O.max_rel_err(dtype, hC[r0:], m, want, 64, n, floor=floor)
    return rel, U.tol(dtype, k), (hA, hB)


def dgemm_legs(G, torch, steps, warmup):
    """fp64: the reference's HPL trailing update (src/gemm/test.cc:20-21, src/gemm/run.sh:2-5: NT, alpha = -1,
    beta = 1, inputs in [0, 1)) and NN 8192^3.  Returns the entries for "also"."""
    import numpy as np
    from oracle import oracle as O
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import util as U
    stream = torch.cuda.current_stream()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4321)
    out = {}
    for tag, (ta, tb, m, n, k, alpha, beta) in (("hpl", (0, 1, 44160, 2048, 384, -1.0, 1.0)),
                                                ("8192", (0, 0, 8192, 8192, 8192, 1.0, 0.0))):
        lda, ldb = (k if ta else m), (n if tb else k)
        A = torch.rand(m * k, device="cuda", generator=gen, dtype=torch.float64)
        B = torch.rand(k * n, device="cuda", generator=gen, dtype=torch.float64)
        C0 = torch.rand(m * n, device="cuda", generator=gen, dtype=torch.float64)
        C = C0.clone()
        cid = G.select_config(G.F64, ta, tb, m, n, k, 1)
        nsteps = max(10, steps // 2) if tag == "8192" else max(10, steps)
        ms = timed_launches(torch, stream, lambda: G.gemm(G.F64, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, m, cid, stream),
                            nsteps, max(2, warmup // 4), settle=False)["median_ms"]
        # parity on a band of 64 rows of one fresh application (beta = 1 accumulates over the timed launches)
        C.copy_(C0)
        G.gemm(G.F64, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, m, cid, stream)
        torch.cuda.synchronize()
        r0 = 4000
        hA, hB, hC0, hC = A.cpu().numpy(), B.cpu().numpy(), C0.cpu().numpy(), C.cpu().numpy()
        want = O.gemm_f64(O.F64, ta, tb, 64, n, k, alpha, hA[r0:], lda, hB, ldb, beta, hC0[r0:] if beta else None, m)
        rel, _ = O.max_rel_err(O.F64, hC[r0:], m, want, 64, n, floor=float(np.sqrt(np.mean(want * want))))
        tf = 2.0 * m * n * k / ms * 1e-9
        out[f"fp64_{tag}_tflops"] = round(tf, 2)
        out[f"fp64_{tag}_ms_per_step"] = round(ms, 4)
        out[f"fp64_{tag}_frac_of_peak"] = round(tf / PEAK_TFLOPS["f64"], 4)
        out[f"fp64_{tag}_tile_config"] = G.config_info(G.F64, cid)["name"]
        out[f"fp64_{tag}_max_rel_err"] = float(f"{rel:.3e}")
        out[f"fp64_{tag}_rel_err_limit"] = float(f"{U.tol(U.F64, k):.3e}")
        if tag == "hpl":
            out["fp64_hpl_workload"] = "DGEMM NT M=44160 N=2048 K=384 alpha=-1 beta=1, A,B,C ~ U[0,1)"
            out["fp64_hpl_algorithmic_GBps"] = round((m * k + k * n + 2 * m * n) * 8 / ms * 1e-6, 1)
        del A, B, C, C0
        torch.cuda.empty_cache()
    out["fp64_peak"] = PEAK_TFLOPS["f64"]
    return out


def skinny_legs(G, torch, steps, warmup):
    """The two HBM-bound shapes of the benchmark set (NN, alpha = 1, beta = 0, U[-1,1] inputs) in both element types:
    time per GEMM (split-K main kernel + reduction) from events on the launch stream, algorithmic bytes / time against
    the 8 TB/s HBM peak.  Parity of these shapes at full size is in tests/test_gemm_gpu.py."""
    stream = torch.cuda.current_stream()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    out = {}
    for dname, dtype, tdt, esz in (("fp16", G.F16, torch.float16, 2), ("fp32", G.F32, torch.float32, 4)):
        for (m, n, k) in ((4096, 128, 4096), (128, 4096, 8192)):
            A = (torch.rand(m * k, device="cuda", generator=gen) * 2 - 1).to(tdt)
            B = (torch.rand(k * n, device="cuda", generator=gen) * 2 - 1).to(tdt)
            C = torch.empty(m * n, device="cuda", dtype=tdt)
            cid = G.select_config(dtype, 0, 0, m, n, k, 1)
            # small kernels: ten groups of at least twenty back-to-back launches each, median over the groups
            us = timed_launches(torch, stream, lambda: G.gemm(dtype, 0, 0, m, n, k, 1.0, A, m, B, k, 0.0, C, m, cid, stream),
                                max(steps, 200), max(warmup, 20), groups=10, settle_min_ms=30.0, settle_max_ms=200.0)["median_ms"] * 1e3
            nbytes = (m * k + k * n + m * n) * esz
            # a plain streaming kernel with the same bytes read and written, on this box, launched the same way
            stream_us = G.probe_stream((m * k + k * n) * esz, m * n * esz, 50) * 1e6
            out[f"{dname}_{m}x{n}x{k}"] = {"us": round(us, 2), "algorithmic_GBps": round(nbytes / us * 1e-3, 1),
                                            "frac_of_hbm_peak": round(nbytes / us * 1e-3 / 8000.0, 4),
                                            "stream_kernel_same_bytes_us": round(stream_us, 2),
                                            "tflops": round(2.0 * m * n * k / us * 1e-6, 1),
                                            "tile_config": G.config_info(dtype, cid)["name"]}
    return out


def ragged_legs(G, torch, steps, warmup):
    """Shapes that end inside a tile and inside a slice of k (alpha = 1, beta = 0, tightly packed operands), one launch
    each through the automatic pick: time per GEMM from events on the launch stream, TFLOP/s against the matrix peak.
    Parity of ragged shapes is in tests/test_gemm_gpu.py."""
    stream = torch.cuda.current_stream()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(98)
    out = {}
    for dname, dtype, tdt, ta, tb, m, n, k in (("fp16", G.F16, torch.float16, 0, 0, 3000, 3000, 3000),
                                               ("fp16", G.F16, torch.float16, 1, 0, 8192, 8192, 8200),
                                               ("fp32", G.F32, torch.float32, 0, 1, 4100, 4100, 4096)):
        A = (torch.rand(m * k, device="cuda", generator=gen) * 2 - 1).to(tdt)
        B = (torch.rand(k * n, device="cuda", generator=gen) * 2 - 1).to(tdt)
        C = torch.empty(m * n, device="cuda", dtype=tdt)
        lda, ldb = (k if ta else m), (n if tb else k)
        cid = G.select_config(dtype, ta, tb, m, n, k, 1)

        def run():
            G.gemm(dtype, ta, tb, m, n, k, 1.0, A, lda, B, ldb, 0.0, C, m, G.CONFIG_AUTO, stream)
        us = timed_launches(torch, stream, run, max(steps, 20), max(warmup, 5), groups=10, settle_min_ms=30.0, settle_max_ms=200.0)["median_ms"] * 1e3
        tf = 2.0 * m * n * k / us * 1e-6
        out[f"{dname}_{'NT'[ta]}{'NT'[tb]}_{m}x{n}x{k}"] = {"us": round(us, 1), "tflops": round(tf, 1),
                                                            "frac_of_peak": round(tf / PEAK_TFLOPS["f16" if dtype == G.F16 else "f32"], 4),
                                                            "tile_config": G.config_info(dtype, cid)["name"]}
        del A, B, C
    return out


def config_legs(G, torch, steps, warmup):
    """The benchmark configurations that are not the headline: SGEMM NN 1024^3 (alpha = 1, beta = 0), SGEMM NT and TN
    4096^3 (alpha = 1.5, beta = 0.5) and the strided-batched HGEMM TN 64 x 512^3 (alpha = 1, beta = 1), one launch each
    through the automatic pick, timed with events on the launch stream.  Algorithmic bytes count C twice where
    beta != 0.  Parity of these configurations is in tests/test_gemm_gpu.py."""
    stream = torch.cuda.current_stream()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    out = {}
    for key, dtype, tdt, ta, tb, m, n, k, batch, alpha, beta in (
            ("cfg1_sgemm_nn_1024", G.F32, torch.float32, 0, 0, 1024, 1024, 1024, 1, 1.0, 0.0),
            ("cfg2a_sgemm_nt_4096", G.F32, torch.float32, 0, 1, 4096, 4096, 4096, 1, 1.5, 0.5),
            ("cfg2b_sgemm_tn_4096", G.F32, torch.float32, 1, 0, 4096, 4096, 4096, 1, 1.5, 0.5),
            ("cfg5_hgemm_tn_512_batch64", G.F16, torch.float16, 1, 0, 512, 512, 512, 64, 1.0, 1.0)):
        scale = 0.1 if dtype == G.F16 else 1.0
        A = ((torch.rand(m * k * batch, device="cuda", generator=gen) * 2 - 1) * scale).to(tdt)
        B = ((torch.rand(k * n * batch, device="cuda", generator=gen) * 2 - 1) * scale).to(tdt)
        C = (torch.rand(m * n * batch, device="cuda", generator=gen) * 2 - 1).to(tdt)
        lda, ldb = (k if ta else m), (n if tb else k)
        cid = G.select_config(dtype, ta, tb, m, n, k, batch)

        def run():
            G.gemm_strided_batched(dtype, ta, tb, m, n, k, alpha, A, lda, m * k, B, ldb, k * n, beta, C, m, m * n, batch,
                                   G.CONFIG_AUTO, stream)
        reps = max(steps, 20) if m >= 4096 else max(steps, 200)
        us = timed_launches(torch, stream, run, reps, max(warmup, 10), groups=10, settle_min_ms=30.0, settle_max_ms=200.0)["median_ms"] * 1e3
        tf = 2.0 * m * n * k * batch / us * 1e-6
        esz = 2 if dtype == G.F16 else 4
        gbps = batch * (m * k + k * n + m * n * (2 if beta != 0 else 1)) * esz / us * 1e-3
        out[key] = {"us": round(us, 1), "tflops": round(tf, 1),
                    "frac_of_peak": round(tf / PEAK_TFLOPS["f16" if dtype == G.F16 else "f32"], 4),
                    "algorithmic_GBps": round(gbps, 1), "tile_config": G.config_info(dtype, cid)["name"]}
        if batch > 1:
            # the memory-bound one: a plain streaming kernel with the same bytes read (A, B, old C) and written, on this box
            out[key]["stream_kernel_same_bytes_us"] = round(
                G.probe_stream(batch * (m * k + k * n + (m * n if beta != 0 else 0)) * esz, batch * m * n * esz, 50, in_place=beta != 0) * 1e6, 1)
        del A, B, C
    return out


def cpu_baseline(dtype, m, n, k, hA, hB):
    """The oracle's native-precision CPU GEMM (fp16 operands widened to fp32, fp32 multiply-add chains) on
    the same operands, all host cores, whole problem once."""
    import numpy as np
    from oracle import oracle as O
    hC = np.zeros(m * n, dtype=hA.dtype)
    O.gemm_native(dtype, 0, 0, 256, 256, 256, 1.0, hA, m, hB, k, 0.0, hC, m)       # spin up the thread pool
    t0 = time.perf_counter()
    O.gemm_native(dtype, 0, 0, m, n, k, 1.0, hA, m, hB, k, 0.0, hC, m)
    dt = time.perf_counter() - t0
    return {"value": round(2.0 * m * n * k / dt * 1e-12, 4), "unit": "TFLOP/s", "cores": O.num_threads(),
            "kind": "port", "seconds": round(dt, 2),
            "sample": f"the whole {m}x{n}x{k} problem once, same operands as the GPU run"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", choices=["f16", "f32", "f64"], default=None, help="run one leg only (profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library runs one GEMM on one GPU; --gpus must be 1 "
              "(sharding over M/N needs no exchange and is not part of this build)", file=sys.stderr)
        sys.exit(2)

    import torch
    import gemm_mmbo_amd as G
    G.lib()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    m = n = k = 8192
    flops = 2.0 * m * n * k
    out = {}
    res = {}
    for name, dtype in (("f16", G.F16), ("f32", G.F32)):
        if args.only and args.only != name:
            continue
        # (the fp32 launch takes ten times as long: half the launches, but never fewer than ten timed groups)
        steps = args.steps if name == "f16" else max(10, args.steps // 2)
        warm = args.warmup if name == "f16" else max(2, args.warmup // 5)
        t, cfg, tensors = time_gemm(G, torch, dtype, m, n, k, steps, warm, seed=1234)
        rel, limit, host = spot_check(G, dtype, m, n, k, *tensors)
        res[name] = dict(t=t, wall_ms=t["wall_ms"], ev_ms=t["median_ms"], cfg=cfg, rel=rel, limit=limit, steps=steps)
        if name == "f16" and not args.no_cpu:
            res[name]["cpu"] = cpu_baseline(dtype, m, n, k, *host)
        del tensors, host
        torch.cuda.empty_cache()

    # The same HGEMM on constant operands (all ones): the matrix pipes then draw far less power and the clock stays up,
    # which separates what the kernel's structure costs from what the chip's power limit costs on real data.
    ones_tflops = None
    if not args.only:
        A1 = torch.ones(m * k, device="cuda", dtype=torch.float16)
        B1 = torch.ones(k * n, device="cuda", dtype=torch.float16)
        C1 = torch.empty(m * n, device="cuda", dtype=torch.float16)
        st = torch.cuda.current_stream()
        cid1 = G.select_config(G.F16, 0, 0, m, n, k, 1)
        t1 = timed_launches(torch, st, lambda: G.gemm(G.F16, G.OP_N, G.OP_N, m, n, k, 1.0, A1, m, B1, k, 0.0, C1, m, cid1, st),
                            40, 10, settle=True)
        ones_tflops = flops / t1["median_ms"] * 1e-9
        assert float(C1[12345]) == float(k)          # 8192 ones: exact in fp16
        del A1, B1, C1
        torch.cuda.empty_cache()

    f64 = dgemm_legs(G, torch, args.steps, args.warmup) if args.only in (None, "f64") else {}
    skinny = skinny_legs(G, torch, args.steps, args.warmup) if not args.only else {}
    ragged = ragged_legs(G, torch, min(args.steps, 10), min(args.warmup, 3)) if not args.only else {}
    configs = config_legs(G, torch, min(args.steps, 20), min(args.warmup, 5)) if not args.only else {}
    if args.only == "f64":
        print(json.dumps({"metric": METRIC, "also": f64}))
        return
    ceilings = {}
    for name, dtype in (("f16", G.F16), ("f32", G.F32), ("f64", G.F64)):
        if not args.only or args.only == name:          # (a one-leg run, as the profiles use, probes that leg's type only)
            for rnd in (0, 1):
                tf, mhz = G.probe_mfma_ceiling(dtype, bool(rnd))
                ceilings[f"{name}_{'random' if rnd else 'ones'}_operands"] = {"tflops": round(tf, 1), "shader_mhz": round(mhz)}
    head = "f16" if "f16" in res else "f32"
    r = res[head]
    t = r["t"]
    tflops = flops / t["median_ms"] * 1e-9
    achieved = tflops                               # the same K launches, timed by events on the launch stream
    traffic, traffic_source = profiled_traffic(head, r["cfg"]["name"])
    alg_bytes = (m * k + k * n + m * n) * (2 if head == "f16" else 4)
    out = {
        "metric": METRIC, "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": r["steps"],
        "warmup": args.warmup, "ms_per_step": round(t["median_ms"], 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": head, "data": "synthetic",
        "config": {"workload": f"{'H' if head == 'f16' else 'S'}GEMM NN M=N=K=8192 lda=ldb=ldc=8192 alpha=1 beta=0, "
                               + ("A,B ~ N(0,1)*0.1 rounded to fp16, fp32 accumulate" if head == "f16" else "A,B ~ U[-1,1]"),
                   "tile_config": r["cfg"]["name"]},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS[head], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS[head], 4), "traffic": traffic, "traffic_source": traffic_source,
                     "algorithmic_bytes": alg_bytes, "flops_per_launch": flops,
                     "kernel_ms": round(t["median_ms"], 4)},
        "timing": {"statistic": "median over the groups of the timed region; value and ms_per_step use it",
                   "groups": t["groups"], "median_ms": round(t["median_ms"], 4), "mean_ms": round(t["mean_ms"], 4),
                   "min_ms": round(t["min_ms"], 4), "max_ms": round(t["max_ms"], 4),
                   "wall_ms_per_step": round(t["wall_ms"], 4), "settle_ms": round(t["settle_ms"], 1),
                   "settle_launches": t["settle_launches"],
                   "mean_tflops": round(flops / t["mean_ms"] * 1e-9, 2), "best_tflops": round(flops / t["min_ms"] * 1e-9, 2)},
        "max_rel_err": float(f"{r['rel']:.3e}"), "rel_err_limit": float(f"{r['limit']:.3e}"),
        "parity_ok": bool(r["rel"] <= r["limit"]),
    }
    if "cpu" in r:
        out["cpu_baseline"] = r["cpu"]
    if ceilings:
        # what a register-only MFMA loop sustains on this box (the chip lowers its clock under power)
        out["mfma_issue_ceiling"] = ceilings
        c = ceilings.get(f"{head}_random_operands")
        if c:
            out["roofline"]["frac_of_measured_mfma_ceiling"] = round(achieved / c["tflops"], 4)
    if head == "f16" and "f32" in res:
        q = res["f32"]
        out["also"] = {"fp32_tflops": round(flops / q["ev_ms"] * 1e-9, 2), "fp32_ms_per_step": round(q["ev_ms"], 4),
                       "fp32_frac_of_peak": round(flops / q["ev_ms"] * 1e-9 / PEAK_TFLOPS["f32"], 4),
                       "fp32_peak": PEAK_TFLOPS["f32"], "fp32_tile_config": q["cfg"]["name"], "fp32_steps": q["steps"],
                       "fp32_groups": q["t"]["groups"],
                       "fp32_max_rel_err": float(f"{q['rel']:.3e}"), "fp32_rel_err_limit": float(f"{q['limit']:.3e}")}
    if ones_tflops is not None:
        out.setdefault("also", {})["fp16_constant_operands_tflops"] = round(ones_tflops, 1)
        out["also"]["fp16_constant_operands_frac_of_peak"] = round(ones_tflops / PEAK_TFLOPS["f16"], 4)
    if skinny:
        out.setdefault("also", {})["skinny_nn_hbm_bound"] = skinny
    if ragged:
        out.setdefault("also", {})["ragged_one_launch"] = ragged
    if configs:
        out.setdefault("also", {})["other_benchmark_configs"] = configs
    if f64:
        out.setdefault("also", {}).update(f64)
        out["parity_ok"] = bool(out["parity_ok"] and f64["fp64_hpl_max_rel_err"] <= f64["fp64_hpl_rel_err_limit"]
                                and f64["fp64_8192_max_rel_err"] <= f64["fp64_8192_rel_err_limit"])
    print(json.dumps(out))
    if not out["parity_ok"]:
        sys.exit(3)


if __name__ == "__main__":
    main()
