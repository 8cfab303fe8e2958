"""Offline tuner: time every tile config on a list of shapes and print rows for csrc/tuned_table.hpp.

The reference keeps an exact-size table for its Tensile kernels, size -> (solution index, measured GFLOP/s)
(src/gemm/ref/vega20_Cijk_Ailk_Bjlk_DB.yaml:929-1177), and finds the fastest kernel for a size by running all of
them (src/gemm/benchmark.cc:89-109).  This does the same over this library's config ids, through the C ABI, on the
GPU it runs on:

    python -m gemm_mmbo_amd.tune                      # the built-in shape list (benchmark configs + HPL sweep points)
    python -m gemm_mmbo_amd.tune shapes.txt           # one shape per line:  dtype ta tb m n k batch alpha beta
                                                      # (dtype 0 fp32, 1 fp16, 2 fp64; ta/tb 0 = N, 1 = T)
    python -m gemm_mmbo_amd.tune shapes.txt --dump t.json    # also write every config's time per shape

For every shape it prints the ranking and one line in the table's syntax; paste the lines into kTuned[] and rebuild.
The fastest config only enters a line after its result has passed a check against the library's fp64 kernel.
Configs that do not apply to a shape (the ring kernels on ragged shapes or on operands that are not 16-byte aligned: the
operands here are tightly packed) are skipped, as the C ABI refuses them.
"""
import sys

BUILTIN = [
    # dtype ta tb m n k batch alpha beta
    (0, 0, 0, 1024, 1024, 1024, 1, 1.0, 0.0),
    (0, 0, 1, 4096, 4096, 4096, 1, 1.5, 0.5), (0, 1, 0, 4096, 4096, 4096, 1, 1.5, 0.5),
    (0, 0, 0, 1023, 777, 513, 1, 1.0, 0.0), (1, 0, 0, 1023, 777, 513, 1, 1.0, 0.0),
    (0, 0, 0, 4096, 128, 4096, 1, 1.0, 0.0), (1, 0, 0, 4096, 128, 4096, 1, 1.0, 0.0),
    (0, 0, 0, 128, 4096, 8192, 1, 1.0, 0.0), (1, 0, 0, 128, 4096, 8192, 1, 1.0, 0.0),
    (1, 1, 0, 512, 512, 512, 64, 1.0, 1.0),
    (0, 0, 0, 2048, 2048, 2048, 1, 1.0, 0.0), (1, 0, 0, 2048, 2048, 2048, 1, 1.0, 0.0),
    (0, 0, 0, 4096, 4096, 4096, 1, 1.0, 0.0), (1, 0, 0, 4096, 4096, 4096, 1, 1.0, 0.0),
    (0, 0, 0, 8192, 8192, 8192, 1, 1.0, 0.0), (1, 0, 0, 8192, 8192, 8192, 1, 1.0, 0.0),
    (0, 0, 1, 44160, 2048, 384, 1, -1.0, 1.0), (2, 0, 1, 44160, 2048, 384, 1, -1.0, 1.0),
    (2, 0, 0, 8192, 8192, 8192, 1, 1.0, 0.0),
]


def time_config(G, torch, dtype, ta, tb, m, n, k, batch, alpha, beta, cfg, reps):
    """Milliseconds per launch of one config, or None when the config does not apply to the shape."""
    tdt = {G.F32: torch.float32, G.F16: torch.float16, G.F64: torch.float64}[dtype]
    A = (torch.rand(m * k * batch, device="cuda") - 0.5).to(tdt)
    B = (torch.rand(k * n * batch, device="cuda") - 0.5).to(tdt)
    C = torch.zeros(m * n * batch, device="cuda", dtype=tdt)
    lda, ldb = (k if ta else m), (n if tb else k)
    stream = torch.cuda.current_stream()

    def run():
        G.gemm_strided_batched(dtype, ta, tb, m, n, k, alpha, A, lda, m * k, B, ldb, k * n, beta, C, m, m * n, batch,
                               cfg, stream)
    try:
        for _ in range(2):
            run()
    except G.MmboError:
        return None
    torch.cuda.synchronize()
    # median over five groups of `reps` back-to-back launches
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
    ev[0].record(stream)
    for g in range(5):
        for _ in range(reps):
            run()
        ev[g + 1].record(stream)
    torch.cuda.synchronize()
    return sorted(ev[g].elapsed_time(ev[g + 1]) / reps for g in range(5))[2]


def table_id(G, dtype, cfg):
    """A config id in the syntax of csrc/tuned_table.hpp: ring_id(tile, GlobalSplitU) / x16_id(tile, GlobalSplitU) for the
    direct-to-LDS families (tile = row of kRingTiles / kX16Tiles), the plain number otherwise (staged ids, fp64 rows)."""
    if dtype == G.F64:
        return str(cfg)
    d = G.config_info(dtype, cfg)
    if "DTL1" not in d["name"]:
        return str(cfg)
    fam = [c for c in range(G.num_configs(dtype))
           if ("DTL1" in G.config_info(dtype, c)["name"]) and (("_ACC" in G.config_info(dtype, c)["name"]) == ("_ACC" in d["name"]))
           and G.config_info(dtype, c)["split_k"] == 1]
    ntiles = len(fam)
    tile = (cfg - fam[0]) % ntiles
    return f"{'x16_id' if '_ACC' in d['name'] else 'ring_id'}({tile}, {d['split_k']})"


def passes_check(G, torch, dtype, ta, tb, m, n, k, batch, alpha, beta, cfg):
    """The candidate's result against this library's fp64 kernel on the same operands (gemm_mmbo_amd.report), within the
    library's tolerances: a config that is fast and wrong must never enter the table."""
    from . import report
    d = {G.F32: "s", G.F16: "h", G.F64: "d"}[dtype]
    rec = report.run_shape(G, torch, (d, "NT"[ta], "NT"[tb], m, n, k, batch, alpha, beta, None), 1, 1, cfg, True)
    limit = {G.F32: 1e-5 * max(k, 1) ** 0.5, G.F16: 2e-2, G.F64: 2e-15 * max(k, 1) ** 0.5}[dtype]
    return rec["max_rel_err"] is None or rec["max_rel_err"] <= limit


def tune(shapes, out=sys.stdout, dump=None):
    import torch

    import gemm_mmbo_amd as G
    if not torch.cuda.is_available():
        raise RuntimeError("the tuner times kernels: it needs the GPU")
    rows, table = [], []
    for (dtype, ta, tb, m, n, k, batch, alpha, beta) in shapes:
        flops = 2.0 * m * n * k * batch
        reps = 3 if flops > 1e11 else 20
        res = []
        for cfg in range(G.num_configs(dtype)):
            d = G.config_info(dtype, cfg)
            # split-K and small tiles on the largest problems only cost sweep time
            if flops > 5e11 and (d["split_k"] > 1 or d["macro_tile_m"] * d["macro_tile_n"] < 128 * 128):
                continue
            t = time_config(G, torch, dtype, ta, tb, m, n, k, batch, alpha, beta, cfg, reps)
            if t is not None:
                res.append((t, cfg))
        res.sort()
        pick = G.select_config(dtype, ta, tb, m, n, k, batch)
        t_pick = next((t for t, c in res if c == pick), None)
        while res and not passes_check(G, torch, dtype, ta, tb, m, n, k, batch, alpha, beta, res[0][1]):
            print(f"# config {res[0][1]} FAILS the result check on this shape: left out", file=out)
            res.pop(0)
        best_t, best = res[0]
        row = f"    {{{dtype}, {ta}, {tb}, {m}, {n}, {k}, {batch}, {table_id(G, dtype, best)}, {flops / best_t * 1e-9:.1f}f}},"
        rows.append(row)
        print(f"# dtype {dtype} {'NT'[ta]}{'NT'[tb]} {m}x{n}x{k} batch {batch}: current pick {pick} "
              f"({'%.1f us' % (t_pick * 1e3) if t_pick else 'not timed'}); fastest: "
              + "  ".join(f"{c} {G.config_info(dtype, c)['name']} {t * 1e3:.1f} us" for t, c in res[:4]), file=out)
        print(row, file=out, flush=True)
        table.append({"shape": [dtype, ta, tb, m, n, k, batch, alpha, beta], "pick": pick,
                      "ms": {str(c): t for t, c in res}})
    if dump:
        import json
        with open(dump, "w") as f:
            json.dump(table, f)
    return rows


def main(argv):
    shapes = BUILTIN
    dump = None
    if "--dump" in argv:                      # every config's time per shape, as JSON
        i = argv.index("--dump")
        dump = argv[i + 1]
        argv = argv[:i] + argv[i + 2:]
    if len(argv) > 1:
        shapes = []
        for line in open(argv[1]):
            f = line.split("#")[0].split()
            if f:
                shapes.append(tuple(int(x) for x in f[:7]) + (float(f[7]), float(f[8])))
    tune(shapes, dump=dump)


if __name__ == "__main__":
    main(sys.argv)
