"""The entry point that allocates nothing (mmbo_gemm_strided_batched_static_workspace): split-K partial sums and arrival
counters live in an array of the library's own device image instead of in memory from hipMalloc.  Its results must be
those of mmbo_gemm_strided_batched bit for bit, call after call (all calls on a GPU share the array, which keeps the last
call's contents), and a call whose partial sums do not fit must be refused without launching anything."""
import numpy as np
import pytest

import util as U

pytestmark = pytest.mark.gpu

F32, F16 = 0, 1


def _both(p, cid):
    """C from the ordinary entry point and from the static-workspace one, on the same device operands."""
    import torch
    import gemm_mmbo_amd as G
    dA, dB = torch.from_numpy(p.A).cuda(), torch.from_numpy(p.B).cuda()
    outs = []
    for fn in (G.gemm_strided_batched, G.gemm_strided_batched_static_workspace):
        dC = torch.from_numpy(p.C).cuda()
        fn(p.dtype, p.ta, p.tb, p.m, p.n, p.k, p.alpha, dA, p.lda, p.sa, dB, p.ldb, p.sb, p.beta, dC, p.ldc, p.sc, p.batch, cid)
        torch.cuda.synchronize()
        outs.append(dC.cpu().numpy())
    return outs


def test_static_workspace_entry_point_matches_the_allocating_one_on_consecutive_calls():
    import gemm_mmbo_amd as G
    assert G.static_workspace_bytes() == 32 << 20
    # two calls in a row, the second with a smaller input; then more, over every kernel family and the automatic pick
    cases = [(F16, 0, 0, 4096, 128, 4096, 1.0, 0.0, 1, None), (F16, 0, 0, 1000, 72, 1500, 1.0, 0.0, 1, "x16"),
             (F32, 0, 1, 128, 4096, 2048, 1.5, 0.5, 1, None), (F32, 1, 0, 257, 131, 1000, -1.0, 1.0, 2, "staged"),
             (F16, 1, 1, 256, 256, 2048, 1.0, 0.0, 4, "ring"), (F32, 0, 0, 512, 512, 512, 1.0, 0.0, 1, None)]
    for (dtype, ta, tb, m, n, k, alpha, beta, batch, family) in cases:
        if family is None:
            cid = G.select_config(dtype, ta, tb, m, n, k, batch)
        else:
            names = {c: G.config_info(dtype, c) for c in range(G.num_configs(dtype))}
            want = {"x16": lambda d: "_ACC" in d["name"], "ring": lambda d: "DTL1" in d["name"] and "_ACC" not in d["name"],
                    "staged": lambda d: "DTL1" not in d["name"]}[family]
            cid = [c for c, d in names.items() if want(d) and d["split_k"] == 4 and d["macro_tile_m"] == 64][0]
        p = U.Problem(dtype, ta, tb, m, n, k, alpha, beta, batch=batch, seed=90 + m, dist="normal" if dtype == F16 else "uniform",
                      c_fill="uniform" if beta else "nan")
        ordinary, static = _both(p, cid)
        assert np.array_equal(ordinary.view(np.uint8), static.view(np.uint8)), (dtype, m, n, k, cid)
        U.check(p, static, f"static workspace {m}x{n}x{k} config {cid}")


def test_static_workspace_entry_point_refuses_what_does_not_fit():
    import torch
    import gemm_mmbo_amd as G
    # 16 splits x 2048 x 2048 x 4 bytes = 256 MiB of partial sums: beyond the 32 MiB array
    cid = [c for c in range(G.num_configs(F32)) if G.config_info(F32, c)["split_k"] == 16][0]
    m = n = 2048
    k = 4096
    dA = torch.zeros(m * k, device="cuda")
    dB = torch.zeros(k * n, device="cuda")
    dC = torch.full((m * n,), 3.0, device="cuda")
    with pytest.raises(G.MmboError) as e:
        G.gemm_strided_batched_static_workspace(F32, 0, 0, m, n, k, 1.0, dA, m, 0, dB, k, 0, 0.0, dC, m, 0, 1, cid)
    assert e.value.status == 8
    torch.cuda.synchronize()
    assert float(dC.min()) == 3.0 and float(dC.max()) == 3.0          # nothing ran
    # the same shape without split-K needs no workspace and runs
    G.gemm_strided_batched_static_workspace(F32, 0, 0, m, n, k, 1.0, dA, m, 0, dB, k, 0, 0.0, dC, m, 0, 1,
                                            [c for c in range(G.num_configs(F32)) if G.config_info(F32, c)["split_k"] == 1][0])
    torch.cuda.synchronize()
    assert float(dC.abs().max()) == 0.0
