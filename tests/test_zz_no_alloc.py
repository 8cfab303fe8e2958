"""The entry point that allocates nothing (mmbo_gemm_strided_batched_static_workspace): split-K partial sums live in an
array of the library's own device image instead of in memory from hipMalloc.  Its results must be those of
mmbo_gemm_strided_batched bit for bit, call after call (all calls on a GPU share the array, which keeps the last call's
contents); it must not allocate; a named config whose partial sums do not fit must be refused without launching
anything, and the automatic pick must then run with a smaller split instead."""
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


def test_static_workspace_entry_point_allocates_no_device_memory():
    """The property the entry point exists for: a first-time split-K shape through it leaves the device's free memory
    unchanged and the library's workspace table empty, while the same shape through the ordinary entry point takes a
    workspace from hipMalloc."""
    import torch
    import gemm_mmbo_amd as G
    m, n, k = 2048, 1024, 4096                       # 4 splits x 2048 x 1024 x 4 bytes = 32 MiB: exactly the array
    cid = [c for c in range(G.num_configs(F16)) if G.config_info(F16, c)["split_k"] == 4 and G.config_info(F16, c)["macro_tile_m"] == 128][0]
    dA = torch.ones(m * k, device="cuda", dtype=torch.float16)
    dB = torch.ones(k * n, device="cuda", dtype=torch.float16)
    dC = torch.zeros(m * n, device="cuda", dtype=torch.float16)
    # warm both entry points on a shape without split-K, so that code-object loading and the lookup of the array's
    # address are behind us
    nosplit = [c for c in range(G.num_configs(F16)) if G.config_info(F16, c)["split_k"] == 1 and G.config_info(F16, c)["macro_tile_m"] == 128][0]
    for fn in (G.gemm_strided_batched, G.gemm_strided_batched_static_workspace):
        fn(F16, 0, 0, m, n, k, 1.0, dA, m, 0, dB, k, 0, 0.0, dC, m, 0, 1, nosplit)
    G.gemm_strided_batched_static_workspace(F16, 0, 0, 256, 128, 512, 1.0, dA, 256, 0, dB, 512, 0, 0.0, dC, 256, 0, 1, cid)
    torch.cuda.synchronize()
    G.release_workspace()
    assert G.workspace_info() == (0, 0)
    free0 = torch.cuda.mem_get_info()[0]
    G.gemm_strided_batched_static_workspace(F16, 0, 0, m, n, k, 1.0, dA, m, 0, dB, k, 0, 0.0, dC, m, 0, 1, cid)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the static-workspace entry point changed the device's free memory"
    assert G.workspace_info() == (0, 0)
    assert float(dC.min()) == float(k) and float(dC.max()) == float(k)          # 4096 ones: exact in fp16
    dC.zero_()
    G.gemm_strided_batched(F16, 0, 0, m, n, k, 1.0, dA, m, 0, dB, k, 0, 0.0, dC, m, 0, 1, cid)
    torch.cuda.synchronize()
    slots, nbytes = G.workspace_info()
    assert slots == 1 and nbytes >= 4 * m * n * 4
    assert torch.cuda.mem_get_info()[0] <= free0 - 4 * m * n * 4, "the ordinary entry point should have taken a workspace"
    assert float(dC.min()) == float(k) and float(dC.max()) == float(k)
    G.release_workspace()


def test_static_workspace_automatic_pick_lowers_the_split_until_it_fits():
    """HGEMM 2048 x 2048 x 32768: the automatic pick is a split-K config whose partial sums (GlobalSplitU x 16 MiB) are
    beyond the 32 MiB array.  Under MMBO_CONFIG_AUTO the static entry point runs the same tile with a smaller split
    and delivers the product; the config named outright is still refused."""
    import torch
    import gemm_mmbo_amd as G
    m = n = 2048
    k = 32768
    cid = G.select_config(F16, 0, 0, m, n, k, 1)
    split = G.config_info(F16, cid)["split_k"]
    assert split * m * n * 4 > G.static_workspace_bytes(), "pick a shape whose automatic split does not fit"
    p = U.Problem(F16, 0, 0, m, n, k, 1.0, 0.0, seed=97, dist="normal", c_fill="nan")
    dA, dB, dC = (torch.from_numpy(x).cuda() for x in (p.A, p.B, p.C))
    with pytest.raises(G.MmboError) as e:
        G.gemm_strided_batched_static_workspace(F16, 0, 0, m, n, k, 1.0, dA, p.lda, 0, dB, p.ldb, 0, 0.0, dC, p.ldc, 0, 1, cid)
    assert e.value.status == 8
    G.gemm_strided_batched_static_workspace(F16, 0, 0, m, n, k, 1.0, dA, p.lda, 0, dB, p.ldb, 0, 0.0, dC, p.ldc, 0, 1, G.CONFIG_AUTO)
    torch.cuda.synchronize()
    U.check(p, dC.cpu().numpy(), "static workspace, automatic pick, split lowered")
