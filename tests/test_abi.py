"""Host-side tests of the C-ABI library: it loads, exports every symbol include/mmbo_gemm.h declares,
validates arguments with status codes (never exit()), and its pure-host logic -- the tile-config table,
the per-shape selection and the work-group remap -- behaves.  No compute call is made: no GPU needed.
"""
import ctypes
import os
import re

import numpy as np
import pytest

import gemm_mmbo_amd as G
from gemm_mmbo_amd import api
from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mmbo_gemm.h")


def test_library_is_built_in_tree_and_loads():
    assert os.path.exists(api.LIB_PATH), "build with `python -m gemm_mmbo_amd.build`"
    assert "gfx950" in G.version()


def test_every_declared_symbol_is_exported():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(mmbo_[a-z0-9_]+)\s*\(", text))
    assert declared == set(api.EXPORTS), declared ^ set(api.EXPORTS)
    L = ctypes.CDLL(api.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), f"{name} declared in the header but not exported"


def test_config_table_rows_are_consistent():
    for dtype in (G.F32, G.F16, G.F64):
        n = G.num_configs(dtype)
        assert n >= 4
        mfma = 16 if dtype == G.F64 else 32          # MFMA block edge: 16x16x4 fp64, 32x32 otherwise
        names = set()
        for cid in range(n):
            d = G.config_info(dtype, cid)
            names.add(d["name"])
            assert d["threads"] % 64 == 0 and 64 <= d["threads"] <= 1024
            assert d["macro_tile_m"] % d["wave_tile_m"] == 0 and d["macro_tile_n"] % d["wave_tile_n"] == 0
            waves = (d["macro_tile_m"] // d["wave_tile_m"]) * (d["macro_tile_n"] // d["wave_tile_n"])
            assert waves * 64 == d["threads"]
            assert d["wave_tile_m"] % mfma == 0 and d["wave_tile_n"] % mfma == 0
            assert 0 < d["lds_bytes"] <= 160 * 1024                                # gfx950: 160 KB per CU
            assert d["split_k"] in (1, 2, 4, 8, 16)
        assert len(names) == n
    with pytest.raises(G.MmboError):
        G.config_info(G.F32, G.num_configs(G.F32))
    with pytest.raises(G.MmboError):
        G.config_info(7, 0)


def test_select_config_headline_and_skinny_shapes():
    big16 = G.config_info(G.F16, G.select_config(G.F16, 0, 0, 8192, 8192, 8192))
    assert big16["macro_tile_m"] * big16["macro_tile_n"] >= 256 * 128 and big16["split_k"] == 1
    big32 = G.config_info(G.F32, G.select_config(G.F32, 0, 0, 8192, 8192, 8192))
    assert big32["macro_tile_m"] * big32["macro_tile_n"] >= 128 * 128 and big32["split_k"] == 1
    # 4096 x 128 x 4096 has only a few dozen large output tiles: the pick must spread the work over the
    # 256 CUs, by smaller tiles or by splitting K
    for dtype in (G.F32, G.F16):
        for (m, n, k) in ((4096, 128, 4096), (128, 4096, 8192)):
            d = G.config_info(dtype, G.select_config(dtype, 0, 0, m, n, k))
            tiles = -(-m // d["macro_tile_m"]) * -(-n // d["macro_tile_n"]) * d["split_k"]
            assert tiles >= 128, d
    # tiny problem: a small tile, no split
    d = G.config_info(G.F32, G.select_config(G.F32, 0, 0, 40, 40, 64))
    assert d["macro_tile_m"] <= 64 and d["split_k"] == 1
    assert G.select_config(G.F32, 0, 0, 0, 5, 5) == 0
    # fp64 has its own table: the reference's HPL trailing update gets the tile its sweep found fastest (with K = 384
    # the 64 x 64 tile, five work-groups to a CU, edges out the 128 x 128 ones), a tiny problem a small one
    hpl = G.config_info(G.F64, G.select_config(G.F64, 0, 1, 44160, 2048, 384))
    assert hpl["macro_tile_m"] * hpl["macro_tile_n"] >= 64 * 64 and hpl["split_k"] == 1
    assert G.config_info(G.F64, G.select_config(G.F64, 0, 1, 40, 40, 64))["macro_tile_m"] <= 64
    with pytest.raises(G.MmboError):
        G.select_config(3, 0, 0, 1, 1, 1)
    with pytest.raises(G.MmboError):
        G.select_config(G.F32, 2, 0, 1, 1, 1)


def test_wg_remap_host_twin_matches_reference_golden():
    """With one XCD and id = wg0 + wg1*nwg0 the kernels' mapping is the reference's WGM remap: all 29,440
    pairs of src/gemm/ref/res."""
    gold = np.load(os.path.join(ROOT, "tests", "golden", "wg_remap_460x64_wgm8.npy")).astype(np.int64)
    for wg0, wg1, e0, e1 in gold:
        assert G.wg_remap(int(wg0 + wg1 * 460), 460, 64, 8, 1) == (int(e0), int(e1))


@pytest.mark.parametrize("nwg0,nwg1", [(32, 32), (7, 13), (1, 1), (5, 3), (16, 9), (33, 2), (2, 33)])
@pytest.mark.parametrize("wgm,nxcd", [(8, 8), (8, 1), (4, 8), (1, 8)])
def test_wg_remap_host_twin_bijection_and_oracle(nwg0, nwg1, wgm, nxcd):
    seen = set()
    for lid in range(nwg0 * nwg1):
        t = G.wg_remap(lid, nwg0, nwg1, wgm, nxcd)
        assert 0 <= t[0] < nwg0 and 0 <= t[1] < nwg1
        seen.add(t)
        if nxcd == 1:
            assert t == O.wg_remap(lid % nwg0, lid // nwg0, nwg0, nwg1, wgm)
    assert len(seen) == nwg0 * nwg1


def test_wg_remap_groups_each_xcd_on_neighbouring_tiles():
    """8192^3 with 256x256 tiles: 32 x 32 tiles.  Ids congruent mod 8 run on one XCD; the first 32 of them
    (one per CU of that XCD) must cover a compact block: at most 8 tile columns x 4 tile rows."""
    for x in range(8):
        tiles = [G.wg_remap(x + 8 * i, 32, 32, 8, 8) for i in range(32)]
        rows = {t[0] for t in tiles}
        cols = {t[1] for t in tiles}
        assert len(cols) <= 8 and len(rows) <= 5


@pytest.mark.parametrize("nwg0,nwg1", [(32, 32), (16, 16), (17, 16), (16, 19), (35, 50), (48, 33)])
def test_chip_block_remap_bijection_and_block_structure(nwg0, nwg1):
    """The chip-wide block order of the 256 x 256 HGEMM tiles: a bijection; every run of 256 consecutive ids inside
    the whole blocks covers exactly one 16 x 16 block of tiles, and the 32 ids of one XCD (id % 8) in it a 4 x 8
    sub-block; consecutive blocks share their tile rows or their tile columns (one operand panel stays cached)."""
    seen = set()
    tiles = [G.chip_block_remap(lid, nwg0, nwg1) for lid in range(nwg0 * nwg1)]
    for t in tiles:
        assert 0 <= t[0] < nwg0 and 0 <= t[1] < nwg1
        seen.add(t)
    assert len(seen) == nwg0 * nwg1
    nblk = (nwg0 // 16) * (nwg1 // 16)
    prev = None
    for b in range(nblk):
        blk = tiles[256 * b:256 * (b + 1)]
        r0, c0 = min(t[0] for t in blk), min(t[1] for t in blk)
        assert r0 % 16 == 0 and c0 % 16 == 0
        assert {(t[0] - r0, t[1] - c0) for t in blk} == {(i, j) for i in range(16) for j in range(16)}
        for x in range(8):
            sub = blk[x::8]
            assert max(t[0] for t in sub) - min(t[0] for t in sub) == 3
            assert max(t[1] for t in sub) - min(t[1] for t in sub) == 7
        if prev is not None:
            assert prev[0] == r0 or prev[1] == c0
        prev = (r0, c0)


@pytest.mark.parametrize("tiles,batch", [(4, 64), (1, 8), (16, 16), (32, 24), (3, 40)])
def test_batch_xcd_remap_bijection_and_one_problem_per_xcd(tiles, batch):
    """Batches of small problems: a bijection of the dispatch indices onto (tile, batch index); all tiles of one
    problem fall on one XCD (dispatch index % 8), on consecutive turns of that XCD."""
    got = [G.batch_xcd_remap(lid, tiles, batch) for lid in range(tiles * batch)]
    assert sorted(got) == [(t, z) for t in range(tiles) for z in range(batch)]
    for z in range(batch):
        lids = [lid for lid, (t, zz) in enumerate(got) if zz == z]
        assert len({lid % 8 for lid in lids}) == 1
        turns = sorted(lid // 8 for lid in lids)
        assert turns == list(range(turns[0], turns[0] + tiles))
        assert [got[lid][0] for lid in sorted(lids)] == list(range(tiles))
    with pytest.raises(G.MmboError):
        G.batch_xcd_remap(0, tiles, batch + 1)
    with pytest.raises(G.MmboError):
        G.batch_xcd_remap(tiles * batch, tiles, batch)


def test_chip_block_remap_rejects_bad_arguments():
    with pytest.raises(G.MmboError):
        G.chip_block_remap(0, 15, 16)        # fewer than 16 tile rows
    with pytest.raises(G.MmboError):
        G.chip_block_remap(16 * 16, 16, 16)  # id out of range


def test_wg_remap_rejects_bad_arguments():
    with pytest.raises(G.MmboError):
        G.wg_remap(10, 2, 5, 8, 8)          # id out of range
    with pytest.raises(G.MmboError):
        G.wg_remap(0, 0, 5, 8, 8)


def _call(dtype=0, ta=0, tb=0, m=4, n=4, k=4, lda=4, ldb=4, ldc=4, A=16, B=16, C=16, cfg=-1, alpha=True, beta=True):
    """Raw C-ABI call with fake non-null device addresses; every case here must fail validation before any
    device work."""
    al, be = ctypes.c_float(1.0), ctypes.c_float(0.0)
    return api.lib().mmbo_gemm(dtype, ta, tb, m, n, k, ctypes.byref(al) if alpha else None, A, lda, B, ldb,
                               ctypes.byref(be) if beta else None, C, ldc, cfg, None)


def test_argument_validation_returns_status_codes():
    assert _call(dtype=5) == 1
    assert _call(ta=2) == 2
    assert _call(tb=-1) == 2
    assert _call(lda=3) == 3
    assert _call(ta=1, k=8, lda=4) == 3          # A^T is stored k x m: lda >= k
    assert _call(ldb=3) == 3
    assert _call(tb=1, n=8, ldb=4, ldc=4) == 3   # B^T is stored n x k: ldb >= n
    assert _call(ldc=3) == 3
    assert _call(m=2 ** 31) == 3
    assert _call(alpha=False) == 4
    assert _call(beta=False) == 4
    assert _call(C=None) == 4
    assert _call(A=None) == 4
    assert _call(cfg=10 ** 6) == 5
    assert _call(cfg=-2) == 5
    assert _call(dtype=2, cfg=G.num_configs(G.F64)) == 5      # ids are per element type: fp64 has fewer rows
    assert _call(dtype=2, lda=3) == 3
    # empty problems succeed without touching anything (null pointers allowed)
    assert _call(m=0, A=None, B=None, C=None, lda=1, ldc=1) == 0
    assert _call(n=0, A=None, B=None, C=None) == 0
    for s in range(0, 9):
        assert api.lib().mmbo_status_string(s)
    # strided-batched: negative batch or stride
    al, be = ctypes.c_float(1.0), ctypes.c_float(0.0)
    f = api.lib().mmbo_gemm_strided_batched
    assert f(0, 0, 0, 4, 4, 4, ctypes.byref(al), 16, 4, 16, 16, 4, 16, ctypes.byref(be), 16, 4, 16, -1, -1, None) == 3
    assert f(0, 0, 0, 4, 4, 4, ctypes.byref(al), 16, 4, -16, 16, 4, 16, ctypes.byref(be), 16, 4, 16, 2, -1, None) == 3
    assert f(0, 0, 0, 4, 4, 4, ctypes.byref(al), 16, 4, 16, 16, 4, 16, ctypes.byref(be), 16, 4, 16, 0, -1, None) == 0


def test_python_front_ends_keep_reference_argument_order():
    """src/gemm/gemm.h:4-5: (m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId)."""
    import inspect
    want = ["m", "n", "k", "alpha", "A", "lda", "B", "ldb", "beta", "C", "ldc", "kernelId"]
    for f in (G.naive_dgemm, G.dgemm_NT, G.naive_sgemm, G.naive_hgemm, G.sgemm_NT, G.sgemm_TN, G.hgemm_NN, G.hgemm_TT):
        assert list(inspect.signature(f).parameters) == want


def test_tuner_shape_list_is_valid_and_rows_parse():
    """Every shape of the offline tuner's built-in list is one the library accepts, and its picks are valid ids."""
    from gemm_mmbo_amd import tune
    for (dtype, ta, tb, m, n, k, batch, alpha, beta) in tune.BUILTIN:
        cid = G.select_config(dtype, ta, tb, m, n, k, batch)
        assert 0 <= cid < G.num_configs(dtype)
    # (the timing part needs the GPU: tests/test_gemm_gpu.py)


def test_ragged_shapes_go_to_the_fast_kernels():
    """The x16 kernel takes ragged m, n and k; a dimension smaller than the smallest fast tile mostly keeps a shape with
    the general kernel (unaligned operands do too, but that is decided at the call, not from the shape)."""
    def name(dtype, ta, tb, m, n, k):
        return G.config_info(dtype, G.select_config(dtype, ta, tb, m, n, k))["name"]
    assert "MFMA16x16" in name(G.F16, 0, 0, 3000, 3000, 3000)
    assert "MFMA16x16" in name(G.F32, 0, 1, 4100, 4100, 4099)
    assert "MFMA16x16" in name(G.F16, 1, 0, 3001, 3003, 3005)
    assert "MFMA16x16" in name(G.F16, 0, 0, 3001, 3000, 3008)
    assert "MFMA16x16" in name(G.F32, 0, 1, 1001, 1002, 1000)
    assert "DTL1" not in name(G.F32, 0, 0, 8, 4096, 4096)                          # a dimension below the smallest fast tile:
    assert "DTL1" not in name(G.F16, 0, 0, 40, 40, 64)                             # general kernel, except fp16 on a long k
    assert "MT064x064" in name(G.F16, 0, 0, 8, 4096, 4096) and "DTL1" in name(G.F16, 0, 0, 8, 4096, 4096)
    assert "DTL1" in name(G.F16, 0, 0, 72, 4096, 4096)
    # large ragged shapes whose packed rows split cache lines: the 256 x 256 tile, not the bandwidth-bound smaller ones
    assert G.config_info(G.F16, G.select_config(G.F16, 1, 0, 7000, 7000, 7008))["macro_tile_m"] == 256


def test_sizes_between_rounds_of_the_cus_get_the_192_tiles():
    """3000^2 is 144 tiles of 256 x 256 -- little more than half of the 256 CUs -- but 256 tiles of 192 x 192; the pick
    follows the tile counts (the reference keeps such knowledge in its exact-size table,
    src/gemm/ref/vega20_Cijk_Ailk_Bjlk_DB.yaml:929-1177).  Sizes that fill whole rounds keep the 256 x 256 tile."""
    def tile(dtype, m, n, k, ta=0, tb=0):
        d = G.config_info(dtype, G.select_config(dtype, ta, tb, m, n, k))
        return d["macro_tile_m"], d["macro_tile_n"]
    assert tile(G.F16, 3000, 3000, 3000) == (192, 192) and tile(G.F16, 3072, 3072, 3072) == (192, 192)
    assert tile(G.F32, 3072, 3072, 3072) == (192, 192)
    assert tile(G.F16, 3328, 3328, 3328) in ((256, 192), (192, 256)) and tile(G.F16, 4608, 4608, 4608) in ((256, 192), (192, 256))
    for s in (3584, 4096, 5120, 8192):
        assert tile(G.F16, s, s, s) == (256, 256), s
    assert tile(G.F16, 2048, 2048, 2048) == (128, 128) and tile(G.F16, 2560, 2560, 2560) == (128, 128)
    # the three tiles exist for both element types and every GlobalSplitU, one work-group per CU (more than 80 KB of LDS)
    for dtype in (G.F16, G.F32):
        big = [G.config_info(dtype, c) for c in range(G.num_configs(dtype))]
        for mt in ((192, 192), (256, 192), (192, 256)):
            rows = [d for d in big if (d["macro_tile_m"], d["macro_tile_n"]) == mt]
            assert sorted(d["split_k"] for d in rows) == [1, 2, 4, 8, 16] and all(d["lds_bytes"] > 80 * 1024 and d["threads"] == 256 for d in rows)
