"""Parity of the HIP kernels with the fp64 oracle, through the C ABI, on a real MI355X.

Covers the five benchmark configurations at their full sizes, every tile config and split-K factor on
ragged shapes, all four transposes, leading dimensions larger than the matrix, unaligned operands, the
beta == 0 "never read C" rule, k = 0, strided batches, and size-independent properties (identity, all
ones, linearity in alpha/beta) at full size.  Tolerances are in tests/util.py:
fp32 <= 1e-5*sqrt(K), fp16 <= 2e-2, relative to max(|exact|, rms(exact)).
"""
import os

import numpy as np
import pytest

import util as U
from oracle import oracle as O

pytestmark = pytest.mark.gpu

F32, F16 = 0, 1
NAMES = {F32: "f32", F16: "f16"}


def _run_and_check(p, config_id=-1, label="", offsets=(0, 0, 0)):
    got, guard = U.run_gpu(p, config_id, offsets)
    U.check(p, got, label)
    assert np.all(guard == 0), "wrote past the end of C"
    return got


# ------------------------------------------------------------------ the five benchmark configurations

def test_cfg1_sgemm_nn_1024():
    """SGEMM NN 1024^3, ld = 1024, U[-1,1] from seed 0 (A then B from one stream), alpha=1, beta=0."""
    p = U.Problem(F32, 0, 0, 1024, 1024, 1024, 1.0, 0.0, seed=0, c_fill="nan")
    _run_and_check(p, label="cfg1")


@pytest.mark.parametrize("ta,tb", [(0, 1), (1, 0)])
def test_cfg2_sgemm_nt_tn_4096(ta, tb):
    """SGEMM NT and TN 4096^3, C pre-filled, alpha=1.5, beta=0.5: transposed load paths and C read-modify-write."""
    p = U.Problem(F32, ta, tb, 4096, 4096, 4096, 1.5, 0.5, seed=2)
    _run_and_check(p, label=f"cfg2 {'NT'[ta]}{'NT'[tb]}")


def test_cfg3_hgemm_nn_8192():
    """HGEMM NN 8192^3, A/B ~ N(0,1)*0.1 rounded to fp16, fp32 accumulate, alpha=1, beta=0; full check of
    all 67M outputs against the fp64 oracle."""
    p = U.Problem(F16, 0, 0, 8192, 8192, 8192, 1.0, 0.0, seed=3, dist="normal", c_fill="nan")
    _run_and_check(p, label="cfg3")


def test_cfg3_fp32_sgemm_nn_8192():
    """The metric's fp32 leg: SGEMM NN 8192^3, U[-1,1]."""
    p = U.Problem(F32, 0, 0, 8192, 8192, 8192, 1.0, 0.0, seed=33, c_fill="nan")
    _run_and_check(p, label="cfg3' f32")


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
@pytest.mark.parametrize("m,n,k", [(1023, 777, 513), (4096, 128, 4096), (128, 4096, 8192)])
def test_cfg4_irregular_and_skinny(dtype, m, n, k):
    p = U.Problem(dtype, 0, 0, m, n, k, 1.0, 0.0, seed=4, c_fill="nan")
    _run_and_check(p, label=f"cfg4 {m}x{n}x{k}")


def test_cfg5_strided_batched_hgemm_tn():
    """64 x (512^3) HGEMM TN, stride = one full matrix per operand, alpha=1, beta=1, C ~ U[-1,1]."""
    p = U.Problem(F16, 1, 0, 512, 512, 512, 1.0, 1.0, batch=64, seed=5, dist="normal")
    assert (p.sa, p.sb, p.sc) == (262144, 262144, 262144)
    _run_and_check(p, label="cfg5")


def test_batches_of_small_problems_one_per_xcd():
    """Batches that are multiples of 8, of problems of at most 32 tiles: every kernel family lays one problem on one
    XCD (mmbo_batch_xcd_remap) instead of the dispatcher's order.  Every GlobalSplitU = 1 config of each family (fp32,
    fp16) and the fp64 configs, 1 to 32 tiles per problem, ragged sizes for the kernels that take them, gaps between
    the matrices of the batch, beta != 0; and neighbours that must stay on the plain order (batch 12, 36 tiles, split-K)."""
    import gemm_mmbo_amd as G
    ran = 0
    for dtype in (F32, F16, U.F64):
        dist = "normal" if dtype == F16 else "uniform"
        for cid in range(G.num_configs(dtype)):
            d = G.config_info(dtype, cid)
            name = d["name"]
            ring_only = "DTL1" in name and "_ACC" not in name
            if "GSU01" not in name:
                continue
            bm, bn = d["macro_tile_m"], d["macro_tile_n"]
            bk = d["depth_u"]
            shapes = [(bm, bn, 4 * bk, 8), (2 * bm, 2 * bn, 2 * bk, 16), (4 * bm, 8 * bn, 2 * bk, 8)]
            if not ring_only and bm <= 128:
                shapes.append((2 * bm - 3, 3 * bn - 5, 3 * bk + 1, 24))
            for (m, n, k, batch) in shapes:
                if m * n * batch > 48 << 20:
                    continue
                ta, tb = cid % 2, (cid // 2) % 2
                (ar, ac), (br, bc) = U.stored_shape(ta, m, k), U.stored_shape(tb, k, n)
                gap = 8
                p = U.Problem(dtype, ta, tb, m, n, k, 1.0, 0.5, batch=batch, seed=40 + cid, dist=dist, c_fill="uniform",
                              strides=(ar * ac + gap, br * bc + gap, m * n + gap))
                _run_and_check(p, cid, label=f"{name} {m}x{n}x{k} b{batch}")
                ran += 1
    assert ran >= 60
    for (dtype, m, n, k, batch, cid) in ((F16, 256, 256, 256, 12, -1), (F16, 384, 384, 128, 8, _x16_ids(F16)[4]),
                                         (F32, 128, 128, 512, 8, _x16_ids(F32)[4 + 8])):
        p = U.Problem(dtype, 1, 0, m, n, k, 1.0, 1.0, batch=batch, seed=3, dist="normal" if dtype == F16 else "uniform", c_fill="uniform")
        _run_and_check(p, cid, label=f"plain order {m}x{n}x{k} b{batch}")


# ------------------------------------------------------------------ every config id on ragged shapes

@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_every_config_every_transpose_ragged(dtype, ta, tb):
    """257 x 131 x 1000 with tightly packed operands through every config id.  The general kernel and the x16 family
    take it in every config and transpose (odd m and n, also where they are the contiguous dimension; columns that
    start off 16-byte boundaries; 31 or 62 whole slices of k and a partial one, split unevenly); the ring family only
    takes whole tiles and must refuse it, never compute it wrongly."""
    import gemm_mmbo_amd as G
    taken = 0
    for cid in range(G.num_configs(dtype)):
        name = G.config_info(dtype, cid)["name"]
        p = U.Problem(dtype, ta, tb, 257, 131, 1000, 1.5, 0.5, lda=None, ldc=260, seed=10 + cid)
        if "DTL1" in name and "MFMA16x16" not in name:
            with pytest.raises(G.MmboError) as e:
                U.run_gpu(p, cid)
            assert e.value.status == 5
            continue
        _run_and_check(p, cid, label=f"config {cid} {name}")
        taken += "MFMA16x16" in name
    assert taken == 40


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_every_config_aligned_interior(dtype):
    """Sizes that are multiples of every tile: only the unpredicated fast path runs."""
    import gemm_mmbo_amd as G
    for cid in range(G.num_configs(dtype)):
        p = U.Problem(dtype, 0, 0, 512, 512, 1024, 1.0, 0.0, seed=50 + cid, c_fill="nan")
        _run_and_check(p, cid, label=f"config {cid}")


def _ring_ids(dtype):
    """Config ids of the generic direct-to-LDS ring kernel (32x32 MFMA blocks)."""
    import gemm_mmbo_amd as G
    names = {c: G.config_info(dtype, c)["name"] for c in range(G.num_configs(dtype))}
    return [c for c, nm in names.items() if "DTL1" in nm and "_ACC" not in nm]


def _x16_ids(dtype=F16):
    """Config ids of the ring kernel on 16x16 MFMA blocks with accumulation-register accumulators."""
    import gemm_mmbo_amd as G
    mark = "MFMA16x16x32_ACC" if dtype == F16 else "MFMA16x16x4_ACC"
    return [c for c in range(G.num_configs(dtype)) if mark in G.config_info(dtype, c)["name"]]


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_ring_kernel_every_config_every_transpose(dtype, ta, tb):
    """The direct-to-LDS ring kernel by explicit config id: every ring tile and split-K factor, with K shorter
    and longer than the ring (fewer slices than buffers, odd slice counts), beta read-modify-write, batches."""
    import gemm_mmbo_amd as G
    ids = _ring_ids(dtype)
    assert len(ids) == 20
    bk = 16 if dtype == F32 else 32
    ran = 0
    for cid in ids:
        d = G.config_info(dtype, cid)
        bm, bn, sp = d["macro_tile_m"], d["macro_tile_n"], d["split_k"]
        for (tm, tn, slices, alpha, beta, batch) in ((1, 1, 1, 1.0, 0.0, 1), (2, 1, 3, 1.5, 0.5, 1), (1, 3, 7, -1.0, 1.0, 2),
                                                     (3, 2, 33, 1.0, 0.0, 1)):
            m, n, k = bm * tm, bn * tn, bk * slices * sp
            p = U.Problem(dtype, ta, tb, m, n, k, alpha, beta, batch=batch, seed=70 + cid + slices,
                          dist="normal" if dtype == F16 else "uniform", c_fill="uniform" if beta else "nan")
            _run_and_check(p, cid, label=f"{d['name']} {m}x{n}x{k} b{batch}")
            ran += 1
    assert ran == 80


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_x16_kernel_every_config_every_transpose(dtype, ta, tb):
    """The ring kernel on 16x16 MFMA blocks (v_mfma_f32_16x16x32_f16 / v_mfma_f32_16x16x4_f32) with accumulators pinned
    to the accumulation registers, by explicit config id: every tile (4 and 8 wavefronts, 64 to 256 accumulator
    registers, the 192 x 192 tile whose row-contiguous operands lie in LDS as three sub-tiles of 64 rows) and split-K factor, K shorter and longer than the ring, odd slice counts (the paired-load schedule has an
    even/odd rhythm), beta read-modify-write, batches."""
    import gemm_mmbo_amd as G
    ids = _x16_ids(dtype)
    assert len(ids) == 40
    bk = 16 if dtype == F32 else 32
    ran = 0
    for cid in ids:
        d = G.config_info(dtype, cid)
        assert d["depth_u"] == bk
        bm, bn, sp = d["macro_tile_m"], d["macro_tile_n"], d["split_k"]
        for (tm, tn, slices, alpha, beta, batch) in ((1, 1, 1, 1.0, 0.0, 1), (2, 1, 3, 1.5, 0.5, 1), (1, 3, 7, -1.0, 1.0, 2),
                                                     (3, 2, 33, 1.0, 0.0, 1), (1, 1, 6, 1.0, 0.0, 1)):
            m, n, k = bm * tm, bn * tn, bk * slices * sp
            p = U.Problem(dtype, ta, tb, m, n, k, alpha, beta, batch=batch, seed=170 + cid + slices,
                          dist="normal" if dtype == F16 else "uniform", c_fill="uniform" if beta else "nan")
            _run_and_check(p, cid, label=f"{d['name']} {m}x{n}x{k} b{batch}")
            ran += 1
    assert ran == 200


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_x16_kernel_edge_tiles_and_partial_last_slice(dtype, ta, tb):
    """Ragged problems in the x16 kernel, by explicit config id, every tile and split-K factor: m and n that end inside
    a tile (loads repeat the last rows, stores are guarded: the reference's edge handling, src/gemm/ref/Kernels.cpp:
    1007-1121), down to a single row or column, odd sizes also where the dimension is the contiguous one; a k that ends
    inside a slice (zero-filled: the reference's tail loop, :921-1005), down to k smaller than one slice; with beta,
    batches, padded leading dimensions whose padding rows of C must stay untouched, and operands whose columns start off
    16-byte boundaries (the direct loads take any element-aligned address)."""
    import gemm_mmbo_amd as G
    bk = 16 if dtype == F32 else 32
    g = 4 if dtype == F32 else 8                                # elements per 16 bytes
    ran = 0
    for cid in _x16_ids(dtype):
        d = G.config_info(dtype, cid)
        bm, bn, sp = d["macro_tile_m"], d["macro_tile_n"], d["split_k"]
        #        m            n        slices alpha beta batch pad k tail
        cases = [(bm + g, 2 * bn - g, 3, 1.0, 0.0, 1, 0, 0), (2 * bm - 3 * g, bn + 5 * g, 7, 1.5, 0.5, 2, 8, 0), (g, bn, 2, 1.0, 0.0, 1, 0, 0),
                 (bm, bn, 2, 1.0, 0.0, 1, 0, 1), (bm + g, bn - g, 3, 1.5, 0.5, 2, 8, bk - 1), (2 * bm, bn, 0 if sp == 1 else 1, 1.0, 0.0, 1, 0, 5),
                 (bm, 2 * bn, 6, -1.0, 1.0, 1, 0, g), (bm - g, bn + g, 11, 1.0, 0.0, 1, 8, bk // 2 + 1)]
        if sp > 1:              # uneven splits: the last one gets fewer slices, only the partial one, or the count shrinks
            cases += [(bm, bn + g, 5, 1.0, 0.0, 1, 0, bk * (sp - 1) + 3), (bm + g, bn, 1, 1.5, 0.5, 1, 0, bk + 1), (bm, bn, 0, 1.0, 0.0, 1, 0, bk * 2 + 9)]
        # m, n that end inside a 16-byte group (also where that dimension is the contiguous one) and inside a 4-row group
        cases += [(bm + 3, bn + g, 5, -1.0, 1.0, 1, 0, 0), (bm + g, bn - 1, 6, 1.0, 0.5, 1, 0, 3), (bm - 1, 2 * bn + 1, 4, 1.0, 0.0, 2, 8, 7),
                  (1, 1, 1, 1.0, 0.0, 1, 0, 1), (bm + g + 1, 3, 2, 1.5, 0.5, 1, 8, 0)]
        cases = [c + (True,) for c in cases]
        # tightly packed or oddly padded operands at element offsets: columns of A and B start off 16-byte boundaries
        cases += [(bm + 3, bn + 5, 3, 1.0, 0.0, 1, 0, 1, False), (2 * bm - 1, bn - 7, 2, 1.5, 0.5, 2, 0, bk - 3, False),
                  (g + 1, bn + 1, 1, 1.0, 1.0, 1, 0, 0, False), (bm + 1, g, 5, 1.0, 0.0, 1, 0, 5, False), (bm, bn, 4, 1.0, 0.0, 1, 0, 0, False)]
        for (m, n, slices, alpha, beta, batch, pad, kt, aligned) in cases:
            k = bk * slices * sp + kt
            ar, br = U.stored_shape(ta, m, k)[0], U.stored_shape(tb, k, n)[0]
            if aligned:
                lda, ldb = -(-ar // g) * g + pad, -(-br // g) * g + pad   # columns of A and B start on 16-byte boundaries
            else:
                lda, ldb = ar + cid % 2, br + (cid % 3 == 0)
            if (not ta and m < g) or (tb and n < g):
                continue                                                # a contiguous dimension shorter than one load: refused
            p = U.Problem(dtype, ta, tb, m, n, k, alpha, beta, lda=lda, ldb=ldb, ldc=m + (3 if pad else 0), batch=batch,
                          seed=900 + cid + slices, dist="normal" if dtype == F16 else "uniform", c_fill="uniform" if beta else "nan")
            _run_and_check(p, cid, label=f"{d['name']} {'NT'[ta]}{'NT'[tb]} {m}x{n}x{k} b{batch} ld {lda},{ldb}",
                           offsets=(0, 0, 0) if aligned else (1, 3, 1))
            ran += 1
    assert ran >= 40 * 16


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (1, 1), (0, 1)])
def test_x16_kernel_old_c_fetched_under_the_last_slices(ta, tb):
    """fp16 with beta != 0: on whole tiles with at least ring-depth + 1 whole slices the x16 kernel fetches the tile's old C
    into the LDS ring buffers its last four slices leave (a kernel variant of its own, in both load schedules: the paired one
    of NN, TN, TT and the plain one of NT).  Slice counts on both sides of that limit and of either parity, every
    tile (those of 128 x 128 and more have the variant; the 192 x 192 one carries fewer groups under the last of the four slices), several tiles per resident work-group, batches, ldc > m; the
    reference's own epilogue order is t = alpha * acc, then fma(beta, C, t) (MT192x096x08 kernel :2300-2316, :3037-3056)."""
    import gemm_mmbo_amd as G
    ids = [c for c in _x16_ids(F16) if G.config_info(F16, c)["split_k"] == 1]
    assert len(ids) == 8
    ran = 0
    for cid in ids:
        d = G.config_info(F16, cid)
        bm, bn = d["macro_tile_m"], d["macro_tile_n"]
        depth = d["lds_bytes"] // ((bm + bn) * 64)
        for slices in (depth, depth + 1, depth + 2, depth + 3, depth + 4, 2 * depth + 3):
            tm, tn, batch = (3, 2, 1) if slices == depth + 2 else (1, 1, 2) if slices == depth + 3 else (1, 1, 1)
            m, n, k = bm * tm, bn * tn, 32 * slices
            p = U.Problem(F16, ta, tb, m, n, k, -0.75, 0.5, ldc=m + (8 if slices % 2 else 0), batch=batch, seed=500 + cid + slices,
                          dist="normal", c_fill="uniform")
            _run_and_check(p, cid, label=f"{d['name']} {'NT'[ta]}{'NT'[tb]} {m}x{n}x{k} b{batch}")
            ran += 1
    assert ran == 48


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_x16_tn_with_both_operands_fetched_on_the_even_slices(dtype):
    """TN on a ring of five buffers, every row of A and B starting on a 128-byte memory line (k a multiple of 64 fp16 / 32
    fp32 elements, tight leading dimensions): the kernel variant that fetches both operands' pairs of slices on the even
    iterations.  Even slice counts from below the ring depth to several steady iterations, with and without the old C
    under the last slices (beta), several tiles per resident work-group, batches; and the same shapes with lda or ldb off
    the line, which must take the alternating variant and give the same values."""
    import gemm_mmbo_amd as G
    ids = [c for c in _x16_ids(dtype) if G.config_info(dtype, c)["split_k"] == 1]
    bk = 16 if dtype == F32 else 32
    line = 128 // (4 if dtype == F32 else 2)                  # elements per memory line
    ran = 0
    for cid in ids:
        d = G.config_info(dtype, cid)
        bm, bn = d["macro_tile_m"], d["macro_tile_n"]
        if d["lds_bytes"] // ((bm + bn) * 64) != 5:
            continue
        for slices, (tm, tn, batch), beta in ((2, (1, 1, 1), 0.0), (4, (1, 1, 2), 0.5), (6, (1, 2, 1), 0.0), (8, (2, 1, 1), 0.5),
                                              (10, (1, 1, 1), 0.5), (14, (3, 2, 1), 0.0), (16, (1, 1, 2), 0.5), (36, (1, 1, 1), 0.5)):
            m, n, k = bm * tm, bn * tn, bk * slices
            assert k % line == 0
            for pad in (0, 8):
                p = U.Problem(dtype, 1, 0, m, n, k, 1.25, beta, lda=k + pad, ldb=k + (0 if slices % 4 else pad), batch=batch,
                              seed=900 + cid + slices, dist="normal" if dtype == F16 else "uniform",
                              c_fill="uniform" if beta else "nan")
                _run_and_check(p, cid, label=f"{d['name']} TN {m}x{n}x{k} b{batch} lda {k + pad}")
                ran += 1
        # odd slice counts, a partial last slice and edge tiles under the same variant: the leading dimensions padded up to
        # a whole number of memory lines
        for (m, n, slices, kt, beta, batch) in ((bm, bn, 5, 0, 0.5, 1), (bm + 8, 2 * bn - 8, 7, 0, 0.0, 1), (bm, bn, 9, 5, 0.5, 2),
                                                (2 * bm - 8, bn + 8, 13, bk - 1, 0.0, 1), (bm, bn, 1, 0, 0.5, 1), (bm, bn, 3, 3, 0.0, 1)):
            k = bk * slices + kt
            ld = -(-k // line) * line
            p = U.Problem(dtype, 1, 0, m, n, k, -0.75, beta, lda=ld, ldb=ld, ldc=m + 8, batch=batch, seed=950 + cid + slices,
                          dist="normal" if dtype == F16 else "uniform", c_fill="uniform" if beta else "nan")
            assert (p.sa * (4 if dtype == F32 else 2)) % 128 == 0
            _run_and_check(p, cid, label=f"{d['name']} TN {m}x{n}x{k} b{batch} ld {ld}")
            ran += 1
    assert ran == 5 * (8 * 2 + 6)


def test_x16_kernel_chip_block_order_and_refusals():
    """Grids of at least 16 x 16 tiles of 256 x 256 walk the tiles in chip-wide blocks: whole blocks, blocks plus a
    ragged border of tiles, against the oracle.  Unaligned operands are taken, a contiguous dimension shorter than one
    16-byte load is refused; ld > dim and the automatic pick work."""
    import gemm_mmbo_amd as G
    ids = _x16_ids()
    for cid in ids[:2]:
        assert G.config_info(F16, cid)["macro_tile_m"] == 256
        for (m, n, k) in ((4096, 4096, 64), (4352, 4096, 96), (4096, 4608, 64), (8192, 4352, 32)):
            p = U.Problem(F16, 0, 0, m, n, k, 1.0, 0.0, seed=300 + m // 256, dist="normal", c_fill="nan")
            _run_and_check(p, cid, label=f"chip blocks {m}x{n}x{k}")
    cid = ids[0]
    # unaligned A or B (an element offset, a leading dimension that is not a whole number of 16-byte groups) are taken
    for (dtype, ta, tb, m, n, k, offs) in ((F16, 0, 0, 256, 256, 128, (1, 0, 0)), (F16, 0, 0, 256, 256, 128, (0, 4, 0)),
                                           (F16, 0, 0, 255, 256, 128, (0, 0, 0)), (F32, 0, 1, 256, 254, 136, (3, 1, 0))):
        p = U.Problem(dtype, ta, tb, m, n, k, 1.0, 0.0, seed=5, c_fill="nan", dist="normal" if dtype == F16 else "uniform")
        _run_and_check(p, _x16_ids(dtype)[0], label=f"x16 unaligned {m}x{n}x{k} {offs}", offsets=offs)
    # refused: a memory-contiguous m or n shorter than one 16-byte load
    for (dtype, ta, tb, m, n, k) in ((F16, 0, 0, 7, 256, 128), (F16, 1, 1, 256, 5, 128), (F32, 0, 1, 3, 3, 64)):
        p = U.Problem(dtype, ta, tb, m, n, k, 1.0, 0.0, seed=5, c_fill="nan")
        with pytest.raises(G.MmboError) as e:
            U.run_gpu(p, _x16_ids(dtype)[0])
        assert e.value.status == 5
        _run_and_check(p, -1, label="auto on a thin contiguous dimension")
    p = U.Problem(F16, 1, 0, 512, 512, 320, 1.0, 0.5, lda=1032, ldb=1040, ldc=520, seed=71, dist="normal")
    _run_and_check(p, cid, label="x16 ld>dim")
    # C needs no alignment: an odd element offset and an odd ldc take the element-wise epilogue, with and without beta
    for dtype in (F16, F32):
        for beta in (0.0, 0.5):
            p = U.Problem(dtype, 0, 1, 256, 512, 192, 1.5, beta, ldc=259, seed=72, dist="normal" if dtype == F16 else "uniform",
                          c_fill="uniform" if beta else "nan")
            _run_and_check(p, _x16_ids(dtype)[1], label="x16 unaligned C", offsets=(0, 0, 1))
    assert G.select_config(F16, 0, 0, 8192, 8192, 8192) in ids
    assert G.select_config(F16, 0, 1, 2048, 2048, 2048) in ids
    assert G.select_config(F32, 1, 0, 8192, 8192, 8192) in _x16_ids(F32)
    p = U.Problem(F32, 0, 0, 4096, 4352, 48, 1.0, 0.0, seed=301, c_fill="nan")
    _run_and_check(p, _x16_ids(F32)[0], label="fp32 chip blocks")


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_x16_resident_work_groups_walk_several_tiles(dtype, ta, tb):
    """More 256 x 256 tiles than CUs: a work-group stays resident and takes several tiles, one after the other through
    the same ring -- whole tiles with even and odd slice counts, a partial last slice, a ragged last tile row -- against
    the oracle, with beta = 0 over NaN-filled C and with a read-modify-write, and in a batch of two problems."""
    cid = _x16_ids(dtype)[0]
    slice_k = 32 if dtype == F16 else 16
    dist = "normal" if dtype == F16 else "uniform"
    cases = [(4352, 4352, 10 * slice_k, 1, 0.0),          # 289 tiles, twice the ring depth in slices
             (4352, 4608, 22 * slice_k, 1, 0.5),          # C read and written
             (4608, 4352, 11 * slice_k, 1, 0.0),          # odd slice count
             (4352, 4352, 12 * slice_k + 5, 1, 0.0),      # partial last slice
             (4352 - 8, 4352, 12 * slice_k, 1, 0.0),      # ragged last tile row
             (4352, 4352, 12 * slice_k, 2, 1.0)]          # two problems, 289 tiles each
    for (m, n, k, batch, beta) in cases:
        p = U.Problem(dtype, ta, tb, m, n, k, 1.25, beta, batch=batch, seed=900 + k + batch, dist=dist,
                      c_fill="uniform" if beta else "nan")
        _run_and_check(p, cid, label=f"resident {'NT'[ta]}{'NT'[tb]} {m}x{n}x{k} b{batch} beta={beta}")


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_ring_kernel_refuses_shapes_it_cannot_take(dtype):
    """Ragged m/n, k that does not split into whole slices, unaligned A: MMBO_ERR_INVALID_CONFIG, never a wrong
    result; the automatic pick moves to a kernel that takes the problem and still matches the oracle."""
    import gemm_mmbo_amd as G
    cid = _ring_ids(dtype)[0]
    bk = 16 if dtype == F32 else 32
    for (m, n, k, offs) in ((255, 256, 4 * bk, (0, 0, 0)), (256, 300, 4 * bk, (0, 0, 0)), (256, 256, 4 * bk + 8, (0, 0, 0)),
                            (256, 256, 4 * bk, (1, 0, 0))):
        p = U.Problem(dtype, 0, 0, m, n, k, 1.0, 0.0, seed=5, c_fill="nan")
        with pytest.raises(G.MmboError) as e:
            U.run_gpu(p, cid, offs)
        assert e.value.status == 5
        _run_and_check(p, -1, label="auto fallback", offsets=offs)
    p = U.Problem(dtype, 1, 0, 512, 512, 320, 1.0, 0.5, lda=1032, ldb=1040, ldc=520, seed=71)
    _run_and_check(p, cid, label="ring ld>dim")
    assert "DTL1" in G.config_info(dtype, G.select_config(dtype, 0, 0, 8192, 8192, 8192))["name"]


# ------------------------------------------------------------------ edges

@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 300, 7), (300, 1, 5), (31, 33, 2), (64, 64, 3), (5, 5, 1025),
                                   (129, 65, 64), (33, 257, 100)])
def test_small_and_degenerate_shapes(dtype, m, n, k):
    for ta in (0, 1):
        for tb in (0, 1):
            p = U.Problem(dtype, ta, tb, m, n, k, -1.0, 1.0, seed=m * 7 + n)   # the reference's alpha=-1, beta=1
            _run_and_check(p, label=f"{m}x{n}x{k} {'NT'[ta]}{'NT'[tb]}")


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_k_zero_scales_c_only(dtype):
    p = U.Problem(dtype, 0, 0, 70, 50, 0, 1.0, 0.5, seed=1)
    got = _run_and_check(p, label="k=0 beta=.5")
    p0 = U.Problem(dtype, 0, 0, 70, 50, 0, 1.0, 0.0, seed=1, c_fill="nan")
    got, _ = U.run_gpu(p0)
    assert np.all(got == 0)          # alpha * (empty sum), old NaN contents not read


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_leading_dimensions_larger_than_matrix(dtype):
    """run.sh's precedent: ldc = 44160 > M.  Padding rows of C must stay bit-identical."""
    for (ta, tb) in ((0, 0), (0, 1), (1, 0), (1, 1)):
        p = U.Problem(dtype, ta, tb, 384, 200, 384, -1.0, 1.0, lda=1000, ldb=777, ldc=44160 // 40, seed=6)
        _run_and_check(p, label="ld>dim")
        p = U.Problem(dtype, ta, tb, 100, 90, 80, 1.0, 0.0, lda=101, ldb=93, ldc=107, seed=7, c_fill="nan")
        _run_and_check(p, label="odd ld")


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_unaligned_pointers(dtype):
    """Device pointers offset by one element: no 128-bit access may be assumed aligned."""
    for offs in ((1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 3, 5)):
        p = U.Problem(dtype, 0, 0, 200, 136, 264, 1.5, 0.5, seed=8)
        _run_and_check(p, label=f"offsets {offs}", offsets=offs)
        p = U.Problem(dtype, 1, 1, 256, 128, 256, 1.0, 0.0, seed=9, c_fill="nan")
        _run_and_check(p, label=f"offsets {offs} TT", offsets=offs)


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_beta_zero_ignores_nan_and_inf_in_c(dtype):
    p = U.Problem(dtype, 0, 0, 300, 200, 128, 1.0, 0.0, seed=12, c_fill="nan")
    got, _ = U.run_gpu(p)
    assert np.all(np.isfinite(got.astype(np.float32)))
    p.C[:] = np.inf
    got, _ = U.run_gpu(p, 2 + 6 * 2)          # a split-K config: the reduction must not read C either
    assert np.all(np.isfinite(got.astype(np.float32)))
    U.check(p, got, "beta=0 inf")


def test_strided_batched_with_gaps_and_every_transpose():
    for dtype in (F32, F16):
        for (ta, tb) in ((0, 0), (0, 1), (1, 0), (1, 1)):
            m, n, k, batch = 96, 72, 150, 5
            p = U.Problem(dtype, ta, tb, m, n, k, 0.5, -1.0, batch=batch, seed=13,
                          strides=(m * k + 24, k * n + 8, m * n + 40))
            got = _run_and_check(p, label="batched gaps")
            # the 40-element gap between C matrices is untouched
            for b in range(batch):
                assert np.array_equal(got[b * p.sc + m * n:(b + 1) * p.sc].view(np.uint8),
                                      p.C[b * p.sc + m * n:(b + 1) * p.sc].view(np.uint8))


def test_batched_equals_looped_single_calls_bitwise():
    """Reference semantics (src/gemm/ref/Kernels.cpp:76-78,254): batch b is the same GEMM on offset pointers."""
    import torch
    import gemm_mmbo_amd as G
    m, n, k, batch = 256, 192, 320, 4
    p = U.Problem(F16, 1, 0, m, n, k, 1.0, 1.0, batch=batch, seed=14, dist="normal")
    cid = G.select_config(F16, 1, 0, m, n, k, batch)
    got, _ = U.run_gpu(p, cid)
    dA, dB = torch.from_numpy(p.A).cuda(), torch.from_numpy(p.B).cuda()
    dC = torch.from_numpy(p.C).cuda()
    for b in range(batch):
        G.gemm(F16, 1, 0, m, n, k, 1.0, dA.data_ptr() + 2 * b * p.sa, p.lda, dB.data_ptr() + 2 * b * p.sb, p.ldb,
               1.0, dC.data_ptr() + 2 * b * p.sc, p.ldc, cid)
    torch.cuda.synchronize()
    assert np.array_equal(dC.cpu().numpy().view(np.uint16), got.view(np.uint16))


def test_package_imported_before_torch_still_reaches_the_device():
    """A fresh process that touches the library before it imports torch: the Python layer must end up on the HIP runtime
    torch uses (the wheel ships its own copy; with the system's copy loaded first the library's calls found no device)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = ("import sys; sys.path.insert(0, %r)\n"
            "import gemm_mmbo_amd as G\n"
            "assert G.num_configs(G.F16) > 0\n"
            "import torch\n"
            "m = n = k = 256\n"
            "A = torch.ones(m * k, device='cuda', dtype=torch.float16); B = torch.ones(k * n, device='cuda', dtype=torch.float16)\n"
            "C = torch.zeros(m * n, device='cuda', dtype=torch.float16)\n"
            "G.gemm(G.F16, 0, 0, m, n, k, 1.0, A, m, B, k, 0.0, C, m)\n"
            "torch.cuda.synchronize()\n"
            "assert bool((C == k).all())\n"
            "print('ok')\n") % root
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), (r.stdout[-500:], r.stderr[-1500:])


def test_stream_probe_reports_a_plausible_rate_and_refuses_bad_sizes():
    """mmbo_probe_stream: a plain streaming kernel over given byte counts.  The rate it reports for a copy of 64 MiB
    lies between what any HBM part of this class sustains and the nominal 8 TB/s plus what the last-level cache adds;
    twice the bytes take longer; read-only and write-only runs work; sizes that are not whole 16-byte vectors are refused."""
    import gemm_mmbo_amd as G
    mib = 1 << 20
    t1 = G.probe_stream(64 * mib, 64 * mib, 20)
    t2 = G.probe_stream(256 * mib, 256 * mib, 10)
    assert 1.0e12 < 128 * mib / t1 < 16.0e12, t1
    assert t2 > 1.5 * t1
    assert G.probe_stream(64 * mib, 0, 10) > 0 and G.probe_stream(0, 64 * mib, 10) > 0
    assert G.probe_stream(96 * mib, 32 * mib, 10, in_place=True) > 0
    for args in ((24, 16, 1), (16, 8, 1), (0, 0, 1), (16, 16, 0), (16, 32, 1, True)):
        with pytest.raises(G.MmboError) as e:
            G.probe_stream(*args)
        assert e.value.status != 0


# ------------------------------------------------------------------ size-independent properties at full size

@pytest.mark.parametrize("dtype,size", [(F32, 4096), (F16, 8192)], ids=["f32-4096", "f16-8192"])
def test_identity_and_ones_closed_forms_full_size(dtype, size):
    """op(A) = I gives C = alpha*B exactly; all-ones operands give alpha*K exactly (K is a power of two,
    so every partial sum is representable): bitwise checks that need no oracle run."""
    import torch
    import gemm_mmbo_amd as G
    tdt = torch.float32 if dtype == F32 else torch.float16
    n = size
    eye = torch.eye(n, dtype=tdt, device="cuda")
    B = torch.from_numpy(O.fill_uniform(n * n, dtype, 21)).cuda()
    C = torch.full((n * n,), float("nan"), dtype=tdt, device="cuda")
    for (ta, tb) in ((0, 0), (1, 0)):
        G.gemm(dtype, ta, tb, n, n, n, 1.0, eye, n, B, n, 0.0, C, n)
        torch.cuda.synchronize()
        assert torch.equal(C, B)
    ones = torch.ones(n * n, dtype=tdt, device="cuda")
    G.gemm(dtype, 0, 1, n, n, n, 0.25, ones, n, ones, n, 0.0, C, n)
    torch.cuda.synchronize()
    assert torch.all(C == 0.25 * n)


def test_x16_c_whose_tile_span_passes_32_bit_offsets():
    """The whole-tile epilogue of the x16 kernels addresses C through a buffer descriptor with 32-bit offsets.  With
    ldc so large that one tile's span of C (256 columns x ldc x 2 bytes) passes 2 GiB the library must take the
    element-wise epilogue instead: same values, and nothing written outside the m x n window."""
    import torch
    import gemm_mmbo_amd as G
    m, n, k = 256, 256, 64
    ldc = (1 << 22) + 64                                  # 256 * ldc * 2 bytes > 2^31
    cid = _x16_ids(F16)[0]
    assert G.config_info(F16, cid)["macro_tile_n"] == 256
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    A = (torch.randn(m * k, device="cuda", generator=gen) * 0.1).half()
    B = (torch.randn(k * n, device="cuda", generator=gen) * 0.1).half()
    C = torch.zeros(ldc * n, device="cuda", dtype=torch.float16)
    Cv = C.view(n, ldc)
    C0 = (torch.rand(n, m, device="cuda", generator=gen) * 2 - 1).half()
    Cv[:, :m] = C0
    Cv[:, m:m + 16] = 7.0                                 # sentinels right below the window
    G.gemm(F16, 0, 0, m, n, k, 1.5, A, m, B, k, 0.5, C, ldc, cid)
    torch.cuda.synchronize()
    want = 1.5 * (B.view(n, k).float() @ A.view(k, m).float()) + 0.5 * C0.float()      # column-major C = row-major C^T
    got = Cv[:, :m].float()
    assert float((got - want).abs().max()) <= 2e-2 * float(want.abs().max())
    assert bool((Cv[:, m:m + 16] == 7.0).all()) and float(Cv[:, m + 16:].abs().max()) == 0.0
    del C, Cv
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_old_c_closed_form_where_c_leaves_with_the_streaming_hint(dtype):
    """8192 x 8192 x 4096 on the 256 x 256 tile is 1,024 tiles with k >= 4096: the shape class whose C is stored with the
    non-temporal hint.  With beta != 0 and alpha != 1 on all-ones operands every result is 0.25*K + 0.5*C0, exact for
    small even integers in C0 -- a bitwise check of that store sequence (and of the old C fetched ahead of it) without an
    oracle run; the plain-store copies of the same sequences are what every smaller test exercises."""
    import torch
    import gemm_mmbo_amd as G
    tdt = torch.float32 if dtype == F32 else torch.float16
    m = n = 8192
    k = 4096
    cid = G.select_config(dtype, 0, 0, m, n, k)
    assert "MT256x256" in G.config_info(dtype, cid)["name"]
    ones_a = torch.ones(m * k, dtype=tdt, device="cuda")
    ones_b = torch.ones(k * n, dtype=tdt, device="cuda")
    C0 = (torch.arange(m * n, device="cuda", dtype=torch.int64) % 32 * 2).to(tdt)
    want = 0.25 * k + 0.5 * C0
    for (ta, tb) in ((0, 0), (0, 1)):
        C = C0.clone()
        G.gemm(dtype, ta, tb, m, n, k, 0.25, ones_a, m if not ta else k, ones_b, k if not tb else n, 0.5, C, m)
        torch.cuda.synchronize()
        assert torch.equal(C, want), (ta, tb)


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_linearity_in_alpha_and_beta(dtype):
    """gemm(2a, 2b) == 2 * gemm(a, b) bit for bit: scaling by two is exact in binary floating point
    (outside the fp16 subnormal range, where the doubled value has one more significant bit to round)."""
    p = U.Problem(dtype, 0, 1, 1000, 600, 700, 0.75, -0.5, seed=30, dist="normal")
    g1, _ = U.run_gpu(p)
    p2 = U.Problem(dtype, 0, 1, 1000, 600, 700, 1.5, -1.0, seed=30, dist="normal")
    g2, _ = U.run_gpu(p2)
    doubled = (g1.astype(np.float32) * 2).astype(g1.dtype)
    normal = np.abs(g2.astype(np.float32)) >= 2.0 ** -13
    assert normal.mean() > 0.99
    assert np.array_equal(doubled[normal], g2[normal])


def test_repeatable_bitwise_including_split_k():
    """Split-K partials are reduced in a fixed order: two runs give identical bits."""
    import gemm_mmbo_amd as G
    for dtype in (F32, F16):
        p = U.Problem(dtype, 0, 0, 4096, 128, 4096, 1.0, 0.0, seed=31, c_fill="nan")
        for cid in (G.select_config(dtype, 0, 0, 4096, 128, 4096), 2 + 6 * 3):
            a, _ = U.run_gpu(p, cid)
            b, _ = U.run_gpu(p, cid)
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))


def test_split_k_every_family_ragged_and_batched():
    """GlobalSplitU > 1 in every kernel family: whole tiles, edge tiles with m % 4 != 0 (the partial sums are then stored
    and added element by element) and with m % 4 == 0, uneven splits of k, batches, beta; one call after the other on
    one stream, so on one workspace."""
    import gemm_mmbo_amd as G
    ran = 0
    for dtype in (F32, F16):
        for cid in range(G.num_configs(dtype)):
            d = G.config_info(dtype, cid)
            name, sp, bm, bn, bk = d["name"], d["split_k"], d["macro_tile_m"], d["macro_tile_n"], d["depth_u"]
            if sp == 1 or bm > 128 and sp > 4:
                continue
            ring_only = "DTL1" in name and "_ACC" not in name
            ta, tb = cid % 2, (cid // 2) % 2
            cases = [(ta, tb, 2 * bm, 3 * bn, sp * 3 * bk, 1.0, 0.0, 1, 0), (tb, ta, bm, 2 * bn, sp * 2 * bk, -1.5, 0.5, 3, 4)]
            if not ring_only:
                cases += [(ta, tb, 2 * bm - 3, bn + 5, sp * 2 * bk + bk + 7, 1.0, 0.0, 1, 1),
                          (1, 0, bm + 12, 2 * bn - 1, sp * 4 * bk - 3, 0.5, 1.0, 2, 0)]
            for (a, b, m, n, k, alpha, beta, batch, pad) in cases:
                p = U.Problem(dtype, a, b, m, n, k, alpha, beta, ldc=m + pad, batch=batch, seed=70 + cid,
                              dist="normal" if dtype == F16 else "uniform", c_fill="uniform" if beta else "nan")
                _run_and_check(p, cid, label=f"config {cid} {name} {m}x{n}x{k} b{batch}")
                ran += 1
    assert ran >= 100


def test_split_k_on_two_streams_at_the_same_time():
    """Every stream has its own split-K workspace: GEMMs with GlobalSplitU > 1 queued on two streams without any
    synchronisation between them (the reference's launcher is not re-entrant at all, src/gemm/driver.h:41)."""
    import torch
    import gemm_mmbo_amd as G
    probs = [U.Problem(F16, 0, 0, 4096, 128, 4096, 1.0, 0.0, seed=81, c_fill="nan"),
             U.Problem(F32, 0, 0, 128, 4096, 2048, 1.0, 0.5, seed=82, c_fill="uniform")]
    cids = [G.select_config(p.dtype, 0, 0, p.m, p.n, p.k) for p in probs]
    for p, cid in zip(probs, cids):
        assert G.config_info(p.dtype, cid)["split_k"] > 1
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    tdt = {F32: torch.float32, F16: torch.float16}
    dev = [[torch.from_numpy(x).cuda() for x in (p.A, p.B, p.C)] for p in probs]
    outs = [[torch.empty_like(d[2]) for _ in range(6)] for d in dev]
    torch.cuda.synchronize()
    for rep in range(6):
        for i, (p, cid) in enumerate(zip(probs, cids)):
            with torch.cuda.stream(streams[i]):
                outs[i][rep].copy_(dev[i][2], non_blocking=True)
                G.gemm(p.dtype, 0, 0, p.m, p.n, p.k, p.alpha, dev[i][0], p.lda, dev[i][1], p.ldb, p.beta, outs[i][rep], p.ldc,
                       cid, streams[i])
    torch.cuda.synchronize()
    for i, p in enumerate(probs):
        first = outs[i][0].cpu().numpy()
        U.check(p, first, f"stream {i}")
        for rep in range(1, 6):
            assert np.array_equal(first.view(np.uint8), outs[i][rep].cpu().numpy().view(np.uint8))


def test_split_k_workspaces_stay_bounded_over_many_short_lived_streams():
    """The library keeps one split-K workspace per stream, at most eight per device: a process that keeps creating and
    destroying streams does not keep one buffer per stream handle it ever used (the launcher this replaces never frees
    anything, src/gemm/driver.h:41).  Results stay those of the first call bit for bit; a stream's slot can be handed
    back by name; release_workspace empties the table."""
    import torch
    import gemm_mmbo_amd as G
    G.release_workspace()
    assert G.workspace_info() == (0, 0)
    p = U.Problem(F16, 0, 0, 1024, 128, 2048, 1.0, 0.0, seed=83, c_fill="nan")
    cid = [c for c in range(G.num_configs(F16)) if G.config_info(F16, c)["split_k"] == 4 and G.config_info(F16, c)["macro_tile_m"] == 64][0]
    dA, dB = torch.from_numpy(p.A).cuda(), torch.from_numpy(p.B).cuda()
    first = None
    most = 0
    for i in range(64):
        st = torch.cuda.Stream()
        dC = torch.from_numpy(p.C).cuda()
        st.wait_stream(torch.cuda.current_stream())
        G.gemm(F16, 0, 0, p.m, p.n, p.k, 1.0, dA, p.lda, dB, p.ldb, 0.0, dC, p.ldc, cid, st)
        st.synchronize()
        out = dC.cpu().numpy()
        if first is None:
            first = out
            U.check(p, first, "first short-lived stream")
        else:
            assert np.array_equal(first.view(np.uint8), out.view(np.uint8)), i
        slots, nbytes = G.workspace_info()
        most = max(most, slots)
        assert 1 <= slots <= 8 and nbytes >= 4 * p.m * p.n * 4 * slots, (i, slots, nbytes)
        if i % 16 == 5:
            G.release_stream_workspace(st)              # hand this stream's slot back before the stream goes away
            assert G.workspace_info()[0] == slots - 1
        del st
    assert most >= 2                                    # (distinct stream handles did get distinct slots)
    G.release_stream_workspace(torch.cuda.Stream())     # a stream without a workspace: not an error
    G.release_workspace()
    assert G.workspace_info() == (0, 0)


def test_every_shape_of_the_tuned_table_under_the_automatic_pick():
    """Each exact-shape row of csrc/tuned_table.hpp names a config by id: run the row's shape through MMBO_CONFIG_AUTO
    against the oracle, so a row that points at a config that cannot take its shape, or computes it wrongly, is found.
    (The two 8192^3 rows are test_cfg3_*; fp64 rows are in tests/test_dgemm_gpu.py.)"""
    import os
    import re
    import gemm_mmbo_amd as G
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "gemm_mmbo_amd", "csrc", "tuned_table.hpp")).read()
    rows = re.findall(r"^\s*\{(\d), (\d), (\d), (\d+), (\d+), (\d+), (\d+), (\w+)\((\d), (\d+)\)", text, flags=re.M)
    assert len(rows) >= 15
    ran = 0
    for (dtype, ta, tb, m, n, k, batch, fam, tile, split) in rows:
        dtype, ta, tb, m, n, k, batch, tile, split = (int(v) for v in (dtype, ta, tb, m, n, k, batch, tile, split))
        cid = G.select_config(dtype, ta, tb, m, n, k, batch)
        d = G.config_info(dtype, cid)
        assert d["split_k"] == split and ("_ACC" in d["name"]) == (fam == "x16_id"), (d["name"], fam, tile, split)
        if m * n * k >= 8192 ** 3:
            continue
        p = U.Problem(dtype, ta, tb, m, n, k, 1.0, 0.0, batch=batch, seed=60 + ran, dist="normal" if dtype == F16 else "uniform",
                      c_fill="nan")
        _run_and_check(p, -1, label=f"tuned row {dtype} {ta}{tb} {m}x{n}x{k} b{batch}")
        ran += 1
    assert ran >= 13


def test_async_on_user_stream():
    """The launch goes to the caller's stream (reference: null stream only, src/gemm/common.h:12)."""
    import torch
    import gemm_mmbo_amd as G
    p = U.Problem(F32, 0, 0, 512, 512, 512, 1.0, 0.0, seed=32, c_fill="nan")
    s = torch.cuda.Stream()
    dA, dB, dC = (torch.from_numpy(x).cuda() for x in (p.A, p.B, p.C))
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        G.gemm(F32, 0, 0, 512, 512, 512, 1.0, dA, 512, dB, 512, 0.0, dC, 512, -1, s)
    s.synchronize()
    U.check(p, dC.cpu().numpy(), "stream")


# ------------------------------------------------------------------ C++ harness shaped like the reference's

def _harness(path, *args):
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, path)
    if not os.path.exists(exe):
        pytest.skip(f"{path} not built (run __graft_entry__.build())")
    return subprocess.run([exe, *map(str, args)], capture_output=True, text=True, timeout=280)


def test_cpp_verify_main_reference_defaults_and_failure_exit_code():
    """tests/harness/test: the reference's test.cc flow (NT, alpha=-1, beta=1, M=44160 N=2048 K=384) through the
    C++ front-ends; exit status 0 only when every element matches the oracle."""
    r = _harness("tests/harness/test")
    assert r.returncode == 0 and "result check passed" in r.stdout, r.stdout + r.stderr
    r = _harness("tests/harness/test", 1023, 777, 513, "N", "N", "h", 1, 0)
    assert r.returncode == 0 and "result check passed" in r.stdout, r.stdout + r.stderr
    r = _harness("tests/harness/test", 64, 64, 64, "N", "N", "s", 1, 0, 999)      # bad kernelId: error, not exit(0)
    assert r.returncode != 0


def test_cpp_benchmark_main_modes():
    """gemm_mmbo_amd/host/benchmark: `type M N K lda ldb ldc` like the reference's; type 1 sweeps every config."""
    r = _harness("gemm_mmbo_amd/host/benchmark", 0, 1024, 1024, 1024, 1024, 1024, 1024, "N", "N", "s", 1, 1, 0)
    assert r.returncode == 0 and "sgemm(NN): kernel" in r.stdout, r.stdout + r.stderr
    r = _harness("gemm_mmbo_amd/host/benchmark", 1, 512, 512, 512, 512, 512, 512, "T", "N", "h", 4, 1, 1)
    assert r.returncode == 0 and "hgemm(TN): kernel" in r.stdout, r.stdout + r.stderr
    r = _harness("gemm_mmbo_amd/host/benchmark", 0, 64, 64)
    assert r.returncode == 2


def test_report_driver_writes_parsable_records(tmp_path):
    """python -m gemm_mmbo_amd.report (the sweep driver behind host/run.sh report; reference: src/gemm/run.sh:1-5 over
    src/gemm/benchmark.cc:89-109): two small shapes, JSON lines on stdout and in a file, a CSV with the same rows, the
    roofline arithmetic, the fp64 cross-check and the profiling commands."""
    import csv
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    jpath, cpath = str(tmp_path / "r.jsonl"), str(tmp_path / "r.csv")
    r = subprocess.run([sys.executable, "-m", "gemm_mmbo_amd.report", "shapes", "h,T,N,512,384,1024,2,1,0.5", "s,N,N,257,131,1000",
                        "--json", jpath, "--csv", cpath, "--reps", "5", "--print-profile-commands"],
                       cwd=root, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stderr[-2000:]
    recs = [json.loads(l) for l in r.stdout.splitlines() if l.startswith("{")]
    assert recs == [json.loads(l) for l in open(jpath)]
    rows = list(csv.DictReader(open(cpath)))
    assert len(recs) == 2 and len(rows) == 2
    h, s = recs
    assert (h["dtype"], h["transA"], h["transB"], h["m"], h["n"], h["k"], h["batch"], h["beta"]) == ("h", "T", "N", 512, 384, 1024, 2, 0.5)
    assert h["algorithmic_bytes"] == 2 * (512 * 1024 + 1024 * 384 + 2 * 512 * 384) * 2          # beta != 0: C counted twice
    assert s["algorithmic_bytes"] == (257 * 1000 + 1000 * 131 + 257 * 131) * 4
    for rec, row, limit in ((h, rows[0], 2e-2), (s, rows[1], 1e-5 * 1000 ** 0.5)):
        assert 0 < rec["gpu_ms_min"] <= rec["gpu_ms_median"] <= rec["gpu_ms_max"]
        flops = 2.0 * rec["m"] * rec["n"] * rec["k"] * rec["batch"]
        assert abs(rec["tflops"] - flops / rec["gpu_ms_median"] * 1e-9) <= 0.02 * rec["tflops"] + 0.01
        assert rec["bound"] in ("mfma", "hbm") and 0 < rec["frac_of_bound"] <= 1.0 and 0 < rec["frac_of_peak"] <= 1.0
        assert rec["frac_of_bound"] >= rec["frac_of_peak"]
        assert rec["max_rel_err"] <= limit and "fp64" in rec["checked_against"]
        assert rec["config"] and row["config"] == rec["config"] and float(row["gpu_ms_median"]) == rec["gpu_ms_median"]
    cmds = [l for l in r.stdout.splitlines() if l.startswith("# ")]
    assert len(cmds) == 8 and all("rocprofv3" in c and " -- python3 -m gemm_mmbo_amd.report shapes " in c for c in cmds)
    assert sum("--kernel-trace --stats" in c for c in cmds) == 2 and sum("FETCH_SIZE" in c for c in cmds) == 2
    bad = subprocess.run([sys.executable, "-m", "gemm_mmbo_amd.report", "shapes", "q,N,N,1,1,1"], cwd=root, capture_output=True, text=True)
    assert bad.returncode != 0


def test_mfma_ceiling_probe_reports_plausible_numbers():
    """mmbo_probe_mfma_ceiling: a register-only MFMA loop cannot beat the published peaks, and constant operands
    are never slower than random ones (the chip clocks down under power)."""
    import gemm_mmbo_amd as G
    ones16, mhz1 = G.probe_mfma_ceiling(F16, False)
    rnd16, mhz2 = G.probe_mfma_ceiling(F16, True)
    ones32, mhz3 = G.probe_mfma_ceiling(F32, False)
    assert 500 < rnd16 <= ones16 * 1.05 and ones16 < 2600
    assert 50 < ones32 < 165
    for mhz in (mhz1, mhz2, mhz3):
        assert 500 < mhz < 2600


def test_offline_tuner_emits_table_rows_for_small_shapes():
    """gemm_mmbo_amd/tune.py times every config id and prints rows in tuned_table.hpp's syntax."""
    import io
    import re

    import gemm_mmbo_amd as G
    from gemm_mmbo_amd import tune
    out = io.StringIO()
    shapes = [(0, 0, 1, 256, 256, 128, 1, -1.0, 1.0), (1, 1, 0, 300, 200, 96, 2, 1.0, 0.0), (2, 0, 1, 256, 128, 64, 1, -1.0, 1.0)]
    rows = tune.tune(shapes, out)
    assert len(rows) == 3
    for row, s in zip(rows, shapes):
        m = re.match(r"\s*\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+|ring_id\(\d, \d+\)|x16_id\(\d, \d+\)), ([\d.]+)f\},", row)
        assert m and tuple(int(x) for x in m.groups()[:7]) == s[:7], row
        assert float(m.group(9)) > 0
        if m.group(8).isdigit():
            assert 0 <= int(m.group(8)) < G.num_configs(s[0])
    assert "FAILS" not in out.getvalue()
    # the table syntax names the same config the id does
    for dtype in (0, 1):
        for cid in range(G.num_configs(dtype)):
            d = G.config_info(dtype, cid)
            t = tune.table_id(G, dtype, cid)
            if "DTL1" not in d["name"]:
                assert t == str(cid)
            else:
                fam, tile, split = re.match(r"(\w+)\((\d), (\d+)\)", t).groups()
                assert (fam == "x16_id") == ("_ACC" in d["name"]) and int(split) == d["split_k"]
                base = 50 if fam == "x16_id" else 30
                ntile = 8 if fam == "x16_id" else 4
                assert cid == base + int(tile) + ntile * [1, 2, 4, 8, 16].index(int(split))


def test_automatic_pick_never_fails_on_its_own_choice():
    """MMBO_CONFIG_AUTO picks from the shape; the ring kernels also need 16-byte aligned A and B, every direct-to-LDS
    kernel a tile span below 2 GiB.  With operands that do not qualify the call must still succeed (the x16 twin of the
    pick, or the general kernel), while naming the config explicitly is refused."""
    import torch

    import gemm_mmbo_amd as G
    # a whole-tile fp32 shape whose pick is a ring config, A (then B) one element off 16-byte alignment
    m, n, k = 1024, 1024, 512
    cid = G.select_config(F32, 0, 0, m, n, k)
    name = G.config_info(F32, cid)["name"]
    assert "DTL1" in name and "MFMA16x16" not in name
    for offs in ((1, 0, 0), (0, 1, 0)):
        p = U.Problem(F32, 0, 0, m, n, k, 1.0, 0.0, seed=90, c_fill="nan")
        with pytest.raises(G.MmboError) as e:
            U.run_gpu(p, cid, offs)
        assert e.value.status == 5
        _run_and_check(p, -1, label=f"auto with unaligned operand {offs}", offsets=offs)
    # an fp16 pick that is an x16 config takes unaligned operands by name
    m, n, k = 2048, 2048, 1024
    cid = G.select_config(F16, 0, 0, m, n, k)
    assert "MFMA16x16" in G.config_info(F16, cid)["name"]
    for offs in ((1, 0, 0), (0, 1, 0)):
        p = U.Problem(F16, 0, 0, m, n, k, 1.0, 0.0, seed=90, dist="normal", c_fill="nan")
        _run_and_check(p, cid, label=f"x16 by name with unaligned operand {offs}", offsets=offs)
    # a leading dimension so large that the rows of A^T under the picked tile span more than 2 GiB (only the first k rows of
    # each stored column are used): the pick itself is refused by name, the automatic path moves to a tile that fits
    m, n, k = 64, 16384, 100
    pick = G.select_config(F32, 1, 0, m, n, k)
    tm = G.config_info(F32, pick)["macro_tile_m"]
    assert tm >= 64                                             # a smaller tile exists to fall back to
    lda = 2 ** 31 // (tm * 4) + 4096                            # tm rows of A^T span just over 2 GiB (A: 2.1 GB at tm = 64)
    rng = np.random.default_rng(91)
    hA = rng.uniform(-1, 1, (m, k)).astype(np.float32)          # row i = the k values of column i of the stored k x m matrix
    hB = rng.uniform(-1, 1, (n, k)).astype(np.float32)          # B stored k x n, column j = hB[j]
    dA = torch.zeros(m * lda, dtype=torch.float32, device="cuda")
    dA.view(m, lda)[:, :k] = torch.from_numpy(hA).cuda()
    dB = torch.from_numpy(hB.reshape(-1)).cuda()
    dC = torch.full((m * n,), float("nan"), dtype=torch.float32, device="cuda")
    with pytest.raises(G.MmboError) as e:
        G.gemm(F32, 1, 0, m, n, k, 1.0, dA, lda, dB, k, 0.0, dC, m, pick)
    assert e.value.status == 5
    G.gemm(F32, 1, 0, m, n, k, 1.0, dA, lda, dB, k, 0.0, dC, m, -1)
    torch.cuda.synchronize()
    want = hA.astype(np.float64) @ hB.astype(np.float64).T
    got = dC.cpu().numpy().reshape((m, n), order="F")
    assert np.max(np.abs(got - want)) <= U.tol(F32, k) * max(np.max(np.abs(want)), 1.0)


@pytest.mark.parametrize("dtype", [F32, F16], ids=NAMES.get)
def test_large_ragged_problems_through_the_automatic_pick(dtype):
    """MMBO_CONFIG_AUTO on large shapes that are not made of whole tiles: one launch of the x16 kernel (edge tiles, a
    zero-filled last slice of k, contiguous dimensions that end inside a 16-byte group, columns that start off 16-byte
    boundaries).  Against the oracle, with beta, ld > dim (padding rows untouched), every transpose, batches,
    bit-identical on repetition."""
    import gemm_mmbo_amd as G
    dist = "normal" if dtype == F16 else "uniform"
    cases = [(0, 0, 2100, 2300, 2560, 1.0, 0.0, {}), (0, 1, 2100, 2048, 2560, -1.0, 1.0, {}), (1, 0, 2048, 2100, 2560, 1.5, 0.5, {}),
             (1, 1, 1500, 1900, 4096, 1.0, 0.0, {}), (0, 0, 2100, 2300, 2560, 1.0, 1.0, {"lda": 2104, "ldb": 2568, "ldc": 2111}),
             (0, 1, 1200, 1300, 2304, 1.0, 0.5, {"batch": 3}),
             (0, 1, 2306, 2101, 2560, 1.5, 0.5, {"lda": 2312, "ldb": 2104, "ldc": 2307}),
             (0, 0, 2102, 2302, 2576, 1.0, 0.5, {"lda": 2104, "ldb": 2576}),
             (0, 0, 2104, 2304, 2568, 1.0, 0.0, {}), (1, 0, 2048, 2048, 3000, -1.0, 1.0, {}), (0, 1, 2048, 2304, 2570, 1.5, 0.5, {}),
             (1, 1, 2056, 2048, 1208, 1.0, 0.5, {"batch": 2}), (1, 0, 2051, 2049, 2563, 1.0, 0.0, {"lda": 2568, "ldb": 2568})]
    for (ta, tb, m, n, k, alpha, beta, kw) in cases:
        p = U.Problem(dtype, ta, tb, m, n, k, alpha, beta, seed=500 + m + n, dist=dist, c_fill="uniform" if beta else "nan", **kw)
        got = _run_and_check(p, -1, label=f"ragged {'NT'[ta]}{'NT'[tb]} {m}x{n}x{k} {kw}")
        again, _ = U.run_gpu(p, -1)
        assert np.array_equal(got.view(U.BITS[dtype]), again.view(U.BITS[dtype]))
    # unaligned A
    p = U.Problem(dtype, 0, 0, 2100, 2300, 2560, 1.0, 0.0, seed=77, dist=dist, c_fill="nan")
    _run_and_check(p, -1, label="ragged, unaligned A", offsets=(1, 0, 0))


def test_random_shapes_paddings_and_configs_against_the_oracle():
    """240 seeded random problems: both element types, every transpose, m, n, k from 1 up (a few thousand for some),
    leading dimensions padded, tight or off 16-byte alignment, batches, alpha/beta variants, through MMBO_CONFIG_AUTO
    or a random x16 config id.  A named config may refuse the problem (status 5: a contiguous dimension shorter than
    one 16-byte load); whatever runs must match the oracle
    and leave the padding rows and the guard words behind C untouched."""
    import random

    import gemm_mmbo_amd as G
    rnd = random.Random(20240607)
    x16 = {dt: _x16_ids(dt) for dt in (F32, F16)}
    ran = refused = 0
    for it in range(240):
        dt = rnd.choice((F32, F16))
        ta, tb = rnd.randint(0, 1), rnd.randint(0, 1)
        g = 4 if dt == F32 else 8
        big = rnd.random() < 0.15
        m, n = rnd.randint(1, 4400 if big else 700), rnd.randint(1, 4400 if big else 700)
        k = rnd.randint(1, 80 if big else 1500)
        batch = 1 if big else rnd.choice((1, 1, 1, 2, 3))
        ar, br = U.stored_shape(ta, m, k)[0], U.stored_shape(tb, k, n)[0]
        pad = rnd.choice((0, 0, g, 3 * g))
        if rnd.random() < 0.85:
            lda, ldb = -(-ar // g) * g + pad, -(-br // g) * g + pad
        else:
            lda, ldb = ar + rnd.randint(0, 3), br + rnd.randint(0, 3)
        alpha, beta = rnd.choice((1.0, -1.0, 1.5)), rnd.choice((0.0, 0.0, 1.0, 0.5))
        cfg = -1 if rnd.random() < 0.5 else rnd.choice(x16[dt])
        p = U.Problem(dt, ta, tb, m, n, k, alpha, beta, lda=lda, ldb=ldb, ldc=m + rnd.choice((0, 0, 1, 5)), batch=batch,
                      seed=1000 + it, dist="normal" if dt == F16 else "uniform", c_fill="uniform" if beta else "nan")
        label = f"case {it}: {NAMES[dt]} {'NT'[ta]}{'NT'[tb]} {m}x{n}x{k} ld {lda},{ldb},{p.ldc} b{batch} cfg {cfg}"
        try:
            got, guard = U.run_gpu(p, cfg)
        except G.MmboError as e:
            assert cfg >= 0 and e.status == 5, label
            refused += 1
            continue
        U.check(p, got, label)
        assert np.all(guard == 0), label
        ran += 1
    assert ran >= 200
