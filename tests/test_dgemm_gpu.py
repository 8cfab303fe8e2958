"""Parity of the fp64 kernels (v_mfma_f64_16x16x4_f64) with the oracle, through the C ABI, on a real MI355X.

fp64 is the reference's own element type: naive_dgemm / dgemm_NT (src/gemm/gemm.h:4-5,47-48), alpha = -1,
beta = 1, the HPL trailing-update shape 44160 x 2048 x 384 with ldc >= M (src/gemm/test.cc:20-21,
src/gemm/run.sh:2-5).  Tolerance (tests/util.py): <= 2e-15 * sqrt(K) relative to max(|exact|, rms(exact));
integer-valued inputs must come out bit-exact.
"""
import numpy as np
import pytest

import util as U
from oracle import oracle as O

pytestmark = pytest.mark.gpu

F64 = U.F64


def _run_and_check(p, config_id=-1, label="", offsets=(0, 0, 0)):
    got, guard = U.run_gpu(p, config_id, offsets)
    rel = U.check(p, got, label)
    assert np.all(guard == 0), "wrote past the end of C"
    return got, rel


def test_reference_workload_hpl_shape_nt_alpha_minus1_beta1():
    """The reference's test.cc defaults; ldc > M as in run.sh (padding rows must stay bit-identical)."""
    import gemm_mmbo_amd as G
    m, n, k = 44160, 2048, 384
    p = U.Problem(F64, 0, 1, m, n, k, -1.0, 1.0, ldc=m + 64, seed=44160)
    _run_and_check(p, label="HPL NT")
    # and through the reference's own entry-point name
    import torch
    dA, dB, dC = (torch.from_numpy(x).cuda() for x in (p.A, p.B, p.C))
    G.naive_dgemm(m, n, k, -1.0, dA, p.lda, dB, p.ldb, 1.0, dC, p.ldc)
    torch.cuda.synchronize()
    U.check(p, dC.cpu().numpy(), "naive_dgemm")


@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_every_config_every_transpose_ragged(ta, tb):
    import gemm_mmbo_amd as G
    for cid in range(G.num_configs(F64)):
        p = U.Problem(F64, ta, tb, 333, 217, 150, 1.5, 0.5, seed=100 + cid)
        _run_and_check(p, cid, f"cfg {cid} ragged {'NT'[ta]}{'NT'[tb]}")
        p = U.Problem(F64, ta, tb, 512, 256, 256, 1.0, 0.0, seed=200 + cid, c_fill="nan")
        _run_and_check(p, cid, f"cfg {cid} interior {'NT'[ta]}{'NT'[tb]}")


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 300, 7), (300, 1, 5), (15, 17, 2), (64, 64, 3), (5, 5, 1025),
                                   (129, 65, 64), (33, 257, 100)])
def test_small_and_degenerate_shapes(m, n, k):
    for ta in (0, 1):
        for tb in (0, 1):
            p = U.Problem(F64, ta, tb, m, n, k, -1.0, 1.0, seed=m * 7 + n)
            _run_and_check(p, label=f"{m}x{n}x{k} {'NT'[ta]}{'NT'[tb]}")


def test_k_zero_scales_c_only():
    p = U.Problem(F64, 0, 0, 70, 50, 0, 1.0, 0.5, seed=1)
    _run_and_check(p, label="k=0 beta=.5")
    p0 = U.Problem(F64, 0, 0, 70, 50, 0, 1.0, 0.0, seed=1, c_fill="nan")
    got, _ = U.run_gpu(p0)
    assert np.all(got == 0)


def test_leading_dimensions_odd_and_unaligned_pointers():
    for (ta, tb) in ((0, 0), (0, 1), (1, 0), (1, 1)):
        p = U.Problem(F64, ta, tb, 100, 90, 80, 1.0, 0.0, lda=101, ldb=93, ldc=107, seed=7, c_fill="nan")
        _run_and_check(p, label="odd ld")
    for offs in ((1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 3, 5)):
        p = U.Problem(F64, 0, 1, 200, 136, 264, 1.5, 0.5, seed=8)
        _run_and_check(p, label=f"offsets {offs}", offsets=offs)


def test_beta_zero_ignores_nan_in_c():
    p = U.Problem(F64, 0, 1, 300, 200, 128, 1.0, 0.0, seed=12, c_fill="nan")
    got, _ = U.run_gpu(p)
    assert np.all(np.isfinite(got))
    U.check(p, got, "beta=0 over NaN")


def test_integer_inputs_are_bit_exact():
    """Small integers: every product and partial sum is exact in fp64, so any summation order gives the same bits."""
    import torch

    import gemm_mmbo_amd as G
    m, n, k = 640, 384, 512
    rng = np.random.default_rng(5)
    A = rng.integers(-9, 10, (m, k)).astype(np.float64)
    B = rng.integers(-9, 10, (n, k)).astype(np.float64)          # used transposed
    C = rng.integers(-9, 10, (m, n)).astype(np.float64)
    want = -(A @ B.T) + C
    dA, dB, dC = (torch.from_numpy(np.asfortranarray(x).reshape(-1, order="F")).cuda() for x in (A, B, C))
    for cid in range(G.num_configs(F64)):
        dCc = dC.clone()
        G.dgemm_NT(m, n, k, -1.0, dA, m, dB, n, 1.0, dCc, m, cid)
        torch.cuda.synchronize()
        assert np.array_equal(dCc.cpu().numpy().reshape((m, n), order="F"), want), f"config {cid}"


def test_strided_batched_equals_looped_calls_bitwise():
    import torch

    import gemm_mmbo_amd as G
    m, n, k, batch = 96, 80, 72, 5
    p = U.Problem(F64, 1, 0, m, n, k, 1.0, 1.0, batch=batch, seed=31, strides=(k * m + 6, k * n + 2, m * n + 10))
    got, _ = _run_and_check(p, label="batched TN")
    dA, dB, dC = (torch.from_numpy(x).cuda() for x in (p.A, p.B, p.C))
    for b in range(batch):
        G.dgemm_TN(m, n, k, 1.0, dA.data_ptr() + 8 * b * p.sa, p.lda, dB.data_ptr() + 8 * b * p.sb, p.ldb, 1.0,
                   dC.data_ptr() + 8 * b * p.sc, p.ldc)
    torch.cuda.synchronize()
    assert np.array_equal(dC.cpu().numpy().view(np.uint64), got.view(np.uint64))


def test_large_square_and_probe():
    """4096^3 NN (K large enough for the rounding bound to matter) and the fp64 MFMA ceiling probe."""
    import gemm_mmbo_amd as G
    p = U.Problem(F64, 0, 0, 4096, 4096, 4096, 1.0, 0.0, seed=64, c_fill="nan")
    _run_and_check(p, label="4096^3")
    ones, mhz1 = G.probe_mfma_ceiling(F64, False)
    rnd, mhz2 = G.probe_mfma_ceiling(F64, True)
    assert 20 < rnd <= ones * 1.05 and ones < 85           # published fp64 matrix peak: 78.6 TFLOP/s
    assert 500 < mhz1 < 2600 and 500 < mhz2 < 2600
