"""Pins the CPU oracle (oracle/host_gemm.c) before anything is compared against it.

Each check is chosen so that a plausible mistake in the oracle -- a transposed operand, a dropped beta
term, a wrong leading dimension, a rounding-mode slip -- fails at least one of them.  None of these
tests needs a GPU.
"""
import os
import subprocess

import numpy as np
import pytest

from oracle import oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
F32, F16, F64 = O.F32, O.F16, O.F64


# ------------------------------------------------------------------ work-group remap

def test_wg_remap_matches_reference_golden_file():
    """All 29,440 (wg0, wg1) -> (new0, new1) pairs of the reference's src/gemm/ref/res (460 x 64 grid, WGM 8)."""
    gold = np.load(os.path.join(GOLD, "wg_remap_460x64_wgm8.npy")).astype(np.int64)
    assert gold.shape == (460 * 64, 4)
    for wg0, wg1, e0, e1 in gold:
        assert O.wg_remap(int(wg0), int(wg1), 460, 64, 8) == (int(e0), int(e1))


def test_wg_remap_matches_reference_binary_when_built():
    """oracle/_ref/map_ref is the reference's own map.cpp compiled by oracle/Makefile; its output must be
    the golden file's content and the oracle's."""
    exe = os.path.join(os.path.dirname(GOLD), "..", "oracle", "_ref", "map_ref")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/map_ref not built (reference tree absent at build time)")
    out = subprocess.run([exe], capture_output=True, text=True, check=True).stdout.splitlines()
    assert out[-1].strip() == "finished check"
    gold = np.load(os.path.join(GOLD, "wg_remap_460x64_wgm8.npy"))
    import re
    pat = re.compile(r"\((\d+),\s*(\d+)\)--->\s*\((\d+),\s*(\d+)\)")
    got = np.array([[int(x) for x in pat.match(l).groups()] for l in out[:-1]], dtype=np.int16)
    assert np.array_equal(got, gold)


@pytest.mark.parametrize("nwg0,nwg1,wgm", [(460, 64, 8), (7, 13, 8), (32, 32, 8), (5, 3, 8), (16, 9, 4), (3, 17, 1)])
def test_wg_remap_is_a_bijection(nwg0, nwg1, wgm):
    """Every tile is visited exactly once, including grids whose width is not a multiple of WGM
    (the reference's golden grid, 64 = 8*8, never exercises the partial trailing block)."""
    seen = set()
    for wg1 in range(nwg1):
        for wg0 in range(nwg0):
            a, b = O.wg_remap(wg0, wg1, nwg0, nwg1, wgm)
            assert 0 <= a < nwg0 and 0 <= b < nwg1
            seen.add((a, b))
    assert len(seen) == nwg0 * nwg1


# ------------------------------------------------------------------ fp16 conversion

def test_f16_to_f32_every_bit_pattern():
    allh = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, dtype=np.float32)
    O.lib().oracle_f16_to_f32_array(O._ptr(allh), O._ptr(out), 65536)
    want = allh.view(np.float16).astype(np.float32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_round_to_nearest_even():
    rng = np.random.default_rng(1)
    halfs = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    finite = halfs[np.isfinite(halfs)]
    mids = ((finite.astype(np.float64) + np.roll(finite, 1).astype(np.float64)) / 2).astype(np.float32)  # exact ties
    x = np.concatenate([
        finite, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
        (rng.standard_normal(500000) * 10.0 ** rng.uniform(-9, 6, 500000)).astype(np.float32),
        np.array([65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0 ** -25, 2.0 ** -24, 0.0, -0.0],
                 dtype=np.float32)])
    x = np.ascontiguousarray(x, dtype=np.float32)
    got = np.empty(x.size, dtype=np.uint16)
    O.lib().oracle_f32_to_f16_array(O._ptr(x), O._ptr(got), x.size)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    assert np.isnan(np.array([O.lib().oracle_f32_to_f16(float("nan"))], dtype=np.uint16).view(np.float16))[0]


# ------------------------------------------------------------------ RNG

def _mix64(z):
    z = (z + np.uint64(0x9E3779B97F4A7C15))
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _rng_u64(seed, idx):
    with np.errstate(over="ignore"):
        return _mix64(_mix64(np.uint64(seed)) + idx.astype(np.uint64) * np.uint64(0x9E3779B97F4A7C15))


def test_rng_uniform_matches_independent_numpy_restatement():
    n, seed, off = 10000, 7, 123456789
    idx = np.arange(off, off + n, dtype=np.uint64)
    u = (_rng_u64(seed, idx) >> np.uint64(11)).astype(np.float64) / 2.0 ** 53
    want = (2.0 * u - 1.0).astype(np.float32)
    got = O.fill_uniform(n, F32, seed, off)
    assert np.array_equal(got, want)
    assert got.min() >= -1.0 and got.max() < 1.0 + 1e-7
    got16 = O.fill_uniform(n, F16, seed, off)
    assert np.array_equal(got16.view(np.uint16), want.astype(np.float16).view(np.uint16))
    got64 = O.fill_uniform(n, F64, seed, off)          # fp64 keeps all 53 bits of the draw
    assert got64.dtype == np.float64 and np.array_equal(got64, 2.0 * u - 1.0)


def test_rng_streams_are_position_addressed_and_distinct():
    a = O.fill_uniform(1000, F32, 0, 0)
    b = O.fill_uniform(500, F32, 0, 500)
    assert np.array_equal(a[500:], b)                       # "A then B then C from one stream"
    assert not np.array_equal(a, O.fill_uniform(1000, F32, 1, 0))
    assert abs(float(a.mean())) < 0.1 and 0.5 < float(a.std()) < 0.65   # uniform[-1,1): std = 0.577


def test_rng_normal_moments_and_box_muller():
    n, seed = 200000, 11
    z = O.fill_normal(n, F32, seed, 0, 0.1).astype(np.float64)
    assert abs(z.mean()) < 1e-3 and abs(z.std() - 0.1) < 1e-3
    idx = np.arange(n, dtype=np.uint64)
    u1 = ((_rng_u64(seed, 2 * idx) >> np.uint64(11)).astype(np.float64) + 1.0) / 2.0 ** 53
    u2 = (_rng_u64(seed, 2 * idx + 1) >> np.uint64(11)).astype(np.float64) / 2.0 ** 53
    want = np.sqrt(-2 * np.log(u1)) * np.cos(2 * np.pi * u2) * 0.1
    assert np.max(np.abs(z - want)) < 1e-6


# ------------------------------------------------------------------ GEMM

def _load_cases():
    z = np.load(os.path.join(GOLD, "gemm_small.npz"))
    keys = sorted({k.split("_")[0] for k in z.files})
    return [(k, z) for k in keys]


@pytest.mark.parametrize("key,z", _load_cases(), ids=lambda v: v if isinstance(v, str) else "")
def test_oracle_against_numpy_float64_fixtures(key, z):
    """tests/golden/gemm_small.npz: results of numpy's float64 matmul on inputs from numpy's own generator."""
    dtype, ta, tb, m, n, k, lda, ldb, ldc = (int(v) for v in z[key + "_meta"])
    alpha, beta = (float(v) for v in z[key + "_ab"])
    A, B, C, want = z[key + "_A"], z[key + "_B"], z[key + "_C"], z[key + "_want"].reshape((m, n), order="F")
    for fn in (O.gemm_f64, O.gemm_naive):
        got = fn(dtype, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc)
        got = got[:, :, 0] if got.ndim == 3 else got
        assert np.max(np.abs(got - want)) <= 1e-12 * max(1.0, np.max(np.abs(want)))
    # native-precision baseline stays within the library's own tolerance of the exact result
    Cn = C.copy()
    O.gemm_native(dtype, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cn, ldc)
    rel, _ = O.max_rel_err(dtype, Cn, ldc, want, m, n, floor=max(float(np.sqrt(np.mean(want ** 2))), 1e-30))
    assert rel <= {F32: 1e-5 * np.sqrt(k), F16: 2e-2, F64: 2e-15 * np.sqrt(k)}[dtype]
    # rows m..ldc-1 of C are padding: never written
    pad_before = C.reshape((ldc, n), order="F")[m:, :]
    pad_after = Cn.reshape((ldc, n), order="F")[m:, :]
    assert np.array_equal(np.ascontiguousarray(pad_before).view(np.uint8), np.ascontiguousarray(pad_after).view(np.uint8))


@pytest.mark.parametrize("dtype", [F32, F16, F64])
@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
def test_blocked_equals_brute_force(dtype, ta, tb):
    """Sizes that straddle the packing panels (8/4 rows, 4 columns) and the 512-deep k blocks.  For fp64 operands
    the brute-force sum is carried in long double, so this also bounds the blocked fp64 sum's rounding."""
    for (m, n, k) in ((1, 1, 1), (9, 5, 3), (17, 6, 513), (40, 23, 1030)):
        ar, ac = (k, m) if ta else (m, k)
        br, bc = (n, k) if tb else (k, n)
        lda, ldb, ldc = ar + 1, br + 2, m + 3
        A, B, C = O.fill_uniform(lda * ac, dtype, 5), O.fill_uniform(ldb * bc, dtype, 6), O.fill_uniform(ldc * n, dtype, 7)
        fast = O.gemm_f64(dtype, ta, tb, m, n, k, 0.75, A, lda, B, ldb, -2.0, C, ldc)[:, :, 0]
        slow = O.gemm_naive(dtype, ta, tb, m, n, k, 0.75, A, lda, B, ldb, -2.0, C, ldc)
        assert np.max(np.abs(fast - slow)) <= 1e-12 * max(1.0, float(np.max(np.abs(slow))))


@pytest.mark.parametrize("dtype", [F32, F16, F64])
def test_closed_forms(dtype):
    npdt = O.np_dtype(dtype)
    m, n, k = 19, 13, 31
    # all ones: C_ij = alpha*K + beta*C_ij
    A, B = np.ones(m * k, npdt), np.ones(k * n, npdt)
    C = O.fill_uniform(m * n, dtype, 3)
    out = O.gemm_f64(dtype, 0, 0, m, n, k, 2.0, A, m, B, k, 0.5, C, m)[:, :, 0]
    assert np.array_equal(out, 2.0 * k + 0.5 * C.astype(np.float64).reshape((m, n), order="F"))
    # identity on the left: op(A) = I  =>  C = alpha * op(B), for both storage orders of B
    eye = np.eye(k, dtype=npdt).reshape(-1, order="F")
    Bn = O.fill_uniform(k * n, dtype, 4)
    out = O.gemm_f64(dtype, 0, 0, k, n, k, 3.0, eye, k, Bn, k, 0.0, None, k)[:, :, 0]
    assert np.array_equal(out, 3.0 * Bn.astype(np.float64).reshape((k, n), order="F"))
    Bt = O.fill_uniform(n * k, dtype, 4)        # stored n x k, used transposed
    out = O.gemm_f64(dtype, 1, 1, k, n, k, 1.0, eye, k, Bt, n, 0.0, None, k)[:, :, 0]
    assert np.array_equal(out, Bt.astype(np.float64).reshape((n, k), order="F").T)
    # powers of two are exact in every precision: native result equals the fp64 result bit for bit
    rng = np.random.default_rng(0)
    Ap = (2.0 ** rng.integers(-3, 3, m * k)).astype(npdt)
    Bp = (2.0 ** rng.integers(-3, 3, k * n)).astype(npdt)
    exact = O.gemm_f64(dtype, 0, 0, m, n, k, 1.0, Ap, m, Bp, k, 0.0, None, m)[:, :, 0]
    Cn = np.zeros(m * n, npdt)
    O.gemm_native(dtype, 0, 0, m, n, k, 1.0, Ap, m, Bp, k, 0.0, Cn, m)
    # (the sums are exact in fp32; the fp16 output adds one rounding of that exact value)
    assert np.array_equal(Cn.reshape((m, n), order="F"), exact.astype(npdt))


@pytest.mark.parametrize("dtype", [F32, F16, F64])
def test_transpose_identity(dtype):
    """(op(A) op(B))^T = op(B)^T op(A)^T: the TN product equals the NT product of the swapped operands."""
    m, n, k = 21, 34, 55
    A = O.fill_uniform(k * m, dtype, 8)     # stored k x m, used as A^T (m x k)
    B = O.fill_uniform(k * n, dtype, 9)     # stored k x n
    tn = O.gemm_f64(dtype, 1, 0, m, n, k, 1.0, A, k, B, k, 0.0, None, m)[:, :, 0]
    nt = O.gemm_f64(dtype, 1, 0, n, m, k, 1.0, B, k, A, k, 0.0, None, n)[:, :, 0]
    assert np.array_equal(tn, nt.T)
    # and the same data declared the other way round: (B^T stored n x k used T) etc.
    At = np.ascontiguousarray(A.reshape((k, m), order="F").T).reshape(-1, order="F")   # stored m x k
    nn = O.gemm_f64(dtype, 0, 0, m, n, k, 1.0, At, m, B, k, 0.0, None, m)[:, :, 0]
    assert np.array_equal(tn, nn)


def test_beta_zero_never_reads_c():
    """src/gemm/ref/Kernels.cpp:87: with beta == 0 the old C must not enter the result, NaN included."""
    m, n, k = 8, 8, 8
    A, B = O.fill_uniform(m * k, F32, 1), O.fill_uniform(k * n, F32, 2)
    C = np.full(m * n, np.nan, np.float32)
    out = O.gemm_f64(F32, 0, 0, m, n, k, 1.0, A, m, B, k, 0.0, C, m)
    assert np.all(np.isfinite(out))
    O.gemm_native(F32, 0, 0, m, n, k, 1.0, A, m, B, k, 0.0, C, m)
    assert np.all(np.isfinite(C))
    C2 = np.full(m * n, np.nan, np.float32)
    assert np.all(np.isnan(O.gemm_f64(F32, 0, 0, m, n, k, 1.0, A, m, B, k, 1.0, C2, m)))


def test_dgemm_native_is_the_fp64_contraction_in_place():
    """oracle_dgemm_native (the reference's own arithmetic, src/gemm/gemm.h:4-5 with alpha=-1, beta=1 as in
    src/gemm/test.cc:20-21): equals the dense fp64 oracle, leaves padding rows alone, and is exact on integers."""
    m, n, k, ldc = 37, 29, 61, 41
    A, B, C = O.fill_uniform(m * k, F64, 1), O.fill_uniform(n * k, F64, 2), O.fill_uniform(ldc * n, F64, 3)
    want = O.gemm_f64(F64, 0, 1, m, n, k, -1.0, A, m, B, n, 1.0, C, ldc)[:, :, 0]
    Cn = C.copy()
    O.gemm_native(F64, 0, 1, m, n, k, -1.0, A, m, B, n, 1.0, Cn, ldc)
    got = Cn.reshape((ldc, n), order="F")
    assert np.max(np.abs(got[:m] - want)) <= 4 * np.finfo(np.float64).eps * np.max(np.abs(want))
    assert np.array_equal(got[m:], C.reshape((ldc, n), order="F")[m:])
    rng = np.random.default_rng(1)
    Ai, Bi = rng.integers(-9, 10, m * k).astype(np.float64), rng.integers(-9, 10, n * k).astype(np.float64)
    Ci = rng.integers(-9, 10, m * n).astype(np.float64)
    exact = -(Ai.reshape((m, k), order="F") @ Bi.reshape((n, k), order="F").T) + Ci.reshape((m, n), order="F")
    O.gemm_native(F64, 0, 1, m, n, k, -1.0, Ai, m, Bi, n, 1.0, Ci, m)
    assert np.array_equal(Ci.reshape((m, n), order="F"), exact)
    # the float-scalar entry point refuses fp64 operands
    assert O.lib().oracle_gemm_native(F64, 0, 0, 2, 2, 2, 1.0, A.ctypes.data, 2, B.ctypes.data, 2, 0.0, Cn.ctypes.data, 2,
                                      1, 0, 0, 0) != 0


def test_strided_batch_equals_independent_calls():
    """src/gemm/ref/Kernels.cpp:76-78,254: batch b works on A + b*strideA, B + b*strideB, C + b*strideC."""
    m, n, k, batch = 12, 9, 20, 3
    sa, sb, sc = k * m + 5, k * n + 7, m * n + 11
    A, B, C = O.fill_uniform(sa * batch, F16, 1), O.fill_uniform(sb * batch, F16, 2), O.fill_uniform(sc * batch, F16, 3)
    out = O.gemm_f64(F16, 1, 0, m, n, k, 1.0, A, k, B, k, 1.0, C, m, batch, sa, sb, sc)
    for b in range(batch):
        one = O.gemm_f64(F16, 1, 0, m, n, k, 1.0, A[b * sa:], k, B[b * sb:], k, 1.0, C[b * sc:], m)[:, :, 0]
        assert np.array_equal(out[:, :, b], one)


def test_k_zero_and_empty():
    C = O.fill_uniform(12, F32, 1)
    out = O.gemm_f64(F32, 0, 0, 3, 4, 0, 1.0, np.zeros(1, np.float32), 3, np.zeros(1, np.float32), 1, 2.0, C, 3)
    assert np.array_equal(out[:, :, 0], 2.0 * C.astype(np.float64).reshape((3, 4), order="F"))
    assert O.gemm_f64(F32, 0, 0, 0, 4, 5, 1.0, np.zeros(1, np.float32), 1, np.zeros(20, np.float32), 5, 0.0, None, 1).size == 0


def test_bad_arguments_rejected():
    A = np.zeros(16, np.float32)
    with pytest.raises(ValueError):
        O.gemm_f64(F32, 0, 0, 4, 4, 4, 1.0, A, 3, A, 4, 0.0, None, 4)      # lda < m
    with pytest.raises(ValueError):
        O.gemm_f64(F32, 0, 0, 4, 4, 4, 1.0, A, 4, A, 4, 0.0, None, 3)      # ldc < m


# ------------------------------------------------------------------ the comparator itself
# Every tolerance assertion of the parity tests goes through oracle_max_rel_err (the counterpart of the reference's
# compare loop, src/gemm/test.cc:109-120).  These tests feed it results that are wrong in known ways and check that it
# says so: a comparator that overlooked NaNs, a stride, a batch or its own floor would make every parity test pass
# vacuously.

def _cmp_case(dtype, m=7, n=5, ldg=11, batch=3, gap=13, seed=21):
    """want (dense fp64, exactly representable in dtype) and a got buffer (ldg > m, batch stride > ldg*n) that
    holds the same values, padding and gaps filled with a sentinel."""
    npdt = O.np_dtype(dtype)
    rng = np.random.default_rng(seed)
    want = (rng.integers(-64, 65, (m, n, batch)) / 8.0).astype(np.float64)       # eighths: exact in fp16
    want[want == 0] = 0.125
    strideG = ldg * n + gap
    got = np.full(strideG * batch, 777.0, dtype=npdt)
    for b in range(batch):
        got[b * strideG: b * strideG + ldg * n].reshape((ldg, n), order="F")[:m, :] = want[:, :, b].astype(npdt)
    return want, got, ldg, strideG


@pytest.mark.parametrize("dtype", [F32, F16, F64])
def test_comparator_reports_zero_on_an_exact_copy(dtype):
    want, got, ldg, strideG = _cmp_case(dtype)
    m, n, batch = want.shape
    rel, ab = O.max_rel_err(dtype, got, ldg, want, m, n, batch, strideG, floor=1.0)
    assert rel == 0.0 and ab == 0.0


@pytest.mark.parametrize("dtype", [F32, F16, F64])
@pytest.mark.parametrize("where", ["first", "last_of_batch0", "batch1", "last"])
def test_comparator_finds_one_wrong_element_and_prices_it_exactly(dtype, where):
    """One element off by delta (a power of two: exact in every dtype): abs = delta, rel = delta / max(|want|, floor),
    wherever it sits -- first element, last element of a batch, inside batch >= 1 (strideG != ldg*n), the very last."""
    want, got, ldg, strideG = _cmp_case(dtype)
    m, n, batch = want.shape
    i, j, b = {"first": (0, 0, 0), "last_of_batch0": (m - 1, n - 1, 0), "batch1": (3, 2, 1),
               "last": (m - 1, n - 1, batch - 1)}[where]
    delta = 0.5
    got[b * strideG + j * ldg + i] += delta
    w = abs(want[i, j, b])
    for floor in (1e-30, 1.0, 100.0):
        rel, ab = O.max_rel_err(dtype, got, ldg, want, m, n, batch, strideG, floor=floor)
        assert ab == delta
        assert rel == delta / max(w, floor)


@pytest.mark.parametrize("dtype", [F32, F16, F64])
def test_comparator_takes_the_maximum_not_the_last_or_the_sum(dtype):
    want, got, ldg, strideG = _cmp_case(dtype)
    m, n, batch = want.shape
    got[0 * strideG + 1 * ldg + 2] += 0.25
    got[1 * strideG + 4 * ldg + 6] -= 2.0           # the largest, in the middle of the buffer
    got[2 * strideG + 0 * ldg + 0] += 0.125
    rel, ab = O.max_rel_err(dtype, got, ldg, want, m, n, batch, strideG, floor=1e9)
    assert ab == 2.0 and rel == 2.0 / 1e9


@pytest.mark.parametrize("dtype", [F32, F16, F64])
@pytest.mark.parametrize("bad", [np.nan, np.inf, -np.inf])
def test_comparator_treats_nan_and_inf_in_the_result_as_unbounded_error(dtype, bad):
    """An element the kernel never wrote stays NaN in the beta = 0 tests: it must not compare as 'no error'."""
    want, got, ldg, strideG = _cmp_case(dtype)
    m, n, batch = want.shape
    got[2 * strideG + 3 * ldg + 4] = bad
    rel, ab = O.max_rel_err(dtype, got, ldg, want, m, n, batch, strideG, floor=1.0)
    assert rel == np.inf and ab == np.inf


@pytest.mark.parametrize("dtype", [F32, F16, F64])
def test_comparator_ignores_padding_rows_and_batch_gaps(dtype):
    """Rows m..ldg-1 and the elements between two batches are not part of the result (the padding check of the parity
    tests is separate and bitwise); garbage there, NaN included, leaves the error at zero."""
    want, got, ldg, strideG = _cmp_case(dtype)
    m, n, batch = want.shape
    for b in range(batch):
        blk = got[b * strideG: b * strideG + ldg * n].reshape((ldg, n), order="F")
        blk[m:, :] = np.nan
        got[b * strideG + ldg * n: (b + 1) * strideG] = np.inf
    rel, ab = O.max_rel_err(dtype, got, ldg, want, m, n, batch, strideG, floor=1.0)
    assert rel == 0.0 and ab == 0.0


@pytest.mark.parametrize("dtype", [F32, F16, F64])
def test_comparator_honours_the_leading_dimension_and_the_batch_stride(dtype):
    """The same buffer read with a wrong ldg or strideG is a different matrix: the comparator must notice, i.e. it
    really uses both (a comparator that assumed ldg = m or strideG = ldg*n would report zero on the right call only
    by luck and a wrong figure here)."""
    want, got, ldg, strideG = _cmp_case(dtype)
    m, n, batch = want.shape
    assert O.max_rel_err(dtype, got, ldg, want, m, n, batch, strideG, floor=1.0)[0] == 0.0
    assert O.max_rel_err(dtype, got, ldg - 1, want, m, n, 1, strideG, floor=1.0)[0] > 0.0
    assert O.max_rel_err(dtype, got, ldg, want, m, n, batch, strideG - 1, floor=1.0)[0] > 0.0
    # a dense buffer compared as dense: ldg = m, strideG = m*n
    dense = np.ascontiguousarray(want.reshape(-1, order="F").astype(O.np_dtype(dtype)))
    assert O.max_rel_err(dtype, dense, m, want, m, n, batch, m * n, floor=1.0)[0] == 0.0


def test_comparator_sees_every_element_of_a_large_result():
    """The comparison runs threaded (a max-reduction over columns): an error in any column of a result large enough to
    be split over all threads must come back, and the largest of many must win."""
    m, n = 257, 1031
    rng = np.random.default_rng(5)
    want = rng.standard_normal((m, n))
    got = want.astype(np.float32)
    want = got.astype(np.float64)
    for j in (0, 1, 515, 1029, 1030):
        g = got.copy()
        g[m - 1, j] += 4.0
        rel, ab = O.max_rel_err(F32, np.ravel(g, order="F").copy(), m, want, m, n, floor=1e6)
        assert abs(ab - 4.0) < 1e-5 and abs(rel - 4.0e-6) < 1e-11
    g = got.copy()
    g[:, ::7] += 1.0
    g[100, 700] += 16.0
    rel, ab = O.max_rel_err(F32, np.ravel(g, order="F").copy(), m, want, m, n, floor=1e6)
    assert abs(ab - (17.0 if 700 % 7 == 0 else 16.0)) < 1e-4


# ------------------------------------------------------------------ benchmark configuration 1 without a GPU

def test_cfg1_inputs_native_cpu_gemm_against_fp64_oracle():
    """SGEMM NN 1024^3, lda = ldb = ldc = 1024, A then B from one stream of seed 0, alpha = 1, beta = 0 over a poisoned
    C: the native-precision CPU GEMM (fp32 chains, the timed CPU baseline) against the fp64 oracle within the
    library's fp32 tolerance 1e-5 * sqrt(K).  This is the leg of the benchmark set that runs where no GPU is; the
    GPU test of the same inputs is tests/test_gemm_gpu.py::test_cfg1_sgemm_nn_1024."""
    import util as U
    p = U.Problem(F32, 0, 0, 1024, 1024, 1024, 1.0, 0.0, seed=0, c_fill="nan")
    assert np.array_equal(p.A, O.fill_uniform(1024 * 1024, F32, 0, 0))
    assert np.array_equal(p.B, O.fill_uniform(1024 * 1024, F32, 0, 1024 * 1024))
    got = p.C.copy()
    O.gemm_native(F32, 0, 0, p.m, p.n, p.k, p.alpha, p.A, p.lda, p.B, p.ldb, p.beta, got, p.ldc)
    assert np.all(np.isfinite(got))                     # beta = 0: the NaNs of the old C are gone
    rel = U.check(p, got, "cfg1 on the CPU")
    assert 0.0 < rel <= 1e-5 * np.sqrt(1024)
    # a second opinion on a band of the result: numpy's float64 matmul of the same inputs
    A = p.A.astype(np.float64).reshape((1024, 1024), order="F")
    B = p.B.astype(np.float64).reshape((1024, 1024), order="F")
    band = A[100:132, :] @ B
    assert np.max(np.abs(p.exact()[100:132, :, 0] - band)) <= 1e-11
