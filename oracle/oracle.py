"""TEST INFRASTRUCTURE -- ctypes binding of oracle/liboracle.so (the CPU restatement of the
reference's GEMM arithmetic, see oracle/host_gemm.h).

Only tests/, the smoke check and bench.py's cpu_baseline leg import this module; the
shipped package never does.  Arrays are numpy: float32, or uint16 holding IEEE binary16 bits
(numpy.float16 arrays are accepted and viewed as uint16).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32, F16, F64 = 0, 1, 2
OP_N, OP_T = 0, 1

_lib = None


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "all"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        sz, ll, dbl, vp, ci = ctypes.c_size_t, ctypes.c_longlong, ctypes.c_double, ctypes.c_void_p, ctypes.c_int
        L.oracle_gemm_f64.argtypes = [ci, ci, ci, sz, sz, sz, dbl, vp, sz, vp, sz, dbl, vp, sz, vp, ci, ll, ll, ll]
        L.oracle_gemm_f64.restype = ci
        L.oracle_gemm_native.argtypes = [ci, ci, ci, sz, sz, sz, ctypes.c_float, vp, sz, vp, sz, ctypes.c_float,
                                         vp, sz, ci, ll, ll, ll]
        L.oracle_gemm_native.restype = ci
        L.oracle_dgemm_native.argtypes = [ci, ci, sz, sz, sz, dbl, vp, sz, vp, sz, dbl, vp, sz, ci, ll, ll, ll]
        L.oracle_dgemm_native.restype = ci
        L.oracle_gemm_naive.argtypes = [ci, ci, ci, sz, sz, sz, dbl, vp, sz, vp, sz, dbl, vp, sz, vp]
        L.oracle_gemm_naive.restype = ci
        L.oracle_max_rel_err.argtypes = [ci, vp, sz, ll, vp, sz, sz, ci, dbl, ctypes.POINTER(dbl)]
        L.oracle_max_rel_err.restype = dbl
        L.oracle_num_threads.restype = ci
        L.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_f16_array.argtypes = [vp, vp, sz]
        L.oracle_f16_to_f32_array.argtypes = [vp, vp, sz]
        L.oracle_rng_u64.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        L.oracle_rng_u64.restype = ctypes.c_uint64
        L.oracle_fill_uniform.argtypes = [vp, ci, sz, ctypes.c_uint64, ctypes.c_uint64]
        L.oracle_fill_normal.argtypes = [vp, ci, sz, ctypes.c_uint64, ctypes.c_uint64, dbl]
        up = ctypes.POINTER(ctypes.c_uint)
        L.oracle_wg_remap.argtypes = [ctypes.c_uint] * 5 + [up, up]
        _lib = L
    return _lib


def np_dtype(dtype):
    return {F32: np.float32, F16: np.float16, F64: np.float64}[dtype]


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else None


def _check(a, dtype, name):
    want = np.float32 if dtype == F32 else np.float64 if dtype == F64 else (np.float16, np.uint16)
    if a.dtype not in (want if isinstance(want, tuple) else (want,)):
        raise TypeError(f"{name}: dtype {a.dtype} does not match oracle dtype {dtype}")
    if not a.flags["C_CONTIGUOUS"] and not a.flags["F_CONTIGUOUS"]:
        raise ValueError(f"{name} must be contiguous storage")


def gemm_f64(dtype, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
             batch=1, strideA=0, strideB=0, strideC=0):
    """fp64 oracle: returns a dense column-major (m, n, batch) float64 array (Fortran order)."""
    _check(A, dtype, "A"); _check(B, dtype, "B")
    if C is not None:
        _check(C, dtype, "C")
    out = np.empty(m * n * batch, dtype=np.float64)
    rc = lib().oracle_gemm_f64(dtype, transA, transB, m, n, k, float(alpha), _ptr(A), lda, _ptr(B), ldb,
                               float(beta), _ptr(C), ldc, _ptr(out), batch, strideA, strideB, strideC)
    if rc != 0:
        raise ValueError("oracle_gemm_f64: bad arguments")
    return out.reshape((m, n, batch), order="F")


def gemm_native(dtype, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc,
                batch=1, strideA=0, strideB=0, strideC=0):
    """native-precision CPU GEMM, in place on C (the timed CPU baseline)."""
    _check(A, dtype, "A"); _check(B, dtype, "B"); _check(C, dtype, "C")
    if dtype == F64:
        rc = lib().oracle_dgemm_native(transA, transB, m, n, k, float(alpha), _ptr(A), lda, _ptr(B), ldb, float(beta),
                                       _ptr(C), ldc, batch, strideA, strideB, strideC)
        if rc != 0:
            raise ValueError("oracle_dgemm_native: bad arguments")
        return C
    rc = lib().oracle_gemm_native(dtype, transA, transB, m, n, k, float(alpha), _ptr(A), lda, _ptr(B), ldb,
                                  float(beta), _ptr(C), ldc, batch, strideA, strideB, strideC)
    if rc != 0:
        raise ValueError("oracle_gemm_native: bad arguments")
    return C


def gemm_naive(dtype, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc):
    _check(A, dtype, "A"); _check(B, dtype, "B")
    out = np.empty(m * n, dtype=np.float64)
    rc = lib().oracle_gemm_naive(dtype, transA, transB, m, n, k, float(alpha), _ptr(A), lda, _ptr(B), ldb,
                                 float(beta), _ptr(C), ldc, _ptr(out))
    if rc != 0:
        raise ValueError("oracle_gemm_naive: bad arguments")
    return out.reshape((m, n), order="F")


def max_rel_err(dtype, got, ldg, want, m, n, batch=1, strideG=0, floor=1.0):
    """max |got - want| / max(|want|, floor) over the m x n x batch window; returns (rel, abs)."""
    _check(got, dtype, "got")
    want = np.asfortranarray(want, dtype=np.float64)
    abs_err = ctypes.c_double(0.0)
    rel = lib().oracle_max_rel_err(dtype, _ptr(got), ldg, strideG, _ptr(want), m, n, batch, float(floor),
                                   ctypes.byref(abs_err))
    return rel, abs_err.value


def fill_uniform(n, dtype, seed, offset=0):
    out = np.empty(n, dtype=np_dtype(dtype))
    lib().oracle_fill_uniform(_ptr(out), dtype, n, seed, offset)
    return out


def fill_normal(n, dtype, seed, offset=0, scale=1.0):
    out = np.empty(n, dtype=np_dtype(dtype))
    lib().oracle_fill_normal(_ptr(out), dtype, n, seed, offset, scale)
    return out


def wg_remap(wg0, wg1, nwg0, nwg1, wgm=8):
    a, b = ctypes.c_uint(0), ctypes.c_uint(0)
    lib().oracle_wg_remap(wg0, wg1, nwg0, nwg1, wgm, ctypes.byref(a), ctypes.byref(b))
    return a.value, b.value


def num_threads():
    return lib().oracle_num_threads()
