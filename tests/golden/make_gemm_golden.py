"""Writes tests/golden/gemm_small.npz: small GEMM problems with results computed by numpy's float64
matmul -- an implementation independent of oracle/host_gemm.c -- so the oracle can be pinned against it.

Inputs are drawn with numpy's own PCG64 generator (not the oracle's), rounded to the operand type, and
stored with their leading dimensions; `want` is alpha * op(A) @ op(B) + beta * C in float64 on the
exactly representable input values.  The fp64 cases (dtype code 2) are multiplied in numpy's long double
(64-bit significand on x86-64) and the result rounded once to float64.

    python tests/golden/make_gemm_golden.py
"""
import os

import numpy as np

rng = np.random.default_rng(20240607)
cases = {}
idx = 0
for dtype_code, npdt in ((0, np.float32), (1, np.float16), (2, np.float64)):
    wide = np.longdouble if dtype_code == 2 else np.float64
    for ta in (0, 1):
        for tb in (0, 1):
            for (m, n, k, pad, alpha, beta) in ((5, 7, 3, 0, 1.5, 0.5), (33, 17, 41, 3, -1.0, 1.0), (64, 2, 129, 1, 1.0, 0.0)):
                ar, ac = (k, m) if ta else (m, k)
                br, bc = (n, k) if tb else (k, n)
                lda, ldb, ldc = ar + pad, br + 2 * pad, m + pad
                A = rng.uniform(-1, 1, size=(lda, ac)).astype(npdt)
                B = rng.uniform(-1, 1, size=(ldb, bc)).astype(npdt)
                C = rng.uniform(-1, 1, size=(ldc, n)).astype(npdt)
                opA = A[:ar, :].astype(wide)
                opA = opA.T if ta else opA
                opB = B[:br, :].astype(wide)
                opB = opB.T if tb else opB
                want = alpha * (opA @ opB)
                if beta != 0:
                    want = want + beta * C[:m, :].astype(wide)
                want = want.astype(np.float64)
                key = f"c{idx:02d}"
                cases[key + "_meta"] = np.array([dtype_code, ta, tb, m, n, k, lda, ldb, ldc],
                                                dtype=np.int64)
                cases[key + "_ab"] = np.array([alpha, beta], dtype=np.float64)
                # column-major flat buffers
                cases[key + "_A"] = np.asfortranarray(A).reshape(-1, order="F")
                cases[key + "_B"] = np.asfortranarray(B).reshape(-1, order="F")
                cases[key + "_C"] = np.asfortranarray(C).reshape(-1, order="F")
                cases[key + "_want"] = np.asfortranarray(want).reshape(-1, order="F")
                idx += 1
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_small.npz")
np.savez_compressed(out, **cases)
print("wrote", out, idx, "cases", os.path.getsize(out), "bytes")
