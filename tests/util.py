"""Shared helpers for the parity tests: seeded inputs from the oracle's generator, one call through the
C ABI, comparison against the fp64 oracle with the tolerances the library promises.

Tolerances (max over C of |got - exact| / max(|exact|, rms(exact))):
    fp32:  <= 1e-5 * sqrt(K)        fp16 in/out with fp32 accumulate:  <= 2e-2
    fp64:  <= 2e-15 * sqrt(K)  (both sides are fp64 sums of K terms in different orders; a random-walk estimate
           of their difference is ~0.3 * 2^-53 * sqrt(K) * a few sigma, an order of magnitude below the limit)
These are the limits the library promises.  check() also holds every result to regression_bound(), a much tighter
figure taken from what the kernels deliver.
"""
import math

import numpy as np

from oracle import oracle as O

F32, F16, F64 = 0, 1, 2
ESZ = {F32: 4, F16: 2, F64: 8}
BITS = {F32: np.uint32, F16: np.uint16, F64: np.uint64}


def tol(dtype, k):
    if dtype == F64:
        return 2e-15 * math.sqrt(max(k, 1))
    return 1e-5 * math.sqrt(max(k, 1)) if dtype == F32 else 2e-2


def regression_bound(dtype, k):
    """What the kernels actually deliver, with a factor of about four to spare -- far inside the promised tolerances
    above, so that a loss of accuracy by an order of magnitude fails a test although it would still be 'within
    tolerance'.  fp32: chains of K fp32 multiply-adds behave like a random walk of half-ulp steps, observed
    1.2e-7 * sqrt(K) (1.1e-5 at K = 8192); fp16 output: one rounding to binary16 of an fp32 sum, half an ulp = 2^-11 =
    4.9e-4 of the value at worst, plus the fp32 sum's own error."""
    if dtype == F64:
        return tol(dtype, k)
    walk = 5e-7 * math.sqrt(max(k, 1)) + 2.5e-7
    return walk if dtype == F32 else 5.5e-4 + walk


def stored_shape(trans, rows, cols):
    """(stored rows, stored cols) of an operand whose op() is rows x cols."""
    return (cols, rows) if trans else (rows, cols)


class Problem:
    """Host copies of one GEMM problem: A, B, C as flat column-major numpy buffers with leading dimensions."""

    def __init__(self, dtype, ta, tb, m, n, k, alpha=1.0, beta=0.0, lda=None, ldb=None, ldc=None, batch=1,
                 seed=0, dist="uniform", c_fill="uniform", strides=None):
        self.dtype, self.ta, self.tb, self.m, self.n, self.k = dtype, ta, tb, m, n, k
        self.alpha, self.beta, self.batch = alpha, beta, batch
        ar, ac = stored_shape(ta, m, k)
        br, bc = stored_shape(tb, k, n)
        self.lda = lda if lda is not None else max(ar, 1)
        self.ldb = ldb if ldb is not None else max(br, 1)
        self.ldc = ldc if ldc is not None else max(m, 1)
        sa, sb, sc = self.lda * ac, self.ldb * bc, self.ldc * n
        if strides is not None:
            sa, sb, sc = strides
        self.sa, self.sb, self.sc = sa, sb, sc
        na, nb, nc = max(sa * batch, 1), max(sb * batch, 1), max(sc * batch, 1)
        # one stream per problem, drawn A first, then B, then C (reference: src/gemm/test.cc:39-50)
        if dist == "uniform":
            self.A = O.fill_uniform(na, dtype, seed, 0)
            self.B = O.fill_uniform(nb, dtype, seed, na)
        else:
            self.A = O.fill_normal(na, dtype, seed, 0, 0.1)
            self.B = O.fill_normal(nb, dtype, seed, na, 0.1)
        if c_fill == "uniform":
            self.C = O.fill_uniform(nc, dtype, seed, na + nb)
        elif c_fill == "nan":
            self.C = np.full(nc, np.nan, dtype=O.np_dtype(dtype))
        else:
            raise ValueError(c_fill)
        if self.ldc > m and c_fill == "nan":
            # padding rows get a recognisable finite sentinel so "untouched" can be checked bit for bit
            Cv = self.C.reshape(-1)
            for b in range(batch):
                blk = Cv[b * sc: b * sc + self.ldc * n].reshape((self.ldc, n), order="F")
                blk[m:, :] = -7.0

    def exact(self):
        return O.gemm_f64(self.dtype, self.ta, self.tb, self.m, self.n, self.k, self.alpha, self.A, self.lda,
                          self.B, self.ldb, self.beta, self.C if self.beta != 0 else None, self.ldc,
                          self.batch, self.sa, self.sb, self.sc)


def run_gpu(p, config_id=-1, offset_elems=(0, 0, 0)):
    """Upload, call the C ABI, download.  offset_elems shifts each device pointer by that many elements inside a
    larger allocation (to exercise unaligned operands).  Returns C as a flat numpy buffer."""
    import torch

    import gemm_mmbo_amd as G

    def up(h, off):
        t = torch.zeros(h.size + off + 8, dtype={F32: torch.float32, F16: torch.float16, F64: torch.float64}[p.dtype],
                        device="cuda")
        t[off:off + h.size].copy_(torch.from_numpy(h))
        return t

    dA, dB, dC = up(p.A, offset_elems[0]), up(p.B, offset_elems[1]), up(p.C, offset_elems[2])
    esz = ESZ[p.dtype]
    pa = dA.data_ptr() + offset_elems[0] * esz
    pb = dB.data_ptr() + offset_elems[1] * esz
    pc = dC.data_ptr() + offset_elems[2] * esz
    if p.batch == 1:
        G.gemm(p.dtype, p.ta, p.tb, p.m, p.n, p.k, p.alpha, pa, p.lda, pb, p.ldb, p.beta, pc, p.ldc, config_id)
    else:
        G.gemm_strided_batched(p.dtype, p.ta, p.tb, p.m, p.n, p.k, p.alpha, pa, p.lda, p.sa, pb, p.ldb, p.sb,
                               p.beta, pc, p.ldc, p.sc, p.batch, config_id)
    torch.cuda.synchronize()
    out = dC[offset_elems[2]:offset_elems[2] + p.C.size].cpu().numpy()
    guard = dC[offset_elems[2] + p.C.size:].cpu().numpy()
    return out, guard


def check(p, got, label=""):
    """Compare the m x n x batch window with the fp64 oracle; check padding rows are bit-unchanged."""
    want = p.exact()
    rms = float(np.sqrt(np.mean(want * want))) if want.size else 1.0
    floor = max(rms, 1e-30)
    rel, abs_err = O.max_rel_err(p.dtype, got, p.ldc, want, p.m, p.n, p.batch, p.sc, floor)
    limit = tol(p.dtype, p.k)
    assert rel <= limit, f"{label}: max rel err {rel:.3e} (abs {abs_err:.3e}, rms {rms:.3e}) > {limit:.3e}"
    # The regression bound models the rounding of a sum of k terms, which scales with the size of the TERMS.  Where the
    # window is a handful of elements whose terms happen to cancel (1 x 1 x 65: a result of 0.009 from terms of order 1),
    # rms(exact) is far below that size; the floor of this second figure is therefore never below a tenth of the size a
    # sum of k such terms typically has, |alpha| * sqrt(k) * rms(A) * rms(B).
    bound = regression_bound(p.dtype, p.k)
    if rel > bound and want.size:
        a64, b64 = p.A.astype(np.float64), p.B.astype(np.float64)
        typical = abs(p.alpha) * math.sqrt(max(p.k, 1)) * float(np.sqrt(np.mean(a64 * a64))) * float(np.sqrt(np.mean(b64 * b64)))
        rel2, _ = O.max_rel_err(p.dtype, got, p.ldc, want, p.m, p.n, p.batch, p.sc, max(floor, 0.1 * typical))
    else:
        rel2 = rel
    assert rel2 <= bound, (f"{label}: max rel err {rel2:.3e} is within the promised {limit:.3e} but beyond the {bound:.3e} the "
                           f"kernels deliver (abs {abs_err:.3e}, rms {rms:.3e})")
    if p.ldc > p.m:
        g = got.view(BITS[p.dtype])
        c = p.C.view(BITS[p.dtype])
        for b in range(p.batch):
            gb = g[b * p.sc: b * p.sc + p.ldc * p.n].reshape((p.ldc, p.n), order="F")
            cb = c[b * p.sc: b * p.sc + p.ldc * p.n].reshape((p.ldc, p.n), order="F")
            assert np.array_equal(gb[p.m:, :], cb[p.m:, :]), f"{label}: padding rows of C were written"
    return rel
