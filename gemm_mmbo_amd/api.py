"""Python host layer over the C ABI (include/mmbo_gemm.h), loaded with ctypes.

It mirrors the reference's host front-ends (src/gemm/gemm.h:4-5,47-48): the same positional
argument order  (m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId)  with device pointers
for A, B, C.  Operands may be torch tensors (their data_ptr() is used; torch is only the owner of
device memory and streams here) or raw integer device addresses.

There is no CPU path: if the HIP library has not been built this module raises on first use.
"""
import ctypes
import os

F32, F16, F64 = 0, 1, 2
OP_N, OP_T = 0, 1
CONFIG_AUTO = -1

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmmbo_gemm.so")

EXPORTS = (
    "mmbo_gemm", "mmbo_gemm_strided_batched", "mmbo_gemm_strided_batched_static_workspace", "mmbo_static_workspace_bytes",
    "mmbo_num_configs", "mmbo_config_info", "mmbo_select_config",
    "mmbo_wg_remap", "mmbo_chip_block_remap", "mmbo_batch_xcd_remap", "mmbo_release_workspace", "mmbo_release_stream_workspace", "mmbo_workspace_info",
    "mmbo_probe_mfma_ceiling", "mmbo_probe_stream", "mmbo_status_string", "mmbo_last_hip_error", "mmbo_version",
)


class MmboError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"mmbo_gemm status {status}: {message}")
        self.status = status


class ConfigDesc(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("macro_tile_m", ctypes.c_int), ("macro_tile_n", ctypes.c_int),
                ("depth_u", ctypes.c_int), ("threads", ctypes.c_int), ("wave_tile_m", ctypes.c_int),
                ("wave_tile_n", ctypes.c_int), ("split_k", ctypes.c_int), ("lds_bytes", ctypes.c_int)]

    def as_dict(self):
        d = {f: getattr(self, f) for f, _ in self._fields_}
        d["name"] = self.name.decode()
        return d


_lib = None


def lib():
    """The loaded C-ABI library.  Raises if it is not built -- there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MmboError(-1, f"{LIB_PATH} is missing: run `python -m gemm_mmbo_amd.build` (needs hipcc); "
                                "this package has no CPU or PyTorch fallback")
        # PyTorch first, where there is one: its wheel brings a HIP runtime of its own under a different file name, and a process
        # that has loaded the system's copy before (through this library) ends up with two runtimes, of which only the one
        # loaded first finds a device for this library's calls -- on tensors the other one allocated.  Loaded after torch, the
        # library binds to the runtime torch uses.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        sz, ll, vp, ci, cu = ctypes.c_size_t, ctypes.c_longlong, ctypes.c_void_p, ctypes.c_int, ctypes.c_uint
        L.mmbo_gemm.argtypes = [ci, ci, ci, sz, sz, sz, vp, vp, sz, vp, sz, vp, vp, sz, ci, vp]
        L.mmbo_gemm.restype = ci
        L.mmbo_gemm_strided_batched.argtypes = [ci, ci, ci, sz, sz, sz, vp, vp, sz, ll, vp, sz, ll, vp, vp, sz, ll,
                                                ci, ci, vp]
        L.mmbo_gemm_strided_batched.restype = ci
        L.mmbo_gemm_strided_batched_static_workspace.argtypes = L.mmbo_gemm_strided_batched.argtypes
        L.mmbo_gemm_strided_batched_static_workspace.restype = ci
        L.mmbo_static_workspace_bytes.restype = sz
        L.mmbo_num_configs.argtypes = [ci]
        L.mmbo_num_configs.restype = ci
        L.mmbo_config_info.argtypes = [ci, ci, ctypes.POINTER(ConfigDesc)]
        L.mmbo_config_info.restype = ci
        L.mmbo_select_config.argtypes = [ci, ci, ci, sz, sz, sz, ci]
        L.mmbo_select_config.restype = ci
        L.mmbo_wg_remap.argtypes = [cu, cu, cu, cu, cu, ctypes.POINTER(cu), ctypes.POINTER(cu)]
        L.mmbo_wg_remap.restype = ci
        L.mmbo_chip_block_remap.argtypes = [cu, cu, cu, ctypes.POINTER(cu), ctypes.POINTER(cu)]
        L.mmbo_chip_block_remap.restype = ci
        L.mmbo_batch_xcd_remap.argtypes = [cu, cu, cu, ctypes.POINTER(cu), ctypes.POINTER(cu)]
        L.mmbo_batch_xcd_remap.restype = ci
        L.mmbo_release_workspace.restype = ci
        L.mmbo_release_stream_workspace.argtypes = [vp]
        L.mmbo_release_stream_workspace.restype = ci
        L.mmbo_workspace_info.argtypes = [ctypes.POINTER(sz), ctypes.POINTER(sz)]
        L.mmbo_workspace_info.restype = ci
        dp = ctypes.POINTER(ctypes.c_double)
        L.mmbo_probe_mfma_ceiling.argtypes = [ci, ci, dp, dp]
        L.mmbo_probe_mfma_ceiling.restype = ci
        L.mmbo_probe_stream.argtypes = [sz, sz, ci, ci, dp]
        L.mmbo_probe_stream.restype = ci
        L.mmbo_status_string.argtypes = [ci]
        L.mmbo_status_string.restype = ctypes.c_char_p
        L.mmbo_last_hip_error.restype = ci
        L.mmbo_version.restype = ctypes.c_char_p
        _lib = L
    return _lib


def _check(status):
    if status != 0:
        L = lib()
        msg = L.mmbo_status_string(status).decode()
        if status == 6:
            msg += f" (hipError_t {L.mmbo_last_hip_error()})"
        raise MmboError(status, msg)


def _devptr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return ctypes.c_void_p(x)
    return ctypes.c_void_p(x.data_ptr())


def _stream_handle(stream):
    if stream is None:
        return None
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)


def _scalars(dtype, alpha, beta):
    """alpha and beta in the type the C ABI reads them in: double for F64, float otherwise."""
    t = ctypes.c_double if dtype == F64 else ctypes.c_float
    return t(alpha), t(beta)


def gemm(dtype, transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, config_id=CONFIG_AUTO, stream=None):
    """C = alpha*op(A)*op(B) + beta*C on the current device; asynchronous on `stream`."""
    al, be = _scalars(dtype, alpha, beta)
    _check(lib().mmbo_gemm(dtype, transA, transB, m, n, k, ctypes.byref(al), _devptr(A), lda, _devptr(B), ldb,
                           ctypes.byref(be), _devptr(C), ldc, config_id, _stream_handle(stream)))


def gemm_strided_batched(dtype, transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc,
                         strideC, batch, config_id=CONFIG_AUTO, stream=None):
    al, be = _scalars(dtype, alpha, beta)
    _check(lib().mmbo_gemm_strided_batched(dtype, transA, transB, m, n, k, ctypes.byref(al), _devptr(A), lda,
                                           strideA, _devptr(B), ldb, strideB, ctypes.byref(be), _devptr(C), ldc,
                                           strideC, batch, config_id, _stream_handle(stream)))


def gemm_strided_batched_static_workspace(dtype, transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C,
                                          ldc, strideC, batch, config_id=CONFIG_AUTO, stream=None):
    """The same GEMM without any device allocation: split-K partial sums go to the library's static per-device array
    (static_workspace_bytes() of them); a call that needs more raises MmboError with status 8."""
    al, be = _scalars(dtype, alpha, beta)
    _check(lib().mmbo_gemm_strided_batched_static_workspace(dtype, transA, transB, m, n, k, ctypes.byref(al), _devptr(A),
                                                            lda, strideA, _devptr(B), ldb, strideB, ctypes.byref(be),
                                                            _devptr(C), ldc, strideC, batch, config_id,
                                                            _stream_handle(stream)))


def static_workspace_bytes():
    return lib().mmbo_static_workspace_bytes()


def num_configs(dtype):
    n = lib().mmbo_num_configs(dtype)
    if n < 0:
        _check(-n)
    return n


def config_info(dtype, config_id):
    d = ConfigDesc()
    _check(lib().mmbo_config_info(dtype, config_id, ctypes.byref(d)))
    return d.as_dict()


def select_config(dtype, transA, transB, m, n, k, batch=1):
    c = lib().mmbo_select_config(dtype, transA, transB, m, n, k, batch)
    if c < 0:
        _check(-c)
    return c


def wg_remap(linear_id, nwg0, nwg1, wgm=8, num_xcd=8):
    a, b = ctypes.c_uint(0), ctypes.c_uint(0)
    _check(lib().mmbo_wg_remap(linear_id, nwg0, nwg1, wgm, num_xcd, ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def batch_xcd_remap(linear_id, tiles, batch):
    """(tile, batch index) of a work-group of a batch of small problems laid out one problem per XCD."""
    a, b = ctypes.c_uint(0), ctypes.c_uint(0)
    _check(lib().mmbo_batch_xcd_remap(linear_id, tiles, batch, ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def chip_block_remap(linear_id, nwg0, nwg1):
    """(tile row, tile column) of a work-group in the chip-wide block order of the 256 x 256 HGEMM tiles."""
    a, b = ctypes.c_uint(0), ctypes.c_uint(0)
    _check(lib().mmbo_chip_block_remap(linear_id, nwg0, nwg1, ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def probe_stream(read_bytes, write_bytes, launches=20, in_place=False):
    """Seconds per launch of a plain streaming kernel that reads and writes that many bytes on the current device (in_place:
    the writes go over the first of the bytes read, as an update of C with beta != 0 does)."""
    t = ctypes.c_double(0.0)
    _check(lib().mmbo_probe_stream(int(read_bytes), int(write_bytes), 1 if in_place else 0, int(launches), ctypes.byref(t)))
    return t.value


def probe_mfma_ceiling(dtype, random_operands=True):
    """(TFLOP/s, shader MHz) of a register-only MFMA loop on the current device."""
    tf, mhz = ctypes.c_double(0.0), ctypes.c_double(0.0)
    _check(lib().mmbo_probe_mfma_ceiling(dtype, 1 if random_operands else 0, ctypes.byref(tf), ctypes.byref(mhz)))
    return tf.value, mhz.value


def release_workspace():
    _check(lib().mmbo_release_workspace())


def release_stream_workspace(stream):
    """Frees the split-K workspace the library holds for `stream` (waits for that stream only)."""
    _check(lib().mmbo_release_stream_workspace(_stream_handle(stream)))


def workspace_info():
    """(number of split-K workspaces held for the current device, their total bytes)."""
    slots, nbytes = ctypes.c_size_t(0), ctypes.c_size_t(0)
    _check(lib().mmbo_workspace_info(ctypes.byref(slots), ctypes.byref(nbytes)))
    return slots.value, nbytes.value


def version():
    return lib().mmbo_version().decode()


# ---- the reference's front-end names (src/gemm/gemm.h:4-5 naive_dgemm, :47-48 dgemm_NT), per element type
# and transpose pair.  kernelId is the tile-config id; -1 lets the per-shape table choose.

def naive_sgemm(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId=CONFIG_AUTO):
    gemm(F32, OP_N, OP_N, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId)


def naive_dgemm(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId=CONFIG_AUTO):
    """The reference's own entry point (src/gemm/gemm.h:4-5): DGEMM, A not transposed, B transposed."""
    gemm(F64, OP_N, OP_T, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId)


def naive_hgemm(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId=CONFIG_AUTO):
    gemm(F16, OP_N, OP_N, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId)


def _front_end(dtype, ta, tb):
    def f(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId=CONFIG_AUTO):
        gemm(dtype, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, kernelId)
    return f


sgemm_NN, sgemm_NT, sgemm_TN, sgemm_TT = (_front_end(F32, a, b) for a in (0, 1) for b in (0, 1))
hgemm_NN, hgemm_NT, hgemm_TN, hgemm_TT = (_front_end(F16, a, b) for a in (0, 1) for b in (0, 1))
dgemm_NN, dgemm_NT, dgemm_TN, dgemm_TT = (_front_end(F64, a, b) for a in (0, 1) for b in (0, 1))
