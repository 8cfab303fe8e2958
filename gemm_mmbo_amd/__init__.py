"""MI355X (gfx950) SGEMM/HGEMM/DGEMM: hand-written MFMA kernels behind a C ABI (include/mmbo_gemm.h).

`gemm_mmbo_amd.api` is the Python host layer (ctypes); `gemm_mmbo_amd.build` compiles the library;
`gemm_mmbo_amd/host/` holds the C++ front-ends and harness shaped like the reference's src/gemm.
"""
from .api import (  # noqa: F401
    CONFIG_AUTO, F16, F32, F64, OP_N, OP_T, MmboError, batch_xcd_remap, chip_block_remap, config_info, dgemm_NN, dgemm_NT, dgemm_TN, dgemm_TT, gemm,
    gemm_strided_batched, hgemm_NN, hgemm_NT, naive_dgemm,
    hgemm_TN, hgemm_TT, lib, naive_hgemm, naive_sgemm, num_configs, probe_mfma_ceiling, probe_stream, release_stream_workspace, release_workspace, select_config, sgemm_NN,
    sgemm_NT, sgemm_TN, sgemm_TT, version, wg_remap, workspace_info, gemm_strided_batched_static_workspace, static_workspace_bytes,
)
