// Exact-shape picks measured on MI355X by sweeping every config id (gemm_mmbo_amd/host/benchmark type 1 does
// the same sweep).  The reference keeps such a table for its Tensile kernels: exact size -> (solution index,
// measured GFLOP/s), src/gemm/ref/vega20_Cijk_Ailk_Bjlk_DB.yaml:929-1177.  Shapes not listed here go through
// the cost model in mmbo_gemm.hip.
#pragma once

#include <cstddef>

namespace mmbo {

struct TunedRow {
    int dtype, transA, transB;
    size_t m, n, k;
    int batch;
    int config_id;
    float tflops;     // measured with that config, for the record
};

constexpr TunedRow kTuned[] = {
    //dtype ta tb m n k batch id TFLOP/s
    {0, 0, 0, 1024, 1024, 1024, 1, 33, 93.0f},
    {0, 0, 1, 4096, 4096, 4096, 1, 30, 140.2f},
    {0, 1, 0, 4096, 4096, 4096, 1, 51, 145.0f},
    {0, 0, 0, 1023, 777, 513, 1, 55, 46.6f},
    {1, 0, 0, 1023, 777, 513, 1, 55, 82.4f},
    {0, 0, 0, 4096, 128, 4096, 1, 41, 95.0f},
    {1, 0, 0, 4096, 128, 4096, 1, 37, 272.2f},
    {0, 0, 0, 128, 4096, 8192, 1, 45, 108.8f},
    {1, 0, 0, 128, 4096, 8192, 1, 40, 423.9f},
    {1, 1, 0, 512, 512, 512, 64, 51, 442.8f},
    {0, 0, 0, 2048, 2048, 2048, 1, 33, 117.5f},
    {1, 0, 0, 2048, 2048, 2048, 1, 53, 761.2f},
    {0, 0, 1, 44160, 2048, 384, 1, 53, 120.5f},
    {0, 0, 0, 8192, 8192, 8192, 1, 51, 145.3f},
    {1, 0, 0, 8192, 8192, 8192, 1, 51, 1330.0f},
    {0, 0, 0, 4096, 4096, 4096, 1, 51, 143.6f},
    {1, 0, 0, 4096, 4096, 4096, 1, 51, 1245.0f},
    {2, 0, 1, 44160, 2048, 384, 1, 2, 59.3f},      // the reference's HPL trailing update (src/gemm/run.sh:2-5)
    {2, 0, 0, 8192, 8192, 8192, 1, 0, 69.7f},
};

}  // namespace mmbo
