// Exact-shape picks measured on MI355X by sweeping every config id (gemm_mmbo_amd/host/benchmark type 1 does
// the same sweep).  The reference keeps such a table for its Tensile kernels: exact size -> (solution index,
// measured GFLOP/s), src/gemm/ref/vega20_Cijk_Ailk_Bjlk_DB.yaml:929-1177.  Shapes not listed here go through
// the cost model in mmbo_gemm.hip.
#pragma once

#include <cstddef>

#include "configs.hpp"

namespace mmbo {

struct TunedRow {
    int dtype, transA, transB;
    size_t m, n, k;
    int batch;
    int config_id;
    float tflops;     // measured with that config, for the record
};

// Ring tiles (kRingTiles): 0 = 256x256, 1 = 128x128, 2 = 128x64, 3 = 64x64; x16 tiles (kX16Tiles): 0 = 256x256 on four
// wavefronts, 1 = on eight, 2 = 128x128, 3 = 128x64, 4 = 64x64, 5 = 192x192, 6 = 256x192, 7 = 192x256.  The ids are built from (tile, GlobalSplitU), so a row
// keeps its meaning when a tile or a split factor is added to the tables.
constexpr int ring_id(int tile, int split) { return ring_config_id(tile, split_index(split)); }
constexpr int x16_id(int tile, int split) { return x16_config_id(tile, split_index(split)); }

constexpr TunedRow kTuned[] = {
    //dtype ta tb m n k batch id TFLOP/s (one tuner run on one MI355X; boxes differ by a few percent)
    {0, 0, 0, 1024, 1024, 1024, 1, ring_id(3, 1), 99.2f},
    {0, 0, 1, 4096, 4096, 4096, 1, ring_id(1, 1), 146.2f},
    {0, 1, 0, 4096, 4096, 4096, 1, x16_id(0, 1), 147.9f},
    {0, 0, 0, 1023, 777, 513, 1, x16_id(4, 1), 52.2f},
    {1, 0, 0, 1023, 777, 513, 1, x16_id(4, 1), 89.9f},
    {0, 0, 0, 4096, 128, 4096, 1, ring_id(3, 4), 104.8f},
    {1, 0, 0, 4096, 128, 4096, 1, x16_id(4, 2), 288.0f},
    {0, 0, 0, 128, 4096, 8192, 1, ring_id(1, 8), 118.9f},
    {1, 0, 0, 128, 4096, 8192, 1, ring_id(2, 4), 425.8f},
    {1, 1, 0, 512, 512, 512, 64, x16_id(0, 1), 650.0f},
    {0, 0, 0, 2048, 2048, 2048, 1, x16_id(3, 1), 132.6f},
    {1, 0, 0, 2048, 2048, 2048, 1, x16_id(2, 1), 834.2f},
    {0, 0, 1, 44160, 2048, 384, 1, ring_id(1, 1), 128.0f},
    {0, 0, 0, 8192, 8192, 8192, 1, x16_id(0, 1), 149.8f},
    {1, 0, 0, 8192, 8192, 8192, 1, x16_id(0, 1), 1453.7f},
    {0, 0, 0, 4096, 4096, 4096, 1, x16_id(0, 1), 147.2f},
    {1, 0, 0, 4096, 4096, 4096, 1, x16_id(0, 1), 1319.3f},
    {2, 0, 1, 44160, 2048, 384, 1, 2, 60.3f},      // fp64 ids are rows of kTilesF64; the reference's HPL trailing update (src/gemm/run.sh:2-5)
    {2, 0, 0, 8192, 8192, 8192, 1, 0, 70.0f},
};
static_assert(ring_id(3, 1) == 33 && ring_id(3, 2) == 37 && x16_id(0, 1) == 50 && x16_id(7, 16) == 89,
              "config id layout: 30 staged ids, 20 ring ids, 40 x16 ids");

}  // namespace mmbo
