// Tile-config table: the successor of the reference's {MT0I, MT1J, threads} rows
// (src/gemm/constants.h:34-47,106-135), retuned for 256 CUs, 64-wide wavefronts and 32x32 MFMA blocks.
//
// A config id is  tile + NUM_TILES * split_index : every tile shape can run with
// GlobalSplitU = 1, 2, 4, 8 or 16 (the reference's kernels are all GSU01).
#pragma once

namespace mmbo {

struct TileRow {
    int bm, bn, bk;   // macro tile MT0I x MT1J x DepthU
    int wm, wn;       // wavefronts along M and N; wave tile = (bm/wm) x (bn/wn)
};

constexpr int NUM_TILES = 6;
constexpr int NUM_SPLITS = 5;
constexpr int kSplits[NUM_SPLITS] = {1, 2, 4, 8, 16};

//                                              bm   bn  bk wm wn
constexpr TileRow kTilesF32[NUM_TILES] = {
    {256, 256, 16, 2, 4},
    {256, 128, 16, 2, 2},
    {128, 128, 16, 2, 2},
    {128,  64, 16, 2, 2},
    { 64,  64, 32, 2, 2},
    { 32,  32, 32, 1, 1},
};
constexpr TileRow kTilesF16[NUM_TILES] = {
    {256, 256, 64, 2, 4},
    {256, 128, 64, 2, 2},
    {128, 128, 64, 2, 2},
    {128,  64, 64, 2, 2},
    { 64,  64, 64, 2, 2},
    { 32,  32, 64, 1, 1},
};

// fp64 (dgemm.hpp): 16x16 MFMA blocks, no split-K; config id = row.
constexpr int NUM_F64_TILES = 6;
constexpr TileRow kTilesF64[NUM_F64_TILES] = {
    {128, 128, 16, 2, 2},
    {256, 128, 16, 4, 2},
    { 64,  64, 16, 2, 2},
    { 32,  32, 16, 2, 2},
    {128, 128, 16, 4, 2},     // 64 accumulator registers per lane: four wavefronts per SIMD overlap C traffic with MFMAs
    {128,  64, 16, 2, 2},
};

constexpr const TileRow &tile_row(int dtype, int tile) { return dtype == 0 ? kTilesF32[tile] : kTilesF16[tile]; }

// Ring kernel tiles (gemm_ring.hpp), the same for both element types; depthU is 32 (fp16) / 16 (fp32).
// Config ids continue after the staged ones:  NUM_TILES*NUM_SPLITS + ring_tile + NUM_RING_TILES * split_index.
struct RingRow {
    int bm, bn;
    int wm, wn;       // wavefronts along M and N (swapped for TT so the transposed-read operand has fewer fragments)
    int depth;        // LDS ring buffers
};
constexpr int NUM_RING_TILES = 4;
constexpr RingRow kRingTiles[NUM_RING_TILES] = {
    {256, 256, 4, 2, 5},     // 160 KB of LDS, one work-group per CU
    {128, 128, 2, 2, 5},     //  80 KB, two per CU
    {128,  64, 2, 2, 6},     //  72 KB, two per CU
    { 64,  64, 2, 2, 6},     //  48 KB, three per CU
};
constexpr int ring_bk(int dtype) { return dtype == 0 ? 16 : 32; }

// Tiles of the 16x16-block ring kernel with accumulation-register accumulators (gemm_x16.hpp), both element types;
// depthU is 32 (fp16) / 16 (fp32).
// Config ids continue after the ring ones:  x16_tile + NUM_X16_TILES * split_index.
constexpr int NUM_X16_TILES = 8;
constexpr RingRow kX16Tiles[NUM_X16_TILES] = {
    {256, 256, 2, 2, 5},     // four wavefronts of 128 x 128: 256 accumulator registers per lane, one work-group per CU
    {256, 256, 4, 2, 5},     // eight wavefronts of 64 x 128
    {128, 128, 2, 2, 5},     //  80 KB of LDS, two work-groups per CU
    {128,  64, 2, 2, 6},     //  72 KB, two per CU
    { 64,  64, 2, 2, 6},     //  48 KB, three per CU
    {192, 192, 2, 2, 6},     // four wavefronts of 96 x 96, 144 KB: for sizes whose 256 x 256 tiles would leave a round of the
                             // 256 CUs part empty (3000^2 is 144 tiles of 256 x 256 but 256 tiles of 192 x 192)
    {256, 192, 2, 2, 5},     // four wavefronts of 128 x 96, 140 KB: the steps between 192 x 192 and 256 x 256
    {192, 256, 2, 2, 5},     // four wavefronts of 96 x 128
};

// Config ids (fp32 and fp16 share them): [0, kStagedConfigs) the staged kernel's (tile, split) pairs, then the ring
// kernel's (ring tile, split) pairs, then the x16 kernel's.  split_index indexes kSplits.
constexpr int kStagedConfigs = NUM_TILES * NUM_SPLITS;
constexpr int kRingConfigs = NUM_RING_TILES * NUM_SPLITS;
constexpr int kX16Base = kStagedConfigs + kRingConfigs;
constexpr int kX16Configs = NUM_X16_TILES * NUM_SPLITS;
constexpr int kNumConfigs = kX16Base + kX16Configs;
constexpr int split_index(int split)
{
    for (int i = 0; i < NUM_SPLITS; ++i)
        if (kSplits[i] == split) return i;
    return -1;
}
constexpr int staged_config_id(int tile, int split_idx) { return tile + NUM_TILES * split_idx; }
constexpr int ring_config_id(int tile, int split_idx) { return kStagedConfigs + tile + NUM_RING_TILES * split_idx; }
constexpr int x16_config_id(int tile, int split_idx) { return kX16Base + tile + NUM_X16_TILES * split_idx; }

}  // namespace mmbo
