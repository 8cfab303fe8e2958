// Shared device/host definitions for the gfx950 GEMM kernels.
//
// Index convention (reference: src/gemm/ref/Kernels.cpp:76-78): i runs over M, j over N, l over K,
// and the grid's z over the batch; all storage is column-major.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mmbo {

typedef _Float16 half_t;
typedef float    f32x4  __attribute__((ext_vector_type(4)));
typedef float    f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8  __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4  __attribute__((ext_vector_type(4)));
typedef short    i16x4  __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4  __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2  __attribute__((ext_vector_type(2)));
typedef double   f64x4  __attribute__((ext_vector_type(4)));
typedef double   f64x2  __attribute__((ext_vector_type(2)));

#define MMBO_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

// Kernel argument block.  Successor of the reference's packed kernarg structs
// (src/gemm/gemm.h:6-23 and :49-72): same fields -- C/A/B, alpha/beta, the three leading
// dimensions, sizeI/J/L, the batch strides -- plus what split-K and the tile mapping need.
struct GemmArgs {
    const void *A;
    const void *B;
    void *C;
    float *ws;              // split-K partial sums: [split][batch][n][m] fp32, dense
    float alpha;
    float beta;
    double alpha_d, beta_d; // the fp64 kernels' scalars (the reference's own type, src/gemm/gemm.h:31-32)
    uint32_t m, n, k;       // sizeI, sizeJ, sizeL
    uint32_t lda, ldb, ldc; // strideA1L/strideB1L/strideC1J, in elements
    int64_t strideA, strideB, strideC;   // batch strides in elements (strideA2K/B2K/C2K)
    uint32_t nwg0, nwg1;    // tiles along M and N
    uint32_t wgm;           // WorkGroupMapping width (reference: 8)
    uint32_t nxcd;          // XCDs the dispatcher round-robins over (8 on MI355X; 1 = plain order)
    uint32_t splits;        // GlobalSplitU
    uint32_t k_per_split;   // multiple of the config's depthU
    uint32_t batch;
    uint32_t vec_a, vec_b, vec_c;   // 1 when 128-bit accesses to that operand are aligned
    uint32_t chip_block;    // 1: tiles are walked in 16 x 16 chip-wide blocks (chip_block_remap) instead of wg_remap
    uint32_t batch_xcd;     // 1: every problem of the batch runs on one XCD (batch_xcd_remap)
    uint32_t c_prefetch;    // 1: beta != 0 and the old C may be fetched into freed LDS ring buffers ahead of the epilogue
    uint32_t c_stream;      // 1: C leaves with the non-temporal hint (x16 kernel; long k, many rounds of tiles)
    uint32_t line_rows;     // 1: A, B, their leading dimensions and batch strides are multiples of a 128-byte memory line
    uint32_t ws_narrow;     // 1: a tile's span of the split-K workspace (tile columns x m floats) fits 32-bit offsets
};

// Linear work-group id -> (tile row, tile column).
//
// Step 1 (nxcd > 1): hardware hands consecutive ids to XCDs round-robin, each XCD with its own L2.
// Regroup so XCD x gets the contiguous run of ids [start_x, start_x + count_x): neighbours in the
// remapped order then share an L2.
// Step 2: the reference's WorkGroupMapping (src/gemm/ref/Kernels.cpp:204-236): walk `wgm` tile
// columns wide, down all tile rows, then the next block of columns; the trailing block is as wide
// as what is left.  With nxcd == 1 and id = wg0 + wg1*nwg0 this is that remap exactly.
__host__ __device__ inline void wg_remap(uint32_t id, uint32_t nwg0, uint32_t nwg1, uint32_t wgm,
                                         uint32_t nxcd, uint32_t &wg0, uint32_t &wg1)
{
    uint32_t total = nwg0 * nwg1;
    if (nxcd > 1 && total >= nxcd) {
        uint32_t per = (total + nxcd - 1) / nxcd;        // ids on the fuller XCDs
        uint32_t tall = total % nxcd == 0 ? nxcd : total % nxcd;
        uint32_t x = id % nxcd, local = id / nxcd;
        id = x < tall ? x * per + local : tall * per + (x - tall) * (per - 1) + local;
    }
    uint32_t g0 = id % nwg0, g1 = id / nwg0;
    if (wgm <= 1) { wg0 = g0; wg1 = g1; return; }
    uint32_t serial = g0 + (g1 % wgm) * nwg0;
    uint32_t block = g1 / wgm;
    uint32_t rem = (g1 < nwg1 - (nwg1 % wgm)) ? 0u : nwg1 % wgm;
    uint32_t width = rem == 0 ? wgm : rem;
    wg0 = serial / width;
    wg1 = serial % width + block * wgm;
}

// Batches of small problems: linear dispatch index (x + tiles * z, the order the hardware hands work-groups to the
// XCDs round-robin) -> (tile, batch index) such that all tiles of one problem run on one XCD, one after the other in
// that XCD's share of the dispatch order.  The dispatcher's own order spreads a problem with fewer tiles than XCDs over
// as many XCDs as it has tiles: no two work-groups that read the same panel of A or B share an L2, and every panel
// comes from memory once per work-group that reads it (HGEMM TN 64 x 512^3 on 256 x 256 tiles: 128 MB of operand
// reads instead of 64).  Requires batch % nxcd == 0; a bijection of [0, tiles * batch).
__host__ __device__ inline void batch_xcd_remap(uint32_t lin, uint32_t tiles, uint32_t nxcd, uint32_t &tile, uint32_t &z)
{
    const uint32_t x = lin % nxcd, slot = lin / nxcd;
    z = (slot / tiles) * nxcd + x;
    tile = slot % tiles;
}

// What a work-group does: (tile id for wg_remap, z = split * batch + batch index, XCD count for wg_remap) from its
// block indices.  bx = blockIdx.x (or the tile a resident work-group has walked to), bz = blockIdx.z.
__device__ inline void work_of_block(const GemmArgs &args, uint32_t bx, uint32_t bz, uint32_t &tile, uint32_t &z, uint32_t &nxcd)
{
    tile = bx; z = bz; nxcd = args.nxcd;
    if (args.batch_xcd) {
        batch_xcd_remap(bx + args.nwg0 * args.nwg1 * bz, args.nwg0 * args.nwg1, args.nxcd, tile, z);
        nxcd = 1;                                       // the tiles of one problem are on one XCD already
    }
}

// Linear work-group id -> (tile row, tile column) in chip-wide blocks, for a chip of 8 XCDs x 32 CUs that runs one
// work-group per CU (the 256 x 256 tiles).
//
// The 256 work-groups resident at one time form one 16 x 16 block of tiles; inside it XCD x (= id % 8, the
// dispatcher's round-robin) owns a 4 x 8 sub-block, the XCDs arranged 4 down x 2 across.  Blocks are walked down
// the tile rows and then across, serpentine, so consecutive blocks share a panel of B.  What this buys: at
// any moment the chip streams 16 tile rows of A and 16 tile columns of B (64 MB + 64 MB for fp16 at k = 8192), which
// the 256 MB last-level cache holds, instead of all of A and B at once (wg_remap's order at 8192^3: 256 MB, which
// that cache then cannot hold and every XCD's L2 misses go to HBM).  Per XCD the L2 sees the same 12 panels per
// 32 tiles as with wg_remap.  Tiles outside the whole 16 x 16 blocks (grids that are not multiples of 16) follow
// in column-major order.  Requires nwg0 >= 16 and nwg1 >= 16; a bijection of [0, nwg0*nwg1).
__host__ __device__ inline void chip_block_remap(uint32_t id, uint32_t nwg0, uint32_t nwg1, uint32_t &wg0, uint32_t &wg1)
{
    const uint32_t f0 = nwg0 / 16, f1 = nwg1 / 16, full = f0 * f1 * 256;
    if (id < full) {
        const uint32_t blk = id >> 8, r = id & 255, x = r & 7, loc = r >> 3;
        uint32_t b1 = blk / f0, b0 = blk % f0;
        if (b1 & 1) b0 = f0 - 1 - b0;
        wg0 = b0 * 16 + (x & 3) * 4 + (loc & 3);
        wg1 = b1 * 16 + (x >> 2) * 8 + (loc >> 2);
        return;
    }
    uint32_t rem = id - full;
    const uint32_t w0 = nwg0 - f0 * 16, ca = f1 * 16;       // rows below the blocks, columns the blocks span
    if (rem < w0 * ca) { wg0 = f0 * 16 + rem % w0; wg1 = rem / w0; return; }
    rem -= w0 * ca;
    wg0 = rem % nwg0;
    wg1 = ca + rem / nwg0;
}

template <typename T> struct ElemTraits;
template <> struct ElemTraits<float> {
    static constexpr int VEC = 4;      // elements per 128-bit access
    static constexpr int KG = 8;       // k extent covered by one round of LDS fragment reads
    static constexpr int PAD_KC = 4;   // row padding (elements) of a k-contiguous LDS tile: 16 B
    static constexpr int PAD_RC = 8;   // row padding of a row-contiguous LDS tile
};
template <> struct ElemTraits<double> {
    static constexpr int VEC = 2;
    static constexpr int KG = 4;       // one v_mfma_f64_16x16x4 consumes four k values
    static constexpr int PAD_KC = 2;   // 16 B: 16 rows x 2 k of one 64-bit fragment read land on 64 distinct banks
    static constexpr int PAD_RC = 16;  // row length = 16 mod 32 doubles: two k-rows of a read sit 32 banks apart
};
template <> struct ElemTraits<half_t> {
    static constexpr int VEC = 8;
    static constexpr int KG = 16;
    static constexpr int PAD_KC = 8;   // 16 B
    static constexpr int PAD_RC = 32;  // 64 B: the four k-rows of one transposed read land in distinct bank groups
};

// Write-back of one wavefront's FM x FN blocks of 32 x 32 accumulators.
//   acc[i][j][4*q + r] is C(row, col) with  row = wrow0 + i*32 + 8*q + 4*(lane/32) + r,  col = wcol0 + j*32 + lane%32
// (the v_mfma_f32_32x32 result layout: a lane holds four consecutive rows of one column, four times).
// With GlobalSplitU > 1 the raw sums go to the fp32 workspace [split][batch][n][m] and the reduction kernel
// applies alpha and beta.  Otherwise  C = alpha*acc (+ beta*C): the old C is read only when beta != 0
// (reference: src/gemm/ref/Kernels.cpp:87, guarded stores :1064-1121; order of operations alpha*acc first, then
// fma(beta, C, .), as the reference's assembly epilogue does).  INTERIOR = true drops the m/n guards.
template <typename T, int FM, int FN, bool INTERIOR>
__device__ inline void write_back(const f32x16 (&acc)[FM][FN], const GemmArgs &args, uint32_t wrow0, uint32_t wcol0,
                                  uint32_t batch, uint32_t split, int lane)
{
    constexpr int ESZ = sizeof(T);
    const uint32_t m = args.m, n = args.n;
    const int g = lane >> 5, cl = lane & 31;
    if (args.splits > 1) {
        float *ws = args.ws + ((size_t)split * args.batch + batch) * (size_t)m * n;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                uint32_t col = wcol0 + j * 32 + cl;
                if (!INTERIOR && col >= n) continue;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint32_t row = wrow0 + i * 32 + 8 * q + 4 * g;
                    float *p = ws + (size_t)col * m + row;
                    if (INTERIOR || (row + 4 <= m && (m & 3) == 0)) {
                        *reinterpret_cast<f32x4 *>(p) =
                            f32x4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (row + r < m) p[r] = acc[i][j][4 * q + r];
                    }
                }
            }
        return;
    }

    const float alpha = args.alpha, beta = args.beta;
    const uint32_t ldc = args.ldc;
    T *C = static_cast<T *>(args.C) + (int64_t)batch * args.strideC;
    const bool vec_c = args.vec_c != 0;
    // down a column first: the stores that complete one cache line of C follow each other
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            uint32_t col = wcol0 + j * 32 + cl;
            if (!INTERIOR && col >= n) continue;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t row = wrow0 + i * 32 + 8 * q + 4 * g;
                if (!INTERIOR && row >= m) continue;
                T *p = C + (size_t)col * ldc + row;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = alpha * acc[i][j][4 * q + r];
                if (INTERIOR || row + 4 <= m) {
                    // four rows in range: one vector access, aligned or not (unaligned global access is enabled
                    // on gfx950 under ROCm; an odd ldc costs split lines, not four scalar accesses)
                    typedef u32x4 __attribute__((aligned(4))) u32x4_u;
                    typedef u32x2 __attribute__((aligned(2))) u32x2_u;
                    union { T e[4]; u32x4 v4; u32x2 v2; } io;
                    if (beta != 0.0f) {                       // beta == 0: C is never read
                        if constexpr (ESZ == 4) io.v4 = vec_c ? *reinterpret_cast<const u32x4 *>(p) : *reinterpret_cast<const u32x4_u *>(p);
                        else io.v2 = vec_c ? *reinterpret_cast<const u32x2 *>(p) : *reinterpret_cast<const u32x2_u *>(p);
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] = __builtin_fmaf(beta, (float)io.e[r], v[r]);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) io.e[r] = (T)v[r];
                    if constexpr (ESZ == 4) {
                        if (vec_c) *reinterpret_cast<u32x4 *>(p) = io.v4; else *reinterpret_cast<u32x4_u *>(p) = io.v4;
                    } else {
                        if (vec_c) *reinterpret_cast<u32x2 *>(p) = io.v2; else *reinterpret_cast<u32x2_u *>(p) = io.v2;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (INTERIOR || row + r < m) {
                            float o = v[r];
                            if (beta != 0.0f) o = __builtin_fmaf(beta, (float)p[r], o);
                            p[r] = (T)o;
                        }
                }
            }
        }
}

}  // namespace mmbo
