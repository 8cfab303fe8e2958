// DGEMM for gfx950 on v_mfma_f64_16x16x4_f64: the reference's own element type and workload
// (src/gemm/gemm.h:4-5,47-48 naive_dgemm / dgemm_NT; the HPL trailing update of src/gemm/run.sh:2-5).
//
// Same structure as the staged fp32/fp16 kernel (global loads into registers one stage ahead, padded
// double-buffered LDS tile, one barrier per stage; edges, K tail and unaligned operands through the predicated
// loader), with 16 x 16 MFMA blocks: an fp64 MFMA takes 64 clocks for 2,048 flops, so one 64-bit LDS read per
// operand per MFMA and a single-stage prefetch keep the pipes fed.
//
// Register layout of v_mfma_f64_16x16x4_f64 (checked on the device): operand lane l supplies row (column)
// l%16 at k = l/16; result element e of lane l is D[4*e + l/16][l%16].  A lane's four results are therefore
// four rows 4 apart.  The A fragment is read with its 16 rows permuted, MFMA row 4*e + g <- tile row
// 8*(e/2) + 2*g + e%2 (dgemm_row_of), so that lane group g = l/16 holds rows 2g, 2g+1 (e = 0, 1) and 8+2g, 9+2g
// (e = 2, 3) of column l%16: a 128-bit access per pair, and the four lane groups of a column together cover 64
// contiguous bytes per instruction.  (With four consecutive rows per lane instead, an instruction touches 16-byte
// pieces 32 bytes apart; the C update of a tile then takes about twice as long: the store path of a CU is bound by
// the number of pieces.)
#pragma once

#include "gemm_staged.hpp"

namespace mmbo {

// tile row (within a 16-row block) that MFMA row r = 4*e + g of the A operand carries
__host__ __device__ constexpr int dgemm_row_of(int r) { return 8 * (r >> 3) + 2 * (r & 3) + ((r >> 2) & 1); }

template <bool KC, int LDS_LD>
__device__ inline uint32_t dfrag_lane_off(int lane, int row0, bool permute_rows)
{
    int r = lane & 15, g = lane >> 4;
    if (permute_rows) r = dgemm_row_of(r);
    if (KC) return (uint32_t)((row0 + r) * LDS_LD + g) * 8;
    return (uint32_t)(g * LDS_LD + row0 + r) * 8;
}

// fragment of 16-row block rblk for k = 4*kk + lane/16
template <bool KC, int LDS_LD>
__device__ inline double dread_frag(const char *lds, uint32_t lane_off, int rblk, int kk)
{
    uint32_t off = lane_off + (uint32_t)(KC ? rblk * 16 * LDS_LD + kk * 4 : kk * 4 * LDS_LD + rblk * 16) * 8;
    return *reinterpret_cast<const double *>(lds + off);
}

template <bool TA, bool TB, int BM, int BN, int BK, int WM, int WN>
struct DgemmCfg {
    static constexpr int NT = WM * WN * 64;
    static constexpr int TM = BM / WM, TN = BN / WN;
    static constexpr int FM = TM / 16, FN = TN / 16;
    static_assert(TM % 16 == 0 && TN % 16 == 0, "wave tile must be a multiple of the 16x16 MFMA block");
    static_assert(BK % 4 == 0, "depthU must be a multiple of the MFMA's k");
    using TileA = OperandTile<double, TA, BM, BK, NT>;
    using TileB = OperandTile<double, !TB, BN, BK, NT>;
    static constexpr int STAGE_BYTES = TileA::LDS_BYTES + TileB::LDS_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
};

// C = alpha*acc + beta*C for one wavefront's FM x FN blocks; acc[i][j][e] is
// C(wrow0 + 16*i + 8*(e/2) + 2*(lane/16) + e%2, wcol0 + 16*j + lane%16).  beta == 0 never reads C
// (src/gemm/ref/Kernels.cpp:87); alpha*acc first, then fma(beta, C, .), as the reference's epilogue.
// `early`: the old C of the whole wave tile, requested by the caller under the last stage's MFMAs (dgemm_old_c), or null.
template <int FM, int FN>
__device__ inline void dgemm_write_back(const f64x4 (&acc)[FM][FN], const GemmArgs &args, uint32_t wrow0,
                                        uint32_t wcol0, uint32_t batch, int lane, const f64x2 (*early)[2] = nullptr)
{
    const uint32_t m = args.m, n = args.n, ldc = args.ldc;
    const double alpha = args.alpha_d, beta = args.beta_d;
    const int g = lane >> 4, cl = lane & 15;
    double *C = static_cast<double *>(args.C) + (int64_t)batch * args.strideC;
    const bool vec_c = args.vec_c != 0;
    if (vec_c && wrow0 + FM * 16 <= m && wcol0 + FN * 16 <= n) {
        // Whole wave tile in range.  The compiler may not move a load of C above an earlier store to C, so a
        // block-by-block update pays one full memory latency per block; here the old values of HB blocks are
        // requested together before the first of them is needed.
        double *p0 = C + (size_t)(wcol0 + cl) * ldc + wrow0 + 2 * g;
        constexpr int NB = FM * FN, HB = NB < 4 ? NB : 4;
        static_assert(NB % HB == 0, "blocks per wave tile");
        if (beta != 0.0) {
#pragma unroll
            for (int b0 = 0; b0 < NB; b0 += HB) {
                f64x2 c[HB][2];
#pragma unroll
                for (int b = 0; b < HB; ++b) {
                    if (early) {
                        c[b][0] = early[b0 + b][0];
                        c[b][1] = early[b0 + b][1];
                        continue;
                    }
                    const double *p = p0 + (size_t)((b0 + b) / FM) * 16 * ldc + ((b0 + b) % FM) * 16;
                    c[b][0] = *reinterpret_cast<const f64x2 *>(p);
                    c[b][1] = *reinterpret_cast<const f64x2 *>(p + 8);
                }
#pragma unroll
                for (int b = 0; b < HB; ++b) {
                    const f64x4 &a = acc[(b0 + b) % FM][(b0 + b) / FM];
                    double *p = p0 + (size_t)((b0 + b) / FM) * 16 * ldc + ((b0 + b) % FM) * 16;
                    *reinterpret_cast<f64x2 *>(p) = f64x2{__builtin_fma(beta, c[b][0][0], alpha * a[0]),
                                                          __builtin_fma(beta, c[b][0][1], alpha * a[1])};
                    *reinterpret_cast<f64x2 *>(p + 8) = f64x2{__builtin_fma(beta, c[b][1][0], alpha * a[2]),
                                                              __builtin_fma(beta, c[b][1][1], alpha * a[3])};
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const f64x4 &a = acc[b % FM][b / FM];
                double *p = p0 + (size_t)(b / FM) * 16 * ldc + (b % FM) * 16;
                *reinterpret_cast<f64x2 *>(p) = f64x2{alpha * a[0], alpha * a[1]};
                *reinterpret_cast<f64x2 *>(p + 8) = f64x2{alpha * a[2], alpha * a[3]};
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            uint32_t col = wcol0 + j * 16 + cl;
            if (col >= n) continue;
#pragma unroll
            for (int h = 0; h < 2; ++h) {       // rows 2g, 2g+1 (h = 0) and 8+2g, 9+2g (h = 1) of the block
                uint32_t row = wrow0 + i * 16 + 8 * h + 2 * g;
                if (row >= m) continue;
                double *p = C + (size_t)col * ldc + row;
                double v0 = alpha * acc[i][j][2 * h], v1 = alpha * acc[i][j][2 * h + 1];
                if (vec_c && row + 2 <= m) {
                    if (beta != 0.0) {
                        f64x2 c = *reinterpret_cast<const f64x2 *>(p);
                        v0 = __builtin_fma(beta, c[0], v0);
                        v1 = __builtin_fma(beta, c[1], v1);
                    }
                    *reinterpret_cast<f64x2 *>(p) = f64x2{v0, v1};
                } else {
                    if (beta != 0.0) v0 = __builtin_fma(beta, p[0], v0);
                    p[0] = v0;
                    if (row + 1 < m) {
                        if (beta != 0.0) v1 = __builtin_fma(beta, p[1], v1);
                        p[1] = v1;
                    }
                }
            }
        }
}

// OLD_C_EARLY: the variant for beta != 0 that requests the wave tile's old C under the last stage's MFMAs (wave tiles of at
// most four blocks).  A kernel of its own, picked by the host: the 32 registers per lane it holds the old C in take the
// work-groups per CU from five to four, which calls without C to read would pay for nothing (1024^3, beta = 0: -1 %).
template <bool TA, bool TB, int BM, int BN, int BK, int WM, int WN, bool OLD_C_EARLY = false>
// Eight wavefronts with wave tiles of at most eight blocks (64 accumulator registers, two loader chunks per
// operand) are held to 128 registers per lane so that two work-groups share a CU (the second argument is
// wavefronts per SIMD); the others get 256.
__global__ void __launch_bounds__(WM * WN * 64, (WM * WN >= 8 && (BM / WM / 16) * (BN / WN / 16) <= 8) ? 4 : 2)
dgemm_kernel(const GemmArgs args)
{
    using Cfg = DgemmCfg<TA, TB, BM, BN, BK, WM, WN>;
    using TileA = typename Cfg::TileA;
    using TileB = typename Cfg::TileB;
    constexpr int FM = Cfg::FM, FN = Cfg::FN, ESZ = 8, NKK = BK / 4;

    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    uint32_t wg0, wg1, tile_id, batch, nxcd;
    work_of_block(args, blockIdx.x, blockIdx.z, tile_id, batch, nxcd);
    wg_remap(tile_id, args.nwg0, args.nwg1, args.wgm, nxcd, wg0, wg1);

    const uint32_t row0 = wg0 * BM, col0 = wg1 * BN;
    const int rows_a = (int)min((uint32_t)BM, args.m - row0);
    const int rows_b = (int)min((uint32_t)BN, args.n - col0);
    const uint32_t k_len = args.k;
    const int n_full = (int)(k_len / BK);
    const int k_tail = (int)(k_len % BK);
    const int n_iter = n_full + (k_tail ? 1 : 0);

    const uint32_t lda = args.lda, ldb = args.ldb;
    const char *gA = static_cast<const char *>(args.A) +
                     ((int64_t)batch * args.strideA + (TA ? (int64_t)row0 * lda : (int64_t)row0)) * ESZ;
    const char *gB = static_cast<const char *>(args.B) +
                     ((int64_t)batch * args.strideB + (TB ? (int64_t)col0 : (int64_t)col0 * ldb)) * ESZ;
    const int64_t stepA = (TA ? (int64_t)BK : (int64_t)BK * lda) * ESZ;
    const int64_t stepB = (TB ? (int64_t)BK * ldb : (int64_t)BK) * ESZ;

    uint32_t offA[TileA::NCH], offB[TileB::NCH];
#pragma unroll
    for (int c = 0; c < TileA::NCH; ++c) offA[c] = TileA::goff(tid, c, lda);
#pragma unroll
    for (int c = 0; c < TileB::NCH; ++c) offB[c] = TileB::goff(tid, c, ldb);

    const bool fast = rows_a == BM && rows_b == BN && args.vec_a && args.vec_b;

    u32x4 ra[TileA::NCH], rb[TileB::NCH];
    auto load_stage = [&](int it) {
        const char *pa = gA + (int64_t)it * stepA;
        const char *pb = gB + (int64_t)it * stepB;
        if (fast && it < n_full) {
            TileA::load_fast(ra, pa, offA);
            TileB::load_fast(rb, pb, offB);
        } else {
            int kvalid = it < n_full ? BK : k_tail;
            TileA::load_slow(ra, pa, offA, tid, lda, rows_a, kvalid, args.vec_a != 0);
            TileB::load_slow(rb, pb, offB, tid, ldb, rows_b, kvalid, args.vec_b != 0);
        }
    };

    f64x4 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};

    const uint32_t fa_off = dfrag_lane_off<TA, TileA::LDS_LD>(lane, wm * Cfg::TM, true);
    const uint32_t fb_off = dfrag_lane_off<!TB, TileB::LDS_LD>(lane, wn * Cfg::TN, false) + TileA::LDS_BYTES;

    if (n_iter > 0) {
        load_stage(0);
        TileA::store_lds(ra, lds, tid);
        TileB::store_lds(rb, lds + TileA::LDS_BYTES, tid);
    }
    __syncthreads();

    int cur = 0;
    auto multiply_stage = [&](const char *st) {
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
            double fa[FM], fb[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) fa[i] = dread_frag<TA, TileA::LDS_LD>(st, fa_off, i, kk);
#pragma unroll
            for (int j = 0; j < FN; ++j) fb[j] = dread_frag<!TB, TileB::LDS_LD>(st, fb_off, j, kk);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };
    int it = 0;
    if (fast) {
        // interior tiles of aligned operands, while the next stage is a whole one: no test inside the loop, the
        // predicated loader stays out of its body
        for (; it + 1 < n_full; ++it) {
            TileA::load_fast(ra, gA + (int64_t)(it + 1) * stepA, offA);
            TileB::load_fast(rb, gB + (int64_t)(it + 1) * stepB, offB);
            multiply_stage(lds + cur * Cfg::STAGE_BYTES);
            char *nx = lds + (cur ^ 1) * Cfg::STAGE_BYTES;
            TileA::store_lds(ra, nx, tid);
            TileB::store_lds(rb, nx + TileA::LDS_BYTES, tid);
            __syncthreads();
            cur ^= 1;
        }
    }
    // Old C under the last stage's MFMAs (OLD_C_EARLY): requested at the top of the last stage -- no load follows it, so
    // nothing in the loop waits for it -- and the epilogue finds it in registers instead of starting with one memory
    // latency.  With five (now four) work-groups sharing a CU that latency was supposed to hide under the others' MFMAs;
    // measured on the reference's HPL shape (44160 x 2048 x 384 NT, alpha = -1, beta = 1) it did not: 1,150 -> 1,088 us.
    constexpr bool EARLY_C = OLD_C_EARLY && FM * FN <= 4;
    [[maybe_unused]] f64x2 old_c[EARLY_C ? FM * FN : 1][2];
    [[maybe_unused]] bool have_old_c = false;
    for (; it < n_iter; ++it) {
        const bool more = it + 1 < n_iter;
        if (more) load_stage(it + 1);
        if constexpr (EARLY_C) {
            const uint32_t wrow0 = row0 + wm * Cfg::TM, wcol0 = col0 + wn * Cfg::TN;
            if (!more && args.beta_d != 0.0 && args.vec_c && wrow0 + FM * 16 <= args.m && wcol0 + FN * 16 <= args.n) {
                const double *p0 = static_cast<const double *>(args.C) + (int64_t)batch * args.strideC +
                                   (size_t)(wcol0 + (lane & 15)) * args.ldc + wrow0 + 2 * (lane >> 4);
#pragma unroll
                for (int b = 0; b < FM * FN; ++b) {
                    const double *p = p0 + (size_t)(b / FM) * 16 * args.ldc + (b % FM) * 16;
                    old_c[b][0] = *reinterpret_cast<const f64x2 *>(p);
                    old_c[b][1] = *reinterpret_cast<const f64x2 *>(p + 8);
                }
                have_old_c = true;
            }
        }

        multiply_stage(lds + cur * Cfg::STAGE_BYTES);

        if (more) {
            char *nx = lds + (cur ^ 1) * Cfg::STAGE_BYTES;
            TileA::store_lds(ra, nx, tid);
            TileB::store_lds(rb, nx + TileA::LDS_BYTES, tid);
        }
        __syncthreads();
        cur ^= 1;
    }

    if constexpr (EARLY_C) {
        if (have_old_c) {
            dgemm_write_back<FM, FN>(acc, args, row0 + wm * Cfg::TM, col0 + wn * Cfg::TN, batch, lane, old_c);
            return;
        }
    }
    dgemm_write_back<FM, FN>(acc, args, row0 + wm * Cfg::TM, col0 + wn * Cfg::TN, batch, lane);
}

}  // namespace mmbo
