// Register-staged MFMA GEMM kernel for gfx950: the general path (any m, n, k, leading dimension,
// transpose, alpha/beta, batch, split-K).
//
// Per work-group: a BM x BN tile of C.  Per K stage of BK: 128-bit coalesced global loads into
// registers, issued one stage ahead; 128-bit writes into a padded, double-buffered LDS tile; LDS
// fragment reads feeding v_mfma_f32_32x32x16_f16 / v_mfma_f32_32x32x2_f32; one barrier per stage.
// The structure is the reference kernel's (src/gemm/ref/Kernels.cpp:412-488 prologue, :493-747
// unrolled loop with global prefetch + LDS double buffer, :921-1005 tail, :1064-1121 guarded
// write), rebuilt around matrix instructions and 64-wide wavefronts.
#pragma once

#include <type_traits>

#include "gemm_common.hpp"

namespace mmbo {

// One operand tile: R rows (of C's M or N extent) x BK along K, moved by NT threads.
//   KC = true : source is contiguous along K (A under transA=T, B under transB=N).
//               LDS layout [row][BK + PAD_KC]; fragments come out of one 128-bit read.
//   KC = false: source is contiguous along the row index (A under transA=N, B under transB=T).
//               LDS layout [k][R + PAD_RC]; fp32 fragments are 32-bit reads, fp16 fragments are
//               ds_read_b64_tr_b16 transposing reads.
template <typename T, bool KC, int R, int BK, int NT>
struct OperandTile {
    using Tr = ElemTraits<T>;
    static constexpr int VEC = Tr::VEC;
    static constexpr int ESZ = sizeof(T);
    static constexpr int CHUNKS = R * BK / VEC;
    static_assert(CHUNKS % NT == 0, "tile must split evenly over the work-group");
    static constexpr int NCH = CHUNKS / NT;                 // 128-bit chunks per thread per stage
    static constexpr int INNER = KC ? BK / VEC : R / VEC;   // chunks along the contiguous direction
    static_assert(NT % INNER == 0 || INNER % NT == 0, "thread/chunk mapping");
    static constexpr int OUTER_STEP = NT / INNER;           // outer index step between a thread's chunks
    static_assert(NT >= INNER, "more chunks in one line than threads");
    static constexpr int LDS_LD = KC ? BK + Tr::PAD_KC : R + Tr::PAD_RC;   // elements
    static constexpr int LDS_ELEMS = (KC ? R : BK) * LDS_LD;
    static constexpr int LDS_BYTES = LDS_ELEMS * ESZ;

    // chunk c of this thread: outer index (row if KC, else k) and inner chunk index
    __device__ static inline int outer(int tid, int c) { return tid / INNER + c * OUTER_STEP; }
    __device__ static inline int inner(int tid) { return tid % INNER; }

    // byte offset of chunk c from the tile origin in global memory (ld in elements)
    __device__ static inline uint32_t goff(int tid, int c, uint32_t ld)
    {
        return ((uint32_t)outer(tid, c) * ld + (uint32_t)inner(tid) * VEC) * ESZ;
    }
    __device__ static inline uint32_t lds_woff(int tid, int c)
    {
        return (uint32_t)(outer(tid, c) * LDS_LD + inner(tid) * VEC) * ESZ;
    }

    // Interior, aligned stage: plain 128-bit loads.
    __device__ static inline void load_fast(u32x4 (&regs)[NCH], const char *g, const uint32_t (&off)[NCH])
    {
#pragma unroll
        for (int c = 0; c < NCH; ++c) regs[c] = *reinterpret_cast<const u32x4 *>(g + off[c]);
    }

    // Edge tile, K tail or unaligned operand: zero where row >= rows or k >= kvalid.  Whole in-range chunks still
    // use one 128-bit load, aligned or not (gfx950 under ROCm runs with unaligned global access enabled: a leading
    // dimension like 1023 costs split cache-line accesses, not eight 2-byte loads per chunk); only chunks that
    // straddle the matrix edge or the end of K go element by element.
    typedef u32x4 __attribute__((aligned(2))) u32x4_unaligned;
    __device__ static inline void load_slow(u32x4 (&regs)[NCH], const char *g, const uint32_t (&off)[NCH],
                                            int tid, uint32_t /* ld: the offsets already contain it */, int rows, int kvalid, bool vec)
    {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            int o = outer(tid, c), in0 = inner(tid) * VEC;
            int row0 = KC ? o : in0, k0 = KC ? in0 : o;
            int nrow = KC ? 1 : VEC, nk = KC ? VEC : 1;
            bool full = row0 + nrow <= rows && k0 + nk <= kvalid;
            if (full && vec) {
                regs[c] = *reinterpret_cast<const u32x4 *>(g + off[c]);
            } else if (full) {
                regs[c] = *reinterpret_cast<const u32x4_unaligned *>(g + off[c]);
            } else {
                union { u32x4 v; T e[VEC]; } u;
                u.v = u32x4{0, 0, 0, 0};
                const T *p = reinterpret_cast<const T *>(g + off[c]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    int row = KC ? row0 : row0 + e, kk = KC ? k0 + e : k0;
                    if (row < rows && kk < kvalid) u.e[e] = p[e];
                }
                regs[c] = u.v;
            }
        }
    }

    __device__ static inline void store_lds(const u32x4 (&regs)[NCH], char *lds, int tid)
    {
#pragma unroll
        for (int c = 0; c < NCH; ++c) *reinterpret_cast<u32x4 *>(lds + lds_woff(tid, c)) = regs[c];
    }
};

// Fragment of one 32-row block for one k-group (KG k values): what the MFMA operand registers hold.
template <typename T> struct Frag;
template <> struct Frag<float>  { f32x4 v; };    // component t feeds the t-th 32x32x2 MFMA of the group
template <> struct Frag<half_t> { f16x8 v; };    // feeds one 32x32x16 MFMA

// Per-lane LDS byte offset, inside an operand tile, of the fragment for 32-row block 0, k-group 0.
// lane%32 selects the row, lane/32 the half of the k-group: element e of lane group g is
// k = kg*KG + g*VEC + e for both operands, which is all the contraction needs.
template <typename T, bool KC, int LDS_LD>
__device__ inline uint32_t frag_lane_off(int lane, int row0)
{
    using Tr = ElemTraits<T>;
    int r = lane & 31, g = lane >> 5;
    if (KC) return (uint32_t)((row0 + r) * LDS_LD + g * Tr::VEC) * sizeof(T);
    if (sizeof(T) == 4) return (uint32_t)((g * 4) * LDS_LD + row0 + r) * 4;
    // fp16 transposing read: each 16-lane block reads four k-rows x 16 rows; lane j of the block points
    // at k-row j/4, rows 4*(j%4)..+3, and receives (k-rows 0..3) x (row j).
    int j = lane & 15, blk = (lane >> 4) & 1;
    return (uint32_t)((g * 8 + (j >> 2)) * LDS_LD + row0 + blk * 16 + (j & 3) * 4) * 2;
}

template <typename T, bool KC, int LDS_LD>
__device__ inline Frag<T> read_frag(const char *lds, uint32_t lane_off, int rblk, int kg)
{
    using Tr = ElemTraits<T>;
    Frag<T> f;
    if constexpr (KC) {
        uint32_t off = lane_off + (uint32_t)(rblk * 32 * LDS_LD + kg * Tr::KG) * sizeof(T);
        auto raw = *reinterpret_cast<const u32x4 *>(lds + off);
        f.v = __builtin_bit_cast(decltype(f.v), raw);
    } else if constexpr (sizeof(T) == 4) {
        uint32_t off = lane_off + (uint32_t)(kg * Tr::KG * LDS_LD + rblk * 32) * 4;
#pragma unroll
        for (int t = 0; t < 4; ++t) f.v[t] = *reinterpret_cast<const float *>(lds + off + t * LDS_LD * 4);
    } else {
        uint32_t off = lane_off + (uint32_t)(kg * Tr::KG * LDS_LD + rblk * 32) * 2;
        i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) i16x4 *)MMBO_LDS_PTR(lds + off));
        i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) i16x4 *)MMBO_LDS_PTR(lds + off + 4 * LDS_LD * 2));
        f16x4 l4 = __builtin_bit_cast(f16x4, lo), h4 = __builtin_bit_cast(f16x4, hi);
        f.v = f16x8{l4[0], l4[1], l4[2], l4[3], h4[0], h4[1], h4[2], h4[3]};
    }
    return f;
}

__device__ inline void mma(f32x16 &acc, const Frag<float> &a, const Frag<float> &b)
{
#pragma unroll
    for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[t], b.v[t], acc, 0, 0, 0);
}
__device__ inline void mma(f32x16 &acc, const Frag<half_t> &a, const Frag<half_t> &b)
{
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a.v, b.v, acc, 0, 0, 0);
}

template <typename T, bool TA, bool TB, int BM, int BN, int BK, int WM, int WN>
struct StagedCfg {
    static constexpr int NT = WM * WN * 64;
    static constexpr int TM = BM / WM, TN = BN / WN;        // wave tile
    static constexpr int FM = TM / 32, FN = TN / 32;        // 32x32 MFMA blocks per wave
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA block");
    static_assert(BK % ElemTraits<T>::KG == 0, "depthU must be a multiple of the k-group");
    using TileA = OperandTile<T, TA, BM, BK, NT>;           // A is k-contiguous when transposed
    using TileB = OperandTile<T, !TB, BN, BK, NT>;          // B is k-contiguous when not transposed
    static constexpr int STAGE_BYTES = TileA::LDS_BYTES + TileB::LDS_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;       // double buffer
};

// How many stages ahead the global loads run (a ring of register sets).  One stage costs a full memory latency
// when nothing overlaps it, so short-K problems on small tiles -- few stages, little MFMA work per stage -- want
// several in flight; the large tiles spend their registers on accumulators and keep one.
template <typename T, int BM, int BN, int BK, int NT>
constexpr int staged_prefetch()
{
    // registers per thread per stage: 4 per 128-bit chunk
    const int regs = 4 * (BM + BN) * BK / (16 / (int)sizeof(T)) / NT;
    return regs <= 16 ? 3 : regs <= 32 && BM * BN <= 128 * 128 ? 2 : 1;
}

template <typename T, bool TA, bool TB, int BM, int BN, int BK, int WM, int WN>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_staged_kernel(const GemmArgs args)
{
    using Cfg = StagedCfg<T, TA, TB, BM, BN, BK, WM, WN>;
    using TileA = typename Cfg::TileA;
    using TileB = typename Cfg::TileB;
    using Tr = ElemTraits<T>;
    constexpr int NT = Cfg::NT, FM = Cfg::FM, FN = Cfg::FN, ESZ = sizeof(T);
    constexpr int NKG = BK / Tr::KG;
    constexpr int PF = staged_prefetch<T, BM, BN, BK, NT>();

    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    uint32_t wg0, wg1, tile_id, zb, nxcd;
    work_of_block(args, blockIdx.x, blockIdx.z, tile_id, zb, nxcd);
    wg_remap(tile_id, args.nwg0, args.nwg1, args.wgm, nxcd, wg0, wg1);
    const uint32_t split = zb / args.batch, batch = zb % args.batch;

    const uint32_t row0 = wg0 * BM, col0 = wg1 * BN;
    const int rows_a = (int)min((uint32_t)BM, args.m - row0);     // valid rows of the A tile
    const int rows_b = (int)min((uint32_t)BN, args.n - col0);
    const uint32_t k_begin = split * args.k_per_split;
    const uint32_t k_end = min(args.k, k_begin + args.k_per_split);
    const uint32_t k_len = k_end > k_begin ? k_end - k_begin : 0;
    const int n_full = (int)(k_len / BK);
    const int k_tail = (int)(k_len % BK);
    const int n_iter = n_full + (k_tail ? 1 : 0);

    const uint32_t lda = args.lda, ldb = args.ldb;
    // tile origin in global memory; per stage it moves BK along K
    const char *gA = static_cast<const char *>(args.A) +
                     ((int64_t)batch * args.strideA + (TA ? (int64_t)row0 * lda + k_begin
                                                          : (int64_t)k_begin * lda + row0)) * ESZ;
    const char *gB = static_cast<const char *>(args.B) +
                     ((int64_t)batch * args.strideB + (TB ? (int64_t)k_begin * ldb + col0
                                                          : (int64_t)col0 * ldb + k_begin)) * ESZ;
    const int64_t stepA = (TA ? (int64_t)BK : (int64_t)BK * lda) * ESZ;
    const int64_t stepB = (TB ? (int64_t)BK * ldb : (int64_t)BK) * ESZ;

    uint32_t offA[TileA::NCH], offB[TileB::NCH];
#pragma unroll
    for (int c = 0; c < TileA::NCH; ++c) offA[c] = TileA::goff(tid, c, lda);
#pragma unroll
    for (int c = 0; c < TileB::NCH; ++c) offB[c] = TileB::goff(tid, c, ldb);

    // whole-tile-in-range and aligned: every stage but the K tail takes the unpredicated loader
    const bool fast = rows_a == BM && rows_b == BN && args.vec_a && args.vec_b;

    u32x4 ra[PF][TileA::NCH], rb[PF][TileB::NCH];             // register ring: stage `it` lives in set it % PF
    auto load_stage = [&](int it, u32x4 (&xa)[TileA::NCH], u32x4 (&xb)[TileB::NCH]) {
        const char *pa = gA + (int64_t)it * stepA;
        const char *pb = gB + (int64_t)it * stepB;
        if (fast && it < n_full) {
            TileA::load_fast(xa, pa, offA);
            TileB::load_fast(xb, pb, offB);
        } else {
            int kvalid = it < n_full ? BK : k_tail;
            TileA::load_slow(xa, pa, offA, tid, lda, rows_a, kvalid, args.vec_a != 0);
            TileB::load_slow(xb, pb, offB, tid, ldb, rows_b, kvalid, args.vec_b != 0);
        }
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const uint32_t fa_off = frag_lane_off<T, TA, TileA::LDS_LD>(lane, wm * Cfg::TM);
    const uint32_t fb_off = frag_lane_off<T, !TB, TileB::LDS_LD>(lane, wn * Cfg::TN) + TileA::LDS_BYTES;

    // prologue: stages 0 .. PF-1 requested, stage 0 moved into LDS buffer 0
#pragma unroll
    for (int q = 0; q < PF; ++q)
        if (q < n_iter) load_stage(q, ra[q], rb[q]);
    if (n_iter > 0) {
        TileA::store_lds(ra[0], lds, tid);
        TileB::store_lds(rb[0], lds + TileA::LDS_BYTES, tid);
    }
    __syncthreads();

    int cur = 0;
    // Iteration `it` (register set q = it % PF, a compile-time index inside the PF-fold unrolled body): request
    // stage it+PF into set q, whose stage `it` already sits in LDS; multiply stage `it` from LDS buffer `cur`; move
    // stage it+1 (set (q+1) % PF, requested PF-1 iterations ago) into the other LDS buffer; one barrier.
    auto body = [&](int it, u32x4 (&qa)[TileA::NCH], u32x4 (&qb)[TileB::NCH], u32x4 (&na)[TileA::NCH], u32x4 (&nb)[TileB::NCH]) {
        if (it + PF < n_iter) load_stage(it + PF, qa, qb);

        const char *st = lds + cur * Cfg::STAGE_BYTES;
#pragma unroll
        for (int kg = 0; kg < NKG; ++kg) {
            Frag<T> fa[FM], fb[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) fa[i] = read_frag<T, TA, TileA::LDS_LD>(st, fa_off, i, kg);
#pragma unroll
            for (int j = 0; j < FN; ++j) fb[j] = read_frag<T, !TB, TileB::LDS_LD>(st, fb_off, j, kg);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) mma(acc[i][j], fa[i], fb[j]);
        }

        if (it + 1 < n_iter) {
            char *nx = lds + (cur ^ 1) * Cfg::STAGE_BYTES;   // nobody reads this buffer during stage `it`
            TileA::store_lds(na, nx, tid);
            TileB::store_lds(nb, nx + TileA::LDS_BYTES, tid);
        }
        __syncthreads();
        cur ^= 1;
    };
    for (int it0 = 0; it0 < n_iter; it0 += PF) {
        if constexpr (PF == 1) {
            // one set: stage it+1 is requested into it before the multiply and stored after it
            if (it0 + 1 < n_iter) load_stage(it0 + 1, ra[0], rb[0]);
            const char *st = lds + cur * Cfg::STAGE_BYTES;
#pragma unroll
            for (int kg = 0; kg < NKG; ++kg) {
                Frag<T> fa[FM], fb[FN];
#pragma unroll
                for (int i = 0; i < FM; ++i) fa[i] = read_frag<T, TA, TileA::LDS_LD>(st, fa_off, i, kg);
#pragma unroll
                for (int j = 0; j < FN; ++j) fb[j] = read_frag<T, !TB, TileB::LDS_LD>(st, fb_off, j, kg);
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j) mma(acc[i][j], fa[i], fb[j]);
            }
            if (it0 + 1 < n_iter) {
                char *nx = lds + (cur ^ 1) * Cfg::STAGE_BYTES;
                TileA::store_lds(ra[0], nx, tid);
                TileB::store_lds(rb[0], nx + TileA::LDS_BYTES, tid);
            }
            __syncthreads();
            cur ^= 1;
        } else {
#pragma unroll
            for (int q = 0; q < PF; ++q)
                if (it0 + q < n_iter) body(it0 + q, ra[q], rb[q], ra[(q + 1) % PF], rb[(q + 1) % PF]);
        }
    }

    write_back<T, FM, FN, false>(acc, args, row0 + wm * Cfg::TM, col0 + wn * Cfg::TN, batch, split, lane);
}

// Split-K reduction: C = alpha * sum_s ws[s] + beta * C, splits added in ascending order so the
// result does not depend on scheduling.  The workspace is [split][batch][n][m] fp32, dense, so four consecutive
// rows of one column are one 16-byte load per split; a thread owns such a group when m % 4 == 0 (VEC4), one
// element otherwise.  All loads of a thread are independent and issued before the first add (the loop over the
// splits is unrolled for the split factors the library uses); the adds keep the order.
template <typename T, bool VEC4>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const GemmArgs args)
{
    constexpr int W = VEC4 ? 4 : 1;
    const size_t mn = (size_t)args.m * args.n;
    const size_t idx = ((size_t)blockIdx.x * 256 + threadIdx.x) * W;
    const uint32_t batch = blockIdx.z;
    if (idx >= mn) return;
    const uint32_t row = (uint32_t)(idx % args.m), col = (uint32_t)(idx / args.m);
    const size_t stride = (size_t)args.batch * mn;                  // one split further
    const float *w = args.ws + (size_t)batch * mn + idx;
    float s[W];
#pragma unroll
    for (int e = 0; e < W; ++e) s[e] = 0.0f;
    auto add_splits = [&](auto NS, uint32_t first) {
        constexpr int ns = decltype(NS)::value;
        float v[ns][W];
#pragma unroll
        for (int q = 0; q < ns; ++q) {
            const float *p = w + (size_t)(first + q) * stride;
            if constexpr (VEC4) {
                f32x4 t = *reinterpret_cast<const f32x4 *>(p);
                v[q][0] = t[0]; v[q][1] = t[1]; v[q][2] = t[2]; v[q][3] = t[3];
            } else {
                v[q][0] = *p;
            }
        }
#pragma unroll
        for (int q = 0; q < ns; ++q)
#pragma unroll
            for (int e = 0; e < W; ++e) s[e] += v[q][e];
    };
    uint32_t sp = 0;
    for (; sp + 8 <= args.splits; sp += 8) add_splits(std::integral_constant<int, 8>{}, sp);
    if (sp + 4 <= args.splits) { add_splits(std::integral_constant<int, 4>{}, sp); sp += 4; }
    if (sp + 2 <= args.splits) { add_splits(std::integral_constant<int, 2>{}, sp); sp += 2; }
    if (sp < args.splits) add_splits(std::integral_constant<int, 1>{}, sp);

    T *p = static_cast<T *>(args.C) + (int64_t)batch * args.strideC + (size_t)col * args.ldc + row;
    const float alpha = args.alpha, beta = args.beta;
    if (VEC4 && args.vec_c) {
        typedef typename std::conditional<sizeof(T) == 4, u32x4, u32x2>::type cvec;
        union { T e[4]; cvec v; } io;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = alpha * s[e];
        if (beta != 0.0f) {
            io.v = *reinterpret_cast<const cvec *>(p);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = __builtin_fmaf(beta, (float)io.e[e], o[e]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) io.e[e] = (T)o[e];
        *reinterpret_cast<cvec *>(p) = io.v;
    } else {
#pragma unroll
        for (int e = 0; e < W; ++e) {
            float o = alpha * s[e];
            if (beta != 0.0f) o = __builtin_fmaf(beta, (float)p[e], o);
            p[e] = (T)o;
        }
    }
}

}  // namespace mmbo
