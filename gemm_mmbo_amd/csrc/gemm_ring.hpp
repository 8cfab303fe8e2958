// HGEMM fast path for gfx950: 256 x 256 macro tile, 8 wavefronts, K consumed in slices of 32 through a
// five-deep ring of LDS buffers filled by global->LDS direct loads, fragments double-buffered in registers.
//
// It serves problems whose m and n are multiples of 256, k a multiple of 32, and whose operands are
// 16-byte aligned; everything else takes the staged kernel (gemm_staged.hpp).
//
// The reference's recipe (src/gemm/ref/Kernels.cpp:412-747: global prefetch ahead of use, LDS multi-buffer,
// LDS->register prefetch of the next k step while the current one is multiplied) mapped onto CDNA4:
//   - global -> LDS: global_load_lds_dwordx4; no register staging, no LDS write instructions.  Each lane
//     fetches the 16-byte chunk whose XOR-swizzled LDS slot is (wave, instruction, lane); the swizzle
//     removes the bank conflicts that padding would (a direct load writes 1 KB contiguously, so rows
//     cannot be padded).
//   - measured on MI355X, a 64 KB batch of such loads takes about 3,000 clocks to land when all 256 CUs
//     stream (most requests hit in L2 but wait on lines a neighbour's miss is still fetching), while one
//     slice is multiplied in about 1,000.  The ring therefore keeps four slices (128 KB) in flight per CU and
//     gives each batch three slice times to land: 5 x 32 KB = all 160 KB of LDS.
//   - each wavefront issues the LDS fragment reads of slice s+1 into its second register set, then the 16
//     MFMAs of slice s from the first; one barrier per slice hands buffers over.
#pragma once

#include <type_traits>
#include <utility>

#include "gemm_common.hpp"

namespace mmbo {

namespace ring {

constexpr int BM = 256, BN = 256, BK = 32, NT = 512;
constexpr int DEPTH = 5;                         // ring buffers
constexpr int TILE_BYTES = 256 * BK * 2;         // one operand tile of one slice: 16 KB
constexpr int SLICE_BYTES = 2 * TILE_BYTES;      // A then B: 32 KB
constexpr int LDS_BYTES = DEPTH * SLICE_BYTES;   // 160 KB
constexpr int LOADS = 2;                         // direct loads per thread per operand per slice

// ---- swizzled tile layouts (byte offsets inside a 16 KB operand tile) -------------------------------
// KC (source contiguous along k): row r holds its 32 k values in 64 bytes = 4 chunks of 16 B; chunk c is
//   stored at position c ^ ((r >> 2) & 3), so 16 consecutive rows reading the same logical chunk cover
//   all sixteen 16-byte groups of the 256-byte-wide LDS.
__device__ inline uint32_t kc_off(uint32_t row, uint32_t chunk) { return row * 64 + ((chunk ^ ((row >> 2) & 3)) << 4); }
// RC (source contiguous along the row index): k-row k holds 256 rows in 512 bytes = 32 chunks; chunk c is
//   stored at c ^ ((k & 3) << 2): the four k-rows one transposing read touches land in different groups.
__device__ inline uint32_t rc_off(uint32_t k, uint32_t chunk) { return k * 512 + ((chunk ^ ((k & 3) << 2)) << 4); }

// Global byte offset (from the tile origin of this slice) of the chunk thread (wave, lane) must fetch with
// its i-th direct load so that it lands in LDS slot (wave*LOADS + i)*64 + lane.
template <bool KC>
__device__ inline uint32_t load_goff(int wave, int lane, int i, uint32_t ld)
{
    if (KC) {
        uint32_t row = (wave * LOADS + i) * 16 + (lane >> 2);
        uint32_t chunk = (lane & 3) ^ ((row >> 2) & 3);
        return (row * ld + chunk * 8) * 2;
    }
    uint32_t k = (wave * LOADS + i) * 2 + (lane >> 5);
    uint32_t chunk = (lane & 31) ^ ((k & 3) << 2);
    return (k * ld + chunk * 8) * 2;
}

template <int N, typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl<N>(static_cast<F &&>(f), std::make_integer_sequence<int, N>{});
}

// LDS reads are inline assembly with explicit s_waitcnt: the compiler cannot tell that a fragment read
// never aliases an in-flight direct load (they target different ring buffers) and would otherwise drain
// vmcnt before every read, which would serialise the ring.
template <int OFF>
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr)
{
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
template <int OFF>
__device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t addr)
{
    u32x2 r;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}

// One operand of one wavefront for one slice: F row-blocks of 32 x 2 k-groups of 16, fetched by NOPS
// separate LDS reads so the caller can spread them between MFMAs.
template <bool KC, int F>
struct SliceFrags {
    static constexpr int NOPS = KC ? 2 * F : 4 * F;
    u32x4 x[2][KC ? F : 1];          // KC: one 128-bit read per fragment
    u32x2 y[2][KC ? 1 : F][2];       // RC: two transposing 64-bit reads per fragment

    struct Addr { uint32_t a[KC ? 2 : F]; };      // per-lane byte offsets inside the operand tile

    __device__ static inline Addr make_addr(int lane, int r0)
    {
        Addr ad;
        if constexpr (KC) {
            uint32_t r = lane & 31, g = lane >> 5;
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) ad.a[kg] = kc_off(r0 + r, kg * 2 + g);      // + f*32*64 per block
        } else {
            // transposing read: lane j of a 16-lane block points at k-row j/4, rows 4*(j%4)..+3, and
            // receives (k-rows 0..3) x (row j)
            uint32_t j = lane & 15, blk = (lane >> 4) & 1, g = lane >> 5;
#pragma unroll
            for (int f = 0; f < F; ++f) {
                uint32_t m = r0 + f * 32 + blk * 16 + (j & 3) * 4;
                uint32_t k = g * 8 + (j >> 2);                                         // + kg*16 + h*4
                ad.a[f] = rc_off(k, m >> 3) + (m & 7) * 2;
            }
        }
        return ad;
    }

    // tile = LDS byte address of the operand tile (wave-uniform); OP in [0, NOPS)
    template <int OP>
    __device__ __forceinline__ void read_op(uint32_t tile, const Addr &ad)
    {
        if constexpr (KC) {
            constexpr int kg = OP / F, f = OP % F;
            x[kg][f] = lds_read_b128<f * 32 * 64>(tile + ad.a[kg]);
        } else {
            constexpr int kg = OP / (2 * F), f = (OP / 2) % F, h = OP % 2;
            y[kg][f][h] = lds_read_tr16_b64<kg * 16 * 512 + h * 4 * 512>(tile + ad.a[f]);
        }
    }
    __device__ __forceinline__ void read_all(uint32_t tile, const Addr &ad)
    {
        static_for<NOPS>([&](auto OP) { this->template read_op<decltype(OP)::value>(tile, ad); });
    }
    __device__ __forceinline__ f16x8 get(int kg, int f) const
    {
        if constexpr (KC) return __builtin_bit_cast(f16x8, x[kg][f]);
        else return __builtin_bit_cast(f16x8, u32x4{y[kg][f][0][0], y[kg][f][0][1], y[kg][f][1][0], y[kg][f][1][1]});
    }
};

}  // namespace ring

// WM x WN wavefronts; wave tile (256/WM) x (256/WN).  WM*WN == 8.
// ABLATE is a timing probe in the spirit of the reference's error_kernel_000.s / test_main_loop.s (kernels
// with parts removed to find the ceiling of what is left; results are wrong by design): bit 0 drops the
// global->LDS loads, bit 1 the LDS fragment reads, bit 2 the MFMAs, bit 3 writes the main loop's clock64 and
// wall_clock64 spans to args.ws, bit 6 makes every work-group read the same tiles.  The library only instantiates ABLATE = 0.
template <bool TA, bool TB, int WM, int WN, int ABLATE = 0>
__global__ void __launch_bounds__(512)
hgemm_ring_kernel(const GemmArgs args)
{
    using namespace ring;
    static_assert(WM * WN == 8, "eight wavefronts");
    constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
    constexpr bool A_KC = TA, B_KC = !TB;
    using FragA = SliceFrags<A_KC, FM>;
    using FragB = SliceFrags<B_KC, FN>;

    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    uint32_t wg0, wg1;
    wg_remap(blockIdx.x, args.nwg0, args.nwg1, args.wgm, args.nxcd, wg0, wg1);
    if constexpr (ABLATE & 64) { wg0 = 0; wg1 = 0; }          // probe: every work-group reads the same tiles
    const uint32_t batch = blockIdx.z;
    const uint32_t row0 = wg0 * BM, col0 = wg1 * BN;
    const uint32_t lda = args.lda, ldb = args.ldb;
    const int n_slice = (int)(args.k / BK);

    const char *gA = static_cast<const char *>(args.A) +
                     ((int64_t)batch * args.strideA + (TA ? (int64_t)row0 * lda : (int64_t)row0)) * 2;
    const char *gB = static_cast<const char *>(args.B) +
                     ((int64_t)batch * args.strideB + (TB ? (int64_t)col0 : (int64_t)col0 * ldb)) * 2;
    const int64_t stepA = (TA ? (int64_t)BK : (int64_t)BK * lda) * 2;
    const int64_t stepB = (TB ? (int64_t)BK * ldb : (int64_t)BK) * 2;

    uint32_t offA[LOADS], offB[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        offA[i] = load_goff<A_KC>(wave, lane, i, lda);
        offB[i] = load_goff<B_KC>(wave, lane, i, ldb);
    }
    // slice s goes to ring buffer s % DEPTH; `buf` is that index, kept by the caller
    auto issue_slice = [&](int s, int buf) {
        if constexpr (ABLATE & 1) return;
        char *dst = lds + buf * SLICE_BYTES;
        const char *pa = gA + (int64_t)s * stepA, *pb = gB + (int64_t)s * stepB;
#pragma unroll
        for (int i = 0; i < LOADS; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(pa + offA[i]),
                                             MMBO_LDS_PTR(dst + (wave * LOADS + i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < LOADS; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(pb + offB[i]),
                                             MMBO_LDS_PTR(dst + TILE_BYTES + (wave * LOADS + i) * 1024), 16, 0, 0);
    };
    constexpr int BATCH = 2 * LOADS;             // direct loads per thread per slice

    const typename FragA::Addr adA = FragA::make_addr(lane, wm * TM);
    const typename FragB::Addr adB = FragB::make_addr(lane, wn * TN);
    FragA fa[2];
    FragB fb[2];
    if constexpr (ABLATE != 0) {      // keep the probes' registers defined
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t va = 0x3c003c00u + (uint32_t)lane, vb = 0x38003800u + (uint32_t)lane;
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) {
#pragma unroll
                for (int f = 0; f < (A_KC ? FM : 1); ++f) fa[q].x[kg][f] = u32x4{va, va, va, va};
#pragma unroll
                for (int f = 0; f < (A_KC ? 1 : FM); ++f) fa[q].y[kg][f][0] = fa[q].y[kg][f][1] = u32x2{va, va};
#pragma unroll
                for (int f = 0; f < (B_KC ? FN : 1); ++f) fb[q].x[kg][f] = u32x4{vb, vb, vb, vb};
#pragma unroll
                for (int f = 0; f < (B_KC ? 1 : FN); ++f) fb[q].y[kg][f][0] = fb[q].y[kg][f][1] = u32x2{vb, vb};
            }
        }
    }

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const uint32_t lds_base = (uint32_t)(uintptr_t)MMBO_LDS_PTR(lds);
    auto read_slice = [&](FragA &a, FragB &b, int buf) {
        if constexpr (ABLATE & 2) return;
        const uint32_t t = lds_base + buf * SLICE_BYTES;
        a.read_all(t, adA);
        b.read_all(t + TILE_BYTES, adB);
    };
    // The 16 MFMAs of slice s with the LDS reads of slice s+1 spread between them.  Issued as one block, the
    // reads of all eight wavefronts would fill the LDS queue and each wavefront would sit behind its own
    // last read before reaching its first MFMA.
    constexpr int NA = FragA::NOPS, NR = FragA::NOPS + FragB::NOPS, NMFMA = 2 * FM * FN;
    auto mfma_and_read = [&](const FragA &ca, const FragB &cb, FragA &na, FragB &nb, int nbuf) {
        const uint32_t t = lds_base + nbuf * SLICE_BYTES;
        static_for<NMFMA>([&](auto M) {
            constexpr int m = decltype(M)::value;
            constexpr int kg = m / (FM * FN), i = (m / FN) % FM, j = m % FN;
            if constexpr (!(ABLATE & 4))
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ca.get(kg, i), cb.get(kg, j), acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!(ABLATE & 2)) {
                constexpr int r0 = NR * m / NMFMA, r1 = NR * (m + 1) / NMFMA;
                static_for<r1 - r0>([&](auto R) {
                    constexpr int r = r0 + decltype(R)::value;
                    if constexpr (r < NA) na.template read_op<r>(t, adA);
                    else nb.template read_op<r - NA>(t + TILE_BYTES, adB);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
#define MMBO_BARRIER()                           \
    do {                                         \
        __builtin_amdgcn_sched_barrier(0);       \
        __builtin_amdgcn_s_barrier();            \
        __builtin_amdgcn_sched_barrier(0);       \
    } while (0)
#define MMBO_WAIT_VM(n) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory")
#define MMBO_WAIT_LGKM0() asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory")

    long long t_clk = 0, t_wall = 0;
    if constexpr (ABLATE & 8) { t_clk = clock64(); t_wall = wall_clock64(); }

    // Invariant at the top of iteration s (after barrier B_s): register set s&1 holds slice s; slice s+1 is
    // resident in LDS; every wavefront has finished reading slices <= s, so buffer s % DEPTH is free; this
    // wavefront's loads of slices s+2 .. s+DEPTH-1 are in flight.
    //   iteration s:  issue loads(s+DEPTH) -> buffer s % DEPTH;  read slice s+1 -> set (s+1)&1;
    //                 MFMAs of slice s from set s&1;  wait reads;  wait own loads(s+2);  barrier B_{s+1}.
    // Loads return in order, so "all but the newest (DEPTH-2) batches" means loads(s+2) have landed; once
    // the tail stops issuing, the wait is for everything.
#pragma unroll
    for (int s = 0; s < DEPTH; ++s)
        if (s < n_slice) issue_slice(s, s);
    if (n_slice >= DEPTH) MMBO_WAIT_VM(BATCH * (DEPTH - 1)); else MMBO_WAIT_VM(0);
    MMBO_BARRIER();                                                  // slice 0 resident
    read_slice(fa[0], fb[0], 0);
    MMBO_WAIT_LGKM0();
    if (n_slice >= DEPTH) MMBO_WAIT_VM(BATCH * (DEPTH - 2)); else MMBO_WAIT_VM(0);
    MMBO_BARRIER();                                                  // slice 1 resident, slice 0 in registers

    int buf = 0;                                                     // s % DEPTH
    auto step = [&](int s, FragA &ca, FragB &cb, FragA &na, FragB &nb) {
        const int nbuf = buf + 1 == DEPTH ? 0 : buf + 1;
        const bool steady = s + DEPTH < n_slice;
        if (steady) issue_slice(s + DEPTH, buf);
        __builtin_amdgcn_sched_barrier(0);
        // (the last slice reads a stale buffer into the unused register set: harmless, and it keeps the
        // interleaved block free of branches)
        mfma_and_read(ca, cb, na, nb, nbuf);
        MMBO_WAIT_LGKM0();
        if (steady) MMBO_WAIT_VM(BATCH * (DEPTH - 2)); else MMBO_WAIT_VM(0);
        MMBO_BARRIER();
        buf = nbuf;
    };
    for (int s = 0; s < n_slice; s += 2) {
        step(s, fa[0], fb[0], fa[1], fb[1]);
        if (s + 1 < n_slice) step(s + 1, fa[1], fb[1], fa[0], fb[0]);
    }
    if constexpr (ABLATE & 8) {
        if (tid == 0 && blockIdx.x == 300) {
            reinterpret_cast<long long *>(args.ws)[0] = clock64() - t_clk;
            reinterpret_cast<long long *>(args.ws)[1] = wall_clock64() - t_wall;
        }
    }
#undef MMBO_BARRIER
#undef MMBO_WAIT_VM
#undef MMBO_WAIT_LGKM0

    // ---- write-back: same accumulator layout as the staged kernel; every tile is interior here.
    //   acc[i][j][4*q + r] is C(row0 + wm*TM + i*32 + 8*q + 4*(lane/32) + r,  col0 + wn*TN + j*32 + lane%32)
    const float alpha = args.alpha, beta = args.beta;
    const uint32_t ldc = args.ldc;
    half_t *C = static_cast<half_t *>(args.C) + (int64_t)batch * args.strideC;
    const int g = lane >> 5, cl = lane & 31;
    const bool vec_c = args.vec_c != 0;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            uint32_t col = col0 + wn * TN + j * 32 + cl;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                uint32_t row = row0 + wm * TM + i * 32 + 8 * q + 4 * g;
                half_t *p = C + (size_t)col * ldc + row;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = alpha * acc[i][j][4 * q + r];
                if (vec_c) {
                    union { half_t e[4]; u32x2 v2; } io;
                    if (beta != 0.0f) {                       // beta == 0: C is never read
                        io.v2 = *reinterpret_cast<const u32x2 *>(p);
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] = __builtin_fmaf(beta, (float)io.e[r], v[r]);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) io.e[r] = (half_t)v[r];
                    *reinterpret_cast<u32x2 *>(p) = io.v2;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float o = v[r];
                        if (beta != 0.0f) o = __builtin_fmaf(beta, (float)p[r], o);
                        p[r] = (half_t)o;
                    }
                }
            }
        }
}

}  // namespace mmbo
