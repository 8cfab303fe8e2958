// HGEMM 256 x 256 ring kernel, variant for NN and TT: the k-contiguous operand is fetched in units of 64 k
// (128-byte rows) instead of slices of 32 k (64-byte rows).
//
// Why: a 64-byte row segment is half a cache line, so the slice ring asks L2 for every line of the
// k-contiguous operand twice (one 64-byte request per slice); measured on MI355X the NT layout, whose
// operands both arrive as 512-byte segments, ran 10 % faster than NN at the same LDS and MFMA work, and the
// kernel is power-bound (clock x MFMA-busy is constant), so fewer L2 transactions per byte is what is left.
// Here every request of the k-contiguous operand covers a whole 128-byte line.
//
// LDS (160 KB): the row-contiguous operand keeps a ring of four 16 KB slices; the k-contiguous operand has
// three 32 KB unit buffers.  Unit u = slices 2u, 2u+1.  Half of a unit (rows 0-127 or 128-255, all 64 k) is
// fetched per iteration, so every iteration still issues the same four direct loads per thread:
//   iteration s = 2u   : A-side slice s+4, second half of unit u+2
//   iteration s = 2u+1 : A-side slice s+4, first half of unit u+3
// A unit buffer is free once both its slices are in registers (after iteration 2u); unit u+3 reuses the buffer of
// unit u.  Everything a slice needs was issued at least three iterations before it is read, so at the end of
// iteration s the wait is for all loads but those of iterations s-1 and s.
#pragma once

#include "gemm_ring.hpp"

namespace mmbo {

namespace ring {

// k-contiguous operand in 64-k units: 256 rows x 128 bytes; chunk c (16 B) of row r sits at c ^ ((r >> 1) & 7).
struct WideTile {
    static constexpr int R = 256, UNIT_BYTES = R * 128, NBUF = 3, LPW = 2;   // 16 load instructions per half unit / 8 waves
    __device__ static inline uint32_t off(uint32_t row, uint32_t chunk) { return row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4); }
    // global byte offset, inside one unit, of the chunk thread (wave, lane) fetches with load i of half 0;
    // half 1 is 128 rows further
    __device__ static inline uint32_t load_goff(int wave, int lane, int i, uint32_t ld)
    {
        uint32_t row = (wave * LPW + i) * 8 + (lane >> 3);
        uint32_t chunk = (lane & 7) ^ ((row >> 1) & 7);
        return row * ld * 2 + chunk * 16;
    }
};

template <int F>
struct WideFrags {
    static constexpr int NOPS = 2 * F;
    u32x4 x[2][F];
    struct Addr { uint32_t a[2]; };            // per k-group, for the first slice of a unit
    __device__ static inline Addr make_addr(int lane, int r0)
    {
        Addr ad;
        uint32_t r = lane & 31, g = lane >> 5;
#pragma unroll
        for (int kg = 0; kg < 2; ++kg) ad.a[kg] = WideTile::off(r0 + r, kg * 2 + g);
        return ad;
    }
    // SUB = which slice of the unit (0: k 0-31, 1: k 32-63): chunk index + 4, i.e. address bit 6 flipped
    template <int OP, int SUB>
    __device__ __forceinline__ void read_op(uint32_t unit, const Addr &ad)
    {
        constexpr int kg = OP / F, f = OP % F;
        x[kg][f] = lds_read_b128<f * 32 * 128>(unit + (ad.a[kg] ^ (SUB * 64)));
    }
};

}  // namespace ring

template <bool TRANS, int ABLATE = 0>     // TRANS = false: NN (A row-contiguous, B wide);  true: TT (A wide, B row-contiguous)
__global__ void __launch_bounds__(512)
hgemm_ring_wide_kernel(const GemmArgs args)
{
    using namespace ring;
    using T = half_t;
    constexpr int BM = 256, BN = 256, BK = 32, NW = 8, DA = 4;
    // wave tile: the operand with transposing reads (the row-contiguous one) gets the fewer fragments
    constexpr int WM = TRANS ? 2 : 4, WN = TRANS ? 4 : 2;
    constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
    using TileR = RingTile<T, false, 256, NW>;                       // row-contiguous operand, slice ring
    using FragR = SliceFrags<T, false, 256, NW, TRANS ? FN : FM>;
    using FragW = WideFrags<TRANS ? FM : FN>;
    constexpr int RING_BYTES = DA * TileR::BYTES;                    // 64 KB, then three 32 KB units
    constexpr int BATCH = TileR::LPW + WideTile::LPW;                // 4 direct loads per thread per iteration
    constexpr int NMFMA = 2 * FM * FN;

    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    uint32_t wg0, wg1, tile_id, batch, nxcd;
    work_of_block(args, blockIdx.x, blockIdx.z, tile_id, batch, nxcd);
    wg_remap(tile_id, args.nwg0, args.nwg1, args.wgm, nxcd, wg0, wg1);
    const uint32_t row0 = wg0 * BM, col0 = wg1 * BN;
    const uint32_t lda = args.lda, ldb = args.ldb;
    const int n_slice = (int)(args.k / BK);                           // even, >= 8 (checked by the dispatcher)

    // R = the row-contiguous operand (A for NN, B for TT), W = the k-contiguous one
    const uint32_t ldr = TRANS ? ldb : lda, ldw = TRANS ? lda : ldb;
    const char *gR = TRANS ? static_cast<const char *>(args.B) + ((int64_t)batch * args.strideB + col0) * 2
                           : static_cast<const char *>(args.A) + ((int64_t)batch * args.strideA + row0) * 2;
    const char *gW = TRANS ? static_cast<const char *>(args.A) + ((int64_t)batch * args.strideA + (int64_t)row0 * lda) * 2
                           : static_cast<const char *>(args.B) + ((int64_t)batch * args.strideB + (int64_t)col0 * ldb) * 2;
    const int64_t stepR = (int64_t)BK * ldr * 2;                      // one slice further along k
    const int64_t stepW = 2 * BK * 2;                                 // one unit further along k
    const int64_t halfW = (int64_t)128 * ldw * 2;                     // second half of a unit: 128 rows further

    uint32_t offR[TileR::LPW], offW[WideTile::LPW];
#pragma unroll
    for (int i = 0; i < TileR::LPW; ++i) offR[i] = TileR::load_goff(wave, lane, i, ldr);
#pragma unroll
    for (int i = 0; i < WideTile::LPW; ++i) offW[i] = WideTile::load_goff(wave, lane, i, ldw);

    auto load_r = [&](int l, int slice, int rbuf) {
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void *)(gR + (int64_t)slice * stepR + offR[l]),
            MMBO_LDS_PTR(lds + rbuf * TileR::BYTES + (wave * TileR::LPW + l) * 1024), 16, 0, 0);
    };
    auto load_w = [&](int l, int unit, int half, int ubuf) {
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void *)(gW + (int64_t)unit * stepW + half * halfW + offW[l]),
            MMBO_LDS_PTR(lds + RING_BYTES + ubuf * WideTile::UNIT_BYTES + (half * 16 + wave * WideTile::LPW + l) * 1024),
            16, 0, 0);
    };

    const typename FragR::Addr adR = FragR::make_addr(lane, TRANS ? wn * TN : wm * TM);
    const typename FragW::Addr adW = FragW::make_addr(lane, TRANS ? wm * TM : wn * TN);
    FragR fr[2];
    FragW fw[2];

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const uint32_t lds_base = (uint32_t)(uintptr_t)MMBO_LDS_PTR(lds);
    constexpr int NRR = FragR::NOPS, NR = FragR::NOPS + FragW::NOPS;

    // MFMAs of the slice in (cr, cw), interleaved with the fragment reads of the next slice into (nr, nw)
    // and this iteration's four direct loads.  SUB = which half (along k) of its unit the next slice is.
    auto body = [&](auto SUBC, const FragR &cr, const FragW &cw, FragR &nr, FragW &nw, int rbuf_read, int ubuf_read,
                    bool ld_r, int r_slice, int r_buf, bool ld_w, int w_unit, int w_half, int w_buf) {
        constexpr int SUB = decltype(SUBC)::value;
        const uint32_t tr = lds_base + rbuf_read * TileR::BYTES;
        const uint32_t tw = lds_base + RING_BYTES + ubuf_read * WideTile::UNIT_BYTES;
        static_for<NMFMA>([&](auto M) {
            constexpr int m = decltype(M)::value;
            constexpr int kg = m / (FM * FN), i = (m / FN) % FM, j = m % FN;
            if constexpr (!(ABLATE & 4)) {
                const u32x4 &a = TRANS ? cw.x[kg][i] : cr.x[kg][i];
                const u32x4 &b = TRANS ? cr.x[kg][j] : cw.x[kg][j];
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b),
                                                                   acc[i][j], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (!(ABLATE & 2)) {
                constexpr int r0 = NR * m / NMFMA, r1 = NR * (m + 1) / NMFMA;
                static_for<r1 - r0>([&](auto RR) {
                    constexpr int r = r0 + decltype(RR)::value;
                    if constexpr (r < NRR) nr.template read_op<r>(tr, adR);
                    else nw.template read_op<r - NRR, SUB>(tw, adW);
                });
            }
            if constexpr (!(ABLATE & 1)) {
                constexpr int l0 = (2 * BATCH * m + NMFMA) / (2 * NMFMA), l1 = (2 * BATCH * (m + 1) + NMFMA) / (2 * NMFMA);
                static_for<l1 - l0>([&](auto LL) {
                    constexpr int l = l0 + decltype(LL)::value;
                    if constexpr (l < TileR::LPW) { if (ld_r) load_r(l, r_slice, r_buf); }
                    else if constexpr (l < BATCH) { if (ld_w) load_w(l - TileR::LPW, w_unit, w_half, w_buf); }
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

    // prologue = "iterations" -5 .. -1 of the steady-state pattern
    if constexpr (!(ABLATE & 1)) {
#pragma unroll
        for (int l = 0; l < WideTile::LPW; ++l) load_w(l, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int l = 0; l < TileR::LPW; ++l) load_r(l, t, t);
            const int unit = (t + 1) / 2, half = (t + 1) & 1;        // u0h1, u1h0, u1h1, u2h0
#pragma unroll
            for (int l = 0; l < WideTile::LPW; ++l) load_w(l, unit, half, unit);
        }
    }
    MMBO_WAIT_VM(3 * BATCH);                                         // slice 0 of both operands has landed
    MMBO_BARRIER();
    if constexpr (!(ABLATE & 2)) {
        static_for<FragR::NOPS>([&](auto OP) { fr[0].template read_op<decltype(OP)::value>(lds_base, adR); });
        static_for<FragW::NOPS>([&](auto OP) { fw[0].template read_op<decltype(OP)::value, 0>(lds_base + RING_BYTES, adW); });
    }
    MMBO_WAIT_LGKM0();
    MMBO_WAIT_VM(2 * BATCH);                                         // slice 1 too
    MMBO_BARRIER();

    int rb = 0;         // s % 4: ring buffer of slice s (free for slice s+4)
    int ub = 0;         // u % 3 for u = s / 2
    for (int s = 0; s < n_slice; s += 2) {
        const int u = s >> 1;
        {   // iteration s = 2u: next slice is the second half of unit u; fetch the second half of unit u+2
            const int ub2 = ub + 2 >= 3 ? ub - 1 : ub + 2;
            const bool ld_r = s + 4 < n_slice, ld_w = 2 * (u + 2) < n_slice;
            body(std::integral_constant<int, 1>{}, fr[0], fw[0], fr[1], fw[1], (rb + 1) & 3, ub,
                 ld_r, s + 4, rb, ld_w, u + 2, 1, ub2);
            MMBO_WAIT_LGKM0();
            if (ld_r && ld_w) MMBO_WAIT_VM(2 * BATCH); else MMBO_WAIT_VM(0);
            MMBO_BARRIER();
        }
        {   // iteration s+1 = 2u+1: next slice is the first half of unit u+1; fetch the first half of unit u+3
            const int ub1 = ub + 1 >= 3 ? 0 : ub + 1;
            const bool ld_r = s + 5 < n_slice, ld_w = 2 * (u + 3) < n_slice;
            body(std::integral_constant<int, 0>{}, fr[1], fw[1], fr[0], fw[0], (rb + 2) & 3, ub1,
                 ld_r, s + 5, (rb + 1) & 3, ld_w, u + 3, 0, ub);
            MMBO_WAIT_LGKM0();
            if (ld_r && ld_w) MMBO_WAIT_VM(2 * BATCH); else MMBO_WAIT_VM(0);
            MMBO_BARRIER();
            ub = ub1;
        }
        rb = (rb + 2) & 3;
    }
    if constexpr (ABLATE & 8) {
        if (tid == 0 && blockIdx.x == args.nwg0 * args.nwg1 / 3) {
            reinterpret_cast<long long *>(args.ws)[0] = clock64() - t_clk;
            reinterpret_cast<long long *>(args.ws)[1] = wall_clock64() - t_wall;
        }
    }
#undef MMBO_BARRIER
#undef MMBO_WAIT_VM
#undef MMBO_WAIT_LGKM0

    write_back<T, FM, FN, true>(acc, args, row0 + wm * TM, col0 + wn * TN, batch, 0, lane);
}

}  // namespace mmbo
