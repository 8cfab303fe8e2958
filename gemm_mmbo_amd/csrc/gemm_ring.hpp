// Ring kernel for gfx950: the fast path for problems made of whole tiles (m % BM == 0, n % BN == 0,
// k % BK == 0 per split, A and B 16-byte aligned).  Everything else takes the staged kernel.
//
// K is consumed in slices of 64 bytes per row (BK = 32 halves / 16 floats) through a DEPTH-deep ring of LDS
// buffers filled by global->LDS direct loads; MFMA operand fragments are double-buffered in registers.
//
// The reference's recipe (src/gemm/ref/Kernels.cpp:412-747: global prefetch ahead of use, LDS multi-buffer,
// LDS->register prefetch of the next k step while the current one is multiplied) mapped onto CDNA4:
//   - global -> LDS: buffer_load_dwordx4 ... lds (the slice's origin in a scalar descriptor, a 32-bit offset per lane);
//     no register staging, no LDS write instructions, no vector address arithmetic in the loop.  Each lane
//     fetches the 16-byte chunk whose XOR-swizzled LDS slot is (wave, instruction, lane); the swizzle removes
//     the bank conflicts that padding would (a direct load writes 1 KB contiguously, so rows cannot be padded).
//   - measured on MI355X, a batch of direct loads takes about 3,000 clocks to land when all 256 CUs stream,
//     while a 256 x 256 fp16 slice is multiplied in about 1,000: the ring keeps DEPTH-1 slices in flight per
//     work-group and gives each batch DEPTH-2 slice times to land.
//   - each wavefront issues its share of slice s+DEPTH, then the MFMAs of slice s from one register set with
//     the LDS fragment reads of slice s+1 (into the other set) spread between them, then one barrier.
#pragma once

#include <type_traits>
#include <utility>

#include "gemm_common.hpp"

namespace mmbo {

namespace ring {

template <typename T> struct Slice;
template <> struct Slice<half_t> { static constexpr int BK = 32; };
template <> struct Slice<float>  { static constexpr int BK = 16; };

template <int N, typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (N > 0) static_for_impl<N>(static_cast<F &&>(f), std::make_integer_sequence<int, N>{});
}

// LDS reads are inline assembly with explicit s_waitcnt: the compiler cannot tell that a fragment read never
// aliases an in-flight direct load (they target different ring buffers) and would otherwise drain vmcnt
// before every read, which would serialise the ring.
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
template <int OFF>
__device__ __forceinline__ uint32_t lds_read_b32(uint32_t addr)
{
    uint32_t r;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}

// A work-group-uniform address as a scalar value (both halves through readfirstlane: the compiler then keeps what is
// derived from it in scalar registers, where a buffer descriptor must live).
__device__ __forceinline__ uint64_t uniform_address(const void *p)
{
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// The direct loads are buffer loads that write LDS (buffer_load_dwordx4 ... lds): 16 bytes per lane from
//     descriptor origin + scalar offset + the lane's 32-bit byte offset      to      LDS at M0 + lane * 16.
// An operand's descriptor lives in four scalar registers and is that operand's cursor: its origin is the next slice to be
// requested and moves on by two scalar adds per slice; the lane offsets never change.  So the slice loop spends no
// vector instruction on addresses (the global form of the load takes a 64-bit address per lane: three 64-bit vector adds
// per pair of loads), and a load is three instructions in all -- M0, the wait state the hardware wants after a write to
// M0, the load -- written as one asm statement so that nothing else lands between the MFMAs around it.  The statement
// leaves M0 changed without saying so (the compiler refuses M0 in a clobber list): these kernels contain no other
// instruction that reads M0, which tests/test_kernel_asm.py checks on the generated assembly.
// The descriptor's range is the 2 GiB a tile's span of an operand is limited to, so it never clips; its last word is the
// raw 32-bit format of this chip family.
__device__ __forceinline__ u32x4 slice_cursor(uint64_t origin)
{
    return u32x4{(uint32_t)origin, (uint32_t)(origin >> 32) & 0xffffu, 0x7fffffffu, 0x00020000u};
}
__device__ __forceinline__ void advance(u32x4 &cursor, uint64_t bytes)
{
    const uint64_t o = (((uint64_t)cursor[1] << 32) | cursor[0]) + bytes;       // (bits 48..63 of the second word stay zero)
    cursor[0] = (uint32_t)o;
    cursor[1] = (uint32_t)(o >> 32);
}
// lds_addr: work-group-uniform LDS byte address.  AHEAD = false: the slice at the cursor; true: the slice `step` bytes
// further (step < 2 GiB by the tile-span limit).  (M0 is written with s_mov, which leaves the condition code alone: the
// statement then writes nothing the compiler knows of, and two of them in a row are not padded apart.)
template <bool AHEAD>
__device__ __forceinline__ void direct_load16(const u32x4 &cursor, uint32_t step, uint32_t lane_offset, uint32_t lds_addr)
{
    if constexpr (AHEAD)
        asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
                     :: "v"(lane_offset), "s"(cursor), "s"(step), "s"(lds_addr) : "memory");
    else
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, 0 offen lds"
                     :: "v"(lane_offset), "s"(cursor), "s"(lds_addr) : "memory");
}

// The same load in two statements, for callers that put another asm statement (an MFMA) between them: that statement is
// then the wait state between the write to M0 and the load, and the s_nop is saved.  The caller guarantees that at least
// one instruction it controls sits between the two.
__device__ __forceinline__ void set_lds_destination(uint32_t lds_addr) { asm volatile("s_mov_b32 m0, %0" :: "s"(lds_addr)); }
template <bool AHEAD>
__device__ __forceinline__ void direct_load16_to_destination(const u32x4 &cursor, uint32_t step, uint32_t lane_offset)
{
    if constexpr (AHEAD) asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" :: "v"(lane_offset), "s"(cursor), "s"(step) : "memory");
    else asm volatile("buffer_load_dwordx4 %0, %1, 0 offen lds" :: "v"(lane_offset), "s"(cursor) : "memory");
}

// One operand tile of one slice: R rows x BK along k = R * 64 bytes, loaded by NW wavefronts.
//   KC (source contiguous along k): LDS row r = its 64 bytes = 4 chunks of 16 B; chunk c sits at position
//     c ^ ((r >> 2) & 3), so 16 consecutive rows reading the same logical chunk cover all sixteen 16-byte
//     groups of the 256-byte-wide LDS.
//   RC (source contiguous along the row index): LDS k-row = R elements; its chunks are XOR-swizzled with a
//     mask that depends on k so that the k-rows one fragment read touches fall in different bank groups:
//       fp16 (ds_read_b64_tr_b16 reads four consecutive k-rows x 32 B): mask from k & 3;
//       fp32 (ds_read_b32: lanes 0-31 one k-row, lanes 32-63 the k-row four further): mask from (k >> 2) & 1.
template <typename T, bool KC, int R, int NW>
struct RingTile {
    static constexpr int ESZ = sizeof(T);
    static constexpr int BK = Slice<T>::BK;
    static constexpr int BYTES = R * 64;
    static constexpr int INSTRS = R / 16;                    // direct-load instructions (1 KB each) per slice
    static_assert(INSTRS % NW == 0, "tile must split evenly over the wavefronts");
    static constexpr int LPW = INSTRS / NW;                  // loads per thread per slice
    static constexpr int ROW_BYTES = R * ESZ;                // RC: one k-row
    static constexpr int CPR = ROW_BYTES / 16;               // RC: chunks per k-row
    static constexpr int KPI = 1024 / ROW_BYTES;             // RC: k-rows per load instruction
    static_assert(KC || (ROW_BYTES <= 1024 && 1024 % ROW_BYTES == 0 && CPR >= (ESZ == 4 ? 16 : 8)),
                  "RC tile: a k-row must be 128 (fp16) or 256 .. 1024 bytes, a power of two");

    __device__ static inline uint32_t rc_mask(uint32_t k)
    {
        if constexpr (ESZ == 4) return ((k >> 2) & 1) << 3;                  // shift by 128 B
        else if constexpr (ROW_BYTES % 256 == 0) return (k & 3) << 2;        // shift by 64 B per k
        else if constexpr (ROW_BYTES % 256 == 128) return ((k >> 1) & 1) << 2;
        else return 0;
    }
    __device__ static inline uint32_t kc_off(uint32_t row, uint32_t chunk) { return row * 64 + ((chunk ^ ((row >> 2) & 3)) << 4); }
    __device__ static inline uint32_t rc_off(uint32_t k, uint32_t chunk) { return k * ROW_BYTES + ((chunk ^ rc_mask(k)) << 4); }

    // Global byte offset (from the tile origin of this slice) of the chunk thread (wave, lane) must fetch with
    // its i-th direct load so that it lands in LDS slot (wave*LPW + i)*64 + lane.
    __device__ static inline uint32_t load_goff(int wave, int lane, int i, uint32_t ld)
    {
        const uint32_t q = wave * LPW + i;
        if constexpr (KC) {
            uint32_t row = q * 16 + (lane >> 2);
            uint32_t chunk = (lane & 3) ^ ((row >> 2) & 3);
            return row * ld * ESZ + chunk * 16;
        } else {
            uint32_t k = q * KPI + lane / CPR;
            uint32_t chunk = (lane % CPR) ^ rc_mask(k);
            return k * ld * ESZ + chunk * 16;
        }
    }
};

// Fragments of one operand of one wavefront for one slice: F row-blocks of 32 x 2 k-groups.  A k-group is what one
// 128-bit register quad per lane feeds: 16 k values (one 32x32x16 f16 MFMA) or 8 (four 32x32x2 f32 MFMAs).
// Lane group g = lane/32, element e holds k = kg*KG + g*VEC + e, for both operands alike.
template <typename T, bool KC, int R, int NW, int F>
struct SliceFrags {
    using Tile = RingTile<T, KC, R, NW>;
    static constexpr int ESZ = sizeof(T);
    static constexpr int RPF = KC ? 1 : (ESZ == 2 ? 2 : 4);     // LDS reads per fragment
    static constexpr int NOPS = 2 * F * RPF;
    u32x4 x[2][F];

    struct Addr { uint32_t a[KC ? 2 : F]; };                    // per-lane byte offsets inside the operand tile

    __device__ static inline Addr make_addr(int lane, int r0)
    {
        Addr ad;
        if constexpr (KC) {
            uint32_t r = lane & 31, g = lane >> 5;
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) ad.a[kg] = Tile::kc_off(r0 + r, kg * 2 + g);   // + f*32*64 per block
        } else if constexpr (ESZ == 2) {
            // transposing read: lane j of a 16-lane block points at k-row j/4, rows 4*(j%4)..+3, and receives
            // (k-rows 0..3) x (row j)
            uint32_t j = lane & 15, blk = (lane >> 4) & 1, g = lane >> 5;
#pragma unroll
            for (int f = 0; f < F; ++f) {
                uint32_t m = r0 + f * 32 + blk * 16 + (j & 3) * 4;
                uint32_t k = g * 8 + (j >> 2);                                           // + kg*16 + h*4
                ad.a[f] = Tile::rc_off(k, m >> 3) + (m & 7) * 2;
            }
        } else {
            uint32_t r = lane & 31, g = lane >> 5;
#pragma unroll
            for (int f = 0; f < F; ++f) {
                uint32_t m = r0 + f * 32 + r;
                uint32_t k = g * 4;                                                      // + kg*8 + t
                ad.a[f] = Tile::rc_off(k, m >> 2) + (m & 3) * 4;
            }
        }
        return ad;
    }

    // tile = LDS byte address of the operand tile (wave-uniform); OP in [0, NOPS)
    template <int OP>
    __device__ __forceinline__ void read_op(uint32_t tile, const Addr &ad)
    {
        constexpr int kg = OP / (F * RPF), f = (OP / RPF) % F, h = OP % RPF;
        if constexpr (KC) {
            x[kg][f] = lds_read_b128<f * 32 * 64>(tile + ad.a[kg]);
        } else if constexpr (ESZ == 2) {
            u32x2 v = lds_read_tr16_b64<(kg * 16 + h * 4) * Tile::ROW_BYTES>(tile + ad.a[f]);
            x[kg][f][2 * h] = v[0];
            x[kg][f][2 * h + 1] = v[1];
        } else {
            x[kg][f][h] = lds_read_b32<(kg * 8 + h) * Tile::ROW_BYTES>(tile + ad.a[f]);
        }
    }
    __device__ __forceinline__ void read_all(uint32_t tile, const Addr &ad)
    {
        static_for<NOPS>([&](auto OP) { this->template read_op<decltype(OP)::value>(tile, ad); });
    }
};

}  // namespace ring

template <typename T, bool TA, bool TB, int BM, int BN, int WM, int WN, int DEPTH>
struct RingCfg {
    static constexpr int NW = WM * WN, NT = NW * 64;
    static constexpr int BK = ring::Slice<T>::BK;
    static constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 32, FN = TN / 32;
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA block");
    using TileA = ring::RingTile<T, TA, BM, NW>;       // A is k-contiguous when transposed
    using TileB = ring::RingTile<T, !TB, BN, NW>;      // B is k-contiguous when not transposed
    using FragA = ring::SliceFrags<T, TA, BM, NW, FM>;
    using FragB = ring::SliceFrags<T, !TB, BN, NW, FN>;
    static constexpr int SLICE_BYTES = TileA::BYTES + TileB::BYTES;
    static constexpr int LDS_BYTES = DEPTH * SLICE_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "ring does not fit the 160 KB of LDS");
    static constexpr int BATCH = TileA::LPW + TileB::LPW;      // direct loads per thread per slice
    static constexpr int MPK = sizeof(T) == 2 ? 1 : 4;         // MFMAs per (k-group, block pair)
    static constexpr int NMFMA = 2 * FM * FN * MPK;
};

template <typename T, bool TA, bool TB, int BM, int BN, int WM, int WN, int DEPTH>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_ring_kernel(const GemmArgs args)
{
    using namespace ring;
    using Cfg = RingCfg<T, TA, TB, BM, BN, WM, WN, DEPTH>;
    using TileA = typename Cfg::TileA;
    using TileB = typename Cfg::TileB;
    using FragA = typename Cfg::FragA;
    using FragB = typename Cfg::FragB;
    constexpr int FM = Cfg::FM, FN = Cfg::FN, BK = Cfg::BK, ESZ = sizeof(T), BATCH = Cfg::BATCH;

    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    uint32_t wg0, wg1, tile_id, zb, nxcd;
    work_of_block(args, blockIdx.x, blockIdx.z, tile_id, zb, nxcd);
    wg_remap(tile_id, args.nwg0, args.nwg1, args.wgm, nxcd, wg0, wg1);
    wg0 = __builtin_amdgcn_readfirstlane(wg0);
    wg1 = __builtin_amdgcn_readfirstlane(wg1);
    // (the division runs on the vector unit: back to scalar registers, so that what follows from it -- the k range, the
    // slice count, the loop test -- stays scalar as well)
    const uint32_t split = __builtin_amdgcn_readfirstlane(zb / args.batch), batch = __builtin_amdgcn_readfirstlane(zb % args.batch);
    const uint32_t row0 = wg0 * BM, col0 = wg1 * BN;
    const uint32_t lda = args.lda, ldb = args.ldb;
    const uint32_t k_begin = split * args.k_per_split;
    const uint32_t k_end = min(args.k, k_begin + args.k_per_split);
    const int n_slice = k_end > k_begin ? (int)((k_end - k_begin) / BK) : 0;

    const char *gA = static_cast<const char *>(args.A) +
                     ((int64_t)batch * args.strideA + (TA ? (int64_t)row0 * lda + k_begin
                                                          : (int64_t)k_begin * lda + row0)) * ESZ;
    const char *gB = static_cast<const char *>(args.B) +
                     ((int64_t)batch * args.strideB + (TB ? (int64_t)k_begin * ldb + col0
                                                          : (int64_t)col0 * ldb + k_begin)) * ESZ;
    const int64_t stepA = (TA ? (int64_t)BK : (int64_t)BK * lda) * ESZ;
    const int64_t stepB = (TB ? (int64_t)BK * ldb : (int64_t)BK) * ESZ;

    uint32_t offA[TileA::LPW], offB[TileB::LPW];
#pragma unroll
    for (int i = 0; i < TileA::LPW; ++i) offA[i] = TileA::load_goff(wave, lane, i, lda);
#pragma unroll
    for (int i = 0; i < TileB::LPW; ++i) offB[i] = TileB::load_goff(wave, lane, i, ldb);

    // cursors of the two operands: the next slice to be requested (slices are requested in order, one per iteration)
    u32x4 curA = slice_cursor(uniform_address(gA)), curB = slice_cursor(uniform_address(gB));
    const uint32_t lds_base = (uint32_t)(uintptr_t)MMBO_LDS_PTR(lds);
    const uint32_t ldsA = lds_base + wave * TileA::LPW * 1024, ldsB = lds_base + TileA::BYTES + wave * TileB::LPW * 1024;
    // the next slice goes to ring buffer `buf` (slice s to buffer s % DEPTH, kept by the caller)
    auto issue_slice = [&](int buf) {
        const uint32_t bo = buf * Cfg::SLICE_BYTES;
        static_for<TileA::LPW>([&](auto I) { direct_load16<false>(curA, 0u, offA[decltype(I)::value], ldsA + bo + decltype(I)::value * 1024); });
        static_for<TileB::LPW>([&](auto I) { direct_load16<false>(curB, 0u, offB[decltype(I)::value], ldsB + bo + decltype(I)::value * 1024); });
        advance(curA, (uint64_t)stepA);
        advance(curB, (uint64_t)stepB);
    };

    const typename FragA::Addr adA = FragA::make_addr(lane, wm * Cfg::TM);
    const typename FragB::Addr adB = FragB::make_addr(lane, wn * Cfg::TN);
    FragA fa[2];
    FragB fb[2];
    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto read_slice = [&](FragA &a, FragB &b, int buf) {
        const uint32_t t = lds_base + buf * Cfg::SLICE_BYTES;
        a.read_all(t, adA);
        b.read_all(t + TileA::BYTES, adB);
    };
    // The MFMAs of slice s with the LDS reads of slice s+1 and the direct loads of slice s+DEPTH spread between
    // them.  A wavefront issues in order: issued as one block at the top of the slice, the reads of all
    // wavefronts fill the LDS queue and the loads the texture-address queue, and every wavefront sits behind
    // its own last memory instruction before it reaches its first MFMA (measured: ~300 clocks per slice lost to
    // the reads, ~450 to the loads).
    constexpr int NA = FragA::NOPS, NR = FragA::NOPS + FragB::NOPS, NMFMA = Cfg::NMFMA, MPK = Cfg::MPK;
    // The reads go out between the first READ_SPAN MFMAs so that the last one has landed by the end of the slice.
    // With one wavefront per SIMD (four-wave work-groups) nothing else covers that latency, and the fewer MFMAs a
    // slice has the larger the exposed share: measured on fp32 4096 x 128 x 4096, reads spread over the whole slice
    // cost 10 us on top of 35 us of MFMAs.
    constexpr int READ_SPAN = Cfg::NW > 4 ? NMFMA : (NMFMA >= 32 ? NMFMA * 3 / 4 : NMFMA / 2);
    auto mfma_and_read = [&](auto ALWAYS, const FragA &ca, const FragB &cb, FragA &na, FragB &nb, int nbuf, bool load, int lbuf) {
        constexpr bool always = decltype(ALWAYS)::value;          // steady state: every slice issues its loads, no flag test
        const uint32_t t = lds_base + nbuf * Cfg::SLICE_BYTES;
        const uint32_t dstA = ldsA + lbuf * Cfg::SLICE_BYTES, dstB = ldsB + lbuf * Cfg::SLICE_BYTES;
        static_for<NMFMA>([&](auto M) {
            constexpr int m = decltype(M)::value;
            // consecutive MFMAs go to different accumulators
            constexpr int kg = m / (FM * FN * MPK), tt = (m / (FM * FN)) % MPK, i = (m / FN) % FM, j = m % FN;
            if constexpr (ESZ == 2)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, ca.x[kg][i]),
                                                                   __builtin_bit_cast(f16x8, cb.x[kg][j]), acc[i][j], 0, 0, 0);
            else {
                // (through locals: bit-casting a vector-element expression directly picked element 0)
                const uint32_t ua = ca.x[kg][i][tt], ub = cb.x[kg][j][tt];
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, ua),
                                                                 __builtin_bit_cast(float, ub), acc[i][j], 0, 0, 0);
            }
            // (one scheduling barrier per MFMA slot, at its end: two of them with nothing in between make the compiler
            // pad the gap with an s_nop, which costs an issue slot like any other instruction)
            if constexpr (m < READ_SPAN) {
                constexpr int r0 = NR * m / READ_SPAN, r1 = NR * (m + 1) / READ_SPAN;
                static_for<r1 - r0>([&](auto RR) {
                    constexpr int r = r0 + decltype(RR)::value;
                    if constexpr (r < NA) na.template read_op<r>(t, adA);
                    else nb.template read_op<r - NA>(t + TileA::BYTES, adB);
                });
            }
            {
                // load l goes out after MFMA number (2l+1) * NMFMA / (2 * BATCH): evenly spaced, none first or last
                constexpr int l0 = (2 * BATCH * m + NMFMA) / (2 * NMFMA), l1 = (2 * BATCH * (m + 1) + NMFMA) / (2 * NMFMA);
                static_for<l1 - l0>([&](auto LL) {
                    constexpr int l = l0 + decltype(LL)::value;
                    if constexpr (l < BATCH) {
                        if (always || load) {
                            if constexpr (l < TileA::LPW) direct_load16<false>(curA, 0u, offA[l], dstA + l * 1024);
                            else direct_load16<false>(curB, 0u, offB[l - TileA::LPW], dstB + (l - TileA::LPW) * 1024);
                        }
                    }
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        if (always || load) {                                     // the cursors move on to the slice after the one just requested
            advance(curA, (uint64_t)stepA);
            advance(curB, (uint64_t)stepB);
        }
    };
#define MMBO_BARRIER()                           \
    do {                                         \
        __builtin_amdgcn_sched_barrier(0);       \
        __builtin_amdgcn_s_barrier();            \
        __builtin_amdgcn_sched_barrier(0);       \
    } while (0)
#define MMBO_WAIT_VM(n) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory")
#define MMBO_WAIT_LGKM0() asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory")

    // Invariant at the top of iteration s (after barrier B_s): register set s&1 holds slice s; slice s+1 is
    // resident in LDS; every wavefront has finished reading slices <= s, so buffer s % DEPTH is free; this
    // wavefront's loads of slices s+2 .. s+DEPTH-1 are in flight.
    //   iteration s:  MFMAs of slice s from set s&1, interleaved with the loads(s+DEPTH) -> buffer s % DEPTH and the
    //                 reads of slice s+1 -> set (s+1)&1;  wait reads;  wait own loads(s+2);  barrier B_{s+1}.
    // Loads return in order, so "all but the newest (DEPTH-2) batches" means loads(s+2) have landed; once the
    // tail stops issuing, the wait is for everything.
#pragma unroll
    for (int s = 0; s < DEPTH; ++s)
        if (s < n_slice) issue_slice(s);
    if (n_slice >= DEPTH) MMBO_WAIT_VM(BATCH * (DEPTH - 1)); else MMBO_WAIT_VM(0);
    MMBO_BARRIER();                                                  // slice 0 resident
    read_slice(fa[0], fb[0], 0);
    MMBO_WAIT_LGKM0();
    if (n_slice >= DEPTH) MMBO_WAIT_VM(BATCH * (DEPTH - 2)); else MMBO_WAIT_VM(0);
    MMBO_BARRIER();                                                  // slice 1 resident, slice 0 in registers

    int buf = 0;                                                     // s % DEPTH
    // steady state: every slice issues its loads; no flag is tested inside the loop (with two MFMAs per slice in the
    // smallest fp16 tile the tests and branches were a third of the instructions a wavefront issued per slice)
    auto steady_step = [&](int s, FragA &ca, FragB &cb, FragA &na, FragB &nb) {
        const int nbuf = buf + 1 == DEPTH ? 0 : buf + 1;
        mfma_and_read(std::true_type{}, ca, cb, na, nb, nbuf, true, buf);
        MMBO_WAIT_LGKM0();
        MMBO_WAIT_VM(BATCH * (DEPTH - 2));
        MMBO_BARRIER();
        buf = nbuf;
    };
    auto step = [&](int s, FragA &ca, FragB &cb, FragA &na, FragB &nb) {
        const int nbuf = buf + 1 == DEPTH ? 0 : buf + 1;
        const bool steady = s + DEPTH < n_slice;
        // (the last slice reads a stale buffer into the unused register set: harmless, and it keeps the
        // interleaved block free of divergent control flow)
        mfma_and_read(std::false_type{}, ca, cb, na, nb, nbuf, steady, buf);
        MMBO_WAIT_LGKM0();
        if (steady) MMBO_WAIT_VM(BATCH * (DEPTH - 2)); else MMBO_WAIT_VM(0);
        MMBO_BARRIER();
        buf = nbuf;
    };
    int s = 0;
    for (; s + 1 + DEPTH < n_slice; s += 2) {
        steady_step(s, fa[0], fb[0], fa[1], fb[1]);
        steady_step(s + 1, fa[1], fb[1], fa[0], fb[0]);
    }
    for (; s < n_slice; s += 2) {
        step(s, fa[0], fb[0], fa[1], fb[1]);
        if (s + 1 < n_slice) step(s + 1, fa[1], fb[1], fa[0], fb[0]);
    }
#undef MMBO_BARRIER
#undef MMBO_WAIT_VM
#undef MMBO_WAIT_LGKM0

    write_back<T, FM, FN, true>(acc, args, row0 + wm * Cfg::TM, col0 + wn * Cfg::TN, batch, split, lane);
}

}  // namespace mmbo
