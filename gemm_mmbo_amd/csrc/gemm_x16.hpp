// Ring kernel on 16 x 16 MFMA blocks (v_mfma_f32_16x16x32_f16 / v_mfma_f32_16x16x4_f32) with the accumulators pinned
// to the accumulation registers.
//
// Same structure as gemm_ring.hpp (K in slices of 64 bytes per row -- 32 halves or 16 floats -- through a ring of LDS
// buffers filled by global->LDS direct loads; fragments double-buffered in registers; one barrier per slice), and the
// same recipe as the reference's kernels (src/gemm/ref/Kernels.cpp:412-747).  Unlike gemm_ring.hpp it also takes
// ragged problems: edge tiles load clamped rows and store under guards, a partial last slice of k is zero-filled.  Two differences, both about energy: MI355X
// lowers its clock under the power that fp16 MFMAs on real data draw, so what a kernel costs per flop outside
// the matrix pipe, and what the matrix instruction itself costs, decide the rate.
//   - 16x16x32 blocks: measured on the same random operands a register-only loop of v_mfma_f32_16x16x32_f16
//     sustains about 11 % more flop/s than one of v_mfma_f32_32x32x16_f16 (the chip holds a higher clock).
//   - a wavefront owns up to 128 x 128 of C (256 accumulator registers per lane): four wavefronts cover a
//     256 x 256 tile and read every LDS byte twice per slice instead of three times with eight 64 x 128 wavefronts.
//     The accumulators live in a[0..255] by name: written by the MFMAs below, read back in the epilogue, never
//     seen by the register allocator (left to choose, it shuttles accumulator tiles between the two register
//     files inside the loop and spills).  Every statement that touches them lists all of them as clobbered, so
//     the compiler neither uses them for anything else nor under-counts the kernel's registers.
#pragma once

#include "gemm_ring.hpp"

namespace mmbo {

namespace x16 {

using ring::advance;
using ring::direct_load16;
using ring::direct_load16_to_destination;
using ring::lds_read_b128;
using ring::lds_read_tr16_b64;
using ring::set_lds_destination;
using ring::slice_cursor;
using ring::static_for;
using ring::uniform_address;

// The 64 accumulator blocks a[4q : 4q+3], spelled out: an asm statement names its registers and its clobbers as literals.
#define MMBO_ACC_BLOCKS(X) \
    X(0,1,2,3) X(4,5,6,7) X(8,9,10,11) X(12,13,14,15) X(16,17,18,19) X(20,21,22,23) X(24,25,26,27) X(28,29,30,31) \
    X(32,33,34,35) X(36,37,38,39) X(40,41,42,43) X(44,45,46,47) X(48,49,50,51) X(52,53,54,55) X(56,57,58,59) X(60,61,62,63) \
    X(64,65,66,67) X(68,69,70,71) X(72,73,74,75) X(76,77,78,79) X(80,81,82,83) X(84,85,86,87) X(88,89,90,91) X(92,93,94,95) \
    X(96,97,98,99) X(100,101,102,103) X(104,105,106,107) X(108,109,110,111) X(112,113,114,115) X(116,117,118,119) X(120,121,122,123) X(124,125,126,127) \
    X(128,129,130,131) X(132,133,134,135) X(136,137,138,139) X(140,141,142,143) X(144,145,146,147) X(148,149,150,151) X(152,153,154,155) X(156,157,158,159) \
    X(160,161,162,163) X(164,165,166,167) X(168,169,170,171) X(172,173,174,175) X(176,177,178,179) X(180,181,182,183) X(184,185,186,187) X(188,189,190,191) \
    X(192,193,194,195) X(196,197,198,199) X(200,201,202,203) X(204,205,206,207) X(208,209,210,211) X(212,213,214,215) X(216,217,218,219) X(220,221,222,223) \
    X(224,225,226,227) X(228,229,230,231) X(232,233,234,235) X(236,237,238,239) X(240,241,242,243) X(244,245,246,247) X(248,249,250,251) X(252,253,254,255)

// acc block BASE/4 += A-fragment x B-fragment.  The statement clobbers exactly the four registers it writes.  (With every
// accumulation register in every MFMA's clobber list the compiler pads each pair of neighbouring asm statements with an
// s_nop: for statements it cannot look into, it assumes a result-forwarding hazard whenever what one writes overlaps what
// the next names.  An s_nop is an issue slot like any other instruction, and there was one for almost every MFMA.)
// Nothing else may ever hold a value in these registers: acc_zero claims all of them for the kernel, and
// tests/test_kernel_asm.py checks that no compiler-generated instruction of these kernels names an accumulation register.
template <int BASE, int NACC>
__device__ __forceinline__ void mfma_acc(const u32x4 &a, const u32x4 &b)
{
    static_assert(BASE % 4 == 0 && BASE + 4 <= NACC, "accumulator block out of range");
#define X(r0, r1, r2, r3)                                                                                     \
    if constexpr (BASE == r0)                                                                                 \
        asm volatile("v_mfma_f32_16x16x32_f16 a[" #r0 ":" #r3 "], %0, %1, a[" #r0 ":" #r3 "]" ::"v"(a), "v"(b) \
                     : "a" #r0, "a" #r1, "a" #r2, "a" #r3);
    MMBO_ACC_BLOCKS(X)
#undef X
}
// fp32: acc block BASE/4 += (one k of four per lane group) A x B; called four times per fragment pair
template <int BASE, int NACC>
__device__ __forceinline__ void mfma_acc_f32(uint32_t a, uint32_t b)
{
    static_assert(BASE % 4 == 0 && BASE + 4 <= NACC, "accumulator block out of range");
#define X(r0, r1, r2, r3)                                                                                    \
    if constexpr (BASE == r0)                                                                                \
        asm volatile("v_mfma_f32_16x16x4_f32 a[" #r0 ":" #r3 "], %0, %1, a[" #r0 ":" #r3 "]" ::"v"(a), "v"(b) \
                     : "a" #r0, "a" #r1, "a" #r2, "a" #r3);
    MMBO_ACC_BLOCKS(X)
#undef X
}
// All NACC accumulation registers = 0, four per statement, each statement clobbering the four it writes (between
// statements that each name every register the compiler would put one s_nop per write); together the statements name
// all of them, which is what keeps the compiler from using any.
template <int NACC>
__device__ __forceinline__ void acc_zero()
{
#define X(r0, r1, r2, r3)                                                                                              \
    if constexpr (r0 < NACC)                                                                                           \
        asm volatile("v_accvgpr_write_b32 a[" #r0 "], 0\n\tv_accvgpr_write_b32 a[" #r1 "], 0\n\t"                      \
                     "v_accvgpr_write_b32 a[" #r2 "], 0\n\tv_accvgpr_write_b32 a[" #r3 "], 0" ::: "a" #r0, "a" #r1, "a" #r2, "a" #r3);
    MMBO_ACC_BLOCKS(X)
#undef X
    asm volatile("s_nop 7" ::: "memory");
}
template <int I>
__device__ __forceinline__ float acc_read()
{
    float x;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(I));
    return x;
}

// One operand tile of one slice: R rows x 32 k = R * 64 bytes, fetched by NW wavefronts with 1 KB direct loads.
//   KC (source contiguous along k): LDS row r = its 64 bytes; 16-byte chunk c sits at position c ^ ((r >> 1) & 3).
//     A fragment read (ds_read_b128, lane l -> row l % 16, chunk l / 16) was timed on MI355X with candidate
//     swizzles: this one runs at the conflict-free rate, the ring kernel's (r >> 2) & 3 at half of it for this
//     lane pattern (and at the full rate for the ring kernel's own row l % 32, chunk l / 32).
//   RC (source contiguous along the row index): LDS k-row = R halves.  A transposing read takes, per 16-lane
//     block, four consecutive k-rows x 32 bytes; its blocks sit 8 k-rows apart.  The chunk index is XORed with a
//     mask of k so that the four k-rows of a block fall into different 64-byte groups and the two blocks served
//     in one pass into different halves of a group.
//     A tile whose row count is not a power of two (192) is laid out as NSUB sub-tiles of SUB rows, SUB the largest
//     power of two that divides R: a 1 KB direct load fills whole k-rows of ONE sub-tile, the sub-tiles of a slice
//     follow each other in LDS, and each is swizzled like a tile of SUB rows (16-row MFMA blocks never straddle two).
template <typename T, bool KC, int R, int NW>
struct Tile {
    static constexpr int ESZ = sizeof(T);
    static constexpr int BYTES = R * 64;
    static constexpr int INSTRS = R / 16;
    static_assert(INSTRS % NW == 0, "tile must split evenly over the wavefronts");
    static constexpr int LPW = INSTRS / NW;
    static constexpr int SUB = KC ? R : (R & -R);                 // rows of a sub-tile (RC operands; the whole tile when R is a power of two)
    static constexpr int NSUB = R / SUB;
    static constexpr int ROW_BYTES = SUB * ESZ;                   // one k-row of one sub-tile
    static constexpr int CPR = ROW_BYTES / 16;
    static constexpr int KPI = 1024 / ROW_BYTES;
    static constexpr int SUB_BYTES = SUB * 64;                    // one sub-tile of one slice
    static constexpr int IPS = INSTRS / NSUB;                     // direct loads per sub-tile
    static_assert(KC || (ROW_BYTES >= 64 * ESZ && ROW_BYTES <= 1024 && (ROW_BYTES & (ROW_BYTES - 1)) == 0),
                  "RC tile: a k-row of a sub-tile is 64 elements to 1024 bytes, a power of two");
    static_assert(KC || IPS * 1024 == SUB_BYTES, "a sub-tile is a whole number of 1 KB loads");

    __device__ static inline uint32_t rc_mask(uint32_t k)
    {
        // fp32 (ds_read_b32: lane group g = l / 16 reads k-row 4g + t, 16 consecutive rows = 64 bytes): the four
        // groups of one read go to the four 64-byte quarters of the 256-byte bank span
        if constexpr (ESZ == 4) return ((k >> 2) & 3) << 2;
        else if constexpr (ROW_BYTES % 256 == 0) return ((k & 3) << 2) | (((k >> 3) & 1) << 1);
        else return (((k >> 1) & 1) << 2) | (((k >> 3) & 1) << 1);    // 128-byte k-rows alternate between bank halves
    }
    __device__ static inline uint32_t kc_swz(uint32_t row) { return (row >> 1) & 3; }
    __device__ static inline uint32_t kc_off(uint32_t row, uint32_t chunk) { return row * 64 + ((chunk ^ kc_swz(row)) << 4); }
    // LDS offset of 16-byte group `chunk` (counted along all R rows) of k-row k
    __device__ static inline uint32_t rc_off(uint32_t k, uint32_t chunk)
    {
        if constexpr (NSUB == 1) return k * ROW_BYTES + ((chunk ^ rc_mask(k)) << 4);
        else return (chunk / CPR) * SUB_BYTES + k * ROW_BYTES + (((chunk % CPR) ^ rc_mask(k)) << 4);
    }

    static constexpr uint32_t EPC = 16 / ESZ;                   // elements per 16-byte group

    // RC operand, edge tile.  `valid` = rows of the tile that exist (R, or fewer for the last tile of a ragged
    // dimension).  Groups before the last one that holds an existing row are fetched in place.  That last group is
    // fetched from the 16 bytes that END at the last existing row (the reference's ShiftPtr, src/gemm/ref/Kernels.cpp:
    // 240-304: no byte outside the operand is touched), so its slot holds rows valid-EPC .. valid-1 instead of
    // last*EPC .. : the epilogue undoes the shift.  The slots of the groups behind it get the same 16 bytes and feed
    // accumulators that are never stored.  A tile with fewer than EPC rows reaches back into the tile before it: the
    // caller moves the tile origin back by `back` = EPC - valid rows (the host refuses a whole dimension that short).
    __device__ static inline uint32_t rc_group_off(uint32_t chunk, uint32_t valid, uint32_t back)
    {
        const uint32_t last = (valid - 1) / EPC;
        return chunk < last ? chunk * 16 : (valid + back - EPC) * ESZ;
    }

    // global byte offset (from the tile origin of this slice) of the chunk that lands in LDS slot (wave*LPW + i)*64 + lane.
    // KC operand, edge tile: the slots of the rows past the edge are filled with a copy of the last existing row.
    __device__ static inline uint32_t load_goff(int wave, int lane, int i, uint32_t ld, uint32_t valid, uint32_t back)
    {
        const uint32_t q = wave * LPW + i;
        if constexpr (KC) {
            uint32_t row = q * 16 + (lane >> 2);
            uint32_t chunk = (lane & 3) ^ kc_swz(row);
            return min(row, valid - 1) * ld * ESZ + chunk * 16;
        } else {
            uint32_t k = (q % IPS) * KPI + lane / CPR;
            uint32_t chunk = (q / IPS) * CPR + ((lane % CPR) ^ rc_mask(k));
            return k * ld * ESZ + rc_group_off(chunk, valid, back);
        }
    }

    // The last, partial slice of a k that is not a whole number of slices (reference: the tail loop,
    // src/gemm/ref/Kernels.cpp:921-1005, zero-fills k >= remainder): the same slots as the direct loads fill, written
    // through registers, with zeros from k_tail on.  g = operand origin of this tile at the tail slice.  Only elements
    // that exist are read: a 16-byte chunk along k that straddles the end goes element by element.
    __device__ static inline void fill_tail(const char *g, uint32_t ld, uint32_t valid, uint32_t back, uint32_t k_tail, char *dst,
                                            int wave, int lane)
    {
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            const uint32_t q = wave * LPW + i;
            u32x4 v = {0u, 0u, 0u, 0u};
            if constexpr (KC) {
                uint32_t row = q * 16 + (lane >> 2);
                uint32_t chunk = (lane & 3) ^ kc_swz(row);
                const char *p = g + min(row, valid - 1) * ld * ESZ + chunk * 16;
                const uint32_t k0 = chunk * EPC;
                if (k0 + EPC <= k_tail) {
                    v = *reinterpret_cast<const u32x4 *>(p);
                } else if (k0 < k_tail) {
                    union { T e[EPC]; u32x4 v; } u;
                    u.v = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
                    for (uint32_t e = 0; e < EPC; ++e)
                        if (k0 + e < k_tail) u.e[e] = reinterpret_cast<const T *>(p)[e];
                    v = u.v;
                }
            } else {
                uint32_t k = (q % IPS) * KPI + lane / CPR;
                uint32_t chunk = (q / IPS) * CPR + ((lane % CPR) ^ rc_mask(k));
                if (k < k_tail) v = *reinterpret_cast<const u32x4 *>(g + k * ld * ESZ + rc_group_off(chunk, valid, back));
            }
            *reinterpret_cast<u32x4 *>(dst + q * 1024 + lane * 16) = v;
        }
    }
};

// Fragments of one operand of one wavefront for one slice: F blocks of 16 rows x one slice of k, four registers each.
// fp16: lane l holds row l % 16, k = (l / 16) * 8 + 0..7 -- the operand layout of the 16x16x32 MFMA.
// fp32: lane l holds row l % 16, k = (l / 16) * 4 + t in register t -- register t of both operands feeds the t-th of
// four 16x16x4 MFMAs (whose lane group g then contracts k = 4g + t: any four k do, as long as A and B agree).
template <typename E, bool KC, int R, int NW, int F>
struct Frags {
    using T = Tile<E, KC, R, NW>;
    static constexpr int ESZ = sizeof(E);
    static constexpr int RPF = KC ? 1 : (ESZ == 2 ? 2 : 4);          // LDS reads per fragment
    static constexpr int NOPS = F * RPF;
    u32x4 x[F];

    static constexpr int NADDR = KC ? 1 : F;                         // distinct read addresses per slice
    struct Addr { uint32_t a[NADDR]; };

    __device__ static inline Addr make_addr(int lane, int r0)
    {
        Addr ad;
        if constexpr (KC) {
            ad.a[0] = T::kc_off(r0 + (lane & 15), lane >> 4);                     // + f*16*64 per block
        } else if constexpr (ESZ == 4) {
            const uint32_t r = lane & 15, g = lane >> 4;
#pragma unroll
            for (int f = 0; f < F; ++f) {
                uint32_t m = r0 + f * 16 + r;
                ad.a[f] = T::rc_off(4 * g, m >> 2) + (m & 3) * 4;                 // + t k-rows: not in the swizzle mask
            }
        } else {
            // transposing read: lane j of a 16-lane block points at k-row j/4, rows 4*(j%4)..+3, and receives
            // (k-rows 0..3) x (row j); block b covers k = 8b + 4h + 0..3 with its h-th read
            const uint32_t j = lane & 15, b = lane >> 4;
#pragma unroll
            for (int f = 0; f < F; ++f) {
                uint32_t m = r0 + f * 16 + (j & 3) * 4;
                uint32_t k = b * 8 + (j >> 2);                                    // + 4h: not in the swizzle mask
                ad.a[f] = T::rc_off(k, m >> 3) + (m & 7) * 2;
            }
        }
        return ad;
    }

    // Read number OP of a slice takes the address tile + ad.a[address_index(OP)] plus a constant; consecutive reads
    // share addresses, and first_use(OP) says whether OP is the first to use its one.
    static constexpr int address_index(int op) { return KC ? 0 : op / RPF; }
    static constexpr bool first_use(int op) { return KC ? op == 0 : op % RPF == 0; }
    template <int OP>
    __device__ __forceinline__ void read_op_at(uint32_t address)
    {
        constexpr int f = OP / RPF, h = OP % RPF;
        if constexpr (KC) {
            x[f] = lds_read_b128<f * 16 * 64>(address);
        } else if constexpr (ESZ == 4) {
            x[f][h] = ring::lds_read_b32<h * T::ROW_BYTES>(address);
        } else {
            u32x2 v = lds_read_tr16_b64<h * 4 * T::ROW_BYTES>(address);
            x[f][2 * h] = v[0];
            x[f][2 * h + 1] = v[1];
        }
    }
    template <int OP>
    __device__ __forceinline__ void read_op(uint32_t tile, const Addr &ad)
    {
        read_op_at<OP>(tile + ad.a[address_index(OP)]);
    }
    __device__ __forceinline__ void read_all(uint32_t tile, const Addr &ad)
    {
        static_for<NOPS>([&](auto OP) { this->template read_op<decltype(OP)::value>(tile, ad); });
    }
};

// How many of a slice's `loads` direct loads have gone out before MFMA slot `slot` of `slots`: load l goes out after MFMA
// number (2l+1) * slots / (2 * loads), evenly spaced, none first or last.
constexpr int gcd_of(int a, int b) { return b == 0 ? a : gcd_of(b, a % b); }

constexpr int loads_before_slot(int loads, int slots, int slot)
{
    const int l = (2 * loads * slot + slots) / (2 * slots);
    return l < loads ? l : loads;
}

}  // namespace x16

template <typename T, bool TA, bool TB, int BM, int BN, int WM, int WN, int DEPTH>
struct X16Cfg {
    static constexpr int NW = WM * WN, NT = NW * 64;
    static constexpr int ESZ = sizeof(T);
    static constexpr int BK = 64 / ESZ;                           // one slice: 64 bytes per row
    static constexpr int MPF = ESZ == 2 ? 1 : 4;                  // MFMAs per fragment pair
    static constexpr int TM = BM / WM, TN = BN / WN, FM = TM / 16, FN = TN / 16;
    static_assert(TM % 16 == 0 && TN % 16 == 0, "wave tile must be a multiple of the 16x16 MFMA block");
    static constexpr int NACC = FM * FN * 4 > 128 ? 256 : FM * FN * 4 > 64 ? 128 : 64;    // accumulation registers claimed
    static_assert(FM * FN * 4 <= 256, "wave tile needs more than 256 accumulator registers");
    using TileA = x16::Tile<T, TA, BM, NW>;
    using TileB = x16::Tile<T, !TB, BN, NW>;
    using FragA = x16::Frags<T, TA, BM, NW, FM>;
    using FragB = x16::Frags<T, !TB, BN, NW, FN>;
    static constexpr int SLICE_BYTES = TileA::BYTES + TileB::BYTES;
    static constexpr int LDS_BYTES = DEPTH * SLICE_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "ring does not fit the 160 KB of LDS");
    static constexpr int BATCH = TileA::LPW + TileB::LPW;         // direct loads per thread per slice
    static constexpr int NMFMA = FM * FN * MPF;
    static_assert(BATCH * (DEPTH - 1) < 64, "more loads in flight than vmcnt can count");
    // Old C ahead of the epilogue (fp16, beta != 0): a wavefront's FM * FN / 2 sixteen-byte groups per lane (two vertically
    // adjacent blocks each, as the epilogue reads them) are fetched with direct loads into the ring buffers the last
    // slices no longer need, a quarter of them under each of the last four slices, evenly spread over the slice's MFMAs.
    static constexpr int C_GROUPS = FM * FN / 2;
    static constexpr int C_PER_SLICE = (C_GROUPS + 3) / 4;                       // (the last of the four slices may carry fewer)
    static constexpr int C_PERIOD = NMFMA / (C_PER_SLICE > 0 ? C_PER_SLICE : 1);  // one load every C_PERIOD MFMAs
    // (wave tiles of 64 x 64 and more: on the 64 x 64 macro tile the variant's longer tails cost more than the read it hides,
    // HGEMM 1000 x 1000 x 1024 with beta = 1: 9.5 -> 9.7 us)
    static constexpr bool C_PREFETCH = ESZ == 2 && FM % 2 == 0 && C_GROUPS >= 8 && C_PERIOD >= 2 &&
                                       C_PER_SLICE * NW * 1024 <= SLICE_BYTES;
};

// PAIR: fetch two slices of one operand per iteration (see mfma_and_read); on when an operand is k-contiguous.
// EVEN_OP: the operand (0 = A, 1 = B) that paired mode fetches on even iterations.  Measured at 8192^3, against
// unpaired: NN and TT +1.0 to +1.5 % with the k-contiguous operand on the even iterations and -1.5 % with the other
// one, TN (both k-contiguous) +0.8 % with four wavefronts and +2.5 % with eight, NT (neither) -1.3 %.
// What decides it is where a pair starts: iteration s fetches slices s+DEPTH-1 and s+DEPTH, two halves of the same 128-byte
// lines only when the first of them is even -- s even for a ring of five buffers, s odd for a ring of six.  The launcher
// therefore gives the k-contiguous operand the even iterations on five buffers and the odd ones on six (six buffers, fp16:
// 3072^3 NN on the 192 x 192 tile 52.2 -> 50.3 us, 1024 x 1024 x 4096 on 64 x 64 21.1 -> 18.9, 2048 x 1024 x 4096 on 128 x 64 27.2 -> 25.3).
// OLD_C_AHEAD: the variant for beta != 0 that fetches a tile's old C into LDS under the tile's last four slices (see c_ahead
// below; both load schedules).  A kernel of its own, chosen by the host: with the code in the one kernel, calls that have no C to read paid
// 1.5-3 % on short-k and mid-size shapes for tails that had grown.
// BOTH_EVEN: the variant for two k-contiguous operands (TN) whose rows start on memory lines: both operands' pairs on the
// even iterations (see BOTH below).  A kernel of its own, chosen by the host.
template <typename T, bool TA, bool TB, int BM, int BN, int WM, int WN, int DEPTH, bool PAIR = (TA || !TB),
          int EVEN_OP = (TA ? 0 : 1), bool OLD_C_AHEAD = false, bool BOTH_EVEN = false>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_x16_kernel(const GemmArgs args)
{
    static_assert(!OLD_C_AHEAD || X16Cfg<T, TA, TB, BM, BN, WM, WN, DEPTH>::C_PREFETCH, "no old-C variant of this kernel");
    using namespace x16;
    using Cfg = X16Cfg<T, TA, TB, BM, BN, WM, WN, DEPTH>;
    using TileA = typename Cfg::TileA;
    using TileB = typename Cfg::TileB;
    using FragA = typename Cfg::FragA;
    using FragB = typename Cfg::FragB;
    constexpr int FM = Cfg::FM, FN = Cfg::FN, BK = Cfg::BK, BATCH = Cfg::BATCH, NACC = Cfg::NACC, ESZ = Cfg::ESZ;
    [[maybe_unused]] constexpr int MPF = Cfg::MPF;
    // Both operands k-contiguous (TN) on a ring of five buffers: the even iterations fetch the pair of slices s+4, s+5 of BOTH
    // operands and the odd ones nothing.  Alternating the operands, the odd iterations' pairs (s+4, s+5 with s odd) start on an
    // odd slice and so straddle two memory lines: half-line requests for half of the traffic.  The waits are the same either
    // way -- the loads of the last two iterations may stay in flight -- and so is the shortest lead (a pair's first slice is
    // requested two to three slices before it is needed).  Measured (fp16, us): 64 x 512^3 27.1 -> 25.0, 2048^3 21.9 -> 20.7,
    // 4096^3 105.8 -> 101.5, 8192^3 777 -> 765.  Only where every row of A and B starts on a memory line (BOTH_EVEN, the host's
    // choice): with rows that straddle lines anyway the bunched requests cost 7 % (8192 x 8192 x 8200, lda = ldb = 8200).
    constexpr bool BOTH = BOTH_EVEN && PAIR && TA && !TB && DEPTH == 5;

    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;

    // A work-group walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ...: the host launches one work-group per tile,
    // or, for the 256 x 256 tiles on grids larger than the chip, one per CU (persistent).  Staying resident saves the
    // dispatch of a new work-group per tile, and the next tile's first loads are in flight while the stores of the
    // last one are still being acknowledged.  Those stores are older than the loads, and the count-based waits below
    // only ever wait for more when something older is still outstanding.
    const uint32_t n_tiles = args.nwg0 * args.nwg1;
    for (uint32_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    uint32_t wg0, wg1, tile_id, zb, nxcd;
    work_of_block(args, tile, blockIdx.z, tile_id, zb, nxcd);
    if (args.chip_block) chip_block_remap(tile_id, args.nwg0, args.nwg1, wg0, wg1);
    else wg_remap(tile_id, args.nwg0, args.nwg1, args.wgm, nxcd, wg0, wg1);
    // (the divisions above run on the vector unit; what follows wants these in scalar registers)
    wg0 = __builtin_amdgcn_readfirstlane(wg0);
    wg1 = __builtin_amdgcn_readfirstlane(wg1);
    zb = __builtin_amdgcn_readfirstlane(zb);
    // (the division runs on the vector unit: back to scalar registers, so that what follows from it -- the k range, the
    // slice count, the loop test -- stays scalar as well)
    const uint32_t split = __builtin_amdgcn_readfirstlane(zb / args.batch), batch = __builtin_amdgcn_readfirstlane(zb % args.batch);
    const uint32_t row0 = wg0 * BM, col0 = wg1 * BN;
    const uint32_t lda = args.lda, ldb = args.ldb;
    const uint32_t k_begin = split * args.k_per_split;
    // every split takes k_per_split (whole slices); the last one also the rest of k, whose last slice may be partial
    const uint32_t k_end = split + 1 == args.splits ? args.k : min(args.k, k_begin + args.k_per_split);
    const int n_slice = k_end > k_begin ? (int)((k_end - k_begin) / BK) : 0;
    const uint32_t k_tail = k_end > k_begin ? (k_end - k_begin) % BK : 0;

    // rows and columns of this tile that exist: less than the tile on the last tile row / column of a ragged problem;
    // a row-contiguous operand with less than one 16-byte group of them starts that many rows early (Tile::rc_group_off)
    const uint32_t m_here = min((uint32_t)BM, args.m - row0), n_here = min((uint32_t)BN, args.n - col0);
    constexpr uint32_t EPC = 16 / ESZ;
    const uint32_t backA = (!TA && m_here < EPC) ? EPC - m_here : 0, backB = (TB && n_here < EPC) ? EPC - n_here : 0;
    const char *gA = static_cast<const char *>(args.A) +
                     ((int64_t)batch * args.strideA + (TA ? (int64_t)row0 * lda + k_begin
                                                          : (int64_t)k_begin * lda + row0 - backA)) * ESZ;
    const char *gB = static_cast<const char *>(args.B) +
                     ((int64_t)batch * args.strideB + (TB ? (int64_t)k_begin * ldb + col0 - backB
                                                          : (int64_t)col0 * ldb + k_begin)) * ESZ;
    const int64_t stepA = (TA ? (int64_t)BK : (int64_t)BK * lda) * ESZ;
    const int64_t stepB = (TB ? (int64_t)BK * ldb : (int64_t)BK) * ESZ;

    uint32_t offA[TileA::LPW], offB[TileB::LPW];
#pragma unroll
    for (int i = 0; i < TileA::LPW; ++i) offA[i] = TileA::load_goff(wave, lane, i, lda, m_here, backA);
#pragma unroll
    for (int i = 0; i < TileB::LPW; ++i) offB[i] = TileB::load_goff(wave, lane, i, ldb, n_here, backB);

    // The direct loads (ring::direct_load16): each operand has a cursor, a buffer descriptor in scalar registers whose
    // origin is the next slice to be requested; the lane's part of the address is the 32-bit offset computed above.
    // Slices are requested in order, so a request is "the slice at the cursor" (or, in paired mode, also the one after
    // it), and the cursor then moves on.
    u32x4 curA = slice_cursor(uniform_address(gA)), curB = slice_cursor(uniform_address(gB));
    const uint32_t stepA32 = (uint32_t)stepA, stepB32 = (uint32_t)stepB;       // below 2 GiB: the tile-span limit
    const uint32_t lds_base = (uint32_t)(uintptr_t)MMBO_LDS_PTR(lds);
    const uint32_t ldsA = lds_base + wave * TileA::LPW * 1024, ldsB = lds_base + TileA::BYTES + wave * TileB::LPW * 1024;
    // load number i of operand OP (0 = A, 1 = B), of the slice at the cursor (AHEAD = false) or the one after it, to
    // dst = this wavefront's first LDS destination of that operand in the ring buffer the slice goes to (op_dst)
    auto op_dst = [&](auto OP, int b) { return (decltype(OP)::value == 0 ? ldsA : ldsB) + (uint32_t)b * Cfg::SLICE_BYTES; };
    auto issue_op_load = [&](auto OP, auto I, auto AHEAD, uint32_t dst, auto DESTINATION_SET) {
        constexpr int op = decltype(OP)::value, i = decltype(I)::value;
        constexpr bool ahead = decltype(AHEAD)::value;
        if constexpr (decltype(DESTINATION_SET)::value) {           // M0 was written before the MFMA just issued
            if constexpr (op == 0) direct_load16_to_destination<ahead>(curA, stepA32, offA[i]);
            else direct_load16_to_destination<ahead>(curB, stepB32, offB[i]);
        } else {
            if constexpr (op == 0) direct_load16<ahead>(curA, stepA32, offA[i], dst + i * 1024);
            else direct_load16<ahead>(curB, stepB32, offB[i], dst + i * 1024);
        }
    };
    auto advance_op = [&](auto OP, int slices) {
        if constexpr (decltype(OP)::value == 0) advance(curA, (uint64_t)stepA * slices);
        else advance(curB, (uint64_t)stepB * slices);
    };
    // direct load number l (A's first, then B's) of the slices at the two cursors into ring buffer `buf`
    auto issue_load = [&](auto L, uint32_t dst_a, uint32_t dst_b, auto DESTINATION_SET) {
        constexpr int l = decltype(L)::value;
        if constexpr (l < TileA::LPW) issue_op_load(std::integral_constant<int, 0>{}, L, std::false_type{}, dst_a, DESTINATION_SET);
        else issue_op_load(std::integral_constant<int, 1>{}, std::integral_constant<int, l - TileA::LPW>{}, std::false_type{}, dst_b, DESTINATION_SET);
    };
    auto issue_slice = [&](int buf) {
        const uint32_t dst_a = op_dst(std::integral_constant<int, 0>{}, buf), dst_b = op_dst(std::integral_constant<int, 1>{}, buf);
        static_for<BATCH>([&](auto L) { issue_load(L, dst_a, dst_b, std::false_type{}); });
        advance(curA, (uint64_t)stepA);
        advance(curB, (uint64_t)stepB);
    };

    const typename FragA::Addr adA = FragA::make_addr(lane, wm * Cfg::TM);
    const typename FragB::Addr adB = FragB::make_addr(lane, wn * Cfg::TN);
    FragA fa[2];
    FragB fb[2];

    // Old C ahead of the epilogue (Cfg::C_PREFETCH; paired mode, whole tiles, whole slices, at least DEPTH + 1 of them).
    // Group q of this wavefront = blocks (i, j), (i + 1, j) with j = q / (FM / 2), i = 2 * (q % (FM / 2)): the lane's 16 bytes
    // start at  C_tile + (lane's column * ldc + lane's row of the pair) + (j * 16 * ldc + i * 16)  elements -- the part in
    // front is the lane's constant offset, the part behind a scalar offset of the load.  Group q goes to the ring buffer of
    // slice n_slice - 4 + q / C_PER_SLICE (free from that slice's iteration on), at wave * C_PER_SLICE KB + (q % C_PER_SLICE) KB.
    const bool c_ahead = OLD_C_AHEAD && args.c_prefetch != 0 && m_here == (uint32_t)BM && n_here == (uint32_t)BN &&
                         k_tail == 0 && n_slice >= DEPTH + 1;
    // (set up whether used or not: a descriptor that is assigned under a branch ends up in vector registers, where a
    // buffer load cannot take it)
    [[maybe_unused]] const u32x4 curC = slice_cursor(uniform_address(
        static_cast<const char *>(args.C) + (OLD_C_AHEAD ? ((int64_t)batch * args.strideC + (int64_t)col0 * args.ldc + row0) * ESZ : 0)));
    [[maybe_unused]] const uint32_t c_lane_off = !OLD_C_AHEAD ? 0u :
        ((wn * Cfg::TN + (lane & 15)) * args.ldc + wm * Cfg::TM + (((lane >> 4) & 1) ? 4 * (lane >> 4) + 12 : 4 * (lane >> 4))) * ESZ;
    [[maybe_unused]] const uint32_t c_col_step = !OLD_C_AHEAD ? 0u : __builtin_amdgcn_readfirstlane(16 * args.ldc * ESZ);

    auto read_slice = [&](FragA &a, FragB &b, int buf) {
        const uint32_t t = lds_base + buf * Cfg::SLICE_BYTES;
        a.read_all(t, adA);
        b.read_all(t + TileA::BYTES, adB);
    };

    // One slice: its MFMAs from register set (ca, cb), with the LDS reads of the next slice (into na, nb) issued
    // between the first READ_SPAN of them and this wavefront's direct loads of slice s+DEPTH spread over all of
    // them.  A wavefront issues in order and here it is alone on its SIMD: memory instructions issued as a block
    // would stall the matrix pipe behind the LDS / texture-address queues, and reads issued late would leave their
    // latency exposed before the barrier.
    constexpr int NA = FragA::NOPS, NR = FragA::NOPS + FragB::NOPS, NMFMA = Cfg::NMFMA;
    constexpr int READ_SPAN = Cfg::NW > 4 ? NMFMA : NMFMA * 3 / 4;     // two wavefronts per SIMD cover each other's read latency
    // Paired mode (PAIR): iteration s fetches TWO slices, s+DEPTH-1 and s+DEPTH, of ONE operand -- A on even s, B on
    // odd s -- and issues the two loads that cover the two halves of the same 128-byte memory lines back to back.
    // With 64-byte LDS rows a k-contiguous operand otherwise asks for every cache line twice, a slice time apart
    // (measured: half-line requests stream at 35-52 B/clk/CU from L2, whole lines at 72-91).  `load` / `load2`
    // say whether the first / second slice of the pair exists.
    auto mfma_and_read = [&](auto LOAD, auto PAR, const FragA &ca, const FragB &cb, FragA &na, FragB &nb, int nbuf, bool load,
                             bool load2, int lbuf, auto OLD_C, int c_first) {
        constexpr bool old_c = decltype(OLD_C)::value;            // this slice carries a quarter of the old C (no operand loads then)
        constexpr int load_mode = decltype(LOAD)::value;          // 0 none, 1 always, 2 if `load` (and `load2`)
        constexpr int par = decltype(PAR)::value;
        constexpr int opn = par ^ EVEN_OP;                         // paired mode: the operand this iteration fetches
        constexpr int LX = EVEN_OP == 0 ? TileA::LPW : TileB::LPW, LY = EVEN_OP == 0 ? TileB::LPW : TileA::LPW;
        // and its loads per slice (BOTH: the even operand's loads, then the other one's; the odd iterations fetch nothing)
        constexpr int LOP = BOTH ? (par == 0 ? LX + LY : 0) : (opn == 0 ? TileA::LPW : TileB::LPW);
        constexpr int load_mode_here = (BOTH && par == 1) ? 0 : load_mode;
        const int pbuf = lbuf == 0 ? DEPTH - 1 : lbuf - 1;        // buffer of slice s+DEPTH-1
        const uint32_t t = lds_base + nbuf * Cfg::SLICE_BYTES;
        // LDS destinations of this iteration's loads, worked out here, once (the empty asm pins them to scalar registers
        // at this point: otherwise the compiler recomputes them next to every load, between two MFMAs)
        uint32_t dst_x0 = op_dst(std::integral_constant<int, opn>{}, pbuf), dst_x1 = op_dst(std::integral_constant<int, opn>{}, lbuf);
        uint32_t dst_a = op_dst(std::integral_constant<int, 0>{}, lbuf), dst_b = op_dst(std::integral_constant<int, 1>{}, lbuf);
        // (BOTH: the other operand's two destinations)
        [[maybe_unused]] uint32_t dst_y0 = op_dst(std::integral_constant<int, 1 - EVEN_OP>{}, pbuf),
                                  dst_y1 = op_dst(std::integral_constant<int, 1 - EVEN_OP>{}, lbuf);
        if constexpr (load_mode_here != 0 && PAIR) asm volatile("" : "+s"(dst_x0), "+s"(dst_x1));
        if constexpr (load_mode_here != 0 && BOTH) asm volatile("" : "+s"(dst_y0), "+s"(dst_y1));
        if constexpr (load_mode_here != 0 && !PAIR) asm volatile("" : "+s"(dst_a), "+s"(dst_b));
        // old C ahead of the epilogue: this iteration's groups c_first .. c_first + C_PER_SLICE - 1 go to buffer lbuf (the
        // one this slice left; no operand load goes there any more), one after every eighth MFMA
        [[maybe_unused]] const uint32_t c_dst = lds_base + (uint32_t)lbuf * Cfg::SLICE_BYTES + wave * (Cfg::C_PER_SLICE * 1024);
        uint32_t read_a[FragA::NADDR], read_b[FragB::NADDR];      // addresses of the LDS reads, each live from its first use to its last
        static_for<NMFMA>([&](auto M) {
            constexpr int m = decltype(M)::value;
            // boustrophedon over the FM x FN blocks: consecutive MFMAs share one operand register, also at the row
            // ends (a register-only loop of these MFMAs runs 3 % faster when one operand repeats than when both change);
            // fp32 walks the blocks four times, once per k register, so an accumulator recurs every FM*FN MFMAs
            constexpr int tt = m / (FM * FN), ij = m % (FM * FN);
            constexpr int i = ij / FN, j = (i & 1) ? FN - 1 - ij % FN : ij % FN;
            // The direct loads that go out after this MFMA (known at compile time).  Paired mode: load l of the first slice
            // of the pair after MFMA number (2l+1) * NMFMA / (2 * LOP), the load of the second slice, which shares its memory
            // lines, one MFMA later.  Unpaired: load l after MFMA number (2l+1) * NMFMA / (2 * BATCH): evenly spaced, none
            // first or last.  Where exactly one load follows the MFMA, its LDS destination goes into M0 BEFORE the MFMA and the
            // load itself after it: the MFMA is the wait state a write to M0 needs, and the load costs two instructions.
            constexpr int LIM = PAIR ? (LOP > 0 ? LOP : 1) : BATCH;
            constexpr int l0 = loads_before_slot(LIM, NMFMA, m), l1 = loads_before_slot(LIM, NMFMA, m + 1),
                          p0 = m == 0 ? 0 : loads_before_slot(LIM, NMFMA, m - 1);
            constexpr int n_first = load_mode_here != 0 ? l1 - l0 : 0, n_second = (load_mode_here != 0 && PAIR) ? l0 - p0 : 0;
            static_assert(!PAIR || m + 1 < NMFMA || n_first == 0, "the last MFMA slot cannot start a pair of loads");
            constexpr bool single = n_first + n_second == 1;
            if constexpr (single) {
                if constexpr (BOTH && n_second == 1) set_lds_destination(p0 < LX ? dst_x1 + p0 * 1024 : dst_y1 + (p0 - LX) * 1024);
                else if constexpr (BOTH) set_lds_destination(l0 < LX ? dst_x0 + l0 * 1024 : dst_y0 + (l0 - LX) * 1024);
                else if constexpr (n_second == 1) set_lds_destination(dst_x1 + p0 * 1024);
                else if constexpr (PAIR) set_lds_destination(dst_x0 + l0 * 1024);
                else if constexpr (l0 < TileA::LPW) set_lds_destination(dst_a + l0 * 1024);
                else set_lds_destination(dst_b + (l0 - TileA::LPW) * 1024);
            }
            // An address that a read of this slot is the first to use is worked out BEFORE the MFMA (the empty asm, which only
            // reads it, keeps the addition there): behind it, the read would wait for the addition with nothing in between,
            // and where the compiler puts it otherwise changes with unrelated code (measured: 2-3 % at 8192^3 fp16 NN).
            constexpr int r0 = m < READ_SPAN ? NR * m / READ_SPAN : 0, r1 = m < READ_SPAN ? NR * (m + 1) / READ_SPAN : 0;
            static_for<r1 - r0>([&](auto RR) {
                constexpr int r = r0 + decltype(RR)::value;
                if constexpr (r < NA) {
                    if constexpr (FragA::first_use(r)) {
                        read_a[FragA::address_index(r)] = t + adA.a[FragA::address_index(r)];
                        asm volatile("" ::"v"(read_a[FragA::address_index(r)]));
                    }
                } else if constexpr (FragB::first_use(r - NA)) {
                    read_b[FragB::address_index(r - NA)] = t + TileA::BYTES + adB.a[FragB::address_index(r - NA)];
                    asm volatile("" ::"v"(read_b[FragB::address_index(r - NA)]));
                }
            });
            if constexpr (ESZ == 2) mfma_acc<(i * FN + j) * 4, NACC>(ca.x[i], cb.x[j]);
            else mfma_acc_f32<(i * FN + j) * 4, NACC>(ca.x[i][tt], cb.x[j][tt]);
            static_for<r1 - r0>([&](auto RR) {
                constexpr int r = r0 + decltype(RR)::value;
                if constexpr (r < NA) na.template read_op_at<r>(read_a[FragA::address_index(r)]);
                else nb.template read_op_at<r - NA>(read_b[FragB::address_index(r - NA)]);
            });
            constexpr std::bool_constant<single> DESTINATION_SET{};
            static_for<n_second>([&](auto LL) {
                constexpr int l = p0 + decltype(LL)::value;
                if constexpr (BOTH && l >= LX) {
                    if (load_mode == 1 || load2) issue_op_load(std::integral_constant<int, 1 - EVEN_OP>{}, std::integral_constant<int, l - LX>{}, std::true_type{}, dst_y1, DESTINATION_SET);
                } else {
                    if (load_mode == 1 || load2) issue_op_load(std::integral_constant<int, opn>{}, std::integral_constant<int, l>{}, std::true_type{}, dst_x1, DESTINATION_SET);
                }
            });
            static_for<n_first>([&](auto LL) {
                constexpr int l = l0 + decltype(LL)::value;
                if constexpr (BOTH && l >= LX) {
                    if (load_mode == 1 || load) issue_op_load(std::integral_constant<int, 1 - EVEN_OP>{}, std::integral_constant<int, l - LX>{}, std::false_type{}, dst_y0, DESTINATION_SET);
                } else if constexpr (PAIR) {
                    if (load_mode == 1 || load) issue_op_load(std::integral_constant<int, opn>{}, std::integral_constant<int, l>{}, std::false_type{}, dst_x0, DESTINATION_SET);
                } else {
                    if (load_mode == 1 || load) issue_load(std::integral_constant<int, l>{}, dst_a, dst_b, DESTINATION_SET);
                }
            });
            if constexpr (old_c && OLD_C_AHEAD && m % Cfg::C_PERIOD == Cfg::C_PERIOD / 2 && m / Cfg::C_PERIOD < Cfg::C_PER_SLICE) {
                constexpr int c = m / Cfg::C_PERIOD;
                const uint32_t q = (uint32_t)c_first + c;             // group q: column block q / (FM / 2), row-block pair q % (FM / 2)
                if (Cfg::C_GROUPS % Cfg::C_PER_SLICE == 0 || q < (uint32_t)Cfg::C_GROUPS) {
                    const uint32_t soff = __builtin_amdgcn_readfirstlane((q / (FM / 2)) * c_col_step + (q % (FM / 2)) * (32 * ESZ));
                    direct_load16<true>(curC, soff, c_lane_off, c_dst + c * 1024);
                }
            }
            // (one scheduling barrier per MFMA slot, at its end: two of them with nothing in between make the compiler
            // pad the gap with an s_nop, which costs an issue slot like any other instruction)
            __builtin_amdgcn_sched_barrier(0);
        });
        // the cursors move past what this iteration requested (past the end of k in the last iterations: never used again).
        // The paired tail moves them itself, behind its choice between two copies of the slice: a cursor that is changed on
        // one side of a branch only comes out of the merge in vector registers, where a buffer load cannot take it.
        if constexpr (load_mode_here == 1 && PAIR) advance_op(std::integral_constant<int, opn>{}, 2);
        if constexpr (load_mode_here == 1 && BOTH) advance_op(std::integral_constant<int, 1 - EVEN_OP>{}, 2);
        if constexpr (load_mode != 0 && !PAIR) {
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
    // resident in LDS; every wavefront has finished reading slices <= s, so buffer s % DEPTH is free (and, for the
    // operand whose turn it is in paired mode, buffer (s-1) % DEPTH too); the loads of the later slices are in flight.
    // Loads return in order.  Unpaired: waiting for all but the newest DEPTH-2 batches means this wavefront's part of
    // slice s+2 has landed.  Paired: everything issued in the last DEPTH-3 iterations belongs to slices >= s+3, so all but
    // that may stay in flight.
    int buf = 0;                                                     // s % DEPTH
    int s = 0;
    if constexpr (!PAIR) {
#pragma unroll
        for (int q = 0; q < DEPTH; ++q)
            if (q < n_slice) issue_slice(q);
        acc_zero<NACC>();                                                // (while the first slices are on their way)
        if (n_slice >= DEPTH) MMBO_WAIT_VM(BATCH * (DEPTH - 1)); else MMBO_WAIT_VM(0);
        MMBO_BARRIER();                                                  // slice 0 resident
        read_slice(fa[0], fb[0], 0);
        MMBO_WAIT_LGKM0();
        if (n_slice >= DEPTH) MMBO_WAIT_VM(BATCH * (DEPTH - 2)); else MMBO_WAIT_VM(0);
        MMBO_BARRIER();                                                  // slice 1 resident, slice 0 in registers

        // steady state: every slice issues loads, no flag tests inside the MFMA stream
        auto steady_step = [&](int s, FragA &ca, FragB &cb, FragA &na, FragB &nb) {
            const int nbuf = buf + 1 == DEPTH ? 0 : buf + 1;
            mfma_and_read(std::integral_constant<int, 1>{}, std::integral_constant<int, 0>{}, ca, cb, na, nb, nbuf, true, true, buf, std::false_type{}, 0);
            MMBO_WAIT_LGKM0();
            MMBO_WAIT_VM(BATCH * (DEPTH - 2));
            MMBO_BARRIER();
            buf = nbuf;
        };
        // (the last slice reads a stale buffer into the unused register set: harmless, and it keeps the
        // interleaved block free of divergent control flow)
        auto tail_step = [&](int s, FragA &ca, FragB &cb, FragA &na, FragB &nb) {
            const int nbuf = buf + 1 == DEPTH ? 0 : buf + 1;
            const bool load = s + DEPTH < n_slice;
            if constexpr (OLD_C_AHEAD) {
                // The last four slices carry the old C (no operand load is issued in the last DEPTH slices).  All operand loads
                // are older than any of these; loads return in order, so leaving at most two slices' worth of C loads in flight
                // also means every operand load has landed -- except, under the first of the four slices, some of the newest
                // C_PER_SLICE operand loads, which belong to the last slice (C_PER_SLICE <= BATCH) and are not needed yet.
                static_assert(Cfg::C_PER_SLICE <= BATCH && 2 * Cfg::C_PER_SLICE < 64, "old-C loads per slice exceed what the wait below assumes");
                const int c_first = __builtin_amdgcn_readfirstlane((c_ahead && s + 4 >= n_slice) ? (s + 4 - n_slice) * Cfg::C_PER_SLICE : -1);
                if (c_first >= 0) {
                    mfma_and_read(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, ca, cb, na, nb, nbuf, false, false, buf, std::true_type{}, c_first);
                    MMBO_WAIT_LGKM0();
                    MMBO_WAIT_VM(2 * Cfg::C_PER_SLICE);
                    MMBO_BARRIER();
                    buf = nbuf;
                    return;
                }
            }
            mfma_and_read(std::integral_constant<int, 2>{}, std::integral_constant<int, 0>{}, ca, cb, na, nb, nbuf, load, load, buf, std::false_type{}, 0);
            MMBO_WAIT_LGKM0();
            if (load) MMBO_WAIT_VM(BATCH * (DEPTH - 2)); else MMBO_WAIT_VM(0);
            MMBO_BARRIER();
            buf = nbuf;
        };
        for (; s + 1 + DEPTH < n_slice; s += 2) {
            steady_step(s, fa[0], fb[0], fa[1], fb[1]);
            steady_step(s + 1, fa[1], fb[1], fa[0], fb[0]);
        }
        for (; s < n_slice; s += 2) {
            tail_step(s, fa[0], fb[0], fa[1], fb[1]);
            if (s + 1 < n_slice) tail_step(s + 1, fa[1], fb[1], fa[0], fb[0]);
        }
    } else {
        static_assert(!PAIR || DEPTH >= 5, "paired loads need a ring of at least five buffers");
        // X = the operand even iterations fetch (EVEN_OP), Y = the other
        constexpr int LA = EVEN_OP == 0 ? TileA::LPW : TileB::LPW, LB = EVEN_OP == 0 ? TileB::LPW : TileA::LPW;
        constexpr std::integral_constant<int, EVEN_OP> OPX{};
        constexpr std::integral_constant<int, 1 - EVEN_OP> OPY{};
        // prologue: X slices 0 .. DEPTH-2, Y slices 0 .. DEPTH-1 (iteration 0 brings X's DEPTH-1 and DEPTH).  Slices 0 and 1 of both
        // operands -- and, with five buffers, X's 2 and 3 -- go out the way the loop's pairs do, the two loads that share a memory
        // line back to back (whole-line requests stream twice as fast as half-line ones, and nothing else is in flight yet);
        // the rest slice by slice, in the order the loop's first waits count on: they let the newest loads of the prologue stay
        // in flight, and none of those may belong to slice 2.
        auto pro_pair = [&](auto OP, auto L, int q) {                    // slices q and q + 1 of one operand
            constexpr int n = decltype(L)::value;
            if (q + 1 < n_slice) {
                static_for<n>([&](auto I) {
                    issue_op_load(OP, I, std::false_type{}, op_dst(OP, q), std::false_type{});
                    issue_op_load(OP, I, std::true_type{}, op_dst(OP, q + 1), std::false_type{});
                });
            } else if (q < n_slice) {
                static_for<n>([&](auto I) { issue_op_load(OP, I, std::false_type{}, op_dst(OP, q), std::false_type{}); });
            }
            advance_op(OP, 2);                                           // (not under the branch: the cursors stay in scalar registers)
        };
        auto pro_one = [&](auto OP, auto L, int q) {
            constexpr int n = decltype(L)::value;
            if (q < n_slice) static_for<n>([&](auto I) { issue_op_load(OP, I, std::false_type{}, op_dst(OP, q), std::false_type{}); });
            advance_op(OP, 1);
        };
        constexpr std::integral_constant<int, LA> NLA{};
        constexpr std::integral_constant<int, LB> NLB{};
        constexpr int X_PAIRED = DEPTH == 5 ? 4 : 2;                     // X's slices below this go out in pairs
        pro_pair(OPX, NLA, 0);
        pro_pair(OPY, NLB, 0);
        if constexpr (BOTH) {
            // (both operands on the even iterations: slices 0 .. 3 of both here, all in pairs; iteration 0 brings 4 and 5)
            pro_pair(OPX, NLA, 2);
            pro_pair(OPY, NLB, 2);
        } else {
            if constexpr (X_PAIRED == 4) pro_pair(OPX, NLA, 2);
#pragma unroll
            for (int q = 2; q < DEPTH; ++q) {
                if (q >= X_PAIRED && q < DEPTH - 1) pro_one(OPX, NLA, q);
                pro_one(OPY, NLB, q);
            }
        }
        constexpr int PRO = BOTH ? (DEPTH - 1) * (LA + LB) : (DEPTH - 1) * LA + DEPTH * LB;       // loads per thread in the prologue
        acc_zero<NACC>();                                                // (while the first slices are on their way)
        if (n_slice >= DEPTH) MMBO_WAIT_VM(PRO - 2 * BATCH); else MMBO_WAIT_VM(0);
        MMBO_BARRIER();                                                  // slices 0 and 1 resident
        read_slice(fa[0], fb[0], 0);
        MMBO_WAIT_LGKM0();
        MMBO_BARRIER();                                                  // slice 0 in registers

        // loads a steady iteration of parity P leaves in flight: those of the last DEPTH-3 iterations, itself included
        auto steady_step = [&](auto PAR, int s, FragA &ca, FragB &cb, FragA &na, FragB &nb) {
            constexpr int par = decltype(PAR)::value;
            constexpr int own = 2 * (par == 0 ? LA : LB), other = 2 * (par == 0 ? LB : LA);
            // (BOTH, five buffers: this iteration and the one before it, of which one fetched both operands' pairs and one nothing)
            constexpr int KEEP = BOTH ? 2 * (LA + LB) : own * ((DEPTH - 3 + 1) / 2) + other * ((DEPTH - 3) / 2);
            static_assert(KEEP < 64, "more loads in flight than vmcnt can count");
            const int nbuf = buf + 1 == DEPTH ? 0 : buf + 1;
            mfma_and_read(std::integral_constant<int, 1>{}, PAR, ca, cb, na, nb, nbuf, true, true, buf, std::false_type{}, 0);
            MMBO_WAIT_LGKM0();
            MMBO_WAIT_VM(KEEP);
            MMBO_BARRIER();
            buf = nbuf;
        };
        // tail: count what was actually issued; hist[0] is the previous iteration, hist[1] the one before
        int hist[2] = {0, 0};
        auto tail_step = [&](auto PAR, int s, FragA &ca, FragB &cb, FragA &na, FragB &nb) {
            constexpr int par = decltype(PAR)::value;
            constexpr int LOP = BOTH ? (par == 0 ? LA + LB : 0) : (par == 0 ? LA : LB);
            constexpr int G = gcd_of(LA, LB);                            // every count below is a multiple of it
            const int nbuf = buf + 1 == DEPTH ? 0 : buf + 1;
            const bool load = LOP != 0 && s + DEPTH - 1 < n_slice, load2 = LOP != 0 && s + DEPTH < n_slice;
            // the last four slices carry the old C of the epilogue (no operand load is left to issue by then)
            // (a copy of the slice of its own, chosen once per slice: a test in front of each of its loads cost the tails of
            // short-k problems without C to fetch 1-3 %)
            // (through readfirstlane: the choice below is then a scalar branch between two straight-line copies; left to the
            // compiler's own view of what is uniform it became a lane-mask test with the two copies chained behind each other)
            const int c_first = !OLD_C_AHEAD ? -1 :
                __builtin_amdgcn_readfirstlane((c_ahead && s + 4 >= n_slice) ? (s + 4 - n_slice) * Cfg::C_PER_SLICE : -1);
            if constexpr (OLD_C_AHEAD) {
                if (c_first >= 0) mfma_and_read(std::integral_constant<int, 0>{}, PAR, ca, cb, na, nb, nbuf, false, false, buf, std::true_type{}, c_first);
                else mfma_and_read(std::integral_constant<int, 2>{}, PAR, ca, cb, na, nb, nbuf, load, load2, buf, std::false_type{}, 0);
            } else {
                mfma_and_read(std::integral_constant<int, 2>{}, PAR, ca, cb, na, nb, nbuf, load, load2, buf, std::false_type{}, 0);
            }
            if constexpr (BOTH) {
                if constexpr (par == 0) { advance_op(OPX, 2); advance_op(OPY, 2); }
            } else {
                advance_op(std::integral_constant<int, par ^ EVEN_OP>{}, 2);
            }
            MMBO_WAIT_LGKM0();
            const int cur = ((load ? 1 : 0) + (load2 ? 1 : 0)) * LOP +
                            (c_first >= 0 ? max(0, min(Cfg::C_PER_SLICE, Cfg::C_GROUPS - c_first)) : 0);
            const int keep = cur + hist[0] + (DEPTH >= 6 ? hist[1] : 0);
            constexpr int KMAX0 = BOTH ? 2 * (LA + LB) : 2 * (LA > LB ? LA : LB) * 3, KC3 = OLD_C_AHEAD ? 3 * Cfg::C_PER_SLICE : 0;
            constexpr int KMAX = ((KMAX0 > KC3 ? KMAX0 : KC3) + G - 1) / G * G;
            bool waited = false;
            static_for<KMAX / G>([&](auto Q) {
                constexpr int c = KMAX - decltype(Q)::value * G;          // KMAX, KMAX-G, ..., G
                if (!waited && keep >= c) { MMBO_WAIT_VM(c); waited = true; }
            });
            if (!waited) MMBO_WAIT_VM(0);
            MMBO_BARRIER();
            hist[1] = hist[0];
            hist[0] = cur;
            buf = nbuf;
        };
        constexpr std::integral_constant<int, 0> EVEN{};
        constexpr std::integral_constant<int, 1> ODD{};
        for (; s + 1 + DEPTH < n_slice; s += 2) {
            steady_step(EVEN, s, fa[0], fb[0], fa[1], fb[1]);
            steady_step(ODD, s + 1, fa[1], fb[1], fa[0], fb[0]);
            hist[0] = BOTH ? 0 : 2 * LB;
            hist[1] = BOTH ? 2 * (LA + LB) : 2 * LA;
        }
        for (; s < n_slice; s += 2) {
            tail_step(EVEN, s, fa[0], fb[0], fa[1], fb[1]);
            if (s + 1 < n_slice) tail_step(ODD, s + 1, fa[1], fb[1], fa[0], fb[0]);
        }
    }
#undef MMBO_BARRIER
#undef MMBO_WAIT_VM
#undef MMBO_WAIT_LGKM0

    if (k_tail != 0) {
        // The partial last slice.  The loop ended on a barrier after every wavefront's last LDS read and with no load in
        // flight, so buffer 0 is free: fill it through registers (zeros from k_tail on), then one more slice of MFMAs.
        TileA::fill_tail(gA + (int64_t)n_slice * stepA, lda, m_here, backA, k_tail, lds, wave, lane);
        TileB::fill_tail(gB + (int64_t)n_slice * stepB, ldb, n_here, backB, k_tail, lds + TileA::BYTES, wave, lane);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        fa[0].read_all(lds_base, adA);
        fb[0].read_all(lds_base + TileA::BYTES, adB);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        static_for<Cfg::NMFMA>([&](auto M) {
            constexpr int m = decltype(M)::value;
            constexpr int tt = m / (FM * FN), ij = m % (FM * FN);
            constexpr int i = ij / FN, j = (i & 1) ? FN - 1 - ij % FN : ij % FN;
            if constexpr (ESZ == 2) mfma_acc<(i * FN + j) * 4, NACC>(fa[0].x[i], fb[0].x[j]);
            else mfma_acc_f32<(i * FN + j) * 4, NACC>(fa[0].x[i][tt], fb[0].x[j][tt]);
        });
        __syncthreads();            // the next tile's direct loads overwrite buffer 0
    }
    // the last MFMAs' results must have landed before they are read back
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // Epilogue, down a column first: the eight 8-byte stores a lane makes into one column of its wave tile follow
    // each other, so every 128-byte line of C is completed within eight instructions (measured at 8192^3: 135 MB
    // written to memory per launch, the algorithmic 134 MB; with the rows as the outer loop it was 318 MB).
    // Block (i, j): lane l holds C(row, col) for row = i*16 + 4*(l/16) + 0..3, col = j*16 + l%16 (the
    // 16x16 MFMA result layout: four consecutive rows of one column).  C = alpha*acc (+ beta*C), the old C read only
    // when beta != 0 (reference: src/gemm/ref/Kernels.cpp:87); with GlobalSplitU > 1 the raw sums go to the fp32
    // workspace [split][batch][n][m] and the reduction kernel applies alpha and beta.
    const uint32_t wrow0 = row0 + wm * Cfg::TM + 4 * (lane >> 4), wcol0 = col0 + wn * Cfg::TN + (lane & 15);
    if (m_here < (uint32_t)BM || n_here < (uint32_t)BN) {
        // Edge tile (reference: the un-shift and the guarded store, src/gemm/ref/Kernels.cpp:1007-1121).  Tile row r is
        // row r of C, except in the last 16-byte group of a row-contiguous A (Tile::rc_group_off): there tile rows
        // gsm+shm .. gsm+EPC-1 are rows gsm .. m_here-1, and tile rows gsm .. gsm+shm-1 repeat rows that the group
        // before already produced.  Columns likewise under a row-contiguous B.  Every element is tested against the
        // tile's extent; four rows go out as one vector where all four exist unshifted and C allows it.
        // (a k-contiguous operand has no shift: gs = the extent, sh = 0, and the tests below reduce to r < extent)
        // The extents and the lane number pass through an empty asm: everything below is derived from them here, after
        // the slice loop.  Otherwise the compiler computes the per-block tests up front and, with the register file full
        // of fragments during the loop, parks them in scratch memory.
        uint32_t e_m = m_here, e_n = n_here, e_lane = lane;
        asm volatile("" : "+s"(e_m), "+s"(e_n), "+v"(e_lane));
        const uint32_t gsm = TA ? e_m : (e_m - 1) / EPC * EPC, shm = TA ? 0u : gsm + EPC - e_m;
        const uint32_t gsn = !TB ? e_n : (e_n - 1) / EPC * EPC, shn = !TB ? 0u : gsn + EPC - e_n;
        const uint32_t vec_rows = shm == 0 ? e_m : gsm;                     // tile rows below this are in place
        const float alpha = args.alpha, beta = args.beta;
        const bool to_ws = args.splits > 1;
        float *ws = args.ws + ((size_t)split * args.batch + batch) * (size_t)args.m * args.n;
        T *C = static_cast<T *>(args.C) + (int64_t)batch * args.strideC;
        const bool vec_c = args.vec_c != 0;
        typedef typename std::conditional<ESZ == 2, u32x2, u32x4>::type cvec;
        const uint32_t lrow0 = wm * Cfg::TM + 4 * (e_lane >> 4), lcol0 = wn * Cfg::TN + (e_lane & 15);
        static_for<FM * FN>([&](auto IJ) {
            constexpr int j = decltype(IJ)::value / FM, i = decltype(IJ)::value % FM, base = (i * FN + j) * 4;
            const uint32_t lr = lrow0 + i * 16, lc = lcol0 + j * 16;
            float v[4] = {acc_read<base>(), acc_read<base + 1>(), acc_read<base + 2>(), acc_read<base + 3>()};
            // the column of C this lane's tile column stands for, if any
            const bool col_ok = lc < gsn || (lc >= gsn + shn && lc - shn < e_n);
            const uint32_t col = col0 + (lc < gsn ? lc : lc - shn);
            if (col_ok) {
                if (!to_ws && vec_c && lr + 3 < vec_rows) {
                    T *p = C + (size_t)col * args.ldc + row0 + lr;
                    union { T e[4]; cvec v; } io;
                    if (beta != 0.0f) {
                        io.v = *reinterpret_cast<const cvec *>(p);
#pragma unroll
                        for (int r = 0; r < 4; ++r) io.e[r] = (T)__builtin_fmaf(beta, (float)io.e[r], alpha * v[r]);
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r) io.e[r] = (T)(alpha * v[r]);
                    }
                    *reinterpret_cast<cvec *>(p) = io.v;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t tr = lr + r;
                        const bool row_ok = tr < gsm || (tr >= gsm + shm && tr - shm < e_m);
                        const uint32_t row = row0 + (tr < gsm ? tr : tr - shm);
                        if (row_ok) {
                            if (to_ws) {
                                ws[(size_t)col * args.m + row] = v[r];
                            } else {
                                T *p = C + (size_t)col * args.ldc + row;
                                float o = alpha * v[r];
                                if (beta != 0.0f) o = __builtin_fmaf(beta, (float)*p, o);
                                *p = (T)o;
                            }
                        }
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);          // one block at a time: keeps the address arithmetic of 64 blocks from piling up
        });
        continue;
    }
    if (args.splits > 1) {
        float *ws = args.ws + ((size_t)split * args.batch + batch) * (size_t)args.m * args.n;
        if (BM * BN < 256 * 256 && args.ws_narrow) {
            // The partial sums as device-scope buffer stores (the tile's part of the workspace as a buffer; args.ws_narrow:
            // its span, BN columns of m floats, fits 32-bit offsets): written through as they are made, so the reduction
            // kernel does not have to wait for the L2s to write them back when this kernel ends (fp16, us: 1280 x 1280 x 4096
            // on 128 x 128 x 2 splits 25.7 -> 24.5, 4096 x 128 x 4096 on 64 x 64 x 2 15.3 -> 14.9, 512 x 512 x 16384 25.4 -> 23.8).
            // Not on the 256 x 256 tiles, whose one work-group per CU then waits on its 64 stores per wavefront itself (2048 x
            // 2048 x 8192 with 2 splits 89.7 -> 92.1).  Scalar offset literal zero, like the stores of C below and for the
            // same reason.
            const __amdgpu_buffer_rsrc_t tile_ws = __builtin_amdgcn_make_buffer_rsrc(
                reinterpret_cast<void *>(uniform_address(ws + (size_t)col0 * args.m + row0)), 0, 0x7fffffff, 0x00020000);
            const uint32_t ws_col = 16 * args.m * 4;
            const uint32_t ws_lane = ((wn * Cfg::TN + (lane & 15)) * args.m + wm * Cfg::TM + 4 * (lane >> 4)) * 4;
            static_for<FM * FN>([&](auto IJ) {
                constexpr int j = decltype(IJ)::value / FM, i = decltype(IJ)::value % FM, base = (i * FN + j) * 4;
                const f32x4 v = {acc_read<base>(), acc_read<base + 1>(), acc_read<base + 2>(), acc_read<base + 3>()};
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), tile_ws, ws_lane + j * ws_col + i * 64, 0, 16);
            });
            continue;
        }
        static_for<FM * FN>([&](auto IJ) {
            constexpr int j = decltype(IJ)::value / FM, i = decltype(IJ)::value % FM, base = (i * FN + j) * 4;
            float *p = ws + (size_t)(wcol0 + j * 16) * args.m + wrow0 + i * 16;
            // with m not a multiple of four the columns of the workspace start at any multiple of four bytes: the vector
            // type only promises that much alignment (the hardware takes a 16-byte store at any dword)
            typedef f32x4 __attribute__((aligned(4))) f32x4_dword_aligned;
            *reinterpret_cast<f32x4_dword_aligned *>(p) = f32x4{acc_read<base>(), acc_read<base + 1>(), acc_read<base + 2>(), acc_read<base + 3>()};
        });
        continue;
    }
    const float alpha = args.alpha, beta = args.beta;
    const uint32_t ldc = args.ldc;
    T *C = static_cast<T *>(args.C) + (int64_t)batch * args.strideC;
    const bool vec_c = args.vec_c != 0;
    typedef typename std::conditional<ESZ == 2, u32x2, u32x4>::type cvec;       // four consecutive rows of one column
    // fp16: a lane's four rows are 8 bytes, a column of one block 32 bytes -- a quarter of a cache line per request.  Two
    // vertically adjacent blocks therefore travel together: v_permlane16_swap hands the lanes of the even 16-lane rows their
    // lower neighbour's four rows of the upper block and the odd rows their upper neighbour's of the lower block, so every
    // lane stores 16 contiguous bytes, from row pair_row0 of the pair on, and a column gets 64 per instruction.  The
    // exchange is its own inverse: applied to a vector loaded from there it returns each lane its rows of both blocks.
    // Two results at a time go through the packed conversion (round to nearest even, like the scalar cast).
    constexpr bool PAIRED_C = ESZ == 2 && FM % 2 == 0;
    const uint32_t pair_row0 = row0 + wm * Cfg::TM + (((lane >> 4) & 1) ? 4 * (lane >> 4) + 12 : 4 * (lane >> 4));
    // The whole-tile store sequences below address C as a buffer whose origin is the tile's first element (the host lets
    // vec_c stand only where a tile's span of C, BN x ldc elements, fits the 32-bit offsets of a buffer access): the lane's
    // part of an address is worked out once, a block adds its column (one vector addition per block column) and, as an
    // immediate, its row.  (The column as the instruction's scalar offset would save that addition, but the compiler then
    // leaves out the wait states between a 16-byte store and the next write to its data registers -- it takes them to be
    // needed only without a scalar offset -- and with the accumulator reads of the next block right behind the store
    // a few lanes stored the next block's value: seen on the 8-wave fp32 tile.)
    // Two cache policies, one copy of each store sequence per policy, chosen once:
    // * device scope (sc1) by default: the stores go through the XCD's L2 to memory as they are made.  Left in the L2 as
    //   ordinary stores are, C is written back when the kernel ends, and where the epilogue is on the critical path (one
    //   round of tiles, short k) that is time added at the end: 64 x 512^3 fp16 26.6 -> 25.7 us, 2048^3 21.6 -> 20.9;
    // * non-temporal where the host asks for it (args.c_stream: a long slice loop and four or more rounds of tiles per CU):
    //   the kernel never reads what it wrote, and a resident work-group's 128 KB per tile (4 MB per XCD and round of tiles:
    //   the size of its L2) otherwise push the operand panels the next tiles share out of the L2 (measured at 8192^3 fp16:
    //   the epilogue itself takes 1 us longer, the next tile's loop 3-6 us less).  Not everywhere: with this hint the two
    //   64-byte halves of a line travel to memory separately (64 x 512^3 fp16: 7.4 us to issue a wavefront's 32 stores
    //   against 3.5).
    const bool c_stream = args.c_stream != 0;
    const T *c_origin = C + (size_t)col0 * ldc + row0;
    // (the descriptor is put together inside each copy, from an address that has just passed through readfirstlane: built once
    // up here it reached some of the copies in vector registers, and every store became a loop over the distinct descriptors)
    auto c_buffer = [&]() {
        return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(uniform_address(c_origin)), 0, 0x7fffffff, 0x00020000);
    };
    const uint32_t c_block_col = 16 * ldc * ESZ;                          // bytes from a block's column to the next block's
    // this lane's first element of the wave tile: four rows of one column per block, or, fp16 pairs, eight rows of two blocks
    const uint32_t c_lane = ((wn * Cfg::TN + (lane & 15)) * ldc + wm * Cfg::TM + 4 * (lane >> 4)) * ESZ;
    const uint32_t c_lane_pair = ((wn * Cfg::TN + (lane & 15)) * ldc + (pair_row0 - row0)) * ESZ;
    auto store_c = [](auto STREAM, auto value, __amdgpu_buffer_rsrc_t tile_c, uint32_t lane_and_row, uint32_t column) {
        constexpr int policy = decltype(STREAM)::value ? 2 : 16;            // nt : sc1
        if constexpr (sizeof(value) == 16) __builtin_amdgcn_raw_buffer_store_b128(value, tile_c, lane_and_row, column, policy);
        else __builtin_amdgcn_raw_buffer_store_b64(value, tile_c, lane_and_row, column, policy);
    };
    auto per_policy = [&](auto &&body) {
        if (c_stream) body(std::true_type{});
        else body(std::false_type{});
    };
    auto two = [](float a, float b) -> uint32_t {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{a, b}), f16x2));
    };
    if (vec_c && beta != 0.0f) {
        if constexpr (PAIRED_C) {
            // the whole wave tile of old C is requested before its first value is used (see below) -- or was requested
            // under the last four slices and is waiting in the ring buffers those slices left (c_ahead)
            u32x4 cold[FM * FN / 2];
            bool from_lds = false;
            if constexpr (OLD_C_AHEAD) {
                if (c_ahead) {
                    from_lds = true;
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // this wavefront's own loads: nobody else reads them
                    const uint32_t first_buf = (uint32_t)(n_slice - 4) % DEPTH;
                    const uint32_t mine = lds_base + wave * (Cfg::C_PER_SLICE * 1024) + lane * 16;
                    static_for<4>([&](auto CC) {
                        constexpr int cc = decltype(CC)::value;
                        uint32_t b = first_buf + cc;
                        if (b >= (uint32_t)DEPTH) b -= DEPTH;
                        const uint32_t at = mine + b * Cfg::SLICE_BYTES;
                        static_for<Cfg::C_PER_SLICE>([&](auto Q) {
                            constexpr int q = decltype(Q)::value;
                            if constexpr (cc * Cfg::C_PER_SLICE + q < Cfg::C_GROUPS) cold[cc * Cfg::C_PER_SLICE + q] = lds_read_b128<q * 1024>(at);
                        });
                    });
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    // (a resident work-group's next tile sends its first loads into these buffers: not before every wavefront
                    // has taken its old C out of them)
                    __syncthreads();
                }
            }
            if (!from_lds)
            static_for<FM * FN / 2>([&](auto IJ) {
                constexpr int j = decltype(IJ)::value / (FM / 2), i = 2 * (decltype(IJ)::value % (FM / 2));
                cold[decltype(IJ)::value] = *reinterpret_cast<const u32x4 *>(C + (size_t)(wcol0 + j * 16) * ldc + pair_row0 + i * 16);
            });
            per_policy([&](auto STREAM) {
            const __amdgpu_buffer_rsrc_t tile_c = c_buffer();
            static_for<FM * FN / 2>([&](auto IJ) {
                constexpr int j = decltype(IJ)::value / (FM / 2), i = 2 * (decltype(IJ)::value % (FM / 2));
                constexpr int b0 = (i * FN + j) * 4, b1 = ((i + 1) * FN + j) * 4;
                const u32x4 c = cold[decltype(IJ)::value];
                auto o0 = __builtin_amdgcn_permlane16_swap(c[0], c[2], false, false);
                auto o1 = __builtin_amdgcn_permlane16_swap(c[1], c[3], false, false);
                union { T e[4]; uint32_t u[2]; } xo, yo;
                xo.u[0] = o0[0]; xo.u[1] = o1[0];
                yo.u[0] = o0[1]; yo.u[1] = o1[1];
                float x[4] = {alpha * acc_read<b0>(), alpha * acc_read<b0 + 1>(), alpha * acc_read<b0 + 2>(), alpha * acc_read<b0 + 3>()};
                float y[4] = {alpha * acc_read<b1>(), alpha * acc_read<b1 + 1>(), alpha * acc_read<b1 + 2>(), alpha * acc_read<b1 + 3>()};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    x[r] = __builtin_fmaf(beta, (float)xo.e[r], x[r]);
                    y[r] = __builtin_fmaf(beta, (float)yo.e[r], y[r]);
                }
                auto s0 = __builtin_amdgcn_permlane16_swap(two(x[0], x[1]), two(y[0], y[1]), false, false);
                auto s1 = __builtin_amdgcn_permlane16_swap(two(x[2], x[3]), two(y[2], y[3]), false, false);
                store_c(STREAM, u32x4{(uint32_t)s0[0], (uint32_t)s1[0], (uint32_t)s0[1], (uint32_t)s1[1]}, tile_c, c_lane_pair + j * c_block_col + i * 16 * ESZ, 0u);
            });
            });
            continue;
        }
        // beta != 0 (reference: the fma(C, beta, .) epilogue, MT192x096x08 kernel :3037-3056): a whole column strip of
        // old C (fp16: the whole wave tile) is requested before its first value is used, so the read-modify-write runs
        // at memory bandwidth instead of one load latency per block.
        constexpr int CHUNK = ESZ == 2 ? FM * FN : FM;                          // blocks requested at once
        per_policy([&](auto STREAM) {
            const __amdgpu_buffer_rsrc_t tile_c = c_buffer();
        static_for<FM * FN / CHUNK>([&](auto CC) {
            constexpr int c0 = decltype(CC)::value * CHUNK;
            cvec cold[CHUNK];
            static_for<CHUNK>([&](auto Q) {
                constexpr int ij = c0 + decltype(Q)::value, j = ij / FM, i = ij % FM;
                cold[decltype(Q)::value] = *reinterpret_cast<const cvec *>(C + (size_t)(wcol0 + j * 16) * ldc + wrow0 + i * 16);
            });
            static_for<CHUNK>([&](auto Q) {
                constexpr int ij = c0 + decltype(Q)::value, j = ij / FM, i = ij % FM, base = (i * FN + j) * 4;
                union { T e[4]; cvec v; } io;
                io.v = cold[decltype(Q)::value];
                float v[4] = {alpha * acc_read<base>(), alpha * acc_read<base + 1>(), alpha * acc_read<base + 2>(), alpha * acc_read<base + 3>()};
#pragma unroll
                for (int r = 0; r < 4; ++r) io.e[r] = (T)__builtin_fmaf(beta, (float)io.e[r], v[r]);
                store_c(STREAM, io.v, tile_c, c_lane + j * c_block_col + i * 16 * ESZ, 0u);
            });
        });
        });
        continue;
    }
    // beta == 0: C is never read.  The aligned and the element-wise variant are separate straight-line sequences: with
    // the choice made per block the epilogue was bound by instruction issue (64 blocks x ~20 instructions with two
    // branches each took 7 us of a 220 us tile at 8192^3, whatever the number of work-groups writing at the time).
    if (vec_c && PAIRED_C) {
        // alpha == 1 gets a copy of the sequence without the multiplications: with the packed conversions that makes 4 (12)
        // instructions per eight results where scalar casts took 16.
        auto store_all = [&](auto UNIT_ALPHA, auto STREAM, __amdgpu_buffer_rsrc_t tile_c) {
            constexpr bool unit = decltype(UNIT_ALPHA)::value;
            static_for<FM * FN / 2>([&](auto IJ) {
                constexpr int j = decltype(IJ)::value / (FM / 2), i = 2 * (decltype(IJ)::value % (FM / 2));
                constexpr int b0 = (i * FN + j) * 4, b1 = ((i + 1) * FN + j) * 4;
                float x[4] = {acc_read<b0>(), acc_read<b0 + 1>(), acc_read<b0 + 2>(), acc_read<b0 + 3>()};
                float y[4] = {acc_read<b1>(), acc_read<b1 + 1>(), acc_read<b1 + 2>(), acc_read<b1 + 3>()};
                if constexpr (!unit) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) { x[r] *= alpha; y[r] *= alpha; }
                }
                auto s0 = __builtin_amdgcn_permlane16_swap(two(x[0], x[1]), two(y[0], y[1]), false, false);
                auto s1 = __builtin_amdgcn_permlane16_swap(two(x[2], x[3]), two(y[2], y[3]), false, false);
                store_c(STREAM, u32x4{(uint32_t)s0[0], (uint32_t)s1[0], (uint32_t)s0[1], (uint32_t)s1[1]}, tile_c, c_lane_pair + j * c_block_col + i * 16 * ESZ, 0u);
            });
        };
        per_policy([&](auto STREAM) {
            const __amdgpu_buffer_rsrc_t tile_c = c_buffer();
            if (alpha == 1.0f) store_all(std::true_type{}, STREAM, tile_c);
            else store_all(std::false_type{}, STREAM, tile_c);
        });
    } else if (vec_c) {
        per_policy([&](auto STREAM) {
            const __amdgpu_buffer_rsrc_t tile_c = c_buffer();
        static_for<FM * FN>([&](auto IJ) {
            constexpr int j = decltype(IJ)::value / FM, i = decltype(IJ)::value % FM, base = (i * FN + j) * 4;
            union { T e[4]; cvec v; } io;
            io.e[0] = (T)(alpha * acc_read<base>());
            io.e[1] = (T)(alpha * acc_read<base + 1>());
            io.e[2] = (T)(alpha * acc_read<base + 2>());
            io.e[3] = (T)(alpha * acc_read<base + 3>());
            store_c(STREAM, io.v, tile_c, c_lane + j * c_block_col + i * 16 * ESZ, 0u);
        });
        });
    } else {
        static_for<FM * FN>([&](auto IJ) {
            constexpr int j = decltype(IJ)::value / FM, i = decltype(IJ)::value % FM, base = (i * FN + j) * 4;
            T *p = C + (size_t)(wcol0 + j * 16) * ldc + wrow0 + i * 16;
            float v[4] = {alpha * acc_read<base>(), alpha * acc_read<base + 1>(), alpha * acc_read<base + 2>(), alpha * acc_read<base + 3>()};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float o = v[r];
                if (beta != 0.0f) o = __builtin_fmaf(beta, (float)p[r], o);
                p[r] = (T)o;
            }
        });
    }
    }   // tiles of this work-group
}

}  // namespace mmbo
