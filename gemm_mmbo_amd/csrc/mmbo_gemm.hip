// C ABI of the gfx950 GEMM library: argument checking, tile-config table, per-shape selection,
// split-K workspace and kernel dispatch.  The reference's counterpart is the header-inline host
// layer src/gemm/gemm.h (front-ends), src/gemm/constants.h (tables) and src/gemm/driver.h (launch).
#include "../../include/mmbo_gemm.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <vector>

#include "configs.hpp"
#include "gemm_common.hpp"
#include "gemm_staged.hpp"
#include "launch.hpp"
#include "tuned_table.hpp"

namespace mmbo {

namespace {

// Config ids (configs.hpp): [0, kStagedConfigs) are the staged kernel's (tile, split) pairs, then the ring kernel's
// (ring tile, split) pairs, then the x16 kernel's.  A ring config applies when m, n are multiples of its tile, k splits
// into whole slices and A, B are 16-byte aligned; otherwise the call is refused with MMBO_ERR_INVALID_CONFIG.
struct ConfigRef {
    bool ring;      // a direct-to-LDS kernel (ring or x16)
    int tile;
    int split;
    bool x16;
};
inline ConfigRef config_ref(int id)
{
    if (id >= kX16Base) return {true, (id - kX16Base) % NUM_X16_TILES, kSplits[(id - kX16Base) / NUM_X16_TILES], true};
    if (id < kStagedConfigs) return {false, id % NUM_TILES, kSplits[id / NUM_TILES], false};
    id -= kStagedConfigs;
    return {true, id % NUM_RING_TILES, kSplits[id / NUM_RING_TILES], false};
}
inline bool valid_dtype(int dtype) { return dtype == MMBO_F32 || dtype == MMBO_F16 || dtype == MMBO_F64; }

// Does the ring (x16 = false) or x16 config (tile, split) take this shape?  Ring: m, n whole tiles, k whole slices, the
// same number for every split; A and B 16-byte aligned (checked at the call).  x16: any shape and alignment (its loads
// repeat or shift the last rows of an edge tile, its edge tiles store under guards, a partial last slice of k is
// zero-filled; the splits take equal runs of whole slices and the last one what is left, fewer splits than asked for
// when k is short) -- except a memory-contiguous m (transA = N) or n (transB = T) shorter than one 16-byte load.
inline bool ring_shape_ok(int dtype, int tile, int split, int transA, int transB, size_t m, size_t n, size_t k, bool x16)
{
    if (k == 0) return false;
    if (x16) {
        const size_t per16 = dtype == MMBO_F32 ? 4 : 8;
        return (transA || m >= per16) && (!transB || n >= per16);
    }
    const RingRow &r = kRingTiles[tile];
    const size_t bk = (size_t)ring_bk(dtype);
    if (m % r.bm || n % r.bn || k % bk) return false;
    return (k / bk) % (size_t)split == 0;
}

thread_local int g_last_hip_error = 0;

int hip_fail(hipError_t e)
{
    g_last_hip_error = (int)e;
    return MMBO_ERR_HIP;
}

// ---- split-K workspace ------------------------------------------------------------------------
// A workspace holds the partial sums of one GEMM with GlobalSplitU > 1: [split][batch][n][m] fp32.
constexpr int kMaxDevices = 64;

// Library-owned workspaces: one per (device, stream), so GEMMs on different streams never share partial sums, grown on
// demand, at most kMaxWsSlots per device (the reference's launcher never frees what it loads, src/gemm/driver.h:41; this
// table is bounded instead).
//   - Each device has its own table and table lock, held only to look a slot up, add one or take one out.
//   - Each slot has its own lock, held by a call from the lookup until both launches that use the buffer (the GEMM and
//     the reduction) are queued: two host threads on one stream cannot interleave their launches, and growing a buffer
//     (wait for that stream, free, allocate) stalls only callers of that same stream.
//   - A new stream that finds the table full retires the least recently used slot nobody holds: the table lock is given
//     up, the device is synchronised (the slot's stream may no longer exist, so it cannot be waited for by handle) and
//     the buffer freed.  mmbo_release_stream_workspace retires one stream's slot at the caller's request.
constexpr size_t kMaxWsSlots = 8;
struct WsSlot {
    hipStream_t stream = nullptr;
    char *base = nullptr;
    size_t bytes = 0;
    unsigned long long last_use = 0;
    bool dead = false;          // taken out of the table; whoever still holds a reference looks the stream up again
    std::mutex use;
};
struct WsTable {
    std::mutex lock;
    std::vector<std::shared_ptr<WsSlot>> slots;
    unsigned long long clock = 0;
};
WsTable g_ws[kMaxDevices];

// A held slot: its buffer may be used until the holder is destroyed.
struct WsHold {
    std::shared_ptr<WsSlot> slot;
    std::unique_lock<std::mutex> held;
};

// The buffer of (current device, stream), at least `bytes` large, held for the caller.
int workspace(hipStream_t stream, size_t bytes, WsHold &hold, char **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    if (dev < 0 || dev >= kMaxDevices) return MMBO_ERR_NO_DEVICE;
    WsTable &tab = g_ws[dev];
    for (;;) {
        std::shared_ptr<WsSlot> slot, victim;
        std::unique_lock<std::mutex> victim_held;
        {
            std::lock_guard<std::mutex> tl(tab.lock);
            for (auto &sl : tab.slots)
                if (sl->stream == stream) slot = sl;
            if (!slot) {
                if (tab.slots.size() >= kMaxWsSlots) {
                    // retire the least recently used slot that no call holds
                    size_t pick = tab.slots.size();
                    for (size_t i = 0; i < tab.slots.size(); ++i) {
                        if (pick < tab.slots.size() && tab.slots[i]->last_use >= tab.slots[pick]->last_use) continue;
                        std::unique_lock<std::mutex> t(tab.slots[i]->use, std::try_to_lock);
                        if (!t.owns_lock()) continue;
                        pick = i;
                        victim_held = std::move(t);
                    }
                    if (pick < tab.slots.size()) {
                        victim = tab.slots[pick];
                        victim->dead = true;
                        tab.slots.erase(tab.slots.begin() + (long)pick);
                    }
                    // (every slot held by a call in flight: the table grows past its bound for now)
                }
                slot = std::make_shared<WsSlot>();
                slot->stream = stream;
                tab.slots.push_back(slot);
            }
            slot->last_use = ++tab.clock;
        }
        if (victim) {
            if (victim->base) {
                e = hipDeviceSynchronize();
                (void)hipFree(victim->base);
                victim->base = nullptr;
                victim->bytes = 0;
            }
            victim_held.unlock();
            if (e != hipSuccess) return hip_fail(e);
        }
        std::unique_lock<std::mutex> held(slot->use);
        if (slot->dead) continue;                    // retired between the lookup and here: look the stream up again
        if (slot->bytes < bytes) {
            if (slot->base) {
                // earlier launches on this stream may still be using the old buffer (fails under stream capture: a captured
                // call must find its workspace already large enough, or use the entry point that allocates nothing)
                e = hipStreamSynchronize(stream);
                if (e != hipSuccess) return hip_fail(e);
                (void)hipFree(slot->base);
                slot->base = nullptr;
                slot->bytes = 0;
            }
            size_t want = bytes + bytes / 4;
            void *p = nullptr;
            if (hipMalloc(&p, want) != hipSuccess) {
                (void)hipGetLastError();
                want = bytes;
                if (hipMalloc(&p, want) != hipSuccess) {
                    (void)hipGetLastError();
                    return MMBO_ERR_WORKSPACE;
                }
            }
            slot->base = static_cast<char *>(p);
            slot->bytes = want;
        }
        *out = slot->base;
        hold.slot = std::move(slot);
        hold.held = std::move(held);
        return MMBO_OK;
    }
}

// Takes the slots `which` selects out of the current device's table and frees their buffers.  `stream_only`: wait for
// that stream alone (its handle is still valid: the caller is about to destroy it); otherwise for the whole device.
int release_slots(bool stream_only, hipStream_t stream)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    if (dev < 0 || dev >= kMaxDevices) return MMBO_ERR_NO_DEVICE;
    WsTable &tab = g_ws[dev];
    std::vector<std::shared_ptr<WsSlot>> out;
    {
        std::lock_guard<std::mutex> tl(tab.lock);
        for (size_t i = 0; i < tab.slots.size();) {
            if (!stream_only || tab.slots[i]->stream == stream) {
                out.push_back(tab.slots[i]);
                tab.slots.erase(tab.slots.begin() + (long)i);
            } else {
                ++i;
            }
        }
    }
    if (out.empty()) return MMBO_OK;
    hipError_t first = hipSuccess;
    for (auto &sl : out) {
        std::lock_guard<std::mutex> held(sl->use);       // a call that holds the slot queues its launches first
        sl->dead = true;
    }
    e = stream_only ? hipStreamSynchronize(stream) : hipDeviceSynchronize();
    if (e != hipSuccess) return hip_fail(e);
    for (auto &sl : out) {
        std::lock_guard<std::mutex> held(sl->use);
        if (sl->base) {
            e = hipFree(sl->base);
            if (e != hipSuccess && first == hipSuccess) first = e;
            sl->base = nullptr;
            sl->bytes = 0;
        }
    }
    return first == hipSuccess ? MMBO_OK : hip_fail(first);
}

// The workspace of the entry point that allocates nothing: one array per device in the library's own image, there from
// the moment the code object is loaded until the process ends.  In host code the array's name is only a handle: the
// device address of each GPU's copy comes from hipGetSymbolAddress, once per device, and that pointer is what the
// kernels get.  Nothing in it has to start at zero: every partial sum a GEMM reads was written by that same GEMM.
constexpr size_t kScratchPartialBytes = 32u << 20;
static __device__ __align__(256) unsigned char scratch[kScratchPartialBytes];
std::mutex g_scratch_mutex;
char *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(char **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    if (dev < 0 || dev >= kMaxDevices) return MMBO_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e);
        if (!p) return MMBO_ERR_WORKSPACE;
        g_scratch_ptr[dev] = static_cast<char *>(p);
    }
    *out = g_scratch_ptr[dev];
    return MMBO_OK;
}

// ---- table ------------------------------------------------------------------------------------
template <int DTYPE, int TILE>
hipError_t dispatch_tile(int tile, int ta, int tb, const GemmArgs &a, hipStream_t s)
{
    if (tile == TILE) return launch_staged<DTYPE, TILE>(ta, tb, a, s);
    if constexpr (TILE + 1 < NUM_TILES) return dispatch_tile<DTYPE, TILE + 1>(tile, ta, tb, a, s);
    return hipErrorInvalidValue;
}

template <int DTYPE, int TILE>
hipError_t dispatch_ring(int tile, int ta, int tb, const GemmArgs &a, hipStream_t s)
{
    if (tile == TILE) return launch_ring<DTYPE, TILE>(ta, tb, a, s);
    if constexpr (TILE + 1 < NUM_RING_TILES) return dispatch_ring<DTYPE, TILE + 1>(tile, ta, tb, a, s);
    return hipErrorInvalidValue;
}

template <int DTYPE, int TILE>
hipError_t dispatch_x16(int tile, int ta, int tb, const GemmArgs &a, hipStream_t s)
{
    if (tile == TILE) return launch_x16<DTYPE, TILE>(ta, tb, a, s);
    if constexpr (TILE + 1 < NUM_X16_TILES) return dispatch_x16<DTYPE, TILE + 1>(tile, ta, tb, a, s);
    return hipErrorInvalidValue;
}

template <int TILE>
hipError_t dispatch_dgemm(int tile, int ta, int tb, const GemmArgs &a, hipStream_t s)
{
    if (tile == TILE) return launch_dgemm<TILE>(ta, tb, a, s);
    if constexpr (TILE + 1 < NUM_F64_TILES) return dispatch_dgemm<TILE + 1>(tile, ta, tb, a, s);
    return hipErrorInvalidValue;
}

template <int TILE>
int dgemm_lds_bytes_of(int tile)
{
    if (tile == TILE) return dgemm_lds_bytes<TILE>();
    if constexpr (TILE + 1 < NUM_F64_TILES) return dgemm_lds_bytes_of<TILE + 1>(tile);
    return 0;
}

template <int DTYPE, int TILE>
int lds_bytes_of(int tile)
{
    if (tile == TILE) return staged_lds_bytes<DTYPE, TILE>();
    if constexpr (TILE + 1 < NUM_TILES) return lds_bytes_of<DTYPE, TILE + 1>(tile);
    return 0;
}

inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

// Relative MFMA-pipe cost of a tile's inner loop (1.0 = the 256 x 256 tile): smaller wave tiles read more
// LDS per MFMA.  Fitted to sweeps of every config on MI355X.
double tile_cost(int dtype, int tile)
{
    static const double c32[NUM_TILES] = {1.00, 1.06, 1.03, 1.03, 1.08, 2.2};
    static const double c16[NUM_TILES] = {1.00, 1.10, 1.15, 1.25, 1.9, 4.0};
    return dtype == MMBO_F32 ? c32[tile] : c16[tile];
}

// Modelled time, in GPU clocks, of running the problem with the staged kernel of (tile, split).
// The staged kernel prefetches one stage ahead, so a stage costs the larger of its MFMA time (shared by the
// work-groups resident on the CU) and the global-load latency; short K and few tiles are latency-bound,
// which is what split-K and small tiles buy back.
double model_time(int dtype, int tile, int split, size_t m, size_t n, size_t k, int batch)
{
    const TileRow &r = tile_row(dtype, tile);
    const double cus = 256.0;
    const double mac_per_clk_cu = dtype == MMBO_F32 ? 128.0 : 2048.0;   // dense MFMA rate of one CU
    const double hbm_bytes_per_clk = 3300.0;                            // ~8 TB/s at ~2.4 GHz
    const double load_latency = 1700.0;                                 // clocks from issue to data in registers
    const double esz = dtype == MMBO_F32 ? 4.0 : 2.0;
    double tiles = (double)ceil_div(m, r.bm) * (double)ceil_div(n, r.bn) * batch * split;
    // work-groups resident per CU, bounded by LDS (160 KB) and by 2048 threads
    int lds = dtype == MMBO_F32 ? lds_bytes_of<0, 0>(tile) : lds_bytes_of<1, 0>(tile);
    int per_cu = 160 * 1024 / (lds > 0 ? lds : 1);
    int thr = r.wm * r.wn * 64;
    if (per_cu > 2048 / thr) per_cu = 2048 / thr;
    if (per_cu < 1) per_cu = 1;
    double slots = cus * per_cu;
    double rounds = (double)ceil_div((size_t)tiles, (size_t)slots);
    double resident = tiles >= slots ? per_cu : (tiles > cus ? tiles / cus : 1.0);   // tiles sharing one CU's pipes
    double stage_mfma = (double)r.bm * r.bn * r.bk * tile_cost(dtype, tile) / mac_per_clk_cu;
    double stage = stage_mfma * resident > load_latency ? stage_mfma * resident : load_latency;
    double stages = (double)ceil_div(ceil_div(k, (size_t)split), (size_t)r.bk);
    double epilogue = (double)r.bm * r.bn * esz * resident / 24.0;      // C tile through one CU's store path
    double compute = rounds * (stages * stage + load_latency + epilogue);
    double bytes = ((double)m * k + (double)k * n + (double)m * n) * batch * esz;
    double t = compute > bytes / hbm_bytes_per_clk ? compute : bytes / hbm_bytes_per_clk;
    t += 9000.0;                                                         // launch
    if (split > 1)   // second launch + partial sums written and read back
        t += 9000.0 + (double)m * n * batch * (2.0 * split * 4.0 + esz) / hbm_bytes_per_clk;
    return t;
}

// fp64: microseconds.  Work-groups run in rounds of (CUs x work-groups per CU); a tile costs a fixed overhead
// (first stage, C update, dispatch of its successor: measured per tile and CU with K swept from 96 to 1536 on the
// HPL shape's M and N) plus its K at the tile's in-loop efficiency (from 8192^3), both shared by the work-groups
// resident on the CU; the last, partial round runs with fewer of them.
double model_time_f64(int tile, size_t m, size_t n, size_t k, int batch)
{
    //                                    128x128/4w 256x128/8w 64x64  32x32  128x128/8w 128x64
    static const double overhead_us[NUM_F64_TILES] = {12.8, 26.5, 1.54, 0.25, 10.6, 5.9};
    static const double in_loop_eff[NUM_F64_TILES] = {0.89, 0.853, 0.846, 0.704, 0.91, 0.84};
    static const int resident[NUM_F64_TILES] = {2, 1, 5, 8, 2, 3};
    const TileRow &r = kTilesF64[tile];
    const double cus = 256.0, flop_per_us_cu = 78.6e6 / 256.0, launch = 5.0;
    const double tiles = (double)ceil_div(m, r.bm) * (double)ceil_div(n, r.bn) * batch;
    const double per_tile = overhead_us[tile] + 2.0 * r.bm * r.bn * (double)(k ? k : 1) / flop_per_us_cu / in_loop_eff[tile];
    const double slots = cus * resident[tile];
    const double full = std::floor(tiles / slots), last = tiles - full * slots;
    double t = launch + full * per_tile * resident[tile];
    if (last > 0) t += per_tile * std::ceil(last / cus);
    return t;
}

}  // namespace

hipError_t launch_splitk_reduce(int dtype, const GemmArgs &args, hipStream_t stream)
{
    size_t mn = (size_t)args.m * args.n;
    const bool vec4 = args.m % 4 == 0;                   // a thread then owns four consecutive rows of one column
    dim3 grid((unsigned)ceil_div(vec4 ? mn / 4 : mn, 256), 1, args.batch);
    if (dtype == MMBO_F32)
        return vec4 ? launch_kernel(splitk_reduce_kernel<float, true>, grid, dim3(256), 0, stream, args)
                    : launch_kernel(splitk_reduce_kernel<float, false>, grid, dim3(256), 0, stream, args);
    return vec4 ? launch_kernel(splitk_reduce_kernel<half_t, true>, grid, dim3(256), 0, stream, args)
                : launch_kernel(splitk_reduce_kernel<half_t, false>, grid, dim3(256), 0, stream, args);
}

}  // namespace mmbo

using namespace mmbo;

extern "C" {

const char *mmbo_version(void) { return "mmbo_gemm 0.1 (gfx950)"; }

int mmbo_last_hip_error(void) { return g_last_hip_error; }

const char *mmbo_status_string(int status)
{
    switch (status) {
        case MMBO_OK: return "ok";
        case MMBO_ERR_INVALID_DTYPE: return "invalid dtype";
        case MMBO_ERR_INVALID_OP: return "invalid transpose op";
        case MMBO_ERR_INVALID_SIZE: return "invalid size, leading dimension, stride or batch";
        case MMBO_ERR_NULL_POINTER: return "null pointer";
        case MMBO_ERR_INVALID_CONFIG: return "invalid config id";
        case MMBO_ERR_HIP: return "HIP runtime error";
        case MMBO_ERR_NO_DEVICE: return "no usable device";
        case MMBO_ERR_WORKSPACE: return "split-K workspace allocation failed";
        default: return "unknown status";
    }
}

int mmbo_num_configs(int dtype)
{
    if (!valid_dtype(dtype)) return -MMBO_ERR_INVALID_DTYPE;
    return dtype == MMBO_F64 ? NUM_F64_TILES : kNumConfigs;
}

int mmbo_config_info(int dtype, int config_id, mmbo_config_desc *out)
{
    if (!valid_dtype(dtype)) return MMBO_ERR_INVALID_DTYPE;
    if (!out) return MMBO_ERR_NULL_POINTER;
    if (config_id < 0 || config_id >= mmbo_num_configs(dtype)) return MMBO_ERR_INVALID_CONFIG;
    std::memset(out, 0, sizeof(*out));
    if (dtype == MMBO_F64) {
        const TileRow &r = kTilesF64[config_id];
        std::snprintf(out->name, sizeof(out->name), "MT%03dx%03dx%02d_WT%03dx%03d_W%d_GSU01_MFMA16x16x4", r.bm, r.bn,
                      r.bk, r.bm / r.wm, r.bn / r.wn, r.wm * r.wn);
        out->macro_tile_m = r.bm; out->macro_tile_n = r.bn; out->depth_u = r.bk; out->threads = r.wm * r.wn * 64;
        out->wave_tile_m = r.bm / r.wm; out->wave_tile_n = r.bn / r.wn; out->split_k = 1;
        out->lds_bytes = dgemm_lds_bytes_of<0>(config_id);
        return MMBO_OK;
    }
    const ConfigRef c = config_ref(config_id);
    if (c.ring) {
        const RingRow &r = c.x16 ? kX16Tiles[c.tile] : kRingTiles[c.tile];
        std::snprintf(out->name, sizeof(out->name), "MT%03dx%03dx%02d_WT%03dx%03d_W%d_GSU%02d_DTL1_RING%d%s", r.bm, r.bn,
                      ring_bk(dtype), r.bm / r.wm, r.bn / r.wn, r.wm * r.wn, c.split, r.depth,
                      !c.x16 ? "" : dtype == MMBO_F16 ? "_MFMA16x16x32_ACC" : "_MFMA16x16x4_ACC");
        out->macro_tile_m = r.bm;
        out->macro_tile_n = r.bn;
        out->depth_u = ring_bk(dtype);
        out->threads = r.wm * r.wn * 64;
        out->wave_tile_m = r.bm / r.wm;
        out->wave_tile_n = r.bn / r.wn;
        out->split_k = c.split;
        out->lds_bytes = r.depth * (r.bm + r.bn) * 64;
        return MMBO_OK;
    }
    int tile = config_id % NUM_TILES, split = kSplits[config_id / NUM_TILES];
    const TileRow &r = tile_row(dtype, tile);
    std::snprintf(out->name, sizeof(out->name), "MT%03dx%03dx%02d_WT%03dx%03d_W%d_GSU%02d", r.bm, r.bn, r.bk,
                  r.bm / r.wm, r.bn / r.wn, r.wm * r.wn, split);
    out->macro_tile_m = r.bm;
    out->macro_tile_n = r.bn;
    out->depth_u = r.bk;
    out->threads = r.wm * r.wn * 64;
    out->wave_tile_m = r.bm / r.wm;
    out->wave_tile_n = r.bn / r.wn;
    out->split_k = split;
    out->lds_bytes = dtype == MMBO_F32 ? lds_bytes_of<0, 0>(tile) : lds_bytes_of<1, 0>(tile);
    return MMBO_OK;
}

// Macro tile (and depthU) of a config id.
static TileRow config_tile(int dtype, int id)
{
    if (dtype == MMBO_F64) return kTilesF64[id];
    const ConfigRef c = config_ref(id);
    if (!c.ring) return tile_row(dtype, c.tile);
    const RingRow &rr = c.x16 ? kX16Tiles[c.tile] : kRingTiles[c.tile];
    return TileRow{rr.bm, rr.bn, ring_bk(dtype), 0, 0};
}

// Per-thread global offsets are 32-bit: one tile's span of an operand must stay below 2 GiB.
static bool tile_span_ok(const TileRow &r, int transA, int transB, size_t lda, size_t ldb, size_t esz)
{
    size_t span_a = (transA ? (size_t)r.bm : (size_t)r.bk) * lda * esz;
    size_t span_b = (transB ? (size_t)r.bk : (size_t)r.bn) * ldb * esz;
    return span_a < 0x7FFFFF00ull && span_b < 0x7FFFFF00ull;
}

// Modelled time, in microseconds, of a whole-tile kernel (ring or x16 family, ring tile index rt: 256x256, 128x128,
// 128x64, 64x64) on a shape made of whole tiles.  Work-groups run in rounds of (CUs x work-groups per CU); a tile costs
// a ring fill, its slices at the family's in-loop efficiency (shared by the work-groups resident on the CU) and its
// C traffic; the last, partial round runs with fewer work-groups per CU; split-K adds the reduction launch.  The
// constants are a least-squares fit to the times of every such config on 45 shapes (gemm_mmbo_amd/tune.py --dump);
// on those shapes the model's pick is within 2.5 % of the fastest config on average, 21 % at worst.
// split_lines: the rows of a packed operand (leading dimension = its stored row count) do not start on 128-byte lines,
// so every request of the direct loads touches one line more.  Measured on fp16: the 128 x 128 and smaller tiles, which
// are bound by that stream, lose 13-26 % of their in-loop rate (3000^3 against 3072^3, 4104^3 against 4096^3, 8200 against
// 8192), the 256 x 256 tile up to 15 % at 3000 and nothing at 4104 or 8200; fp32 tiles, MFMA-bound, lose nothing.
static double model_time_tile(int dtype, const RingRow &r, double e, int split, size_t m, size_t n, size_t k, int batch)
{
    const double launch = 5.9, fill = 0.65, c_us_per_kb = 0.0272, reduce_launch = 1.43, reduce_us_per_mb = 0.28;
    const double esz = dtype == MMBO_F32 ? 4.0 : 2.0;
    const double flop_per_us_cu = dtype == MMBO_F32 ? 0.614e6 : 9.83e6;             // matrix peak of one CU
    const int bk = ring_bk(dtype);
    const int lds = r.depth * (r.bm + r.bn) * 64;
    int per_cu = 160 * 1024 / lds;
    if (per_cu > 3) per_cu = 3;
    if (per_cu < 1) per_cu = 1;
    const double cus = 256.0;
    const double wgs = (double)ceil_div(m, (size_t)r.bm) * (double)ceil_div(n, (size_t)r.bn) * split * batch;
    const double slices = std::ceil(std::ceil((double)k / bk) / split);
    auto tile_time = [&](double resident) {
        return fill + slices * (2.0 * r.bm * r.bn * bk / flop_per_us_cu) * resident / e +
               c_us_per_kb * r.bm * r.bn * esz * resident / 1e3;
    };
    const double slots = cus * per_cu;
    const double full = std::floor(wgs / slots), last = wgs - full * slots;
    double t = launch + full * tile_time(per_cu);
    if (last > 0) {
        // A last round that leaves CUs idle runs faster per tile on fp16: the chip is power-limited on these MFMAs and the
        // clock rises when fewer CUs draw power (HGEMM 3072^3 on 144 tiles of 256 x 256: 54 us against 74 us for a full
        // round of the same tiles; 5120^3, 256 + 144 tiles: the second round takes 0.82 of the first).
        // (with several work-groups to a CU the round lasts as long as the fullest CU's; "busy" is the share of CU time in use)
        const double busy = last / (cus * std::ceil(last / cus));
        // (the tiles that run one to a CU are the power-limited ones; the smaller ones, bound by the L2 -> LDS stream, gain
        // less: HGEMM 1280 x 1280 x 4096 on 100 tiles of 128 x 128 runs at 0.86 of a full round's time per tile)
        const bool one_per_cu = r.depth * (r.bm + r.bn) * 64 > 80 * 1024;
        const double boost = dtype != MMBO_F16 ? 1.0 : one_per_cu ? 0.45 + 0.55 * busy : 0.7 + 0.3 * busy;
        t += tile_time(std::ceil(last / cus)) * boost;
    }
    if (split > 1) t += reduce_launch + reduce_us_per_mb * (double)m * n * batch * (split * 4.0 + esz) / 1e6;
    return t;
}
static double model_time_ring(int dtype, bool x16, int rt, int split, size_t m, size_t n, size_t k, int batch,
                              bool split_lines = false)
{
    static const double eff[2][2][NUM_RING_TILES] = {
        // 256x256 128x128 128x64  64x64
        {{0.9451, 0.9134, 0.8667, 0.9015}, {0.9387, 0.9039, 0.8402, 0.8561}},       // fp32: ring, x16
        {{0.5607, 0.3426, 0.2795, 0.2658}, {0.5879, 0.4873, 0.3151, 0.2560}},       // fp16: ring, x16
    };
    double e = eff[dtype == MMBO_F32 ? 0 : 1][x16 ? 1 : 0][rt];
    if (split_lines && dtype == MMBO_F16) e *= rt == 0 ? 0.95 : 0.78;
    return model_time_tile(dtype, kRingTiles[rt], e, split, m, n, k, batch);      // the x16 tiles of the same macro tile have the same depth
}
// The x16 kernel's tiles without a ring-kernel twin: 192 x 192, 256 x 192, 192 x 256 (kX16Tiles[5..7]).  In-loop
// efficiency: 192 x 192 from HGEMM 6144^3 (four whole rounds, 381 us) and SGEMM 3072^3 (one round, 404 us); the two
// rectangular ones between that and the 256 x 256 tile's.
constexpr int kFirstX16OnlyTile = 5;
static double model_time_x16_only(int dtype, int tile, int split, size_t m, size_t n, size_t k, int batch, bool split_lines)
{
    static const double eff16[3] = {0.50, 0.55, 0.55}, eff32[3] = {0.93, 0.935, 0.935};
    double e = (dtype == MMBO_F32 ? eff32 : eff16)[tile - kFirstX16OnlyTile];
    if (split_lines && dtype == MMBO_F16) e *= 0.90;
    return model_time_tile(dtype, kX16Tiles[tile], e, split, m, n, k, batch);
}

// The cost model's pick among the staged configs (fp32/fp16), which take any shape and any alignment.
static int select_staged(int dtype, size_t m, size_t n, size_t k, int batch)
{
    int best = 0;
    double best_t = 0.0;
    for (int si = 0; si < NUM_SPLITS; ++si) {
        int split = kSplits[si];
        for (int tile = 0; tile < NUM_TILES; ++tile) {
            const TileRow &r = tile_row(dtype, tile);
            if (split > 1 && ceil_div(k, (size_t)split) < (size_t)2 * r.bk) continue;   // slices too thin
            double t = model_time(dtype, tile, split, m, n, k ? k : 1, batch);
            if (best_t == 0.0 || t < best_t) { best_t = t; best = tile + NUM_TILES * si; }
        }
    }
    return best;
}

int mmbo_select_config(int dtype, int transA, int transB, size_t m, size_t n, size_t k, int batch)
{
    if (!valid_dtype(dtype)) return -MMBO_ERR_INVALID_DTYPE;
    if ((transA | transB) & ~1) return -MMBO_ERR_INVALID_OP;
    if (batch < 0) return -MMBO_ERR_INVALID_SIZE;
    if (m == 0 || n == 0 || batch == 0) return 0;
    for (const TunedRow &t : kTuned)
        if (t.dtype == dtype && t.transA == transA && t.transB == transB && t.m == m && t.n == n && t.k == k &&
            t.batch == batch)
            return t.config_id;
    if (dtype == MMBO_F64) {
        int best = 0;
        double best_t = 0.0;
        for (int tile = 0; tile < NUM_F64_TILES; ++tile) {
            double t = model_time_f64(tile, m, n, k, batch);
            if (best_t == 0.0 || t < best_t) { best_t = t; best = tile; }
        }
        return best;
    }
    // Whole-tile kernels (deeper prefetch, no edge handling) measured faster than the staged kernel on every shape
    // they apply to: where one applies, the fastest of them by model_time_ring takes the call.  fp16: the x16 family
    // (16x16x32 MFMAs), except that the 64 x 64 tile is faster on 32x32x16; fp32: the ring family, except that the
    // x16 kernel's 256 x 256 tile (v_mfma_f32_16x16x4_f32, four wavefronts) measures 1.5-2 % faster than the ring
    // kernel's at 8192^3 in NN, TN and TT (0.8 % slower in NT).
    {
        static const int x16_of_ring[NUM_RING_TILES] = {0, 2, 3, 4};       // same macro tile in kX16Tiles (256 x 256: four wavefronts)
        int pick = -1;
        double pick_t = 0.0;
        const size_t esz = dtype == MMBO_F32 ? 4 : 2;
        const bool split_lines = ((transA ? k : m) * esz) % 128 != 0 || ((transB ? n : k) * esz) % 128 != 0;
        for (int rt = 0; rt < NUM_RING_TILES; ++rt)
            for (int si = 0; si < NUM_SPLITS; ++si) {
                const bool ring_ok = ring_shape_ok(dtype, rt, kSplits[si], transA, transB, m, n, k, false);
                const bool x16_ok = ring_shape_ok(dtype, x16_of_ring[rt], kSplits[si], transA, transB, m, n, k, true);
                if (!ring_ok && !x16_ok) continue;
                // A dimension smaller than the tile: only the 64 x 64 fp16 tile on a long k is worth it (measured against
                // the staged kernel's 32 x 32 tile: HGEMM 16 x 4096 x 4096 11.8 against 17.5 us, 48 x 48 x 8192 10.1
                // against 17.1, 32 x 8192 x 1024 9.1 against 8.5-9.4; SGEMM 4096 x 32 x 4096 27.4 against 22.9).
                if (!ring_ok && (m < (size_t)kRingTiles[rt].bm || n < (size_t)kRingTiles[rt].bn) &&
                    !(dtype == MMBO_F16 && rt == 3 && k >= 1024))
                    continue;
                if (kSplits[si] > 1 && (k / ring_bk(dtype)) / (size_t)kSplits[si] < 2) continue;      // slices too thin
                if ((size_t)batch * kSplits[si] > 65535) continue;
                bool x16 = dtype == MMBO_F16 ? rt != 3 : (rt == 0 && !(transA == 0 && transB == 1));
                if (!ring_ok) x16 = true;           // ragged M or N: only the x16 kernel has edge tiles
                if (!x16_ok) x16 = false;
                const double t = model_time_ring(dtype, x16, rt, kSplits[si], m, n, k, batch, split_lines);
                if (pick < 0 || t < pick_t) {
                    pick_t = t;
                    pick = x16 ? x16_config_id(x16_of_ring[rt], si) : ring_config_id(rt, si);
                }
            }
        // the 192-row and 192-column tiles: where they fill the rounds of 256 CUs better than the power-of-two tiles do
        static_assert(kX16Tiles[kFirstX16OnlyTile].bm == 192 && kX16Tiles[kFirstX16OnlyTile].bn == 192 && NUM_X16_TILES == 8,
                      "x16 tiles 5, 6, 7 are 192 x 192, 256 x 192, 192 x 256");
        for (int tile = kFirstX16OnlyTile; tile < NUM_X16_TILES; ++tile) {
            if (m < (size_t)kX16Tiles[tile].bm || n < (size_t)kX16Tiles[tile].bn) continue;
            for (int si = 0; si < NUM_SPLITS; ++si) {
                if (!ring_shape_ok(dtype, tile, kSplits[si], transA, transB, m, n, k, true)) continue;
                if (kSplits[si] > 1 && (k / ring_bk(dtype)) / (size_t)kSplits[si] < 2) continue;
                if ((size_t)batch * kSplits[si] > 65535) continue;
                const double t = model_time_x16_only(dtype, tile, kSplits[si], m, n, k, batch, split_lines);
                if (pick < 0 || t < pick_t) {
                    pick_t = t;
                    pick = x16_config_id(tile, si);
                }
            }
        }
        if (pick >= 0) return pick;
    }
    return select_staged(dtype, m, n, k, batch);
}

int mmbo_wg_remap(unsigned linear_id, unsigned nwg0, unsigned nwg1, unsigned wgm, unsigned num_xcd,
                  unsigned *wg0, unsigned *wg1)
{
    if (!wg0 || !wg1) return MMBO_ERR_NULL_POINTER;
    if (nwg0 == 0 || nwg1 == 0 || wgm == 0 || num_xcd == 0) return MMBO_ERR_INVALID_SIZE;
    if ((unsigned long long)nwg0 * nwg1 > 0xFFFFFFFFull || linear_id >= nwg0 * nwg1) return MMBO_ERR_INVALID_SIZE;
    uint32_t a, b;
    wg_remap(linear_id, nwg0, nwg1, wgm, num_xcd, a, b);
    *wg0 = a;
    *wg1 = b;
    return MMBO_OK;
}

int mmbo_chip_block_remap(unsigned linear_id, unsigned nwg0, unsigned nwg1, unsigned *wg0, unsigned *wg1)
{
    if (!wg0 || !wg1) return MMBO_ERR_NULL_POINTER;
    if (nwg0 < 16 || nwg1 < 16) return MMBO_ERR_INVALID_SIZE;
    if ((unsigned long long)nwg0 * nwg1 > 0xFFFFFFFFull || linear_id >= nwg0 * nwg1) return MMBO_ERR_INVALID_SIZE;
    uint32_t a, b;
    chip_block_remap(linear_id, nwg0, nwg1, a, b);
    *wg0 = a;
    *wg1 = b;
    return MMBO_OK;
}

int mmbo_batch_xcd_remap(unsigned linear_id, unsigned tiles, unsigned batch, unsigned *tile, unsigned *batch_index)
{
    if (!tile || !batch_index) return MMBO_ERR_NULL_POINTER;
    if (tiles == 0 || batch == 0 || batch % 8 != 0) return MMBO_ERR_INVALID_SIZE;
    if ((unsigned long long)tiles * batch > 0xFFFFFFFFull || linear_id >= tiles * batch) return MMBO_ERR_INVALID_SIZE;
    uint32_t t, z;
    batch_xcd_remap(linear_id, tiles, 8, t, z);
    *tile = t;
    *batch_index = z;
    return MMBO_OK;
}

int mmbo_release_workspace(void) { return release_slots(false, nullptr); }

int mmbo_release_stream_workspace(void *stream) { return release_slots(true, static_cast<hipStream_t>(stream)); }

int mmbo_workspace_info(size_t *slots, size_t *bytes)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e);
    if (dev < 0 || dev >= kMaxDevices) return MMBO_ERR_NO_DEVICE;
    WsTable &tab = g_ws[dev];
    std::lock_guard<std::mutex> tl(tab.lock);
    size_t total = 0;
    for (auto &sl : tab.slots) total += sl->bytes;          // (a size being changed right now may be read stale: a diagnostic)
    if (slots) *slots = tab.slots.size();
    if (bytes) *bytes = total;
    return MMBO_OK;
}

size_t mmbo_static_workspace_bytes(void) { return kScratchPartialBytes; }

}  // extern "C"

namespace {

// Where the partial sums of a split-K config go.
enum class WsSource { kLibrary, kStatic };

int gemm_impl(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
              const void *alpha, const void *A, size_t lda, long long strideA,
              const void *B, size_t ldb, long long strideB, const void *beta, void *C,
              size_t ldc, long long strideC, int batch, int config_id, void *stream, WsSource ws_source)
{
    if (!valid_dtype(dtype)) return MMBO_ERR_INVALID_DTYPE;
    if ((transA & ~1) || (transB & ~1)) return MMBO_ERR_INVALID_OP;
    if (!alpha || !beta) return MMBO_ERR_NULL_POINTER;
    const size_t kMaxDim = 0x7FFFFFFFull;
    if (m > kMaxDim || n > kMaxDim || k > kMaxDim || lda > kMaxDim || ldb > kMaxDim || ldc > kMaxDim)
        return MMBO_ERR_INVALID_SIZE;
    if (batch < 0 || batch > 65535) return MMBO_ERR_INVALID_SIZE;
    // BLAS rule: a leading dimension is at least 1 and at least the operand's stored row count
    {
        size_t need_a = transA ? k : m, need_b = transB ? n : k;
        if (lda < (need_a ? need_a : 1) || ldb < (need_b ? need_b : 1) || ldc < (m ? m : 1))
            return MMBO_ERR_INVALID_SIZE;
    }
    if (strideA < 0 || strideB < 0 || strideC < 0) return MMBO_ERR_INVALID_SIZE;
    if (config_id != MMBO_CONFIG_AUTO && (config_id < 0 || config_id >= mmbo_num_configs(dtype)))
        return MMBO_ERR_INVALID_CONFIG;
    if (m == 0 || n == 0 || batch == 0) return MMBO_OK;          // nothing to write
    if (!C) return MMBO_ERR_NULL_POINTER;
    if (k != 0 && (!A || !B)) return MMBO_ERR_NULL_POINTER;

    const bool f64 = dtype == MMBO_F64;
    const double alpha_d = f64 ? *static_cast<const double *>(alpha) : (double)*static_cast<const float *>(alpha);
    const double beta_d = f64 ? *static_cast<const double *>(beta) : (double)*static_cast<const float *>(beta);
    const float alpha_f = (float)alpha_d, beta_f = (float)beta_d;

    const size_t esz_in = f64 ? 8 : dtype == MMBO_F32 ? 4 : 2;
    if (config_id == MMBO_CONFIG_AUTO) {
        config_id = mmbo_select_config(dtype, transA, transB, m, n, k, batch);
        if (config_id < 0) return -config_id;
        // The pick is made from the shape alone.  The ring kernels also need 16-byte aligned A and B, every
        // direct-to-LDS kernel a tile's span of an operand below 2 GiB: where the operands at hand do not qualify, the
        // x16 config of the same tile and split (any alignment), or the staged kernel, takes the call.
        if (!f64) {
            const ConfigRef c = config_ref(config_id);
            if (c.ring && !c.x16) {
                auto al16 = [&](const void *p, size_t ld, long long stride) {
                    return ((uintptr_t)p % 16 == 0) && ((ld * esz_in) % 16 == 0) && (((size_t)stride * esz_in) % 16 == 0);
                };
                if (!al16(A, lda, strideA) || !al16(B, ldb, strideB)) {
                    static const int x16_of_ring[NUM_RING_TILES] = {0, 2, 3, 4};
                    int si = 0;
                    while (si + 1 < NUM_SPLITS && kSplits[si] != c.split) ++si;
                    const int tile = x16_of_ring[c.tile];
                    config_id = ring_shape_ok(dtype, tile, c.split, transA, transB, m, n, k, true)
                                    ? x16_config_id(tile, si) : select_staged(dtype, m, n, k, batch);
                }
            }
        }
        // The entry point that allocates nothing holds kScratchPartialBytes of partial sums: where the pick's GlobalSplitU
        // needs more, the same tile runs with the largest split that fits (down to none), so that every shape still
        // runs under MMBO_CONFIG_AUTO.  (A config the caller names is taken as named, or refused.)
        if (!f64 && ws_source == WsSource::kStatic) {
            const ConfigRef c = config_ref(config_id);
            int si = split_index(c.split);
            auto fits = [&](int sidx) {
                if (kSplits[sidx] == 1) return true;
                if ((double)kSplits[sidx] * batch * (double)m * (double)n * sizeof(float) > (double)kScratchPartialBytes) return false;
                return !c.ring || ring_shape_ok(dtype, c.tile, kSplits[sidx], transA, transB, m, n, k, c.x16);
            };
            while (si > 0 && !fits(si)) --si;
            config_id = c.x16 ? x16_config_id(c.tile, si) : c.ring ? ring_config_id(c.tile, si) : staged_config_id(c.tile, si);
        }
        if (!tile_span_ok(config_tile(dtype, config_id), transA, transB, lda, ldb, esz_in)) {
            // enormous leading dimensions: the first staged tile (no split-K) whose span fits, large tiles first
            const int ntiles = f64 ? NUM_F64_TILES : NUM_TILES;
            config_id = -1;
            for (int tile = 0; tile < ntiles && config_id < 0; ++tile)
                if (tile_span_ok(config_tile(dtype, tile), transA, transB, lda, ldb, esz_in)) config_id = tile;
            if (config_id < 0) return MMBO_ERR_INVALID_SIZE;
        }
    }
    const ConfigRef cref = f64 ? ConfigRef{false, config_id, 1, false} : config_ref(config_id);
    const size_t esz = f64 ? 8 : dtype == MMBO_F32 ? 4 : 2;
    int split = cref.split;
    const RingRow &rr = cref.x16 ? kX16Tiles[cref.tile] : kRingTiles[cref.ring ? cref.tile : 0];
    TileRow r = f64 ? kTilesF64[config_id] : cref.ring ? TileRow{rr.bm, rr.bn, ring_bk(dtype), 0, 0} : tile_row(dtype, cref.tile);
    if (cref.ring && !ring_shape_ok(dtype, cref.tile, split, transA, transB, m, n, k, cref.x16)) return MMBO_ERR_INVALID_CONFIG;

    if (!tile_span_ok(r, transA, transB, lda, ldb, esz)) return MMBO_ERR_INVALID_CONFIG;

    size_t nwg0 = ceil_div(m, r.bm), nwg1 = ceil_div(n, r.bn);
    if (nwg0 * nwg1 > 0x7FFFFFFFull) return MMBO_ERR_INVALID_SIZE;
    // split-K: slices are whole stages; never more slices than stages
    size_t stages = ceil_div(k, r.bk);
    if (stages < 1) stages = 1;
    if ((size_t)split > stages) split = (int)stages;
    size_t k_per_split = ceil_div(stages, (size_t)split) * r.bk;
    split = (int)ceil_div(k ? k : 1, k_per_split);        // the last split takes what is left, a partial slice included
    if ((size_t)batch * split > 65535) return MMBO_ERR_INVALID_SIZE;

    GemmArgs a;
    std::memset(&a, 0, sizeof(a));
    a.A = A; a.B = B; a.C = C; a.ws = nullptr;
    a.alpha = alpha_f; a.beta = beta_f;
    a.alpha_d = alpha_d; a.beta_d = beta_d;
    a.m = (uint32_t)m; a.n = (uint32_t)n; a.k = (uint32_t)k;
    a.lda = (uint32_t)lda; a.ldb = (uint32_t)ldb; a.ldc = (uint32_t)ldc;
    a.strideA = strideA; a.strideB = strideB; a.strideC = strideC;
    a.nwg0 = (uint32_t)nwg0; a.nwg1 = (uint32_t)nwg1;
    a.wgm = 8;
    a.nxcd = 8;
    a.splits = (uint32_t)split;
    a.k_per_split = (uint32_t)(split > 1 ? k_per_split : (k ? k : 1));
    a.batch = (uint32_t)batch;
    // (tiles that run one work-group per CU: 256 x 256 and 192 x 192)
    a.chip_block = cref.x16 && rr.depth * (rr.bm + rr.bn) * 64 > 80 * 1024 && nwg0 >= 16 && nwg1 >= 16;
    // batches of problems of at most 32 tiles (an XCD's CUs hold them at one time): each problem on one XCD
    a.batch_xcd = split == 1 && batch >= a.nxcd && batch % a.nxcd == 0 && nwg0 * nwg1 <= 32;
    auto aligned16 = [&](const void *p, size_t ld, long long stride) {
        return ((uintptr_t)p % 16 == 0) && ((ld * esz) % 16 == 0) && (((size_t)stride * esz) % 16 == 0);
    };
    a.vec_a = aligned16(A, lda, strideA);
    a.vec_b = aligned16(B, ldb, strideB);
    // (the x16 kernel's whole-tile epilogue addresses C as a buffer with 32-bit offsets: where a tile's span of C, its columns x
    // ldc, does not fit them, C goes out element by element instead)
    auto on_lines = [&](const void *p, size_t ld, long long stride) {
        return ((uintptr_t)p % 128 == 0) && ((ld * esz) % 128 == 0) && (batch == 1 || ((size_t)stride * esz) % 128 == 0);
    };
    a.line_rows = on_lines(A, lda, strideA) && on_lines(B, ldb, strideB);
    a.ws_narrow = (size_t)r.bn * m * 4 < 0x7FFFFF00ull;
    a.vec_c = aligned16(C, ldc, strideC) && (!cref.x16 || (size_t)r.bn * ldc * esz < 0x7FFFFF00ull);
    // beta != 0 on the x16 kernel's fp16 path: the old C of a tile is fetched into LDS under the tile's last slices (one
    // tile's span of C, tile columns x ldc, must then fit the 32-bit offsets of a buffer load)
    a.c_prefetch = cref.x16 && dtype == MMBO_F16 && beta_f != 0.0f && split == 1 && a.vec_c &&
                   (size_t)r.bn * ldc * esz < 0x7FFFFF00ull;
    // C with the non-temporal hint: only where resident work-groups walk at least four rounds of tiles (256 CUs) with a long
    // slice loop -- there the operand panels the next tiles share are worth more in the L2 than a fast epilogue (8192^3:
    // +0.3 %); with fewer rounds or a short k plain stores win (fp16 6144^3 +1.6 %, 44160 x 2048 x 384 +2.7 %, 64 x 512^3 +14 %)
    a.c_stream = cref.x16 && rr.depth * (rr.bm + rr.bn) * 64 > 80 * 1024 && (size_t)nwg0 * nwg1 >= 4 * 256 && k >= 4096;

    hipStream_t s = static_cast<hipStream_t>(stream);
    if (cref.ring && !cref.x16 && (!a.vec_a || !a.vec_b)) return MMBO_ERR_INVALID_CONFIG;
    // Split-K: the partial sums go to the stream's own workspace (or the static one), and both launches that use it (the
    // GEMM and the reduction, which adds the splits in ascending order) are queued before the hold on that workspace
    // is given up.
    WsHold ws_hold;
    if (split > 1) {
        const size_t bytes = (size_t)split * batch * m * n * sizeof(float);
        char *base = nullptr;
        if (ws_source == WsSource::kStatic) {
            if (bytes > kScratchPartialBytes) return MMBO_ERR_WORKSPACE;
            int rc = static_scratch(&base);
            if (rc != MMBO_OK) return rc;
        } else {
            int rc = workspace(s, bytes, ws_hold, &base);
            if (rc != MMBO_OK) return rc;
        }
        a.ws = reinterpret_cast<float *>(base);
    }
    hipError_t e;
    if (f64) e = dispatch_dgemm<0>(cref.tile, transA, transB, a, s);
    else if (cref.x16) e = dtype == MMBO_F32 ? dispatch_x16<0, 0>(cref.tile, transA, transB, a, s)
                                        : dispatch_x16<1, 0>(cref.tile, transA, transB, a, s);
    else if (cref.ring) e = dtype == MMBO_F32 ? dispatch_ring<0, 0>(cref.tile, transA, transB, a, s)
                                         : dispatch_ring<1, 0>(cref.tile, transA, transB, a, s);
    else e = dtype == MMBO_F32 ? dispatch_tile<0, 0>(cref.tile, transA, transB, a, s)
                               : dispatch_tile<1, 0>(cref.tile, transA, transB, a, s);
    if (e != hipSuccess) return hip_fail(e);
    if (split > 1) {
        e = launch_splitk_reduce(dtype, a, s);
        if (e != hipSuccess) return hip_fail(e);
    }
    return MMBO_OK;
}

}  // namespace

extern "C" {

int mmbo_gemm_strided_batched(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
                              const void *alpha, const void *A, size_t lda, long long strideA,
                              const void *B, size_t ldb, long long strideB, const void *beta, void *C,
                              size_t ldc, long long strideC, int batch, int config_id, void *stream)
{
    return gemm_impl(dtype, transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch,
                     config_id, stream, WsSource::kLibrary);
}

int mmbo_gemm_strided_batched_static_workspace(int dtype, int transA, int transB, size_t m, size_t n, size_t k,
                                               const void *alpha, const void *A, size_t lda, long long strideA,
                                               const void *B, size_t ldb, long long strideB, const void *beta, void *C,
                                               size_t ldc, long long strideC, int batch, int config_id, void *stream)
{
    return gemm_impl(dtype, transA, transB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC, batch,
                     config_id, stream, WsSource::kStatic);
}

int mmbo_gemm(int dtype, int transA, int transB, size_t m, size_t n, size_t k, const void *alpha,
              const void *A, size_t lda, const void *B, size_t ldb, const void *beta, void *C, size_t ldc,
              int config_id, void *stream)
{
    return mmbo_gemm_strided_batched(dtype, transA, transB, m, n, k, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc,
                                     0, 1, config_id, stream);
}

}  // extern "C"
