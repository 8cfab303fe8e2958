// Instantiates the fp64 kernel for one tile row: compile with -DMMBO_TILE=<row>
#include <atomic>

#include "configs.hpp"
#include "dgemm.hpp"
#include "launch.hpp"

#ifndef MMBO_TILE
#error "MMBO_TILE selects what this translation unit instantiates"
#endif

namespace mmbo {

namespace {
constexpr TileRow R = kTilesF64[MMBO_TILE];

template <bool TA, bool TB, bool OLD_C_EARLY = false>
hipError_t launch_one(const GemmArgs &args, hipStream_t stream)
{
    using Cfg = DgemmCfg<TA, TB, R.bm, R.bn, R.bk, R.wm, R.wn>;
    // beta != 0 on a tile whose wave tiles have at most four blocks: the variant that requests the old C under the last stage
    if constexpr (!OLD_C_EARLY && Cfg::FM * Cfg::FN <= 4) {
        if (args.beta_d != 0.0 && args.vec_c) return launch_one<TA, TB, true>(args, stream);
    }
    auto kernel = dgemm_kernel<TA, TB, R.bm, R.bn, R.bk, R.wm, R.wn, OLD_C_EARLY>;
    static std::atomic<bool> attr_set[64];           // zero-initialised; several host threads may race to set it: harmless
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64 && !attr_set[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set[dev].store(true, std::memory_order_release);
    }
    dim3 grid(args.nwg0 * args.nwg1, 1, args.batch);
    return launch_kernel(kernel, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
}

template <bool TA, bool TB>
constexpr int lds_of() { return DgemmCfg<TA, TB, R.bm, R.bn, R.bk, R.wm, R.wn>::LDS_BYTES; }
}  // namespace

template <>
hipError_t launch_dgemm<MMBO_TILE>(int transA, int transB, const GemmArgs &args, hipStream_t stream)
{
    if (!transA && !transB) return launch_one<false, false>(args, stream);
    if (!transA && transB) return launch_one<false, true>(args, stream);
    if (transA && !transB) return launch_one<true, false>(args, stream);
    return launch_one<true, true>(args, stream);
}

template <>
int dgemm_lds_bytes<MMBO_TILE>()
{
    int a = lds_of<false, false>(), b = lds_of<false, true>(), c = lds_of<true, false>(), d = lds_of<true, true>();
    int m1 = a > b ? a : b, m2 = c > d ? c : d;
    return m1 > m2 ? m1 : m2;
}

}  // namespace mmbo
