// Instantiates the staged kernel for one (element type, tile row): compile with
//   -DMMBO_DTYPE=<0|1> -DMMBO_TILE=<row>
#include <atomic>

#include "configs.hpp"
#include "gemm_staged.hpp"
#include "launch.hpp"

#ifndef MMBO_DTYPE
#error "MMBO_DTYPE and MMBO_TILE select what this translation unit instantiates"
#endif

namespace mmbo {

namespace {
using ElemT = typename std::conditional<MMBO_DTYPE == 0, float, half_t>::type;
constexpr TileRow R = tile_row(MMBO_DTYPE, MMBO_TILE);

template <bool TA, bool TB>
hipError_t launch_one(const GemmArgs &args, hipStream_t stream)
{
    using Cfg = StagedCfg<ElemT, TA, TB, R.bm, R.bn, R.bk, R.wm, R.wn>;
    auto kernel = gemm_staged_kernel<ElemT, TA, TB, R.bm, R.bn, R.bk, R.wm, R.wn>;
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
    dim3 grid(args.nwg0 * args.nwg1, 1, args.batch * args.splits);
    return launch_kernel(kernel, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
}

template <bool TA, bool TB>
constexpr int lds_of() { return StagedCfg<ElemT, TA, TB, R.bm, R.bn, R.bk, R.wm, R.wn>::LDS_BYTES; }
}  // namespace

template <>
hipError_t launch_staged<MMBO_DTYPE, MMBO_TILE>(int transA, int transB, const GemmArgs &args, hipStream_t stream)
{
    if (!transA && !transB) return launch_one<false, false>(args, stream);
    if (!transA && transB) return launch_one<false, true>(args, stream);
    if (transA && !transB) return launch_one<true, false>(args, stream);
    return launch_one<true, true>(args, stream);
}

template <>
int staged_lds_bytes<MMBO_DTYPE, MMBO_TILE>()
{
    int a = lds_of<false, false>(), b = lds_of<false, true>(), c = lds_of<true, false>(), d = lds_of<true, true>();
    int m1 = a > b ? a : b, m2 = c > d ? c : d;
    return m1 > m2 ? m1 : m2;
}

}  // namespace mmbo
