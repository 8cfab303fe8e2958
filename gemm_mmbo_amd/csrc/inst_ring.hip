// Instantiates the ring kernel for one (element type, ring tile row): compile with
//   -DMMBO_DTYPE=<0|1> -DMMBO_TILE=<row>
#include <atomic>

#include "configs.hpp"
#include "gemm_ring.hpp"
#include "launch.hpp"

#ifndef MMBO_DTYPE
#error "MMBO_DTYPE and MMBO_TILE select what this translation unit instantiates"
#endif

namespace mmbo {

namespace {
using ElemT = typename std::conditional<MMBO_DTYPE == 0, float, half_t>::type;
constexpr RingRow R = kRingTiles[MMBO_TILE];

template <bool TA, bool TB, int WM, int WN>
hipError_t launch_one(const GemmArgs &args, hipStream_t stream)
{
    using Cfg = RingCfg<ElemT, TA, TB, R.bm, R.bn, WM, WN, R.depth>;
    auto kernel = gemm_ring_kernel<ElemT, TA, TB, R.bm, R.bn, WM, WN, R.depth>;
    static std::atomic<bool> attr_set[64];           // zero-initialised; several host threads may race to set it: harmless
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64 && !attr_set[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                Cfg::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set[dev].store(true, std::memory_order_release);
    }
    dim3 grid(args.nwg0 * args.nwg1, 1, args.batch * args.splits);
    return launch_kernel(kernel, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
}
}  // namespace

// Wave layout per transpose pair: the operand that needs transposing LDS reads (two or four reads per fragment
// instead of one) gets the fewer fragments.  A needs them under transA = N, B under transB = T.
template <>
hipError_t launch_ring<MMBO_DTYPE, MMBO_TILE>(int transA, int transB, const GemmArgs &args, hipStream_t stream)
{
    if (!transA && !transB) return launch_one<false, false, R.wm, R.wn>(args, stream);
    if (!transA && transB) return launch_one<false, true, R.wm, R.wn>(args, stream);
    if (transA && !transB) return launch_one<true, false, R.wm, R.wn>(args, stream);
    return launch_one<true, true, R.wn, R.wm>(args, stream);
}

}  // namespace mmbo
