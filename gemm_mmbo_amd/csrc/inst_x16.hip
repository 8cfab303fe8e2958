// Instantiates the 16x16x32-MFMA HGEMM ring kernel for one tile row: compile with -DMMBO_TILE=<row>
#include "configs.hpp"
#include "hgemm_x16.hpp"
#include "launch.hpp"

#ifndef MMBO_TILE
#error "MMBO_TILE selects what this translation unit instantiates"
#endif

namespace mmbo {

namespace {
constexpr RingRow R = kX16Tiles[MMBO_TILE];

template <bool TA, bool TB, int WM, int WN>
hipError_t launch_one(const GemmArgs &args, hipStream_t stream)
{
    using Cfg = X16Cfg<TA, TB, R.bm, R.bn, WM, WN, R.depth>;
    auto kernel = hgemm_x16_kernel<TA, TB, R.bm, R.bn, WM, WN, R.depth>;
    static bool attr_set[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64 && !attr_set[dev]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                Cfg::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set[dev] = true;
    }
    dim3 grid(args.nwg0 * args.nwg1, 1, args.batch * args.splits);
    hipLaunchKernelGGL(kernel, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
    return hipGetLastError();
}
}  // namespace

// The operand that needs transposing LDS reads (two per fragment instead of one) gets the fewer fragments:
// A needs them under transA = N, B under transB = T, so TT swaps the wave layout.
template <>
hipError_t launch_x16<MMBO_TILE>(int transA, int transB, const GemmArgs &args, hipStream_t stream)
{
    if (!transA && !transB) return launch_one<false, false, R.wm, R.wn>(args, stream);
    if (!transA && transB) return launch_one<false, true, R.wm, R.wn>(args, stream);
    if (transA && !transB) return launch_one<true, false, R.wm, R.wn>(args, stream);
    return launch_one<true, true, R.wn, R.wm>(args, stream);
}

}  // namespace mmbo
