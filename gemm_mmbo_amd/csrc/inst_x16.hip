// Instantiates the 16x16-block ring kernel for one (element type, tile row): compile with
//   -DMMBO_DTYPE=<0|1> -DMMBO_TILE=<row>
#include <atomic>

#include "configs.hpp"
#include "gemm_x16.hpp"
#include "launch.hpp"

#ifndef MMBO_DTYPE
#error "MMBO_DTYPE and MMBO_TILE select what this translation unit instantiates"
#endif

namespace mmbo {

namespace {
using ElemT = typename std::conditional<MMBO_DTYPE == 0, float, half_t>::type;
constexpr RingRow R = kX16Tiles[MMBO_TILE];

template <bool TA, bool TB, int WM, int WN, bool OLD_C = false, bool BOTH_EVEN = false>
hipError_t launch_one(const GemmArgs &args, hipStream_t stream)
{
    using Cfg = X16Cfg<ElemT, TA, TB, R.bm, R.bn, WM, WN, R.depth>;
    // beta != 0 on fp16 (args.c_prefetch): the variant that fetches the old C ahead of the epilogue, where the tile has one
    if constexpr (!OLD_C && Cfg::C_PREFETCH) {
        if (args.c_prefetch) return launch_one<TA, TB, WM, WN, true, BOTH_EVEN>(args, stream);
    }
    // TN on a ring of five buffers with every row of A and B on a memory line (args.line_rows): both operands' pairs of
    // slices on the even iterations
    if constexpr (!BOTH_EVEN && TA && !TB && R.depth == 5) {
        if (args.line_rows) return launch_one<TA, TB, WM, WN, OLD_C, true>(args, stream);
    }
    // the k-contiguous operand goes to the iterations whose pair of slices starts on an even slice (whole memory lines): the
    // even ones on a ring of five buffers, the odd ones on a ring of six
    constexpr int EVEN_OP = R.depth == 6 ? (TA ? 1 : 0) : (TA ? 0 : 1);
    auto kernel = gemm_x16_kernel<ElemT, TA, TB, R.bm, R.bn, WM, WN, R.depth, (TA || !TB), EVEN_OP, OLD_C, BOTH_EVEN>;
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
    // Tiles of which one work-group per CU fits (256 x 256, 192 x 192): on grids with more tiles than CUs the work-groups
    // stay resident and walk the tiles themselves
    unsigned gx = args.nwg0 * args.nwg1;
    if (Cfg::LDS_BYTES > 80 * 1024) {
        static std::atomic<int> cus[64];
        int n = dev >= 0 && dev < 64 ? cus[dev].load(std::memory_order_acquire) : 0;
        if (n == 0) {
            hipDeviceProp_t prop;
            e = hipGetDeviceProperties(&prop, dev);
            if (e != hipSuccess) return e;
            n = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 1;
            if (dev >= 0 && dev < 64) cus[dev].store(n, std::memory_order_release);
        }
        if (gx > (unsigned)n) gx = (unsigned)n;
    }
    dim3 grid(gx, 1, args.batch * args.splits);
    return launch_kernel(kernel, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, args);
}
}  // namespace

// The operand that needs transposing LDS reads (two or four per fragment instead of one) gets the fewer fragments:
// A needs them under transA = N, B under transB = T, so TT swaps the wave layout.
template <>
hipError_t launch_x16<MMBO_DTYPE, MMBO_TILE>(int transA, int transB, const GemmArgs &args, hipStream_t stream)
{
    if (!transA && !transB) return launch_one<false, false, R.wm, R.wn>(args, stream);
    if (!transA && transB) return launch_one<false, true, R.wm, R.wn>(args, stream);
    if (transA && !transB) return launch_one<true, false, R.wm, R.wn>(args, stream);
    return launch_one<true, true, R.wn, R.wm>(args, stream);
}

}  // namespace mmbo
