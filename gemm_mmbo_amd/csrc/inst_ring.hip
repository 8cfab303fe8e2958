// Instantiates the HGEMM ring kernel for the four transpose pairs.
#include "gemm_ring.hpp"
#include "launch.hpp"

namespace mmbo {

namespace {
template <bool TA, bool TB, int WM, int WN>
hipError_t launch_one(const GemmArgs &args, hipStream_t stream)
{
    auto kernel = hgemm_ring_kernel<TA, TB, WM, WN>;
    static bool attr_set[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64 && !attr_set[dev]) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                ring::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set[dev] = true;
    }
    dim3 grid(args.nwg0 * args.nwg1, 1, args.batch);
    hipLaunchKernelGGL(kernel, grid, dim3(ring::NT), ring::LDS_BYTES, stream, args);
    return hipGetLastError();
}
}  // namespace

// Wave layout per transpose pair: the operand that needs transposing LDS reads (two reads per fragment)
// gets the fewer fragments.
hipError_t launch_hgemm_ring(int transA, int transB, const GemmArgs &args, hipStream_t stream)
{
    if (!transA && !transB) return launch_one<false, false, 4, 2>(args, stream);
    if (!transA && transB) return launch_one<false, true, 4, 2>(args, stream);
    if (transA && !transB) return launch_one<true, false, 4, 2>(args, stream);
    return launch_one<true, true, 2, 4>(args, stream);
}

}  // namespace mmbo
