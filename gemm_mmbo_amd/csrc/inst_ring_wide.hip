// Instantiates the wide-unit HGEMM ring kernel (NN and TT).
#include <atomic>

#include "gemm_ring_wide.hpp"
#include "launch.hpp"

namespace mmbo {

namespace {
template <bool TRANS>
hipError_t launch_one(const GemmArgs &args, hipStream_t stream)
{
    constexpr int LDS = 160 * 1024;
    auto kernel = hgemm_ring_wide_kernel<TRANS>;
    static std::atomic<bool> attr_set[64];           // zero-initialised; several host threads may race to set it: harmless
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64 && !attr_set[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if (e != hipSuccess) return e;
        attr_set[dev].store(true, std::memory_order_release);
    }
    dim3 grid(args.nwg0 * args.nwg1, 1, args.batch);
    return launch_kernel(kernel, grid, dim3(512), LDS, stream, args);
}
}  // namespace

hipError_t launch_hgemm_ring_wide(int transA, int transB, const GemmArgs &args, hipStream_t stream)
{
    if (transA != transB) return hipErrorInvalidValue;
    return transA ? launch_one<true>(args, stream) : launch_one<false>(args, stream);
}

}  // namespace mmbo
