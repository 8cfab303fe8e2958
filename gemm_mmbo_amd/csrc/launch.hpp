// Launchers: one explicit specialisation per (element type, tile row), each defined in its own
// translation unit (inst_staged.hip compiled once per pair) so the kernels build in parallel.
#pragma once

#include "gemm_common.hpp"

namespace mmbo {

// Launches kernel(args) and returns the status of that launch alone (hipGetLastError would also hand back an error
// that an earlier, unrelated HIP call of this thread -- the caller's own, another library's -- left behind).
template <typename Kernel>
inline hipError_t launch_kernel(Kernel kernel, dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream, const GemmArgs &args)
{
    void *kargs[] = {const_cast<GemmArgs *>(&args)};
    return hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, kargs, lds_bytes, stream);
}

// dtype: 0 = fp32, 1 = fp16.  Launches the staged kernel for tile row TILE with the given
// transposes; grid = (nwg0*nwg1, 1, batch*splits).  Returns the launch's hipError_t.
template <int DTYPE, int TILE>
hipError_t launch_staged(int transA, int transB, const GemmArgs &args, hipStream_t stream);

// LDS bytes the staged kernel of that tile needs, worst case over the four transposes.
template <int DTYPE, int TILE>
int staged_lds_bytes();

// Ring kernel of ring tile row TILE; grid = (nwg0*nwg1, 1, batch*splits).
template <int DTYPE, int TILE>
hipError_t launch_ring(int transA, int transB, const GemmArgs &args, hipStream_t stream);

// 16x16-block ring kernel (gemm_x16.hpp) of x16 tile row TILE; grid = (nwg0*nwg1, 1, batch*splits).
template <int DTYPE, int TILE>
hipError_t launch_x16(int transA, int transB, const GemmArgs &args, hipStream_t stream);

// DGEMM kernel of fp64 tile row TILE; grid = (nwg0*nwg1, 1, batch).
template <int TILE>
hipError_t launch_dgemm(int transA, int transB, const GemmArgs &args, hipStream_t stream);
template <int TILE>
int dgemm_lds_bytes();

hipError_t launch_splitk_reduce(int dtype, const GemmArgs &args, hipStream_t stream);

}  // namespace mmbo
