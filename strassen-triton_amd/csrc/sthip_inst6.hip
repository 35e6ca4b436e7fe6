// Instantiates the 64 x 64 fp32 kernel with fused pre-additions (both layouts of B).
#include "sthip_launch.hpp"

namespace sthip {

template __global__ void gemm6_kernel<false>(const Gemm6Params);
template __global__ void gemm6_kernel<true>(const Gemm6Params);

#ifndef __HIP_DEVICE_COMPILE__
hipError_t launch_gemm6(const Gemm6Params& p, bool b_kc, hipStream_t stream) {
    const int nprod = p.nprod > 0 ? p.nprod : 1;
    const dim3 grid((unsigned)(p.tiles_m * p.tiles_n * nprod));
    if (b_kc) hipLaunchKernelGGL(gemm6_kernel<true>, grid, dim3(kThreads6), 0, stream, p);
    else hipLaunchKernelGGL(gemm6_kernel<false>, grid, dim3(kThreads6), 0, stream, p);
    return hipGetLastError();
}
#endif

}  // namespace sthip
