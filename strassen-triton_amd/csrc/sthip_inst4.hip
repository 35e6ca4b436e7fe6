// Instantiates the 256 x 256 pipelined grouped-GEMM kernel for one element type:
// -DSTHIP_INST_TYPE={0:f32,1:f16,2:bf16}.
#include "sthip_launch.hpp"

namespace sthip {

#if STHIP_INST_TYPE == 0
typedef float InstT;
#elif STHIP_INST_TYPE == 1
typedef f16_t InstT;
#else
typedef bf16_t InstT;
#endif

template __global__ void gemm4_kernel<InstT, false>(const Gemm2Params);
template __global__ void gemm4_kernel<InstT, true>(const Gemm2Params);
template __global__ void gemm4p_kernel<InstT, false>(const Gemm2Params);
template __global__ void gemm4p_kernel<InstT, true>(const Gemm2Params);

#ifndef __HIP_DEVICE_COMPILE__
#define STHIP_CAT2(a, b) kLaunch4_##a
#define STHIP_CAT(a) STHIP_CAT2(a, )
extern const LaunchTable3 STHIP_CAT(STHIP_INST_TYPE) = {{&launch_gemm4<InstT, false>, &launch_gemm4<InstT, true>}};
#endif

}  // namespace sthip
