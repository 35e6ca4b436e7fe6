// Instantiates the 256 x 256 pipelined kernel for one (16-bit element type, algorithm) pair:
// -DSTHIP_INST_TYPE={1:f16,2:bf16} -DSTHIP_INST_ALGO={0,1,2}.
#include "sthip_launch.hpp"

namespace sthip {

#if STHIP_INST_TYPE == 1
typedef f16_t InstT;
#else
typedef bf16_t InstT;
#endif

template __global__ void gemm4_kernel<InstT, STHIP_INST_ALGO, false>(const Gemm2Params);
template __global__ void gemm4_kernel<InstT, STHIP_INST_ALGO, true>(const Gemm2Params);

#ifndef __HIP_DEVICE_COMPILE__
#define STHIP_CAT2(a, b, c) kLaunch4_##a##_##b
#define STHIP_CAT(a, b) STHIP_CAT2(a, b, )
extern const LaunchTable3 STHIP_CAT(STHIP_INST_TYPE, STHIP_INST_ALGO) = {
    {&launch_gemm4<InstT, STHIP_INST_ALGO, false>, &launch_gemm4<InstT, STHIP_INST_ALGO, true>}};
#endif

}  // namespace sthip
