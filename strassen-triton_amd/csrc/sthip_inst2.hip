// Instantiates the pipelined grouped-GEMM kernel for one (16-bit element type, algorithm)
// pair: -DSTHIP_INST_TYPE={1:f16,2:bf16} -DSTHIP_INST_ALGO={0,1,2}.
#include "sthip_launch.hpp"

namespace sthip {

#if STHIP_INST_TYPE == 1
typedef f16_t InstT;
#else
typedef bf16_t InstT;
#endif

#define K(akc, bkc) template __global__ void gemm2_kernel<InstT, STHIP_INST_ALGO, akc, bkc>(const Gemm2Params);
K(false, false) K(false, true) K(true, false) K(true, true)
#undef K

#ifndef __HIP_DEVICE_COMPILE__
#define STHIP_CAT2(a, b, c) kLaunch2_##a##_##b
#define STHIP_CAT(a, b) STHIP_CAT2(a, b, )
#define L(akc, bkc) &launch_gemm2<InstT, STHIP_INST_ALGO, akc, bkc>
extern const LaunchTable2 STHIP_CAT(STHIP_INST_TYPE, STHIP_INST_ALGO) = {{{L(false, false), L(false, true)}, {L(true, false), L(true, true)}}};
#endif

}  // namespace sthip
