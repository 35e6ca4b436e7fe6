// Instantiates the fused kernel for one (element type, algorithm) pair, selected with
// -DSTHIP_INST_TYPE={0:f32,1:f16,2:bf16} -DSTHIP_INST_ALGO={0:classic,1:strassen,2:winograd}.
// Split this way so the nine units compile in parallel.
#include "sthip_launch.hpp"

namespace sthip {

#if STHIP_INST_TYPE == 0
typedef float InstT;
#elif STHIP_INST_TYPE == 1
typedef f16_t InstT;
#else
typedef bf16_t InstT;
#endif

// Device pass: emit the eight kernels.  Host pass: emit their launchers and the table.
#define K(akc, bkc, edge) template __global__ void gemm_kernel<InstT, STHIP_INST_ALGO, akc, bkc, edge>(const GemmParams);
K(false, false, false) K(false, false, true) K(false, true, false) K(false, true, true)
K(true, false, false) K(true, false, true) K(true, true, false) K(true, true, true)
#undef K

#ifndef __HIP_DEVICE_COMPILE__
#define STHIP_CAT2(a, b, c) kLaunch_##a##_##b
#define STHIP_CAT(a, b) STHIP_CAT2(a, b, )
#define L(akc, bkc, edge) &launch_gemm<InstT, STHIP_INST_ALGO, akc, bkc, edge>
extern const LaunchTable STHIP_CAT(STHIP_INST_TYPE, STHIP_INST_ALGO) = {{
    {{L(false, false, false), L(false, false, true)}, {L(false, true, false), L(false, true, true)}},
    {{L(true, false, false), L(true, false, true)}, {L(true, true, false), L(true, true, true)}},
}};
#endif

}  // namespace sthip
