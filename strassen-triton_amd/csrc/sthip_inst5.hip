// Instantiates the one-launch Strassen level for one 16-bit element type:
// -DSTHIP_INST_TYPE={1:f16,2:bf16}.
#include "sthip_launch.hpp"

namespace sthip {

#if STHIP_INST_TYPE == 1
typedef f16_t InstT;
#else
typedef bf16_t InstT;
#endif

template __global__ void fused5_kernel<InstT, false>(const Fused5Params);
template __global__ void fused5_kernel<InstT, true>(const Fused5Params);

#ifndef __HIP_DEVICE_COMPILE__
#define STHIP_CAT2(a, b) kLaunch5_##a
#define STHIP_CAT(a) STHIP_CAT2(a, )
extern const LaunchTable5 STHIP_CAT(STHIP_INST_TYPE) = {{&launch_fused5<InstT, false>, &launch_fused5<InstT, true>}};
#endif

}  // namespace sthip
