// Stand-in for <hip/hip_runtime.h> when the kernel headers are compiled for the host (host_shim.h has
// everything they need).
#pragma once
#include "../host_shim.h"
