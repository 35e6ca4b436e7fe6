// Run-time side of the host build of the kernels (see host_runtime.cpp).
#pragma once
#include <functional>
#include <vector>
#include "hip/hip_runtime.h"

struct HostRange { const char* p; size_t n; };
extern std::vector<HostRange> g_host_global;   // what kernels may read through direct-to-LDS / untracked loads
extern bool g_host_late;                       // such loads land at the last moment the waits allow
extern int g_host_compute_units;               // what the library's launcher is told the device has
float host_as_float(uint32_t v, int idx, bool bf16);
namespace sthip { extern char smem[160 * 1024]; }   // the LDS of the workgroup that is running
