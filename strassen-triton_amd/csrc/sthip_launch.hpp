// Launch table shared by the kernel instantiation units and the C-ABI front end.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include "sthip_kernel.hpp"
#include "sthip_kernel2.hpp"
#include "sthip_kernel3.hpp"
#include "sthip_kernel4.hpp"
#include "sthip_kernel5.hpp"
#include "sthip_kernel6.hpp"

namespace sthip {

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };

// More than 64 KiB of dynamic LDS needs an explicit opt-in per kernel, once per device.  `done` is the
// kernel's own flag array; two threads that race here both set the (idempotent) attribute.
struct OptIn { std::atomic<bool> done[64]; };
inline hipError_t opt_in_lds(OptIn& o, const void* kern, int bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64) return hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (!o.done[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return e;
        o.done[dev].store(true, std::memory_order_release);
    }
    return hipSuccess;
}

// Compute units of the current device (0 if the query fails), asked once per device.
inline int compute_units() {
    static std::atomic<int> known[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = known[dev].load(std::memory_order_acquire);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
        known[dev].store(n, std::memory_order_release);
    }
    return n;
}

// One table per (element type, algorithm), indexed [a_kc][b_kc][edge]; each is defined by
// one compilation of sthip_inst.hip.
typedef hipError_t (*LaunchFn)(const GemmParams&, int batch, hipStream_t);
struct LaunchTable { LaunchFn fn[2][2][2]; };
#define STHIP_DECLARE_TABLE(T, A) extern const LaunchTable kLaunch_##T##_##A;
STHIP_DECLARE_TABLE(0, 0) STHIP_DECLARE_TABLE(0, 1) STHIP_DECLARE_TABLE(0, 2)
STHIP_DECLARE_TABLE(1, 0) STHIP_DECLARE_TABLE(1, 1) STHIP_DECLARE_TABLE(1, 2)
STHIP_DECLARE_TABLE(2, 0) STHIP_DECLARE_TABLE(2, 1) STHIP_DECLARE_TABLE(2, 2)
#undef STHIP_DECLARE_TABLE

template <class T, int ALGO, bool A_KC, bool B_KC, bool EDGE>
hipError_t launch_gemm(const GemmParams& p, int batch, hipStream_t stream) {
    using C = Ctx<T, A_KC, B_KC>;
    auto kern = gemm_kernel<T, ALGO, A_KC, B_KC, EDGE>;
    static OptIn opted;
    hipError_t e = opt_in_lds(opted, reinterpret_cast<const void*>(kern), C::SMEM_BYTES);
    if (e != hipSuccess) return e;
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)batch, 1);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), C::SMEM_BYTES, stream, p);
    return hipGetLastError();
}

// Pipelined kernel (16-bit operands): one table per (type, algorithm), indexed [a_kc][b_kc].
typedef hipError_t (*LaunchFn2)(const Gemm2Params&, int batch, hipStream_t);
struct LaunchTable2 { LaunchFn2 fn[2][2]; };
#define STHIP_DECLARE_TABLE2(T, A) extern const LaunchTable2 kLaunch2_##T##_##A;
STHIP_DECLARE_TABLE2(1, 0) STHIP_DECLARE_TABLE2(1, 1) STHIP_DECLARE_TABLE2(1, 2)
STHIP_DECLARE_TABLE2(2, 0) STHIP_DECLARE_TABLE2(2, 1) STHIP_DECLARE_TABLE2(2, 2)
#undef STHIP_DECLARE_TABLE2

template <class T, int ALGO, bool A_KC, bool B_KC>
hipError_t launch_gemm2(const Gemm2Params& p, int batch, hipStream_t stream) {
    auto kern = gemm2_kernel<T, ALGO, A_KC, B_KC>;
    static OptIn opted;
    hipError_t e = opt_in_lds(opted, reinterpret_cast<const void*>(kern), kSmemBytes2);
    if (e != hipSuccess) return e;
    const int nprod = ALGO == ALGO_CLASSIC && p.nprod > 0 ? p.nprod : 1;
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n * nprod), (unsigned)batch, 1);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads), kSmemBytes2, stream, p);
    return hipGetLastError();
}

// 256 x 128 kernel (16-bit operands, A contiguous along k): tables indexed [b_kc].
struct LaunchTable3 { LaunchFn2 fn[2]; };
#define STHIP_DECLARE_TABLE3(T, A) extern const LaunchTable3 kLaunch3_##T##_##A;
STHIP_DECLARE_TABLE3(1, 0) STHIP_DECLARE_TABLE3(1, 1) STHIP_DECLARE_TABLE3(1, 2)
STHIP_DECLARE_TABLE3(2, 0) STHIP_DECLARE_TABLE3(2, 1) STHIP_DECLARE_TABLE3(2, 2)
#undef STHIP_DECLARE_TABLE3

template <class T, int ALGO, bool B_KC>
hipError_t launch_gemm3(const Gemm2Params& p, int batch, hipStream_t stream) {
    auto kern = gemm3_kernel<T, ALGO, B_KC>;
    static OptIn opted;
    hipError_t e = opt_in_lds(opted, reinterpret_cast<const void*>(kern), kSmemBytes3);
    if (e != hipSuccess) return e;
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)batch, 1);
    hipLaunchKernelGGL(kern, grid, dim3(kThreads3), kSmemBytes3, stream, p);
    return hipGetLastError();
}

// 256 x 256 kernel (fp32 or 16-bit operands, A contiguous along k), p.nprod products per launch:
// tables indexed [b_kc].
extern const LaunchTable3 kLaunch4_0;
extern const LaunchTable3 kLaunch4_1;
extern const LaunchTable3 kLaunch4_2;

template <class T, bool B_KC>
hipError_t launch_gemm4(const Gemm2Params& p, int batch, hipStream_t stream) {
    auto kern = gemm4_kernel<T, B_KC>;
    static OptIn opted;
    hipError_t e = opt_in_lds(opted, reinterpret_cast<const void*>(kern), kSmemBytes4);
    if (e != hipSuccess) return e;
    const int nprod = p.nprod > 0 ? p.nprod : 1;
    const int tiles = p.tiles_m * p.tiles_n;
    const int64_t total = (int64_t)tiles * nprod * batch;
    if (total <= 0 || total >= (1 << 30)) return hipErrorInvalidValue;
    // the loader's lane offsets are 32-bit and reach over 32 rows of an operand
    for (int s = 0; s < nprod; ++s)
        if (p.seg[s].a_ld >= (int64_t(1) << 26) || p.seg[s].b_ld >= (int64_t(1) << 26)) return hipErrorInvalidValue;
    Gemm2Params q = p;
    // several small products at once: XCD-chunked numbering (see map_tile4)
    // (measured: grouped launch of config 4 1.585 -> 1.545 ms, two-level 8192^3 0.787 -> 0.766 ms)
    q.xcd_chunks = (tiles == 32 || tiles == 64 || tiles == 128) && p.tiles_m % 4 == 0 && total >= 256 ? 1 : 0;
    q.nbatch = batch;
    // 16-bit results with 16-byte aligned rows, more tiles than CUs: one workgroup per CU walks the tiles
    // as one software pipeline (gemm4p_kernel).  Measured on the grouped launches: 8192^3 one level
    // 0.756 -> 0.729 ms, two levels 0.75 -> 0.72 ms, 4096^3 0.110 -> 0.107 ms, config 4 1.549 -> 1.497 ms;
    // with fewer workgroups than CUs it loses (248: +8 %).
    if constexpr (sizeof(T) == 2) {
        const int cus = compute_units();
        if (!p.one_tile_per_wg && cus > 0 && total > cus && p.c_wide && !p.out_f32 && !p.accumulate) {
            auto kp = gemm4p_kernel<T, B_KC>;
            static OptIn opted_p;
            e = opt_in_lds(opted_p, reinterpret_cast<const void*>(kp), kSmemBytes4p);
            if (e != hipSuccess) return e;
            hipLaunchKernelGGL(kp, dim3((unsigned)cus), dim3(kThreads4), kSmemBytes4p, stream, q);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(kThreads4), kSmemBytes4, stream, q);
    return hipGetLastError();
}

// One-launch Strassen level (16-bit operands, A contiguous along k): tables indexed [b_kc]; `blocks`
// is the length of the work-item list.
typedef hipError_t (*LaunchFn5)(const Fused5Params&, int blocks, hipStream_t);
struct LaunchTable5 { LaunchFn5 fn[2]; };
extern const LaunchTable5 kLaunch5_1;
extern const LaunchTable5 kLaunch5_2;

template <class T, bool B_KC>
hipError_t launch_fused5(const Fused5Params& p, int blocks, hipStream_t stream) {
    auto kern = fused5_kernel<T, B_KC>;
    static OptIn opted;
    hipError_t e = opt_in_lds(opted, reinterpret_cast<const void*>(kern), kSmemBytes4);
    if (e != hipSuccess) return e;
    // the tiles run the loader of the grouped kernel: the same bound on its 32-bit lane offsets
    for (int s = 0; s < 7; ++s)
        if (p.g.seg[s].a_ld >= (int64_t(1) << 26) || p.g.seg[s].b_ld >= (int64_t(1) << 26)) return hipErrorInvalidValue;
    if (blocks <= 0 || p.tiles <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(kThreads4), kSmemBytes4, stream, p);
    return hipGetLastError();
}

// 64 x 64 fp32 kernel with the pre-additions fused into the loads (defined in sthip_inst6.hip).
hipError_t launch_gemm6(const Gemm6Params& p, bool b_kc, hipStream_t stream);

}  // namespace sthip
