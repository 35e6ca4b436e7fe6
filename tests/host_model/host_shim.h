// What the kernel headers under strassen-triton_amd/csrc need in order to compile for the host: the
// HIP keywords as empty macros, the thread coordinates as thread-local variables, and the AMDGPU builtins
// as functions.  One host thread plays one lane; kernel4_host.cpp holds the run-time side.
#pragma once
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <stdio.h>
#include <stdlib.h>
#include <algorithm>
#include <vector>
using std::min;
using std::max;

#define __device__
#define __global__
#define __host__
#define __forceinline__ inline
#define __launch_bounds__(x)
#define __shared__ static   // one copy for all threads: workgroups run one at a time (`extern __shared__` is rewritten to `extern`)

struct HostDim3 { unsigned x, y, z; };
extern thread_local HostDim3 threadIdx, blockIdx, gridDim, blockDim;

void host_syncthreads();                 // barrier over the workgroup's threads
void host_waitcnt(int imm);              // s_waitcnt: completes this lane's pending direct-to-LDS loads
inline void __syncthreads() { host_syncthreads(); }
inline void __builtin_amdgcn_s_waitcnt(int imm) { host_waitcnt(imm); }
inline void __builtin_amdgcn_sched_barrier(int) {}
inline void __builtin_amdgcn_sched_group_barrier(int, int, int) {}
inline void __builtin_amdgcn_s_setprio(int) {}
inline int __builtin_amdgcn_readfirstlane(int x) { return x; }   // only ever applied to uniform values

void host_mfma_16x16x4(float a_inst, float b_inst, float* acc4);   // v_mfma_f32_16x16x4_f32 among the threads of a wave
template <class V> inline V __builtin_amdgcn_mfma_f32_16x16x4f32(float a_inst, float b_inst, V acc, int, int, int) {
    float r[4] = {acc[0], acc[1], acc[2], acc[3]};
    host_mfma_16x16x4(a_inst, b_inst, r);
    return V{r[0], r[1], r[2], r[3]};
}

// v_mfma_f32_32x32x16 (16-bit operands, eight per lane) and v_mfma_f32_32x32x2 (fp32, one per lane) among the
// threads of a wave; `halves` are the raw 16-bit patterns.
void host_mfma_32x32x16(const uint16_t a_inst[8], const uint16_t b_inst[8], float acc16[16], bool bf16);
void host_mfma_32x32x2(float a_inst, float b_inst, float acc16[16]);
template <class A, class V> inline V host_mfma16_wrap(A a, A b, V acc, bool bf16) {
    uint16_t ha[8], hb[8];
    float r[16];
    memcpy(ha, &a, 16); memcpy(hb, &b, 16);
    for (int e = 0; e < 16; ++e) r[e] = acc[e];
    host_mfma_32x32x16(ha, hb, r, bf16);
    V o;
    for (int e = 0; e < 16; ++e) o[e] = r[e];
    return o;
}
template <class A, class V> inline V __builtin_amdgcn_mfma_f32_32x32x16_bf16(A a, A b, V acc, int, int, int) { return host_mfma16_wrap(a, b, acc, true); }
template <class A, class V> inline V __builtin_amdgcn_mfma_f32_32x32x16_f16(A a, A b, V acc, int, int, int) { return host_mfma16_wrap(a, b, acc, false); }
template <class V> inline V __builtin_amdgcn_mfma_f32_32x32x2f32(float a, float b, V acc, int, int, int) {
    float r[16];
    for (int e = 0; e < 16; ++e) r[e] = acc[e];
    host_mfma_32x32x2(a, b, r);
    V o;
    for (int e = 0; e < 16; ++e) o[e] = r[e];
    return o;
}

// Used directly by the fused 128 x 128 kernel of sthip_kernel.hpp, which this build does not run.
typedef short host_s16x4 __attribute__((ext_vector_type(4)));
template <class P> inline host_s16x4 __builtin_amdgcn_ds_read_tr16_b64_v4i16(P) { abort(); }

// The one-launch kernel's counters (sthip_kernel5.hpp): workgroups of that launch would have to run at the
// same time, which this build does not do; the code only has to compile.
#define __HIP_MEMORY_SCOPE_AGENT 4
inline void __builtin_amdgcn_s_sleep(int) {}
inline void __builtin_amdgcn_fence(int, const char*) {}
