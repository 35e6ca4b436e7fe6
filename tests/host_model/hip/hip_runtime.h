// Stand-in for <hip/hip_runtime.h> when the library is compiled for the host: the device-side shims of
// host_shim.h and the few runtime calls the library's host code makes.  A kernel launch runs the kernel at
// once, one workgroup at a time, one host thread per lane (host_launch in kernel4_host.cpp / library_host.cpp).
#pragma once
#include <cstring>
#include <functional>
#include "../host_shim.h"

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1 };
typedef struct HostStream* hipStream_t;
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 63 };
inline const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "invalid value"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
inline hipError_t hipFuncSetAttribute(const void*, hipFuncAttribute, int) { return hipSuccess; }
int host_compute_units();   // how many workgroups the "device" is said to run at once
inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = host_compute_units(); return hipSuccess; }
enum hipMemcpyKind { hipMemcpyDeviceToHost = 2 };
inline hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }   // launches run to completion at once
inline hipError_t hipMemcpy(void* dst, const void* src, size_t n, hipMemcpyKind) { memcpy(dst, src, n); return hipSuccess; }
#define HIP_SYMBOL(x) (&(x))
void host_register_symbol(const void* p, size_t bytes);   // a __device__ array becomes memory that kernels may read
template <class T> inline hipError_t hipGetSymbolAddress(void** p, T* sym) { *p = (void*)sym; host_register_symbol(sym, sizeof(T)); return hipSuccess; }
#define __align__(n) __attribute__((aligned(n)))

void host_launch(dim3 grid, dim3 block, const std::function<void()>& body);
#define hipLaunchKernelGGL(kern, grid, block, shmem, stream, ...) host_launch((grid), (block), [&]() { (kern)(__VA_ARGS__); })
