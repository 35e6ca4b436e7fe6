// Stand-alone timing of the 256 x 256 pipelined kernel on one classical n^3 bf16 product, with
// parts of its main loop compiled out (not part of the library):
//
//   hipcc -O3 -std=c++17 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         -DSTHIP_DBG=<mask> -I . kernel4_microbench.hip -o kernel4_microbench
//   ./kernel4_microbench [n = 8192] [leading-dimension padding in elements = 0]
//
// STHIP_DBG bits: 1 = no global -> LDS loads, 2 = no workgroup barrier, 4 = no LDS fragment reads
// (MFMAs then run on zeros), 8 = no store of the tile, 16 = the kernel returns at once (launch and
// dispatch alone), 32 = the 8-byte store straight from the accumulators, 64 = no MFMAs, 128 = every
// k-step loads the first k-slice again (loads that hit in cache).  0 is the kernel as shipped; 5 is MFMAs alone.
// Results are timings only: with any bit set the product is not computed.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>
#include "sthip_kernel4.hpp"
using namespace sthip;
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
template <bool BKC> void run(int n, int pad) {
  int ld = n + pad;
  size_t bytes = (size_t)n * ld * 2;
  void *A, *B, *C;
  CK(hipMalloc(&A, bytes)); CK(hipMalloc(&B, bytes)); CK(hipMalloc(&C, bytes));
  std::vector<uint16_t> h((size_t)n * ld);
  for (size_t i = 0; i < h.size(); ++i) h[i] = 0x3c00 + (rand() & 0x3ff);
  CK(hipMemcpy(A, h.data(), bytes, hipMemcpyHostToDevice)); CK(hipMemcpy(B, h.data(), bytes, hipMemcpyHostToDevice));
  Gemm2Params p; memset(&p, 0, sizeof(p));
  p.seg[0] = {A, B, ld, ld, 0, 0};
  p.C = C; p.c_rs = ld; p.Mh = n; p.Nh = n; p.Kh = n; p.tiles_m = n / 256; p.tiles_n = n / 256; p.group_m = 4; p.nprod = 1; p.c_wide = (ld % 8 == 0);
  auto kern = gemm4_kernel<bf16_t, BKC>;
  CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kSmemBytes4));
  dim3 grid(p.tiles_m * p.tiles_n, 1);
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  for (int i = 0; i < 5; ++i) hipLaunchKernelGGL(kern, grid, dim3(kThreads4), kSmemBytes4, 0, p);
  CK(hipDeviceSynchronize());
  int reps = 20;
  CK(hipEventRecord(e0));
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(kern, grid, dim3(kThreads4), kSmemBytes4, 0, p);
  CK(hipEventRecord(e1)); CK(hipDeviceSynchronize());
  float ms; CK(hipEventElapsedTime(&ms, e0, e1)); ms /= reps;
  double flops = 2.0 * n * n * (double)n;
  printf("k4 DBG=%d n=%d pad=%d bkc=%d: %.4f ms  %.1f TFLOP/s\n", STHIP_DBG, n, pad, (int)BKC, ms, flops / ms / 1e9);
  fflush(stdout);
  CK(hipFree(A)); CK(hipFree(B)); CK(hipFree(C));
}
int main(int argc, char** argv) {
  int n = argc > 1 ? atoi(argv[1]) : 8192;
  int pad = argc > 2 ? atoi(argv[2]) : 0;
  run<false>(n, pad); run<true>(n, pad);
  return 0;
}
