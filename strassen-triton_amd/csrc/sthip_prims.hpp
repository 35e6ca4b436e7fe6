// The instructions the 256 x 256 and 64 x 64 kernels are built from that the compiler does not generate by itself:
// direct-to-LDS loads, the transposing LDS read, the matrix instructions with their accumulator tied.
// They are kept apart from the kernels so that a build for the host (tests/host_model/) can put
// functions of its own in their place and run the kernels' index arithmetic on the CPU.
#ifndef STHIP_PRIMS_HPP
#define STHIP_PRIMS_HPP

namespace sthip {

// One 1 KiB direct-to-LDS load: lane L moves 16 bytes from sbase + voff to LDS byte address
// lds_addr + 16 L.  Written as inline assembly on purpose: the compiler must not know that
// LDS is being filled asynchronously, or it serialises every later LDS read behind
// vmcnt(0); ordering is enforced by hand with wait_vmcnt() + the workgroup barrier.
__device__ __forceinline__ void lds_dma16(const void* sbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                 :: "s"(sbase), "v"(voff), "s"(lds_addr) : "memory", "m0");
}

// lds_dma16 with the LDS address given as a uniform register plus a constant: one scalar instruction
// for m0 and none for the global address (the rows of the load are part of the lane offset).
__device__ __forceinline__ void lds_dma16_k(const void* sbase, uint32_t voff, uint32_t lds_addr, int k) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0"
                 :: "s"(sbase), "v"(voff), "s"(lds_addr), "n"(k) : "memory", "scc", "m0");
}
// The same under a lane mask that is all ones or zero: with no lane enabled the load is not executed
// (no memory access, nothing to wait for).  Contract: the caller runs with all 64 lanes enabled, and
// the statement leaves them enabled; it is only called from the k-loop of gemm4p_kernel, whose
// control flow depends on blockIdx and kernel arguments alone.  exec is deliberately not in the
// clobber list: the statement restores the value the contract guarantees, and declaring it makes
// the compiler fence every call with hazard nops and re-order the main loop around them.
__device__ __forceinline__ void lds_dma16_km(const void* sbase, uint32_t voff, uint32_t lds_addr, int k, uint32_t mask) {
    asm volatile("s_mov_b32 exec_lo, %4\n\ts_mov_b32 exec_hi, %4\n\ts_add_u32 m0, %2, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %0\n\ts_mov_b64 exec, -1"
                 :: "s"(sbase), "v"(voff), "s"(lds_addr), "n"(k), "s"(mask) : "memory", "scc", "m0");
}

// The transposing LDS read (ds_read_b64_tr_b16): within each group of 16 lanes, lane r addresses four
// consecutive 16-bit elements; lane i receives element i % 4 of lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4.
__device__ __forceinline__ s16x4 lds_read_tr16_b64(const char* p) {
    typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
}

// The lanes of a wave execute in lockstep: what any lane has written to LDS before this point, every lane of
// the same wave may read after it (the waits the compiler places order the accesses).  Nothing is generated
// for it; the build of the kernels for the host synchronises the 64 threads of a wave here.
__device__ __forceinline__ void wave_exchange_point() {}

// acc (16 n x 16 m, transposed so that a lane holds four consecutive n) += B-fragment x A-fragment.
// Written as assembly so that the accumulator is updated in place: given the builtin, the
// register allocator puts result and addend in different registers and permutes the 64
// accumulators back with ~180 register copies per k-step.
// fp32: one v_mfma_f32_16x16x4 on component c of both fragments (k = 4 g + c for lane group g).
__device__ __forceinline__ void mfma16_step_f32(f32x4& acc, uint32_t a, uint32_t b) {
    asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}
template <class T>
__device__ __forceinline__ void mfma16_step(f32x4& acc, const u32x4& a, const u32x4& b) {
    if constexpr (__is_same(T, bf16_t))
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
    else
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
}

// 64 x 64 fp32 kernel (sthip_kernel6.hpp):
// 16-byte global load whose completion the compiler does not track (see run6), and the dependency that
// orders the uses of its result behind a hand-placed wait.
__device__ __forceinline__ void gload16_6(f32x4& dst, const float* p) {
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(p) : "memory");
}
__device__ __forceinline__ void tie6(f32x4& x) { asm volatile("" : "+v"(x)); }

}  // namespace sthip

#endif
