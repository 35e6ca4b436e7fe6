// 256 x 256-tile pipelined grouped-GEMM kernel for gfx950: four waves (one per SIMD) of
// 128 x 128 each, 16-bit operands, A contiguous along k.
//
// The L2 -> LDS path, not the matrix cores, limits the smaller-tile kernels: bytes moved per
// flop go with (1/BM + 1/BN).  A 256 x 256 tile moves two thirds of what 256 x 128 moves, but
// one fp32 accumulator tile then fills all 256 AGPRs of a wave, so no Strassen / Winograd chain
// can stay in registers beside it.  (Parking the chains in per-workgroup fp32 slabs was built
// and measured: every CU parks 256 KiB at the same moment, nine to eighteen times per tile,
// and the kernel ran a third slower than the 256 x 128 one.)  So this kernel only ever runs
// plain products: one launch covers `nprod` independent products of equal shape (the seven
// products of a level, each with its own operand pair and its own output matrix), product-major,
// so that the chip works through one product at a time and each behaves like a classical GEMM.
// The recombination of the seven outputs is a separate elementwise pass.
//
// Pipeline: k-steps of 64 (whole 128-byte lines per row), two LDS stages of 64 KiB, the
// barrier of a step sits just before the next step's first fragments are read, at which
// point the current stage is free and is refilled with the step two ahead.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sthip_kernel3.hpp"

namespace sthip {

constexpr int kThreads4 = 256;
constexpr int kBM4 = 256, kBN4 = 256, kBK4 = 64;
constexpr int kStages4 = 2;
constexpr int kATile4 = kBM4 * kBK4 * 2;                 // 32 KiB
constexpr int kBTile4 = kBN4 * kBK4 * 2;                 // 32 KiB
constexpr int kStageBytes4 = kATile4 + kBTile4;          // 64 KiB
constexpr int kSmemBytes4 = kStages4 * kStageBytes4;     // 128 KiB

// A and k-contiguous B: 256 rows x 8 chunks; wave w loads rows 64 w + 8 i + L/8, i = 0..7,
// chunk (L%8) ^ ((row/2)%8).  n-contiguous B: 64 k-rows x 32 chunks (512 bytes); wave w loads
// k-rows 16 w + 2 i + L/32, i = 0..7, chunk (L%32) ^ ((k%4)*4).
template <bool B_KC>
struct Loader4 {
    const char* a_base; const char* b_base;
    int64_t a_row_bytes, b_row_bytes, a_step_bytes, b_step_bytes;
    uint32_t a_voff[2], b_voff[2];
    int seg, kt, total_seg, KT;
    int batch, tile_m, tile_n, wave;
    const Gemm2Params* P;

    __device__ __forceinline__ void point_at_segment() {
        const Seg2& s = P->seg[seg];
        const int lane = threadIdx.x & 63;
        const char* a = reinterpret_cast<const char*>(s.a) + (int64_t)batch * s.a_bs * 2;
        const char* b = reinterpret_cast<const char*>(s.b) + (int64_t)batch * s.b_bs * 2;
        const int chunk0 = (lane & 7) ^ (lane >> 4);     // (row/2)%8 = 4 (i%2) + L/16
        a_base = a + (int64_t)(tile_m + wave * 64) * s.a_ld * 2;
        a_row_bytes = 8 * s.a_ld * 2;
        a_step_bytes = kBK4 * 2;
        a_voff[0] = (uint32_t)(((lane >> 3) * s.a_ld + chunk0 * 8) * 2);
        a_voff[1] = (uint32_t)(((lane >> 3) * s.a_ld + (chunk0 ^ 4) * 8) * 2);
        if constexpr (B_KC) {
            b_base = b + (int64_t)(tile_n + wave * 64) * s.b_ld * 2;
            b_row_bytes = 8 * s.b_ld * 2;
            b_step_bytes = kBK4 * 2;
            b_voff[0] = (uint32_t)(((lane >> 3) * s.b_ld + chunk0 * 8) * 2);
            b_voff[1] = (uint32_t)(((lane >> 3) * s.b_ld + (chunk0 ^ 4) * 8) * 2);
        } else {
            // k%4 = 2 (i%2) + L/32
            const int chunk = (lane & 31) ^ ((lane >> 5) << 2);
            b_base = b + ((int64_t)(wave * 16) * s.b_ld + tile_n) * 2;
            b_row_bytes = 2 * s.b_ld * 2;
            b_step_bytes = (int64_t)kBK4 * s.b_ld * 2;
            b_voff[0] = (uint32_t)(((lane >> 5) * s.b_ld + chunk * 8) * 2);
            b_voff[1] = (uint32_t)(((lane >> 5) * s.b_ld + (chunk ^ 8) * 8) * 2);
        }
    }

    // The sixteen loads of one k-step (8 for A, 8 for B), then move the cursor on.
    __device__ __forceinline__ void issue(uint32_t stage_addr) {
        const uint32_t sa = stage_addr + wave * 8192, sb = stage_addr + kATile4 + wave * 8192;
#pragma unroll
        for (int i = 0; i < 8; ++i) lds_dma16(a_base + i * a_row_bytes, a_voff[i & 1], sa + i * 1024);
#pragma unroll
        for (int i = 0; i < 8; ++i) lds_dma16(b_base + i * b_row_bytes, b_voff[i & 1], sb + i * 1024);
        a_base += a_step_bytes;
        b_base += b_step_bytes;
        if (++kt == KT) {
            kt = 0;
            if (++seg < total_seg) point_at_segment();
        }
    }

    __device__ __forceinline__ bool done() const { return seg >= total_seg; }
};

// n-contiguous B tile with 512-byte k-rows: same transposing read as the narrower tiles.
__device__ __forceinline__ u32x4 read_frag4_mc(const char* tile, int sub, int kg) {
    const int lane = threadIdx.x & 63;
    const int l16 = lane & 15, grp = lane >> 4;
    const int k = kg * 16 + (grp >> 1) * 8 + (l16 >> 2);
    const int chunk = (sub >> 3) + (grp & 1) * 2 + ((l16 & 3) >> 1);
    const int slot = chunk ^ (((l16 >> 2) & 3) << 2);
    const char* p = tile + k * 512 + slot * 16 + (l16 & 1) * 8;
    typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * 512));
    u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
    u32x4 r = {a[0], a[1], b[0], b[1]};
    return r;
}

struct Acc4 {   // one 128 x 128 wave tile = 4 x 4 MFMA tiles = 256 registers
    f32x16 t[4][4];
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) t[i][j][e] = 0.f;
    }
};

template <class T, bool B_KC>
struct Pipe4 {
    Loader4<B_KC> ld;
    char* smem;
    uint32_t smem_addr;
    int g, total, slot;
    int wm, wn;
    u32x4 fa[2][4], fb[2][4];

    __device__ __forceinline__ void read_frags(int buf, int sl, int kg) {
        const char* s = smem + sl * kStageBytes4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if constexpr (B_KC) fb[buf][j] = read_frag2<true>(s + kATile4, wn + j * 32, kg);
            else fb[buf][j] = read_frag4_mc(s + kATile4, wn + j * 32, kg);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[buf][i] = read_frag2<true>(s, wm + i * 32, kg);
    }

    __device__ __forceinline__ void start() {
        g = 0;
        slot = 0;
        if (STHIP_DBG & 4) {
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i) { fa[b][i] = u32x4{0, 0, 0, 0}; fb[b][i] = u32x4{0, 0, 0, 0}; }
        }
        if (!(STHIP_DBG & 1)) {
            ld.issue(smem_addr);
            if (!ld.done()) ld.issue(smem_addr + kStageBytes4);
            if (total >= 2) wait_vmcnt_imm<16>(); else wait_vmcnt_imm<0>();   // step 0 has landed
        }
        __syncthreads();
        if (!(STHIP_DBG & 4)) read_frags(0, 0, 0);
    }

    __device__ __forceinline__ void run(Acc4& acc, int KT) {
        for (int kt = 0; kt < KT; ++kt, ++g) {
#pragma unroll
            for (int kg = 0; kg < 4; ++kg) {
                const int nb = (kg + 1) & 1, cb = kg & 1;
                if (kg < 3) {
                    if (!(STHIP_DBG & 4)) read_frags(nb, slot, kg + 1);
                } else {
                    // Every wave has read all fragments of this step: after the barrier its stage is
                    // free for the step two ahead.  Step g+1 (the only load batch in flight) must
                    // have landed before its fragments are read.
                    if (!(STHIP_DBG & 1)) wait_vmcnt_imm<0>();
                    if (!(STHIP_DBG & 2)) __syncthreads();
                    if (!(STHIP_DBG & 1) && !ld.done()) ld.issue(smem_addr + slot * kStageBytes4);
                    if (!(STHIP_DBG & 4) && g + 1 < total) read_frags(nb, slot ^ 1, 0);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (!(STHIP_DBG & 64)) mfma_step<T>(acc.t[i][j], fa[cb][i], fb[cb][j]);
                if (!(STHIP_DBG & (4 | 64))) {
#pragma unroll
                    for (int m = 0; m < 16; ++m) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            slot ^= 1;
        }
    }
};

template <class T>
__device__ __forceinline__ void store_tile4(const Acc4& acc, const Gemm2Params& P, char* Cb, int quad, int row, int col) {
    const int lane = threadIdx.x & 63;
    const int esz = P.out_f32 ? 4 : 2;
    const int m0 = (quad >> 1) * P.Mh + row + (lane & 31);
    const int n0 = (quad & 1) * P.Nh + col + 4 * (lane >> 5);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc.t[i][j][4 * g + e];
                char* dst = Cb + ((int64_t)(m0 + i * 32) * P.c_rs + (n0 + j * 32 + 8 * g)) * esz;
                if (P.out_f32) {
                    f32x4* d = reinterpret_cast<f32x4*>(dst);
                    f32x4 o = {v[0], v[1], v[2], v[3]};
                    if (P.accumulate) o += *d;
                    *d = o;
                } else {
                    u32x2* d = reinterpret_cast<u32x2*>(dst);
                    if (P.accumulate) {
                        const u32x2 old = *d;
                        const uint32_t w0 = old[0], w1 = old[1];
                        if constexpr (__is_same(T, bf16_t)) {
                            v[0] += bf16lo(w0); v[1] += bf16hi(w0); v[2] += bf16lo(w1); v[3] += bf16hi(w1);
                        } else {
                            const f16x2 h0 = as_f16x2(w0), h1 = as_f16x2(w1);
                            v[0] += (float)h0[0]; v[1] += (float)h0[1]; v[2] += (float)h1[0]; v[3] += (float)h1[1];
                        }
                    }
                    u32x2 o;
                    if constexpr (__is_same(T, bf16_t)) { o[0] = pack_bf16(v[0], v[1]); o[1] = pack_bf16(v[2], v[3]); }
                    else { o[0] = pack_f16(v[0], v[1]); o[1] = pack_f16(v[2], v[3]); }
                    *d = o;
                }
                if (g == 3) __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}

template <class T, bool B_KC>
__global__ void __launch_bounds__(kThreads4) gemm4_kernel(const Gemm2Params P) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    // blockIdx.x = product * tiles + tile: the XCD-aware renumbering works within one product
    const int tiles = P.tiles_m * P.tiles_n;
    const int prod = __builtin_amdgcn_readfirstlane((int)blockIdx.x / tiles);
    GemmParams tp;
    tp.tiles_m = P.tiles_m; tp.tiles_n = P.tiles_n; tp.group_m = P.group_m;
    int tm, tn;
    tile_coords_in(tp, (int)blockIdx.x - prod * tiles, tiles, tm, tn);
    const int tile_m = tm * kBM4, tile_n = tn * kBN4;
    const int batch = blockIdx.y;
    char* Cb = reinterpret_cast<char*>(P.C) + ((int64_t)batch * P.c_bs + (int64_t)prod * P.c_ps) * (P.out_f32 ? 4 : 2);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int KT = P.Kh / kBK4;

    Pipe4<T, B_KC> pipe;
    pipe.smem = smem;
    pipe.smem_addr = (uint32_t)(uintptr_t)(lptr_t)smem;
    pipe.wm = (wave >> 1) * 128;
    pipe.wn = (wave & 1) * 128;
    pipe.total = KT;
    pipe.ld.P = &P;
    pipe.ld.wave = wave;
    pipe.ld.seg = prod; pipe.ld.kt = 0; pipe.ld.total_seg = prod + 1; pipe.ld.KT = KT;
    pipe.ld.batch = batch; pipe.ld.tile_m = tile_m; pipe.ld.tile_n = tile_n;
    pipe.ld.point_at_segment();
    pipe.start();

    Acc4 r;
    r.zero();
    pipe.run(r, KT);
    store_tile4<T>(r, P, Cb, 0, tile_m + pipe.wm, tile_n + pipe.wn);
}

}  // namespace sthip
