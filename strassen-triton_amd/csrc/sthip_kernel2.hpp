// Pipelined grouped-GEMM kernel for gfx950: the fast path for 16-bit operands.
//
// The kernel runs a short list of "segments" (operand pairs) for one 128 x 128 output tile
// position and recombines their fp32 accumulators in registers:
//   classic : 1 segment,  C = A B
//   Strassen: 7 segments, C11..C22 from M1..M7 with at most three accumulator tiles live
//   Winograd: 7 segments, the U-chain accumulated in place
// Every operand of a segment is a plain matrix (a raw quadrant of A / B, or a quadrant sum
// that a pre-pass wrote once), so tiles go from global memory straight into LDS with
// global_load_lds_dwordx4 -- no staging registers, no VALU work in the main loop.
//
// Pipeline.  LDS holds a ring of four stages (A tile + B tile of 64 k each).  Loads run
// three k-steps ahead of the MFMAs and the ring never drains between segments: while the
// last steps of one product compute, the first tiles of the next product are already in
// flight.  One workgroup barrier per k-step, placed in the middle of the step so that the
// first fragments of the next step are read while the current step's last MFMAs issue.
// LDS rows are XOR-swizzled in units of 16 bytes so that both the direct loads (which must
// fill LDS in lane order) and the fragment reads are bank-conflict free.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sthip_kernel.hpp"
#include "sthip_prims.hpp"

namespace sthip {

constexpr int kMaxSeg = 49;   // seven products of one level, or the 49 of two levels in one launch
constexpr int kStages = 4;
constexpr int kBK2 = 64;                       // k per step (16-bit operands)
constexpr int kTileBytes2 = 128 * kBK2 * 2;    // one operand tile: 16 KiB
constexpr int kStageBytes2 = 2 * kTileBytes2;  // A + B
constexpr int kSmemBytes2 = kStages * kStageBytes2;

struct Seg2 {
    const void* a; const void* b;   // operand bases (batch 0)
    int64_t a_ld, b_ld;             // stride of the non-contiguous index, elements
    int64_t a_bs, b_bs;             // batch strides, elements
};

struct Gemm2Params {
    Seg2 seg[kMaxSeg];
    void* C;
    float* park;          // scratch for one parked accumulator tile per workgroup (256 x 128 kernel, Strassen)
    int64_t c_rs, c_bs;   // C is row-major with unit column stride
    int64_t c_ps;         // classical kernels: element stride between the outputs of consecutive products
    int nprod;            // classical kernels: products in this launch (0 or 1 = plain GEMM)
    int Mh, Nh, Kh;       // extent of one segment product
    int tiles_m, tiles_n;
    int out_f32, accumulate, group_m;
    int c_wide;           // 256 x 256 kernel: C, its rows and its product / batch strides are 16-byte aligned
    int c_stream;         // 256 x 256 kernel: store the result tiles with the streaming hint
    int xcd_chunks;       // 256 x 256 kernel: products of fewer than 256 tiles go to the XCDs 32 tiles at a time (1-D grid)
    int nbatch;           // 256 x 256 kernel: batch entries (its grid is one-dimensional over batch entry, product and tile)
    int one_tile_per_wg;  // 256 x 256 kernel: never let a workgroup walk several tiles (test and timing switch)
};

__device__ __forceinline__ void wait_vmcnt(int n) {
    // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[15:14]; leave the others open
    if (n >= 16) __builtin_amdgcn_s_waitcnt(0x0F70 | (16 & 0xF) | ((16 >> 4) << 14));
    else if (n == 8) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    else __builtin_amdgcn_s_waitcnt(0x0F70 | 0);
}

typedef void __attribute__((address_space(3))) * lptr_t;

// Issues this wave's share (4 + 4 loads of 1 KiB) of one k-step into one LDS stage.
// KC operand tile: 128 rows x 8 chunks of 16 bytes; the load that fills rows R..R+7 has lane
// L fetch row R + L/8, chunk (L%8) ^ ((row/2)%8).  Other layout: 64 k-rows x 16 chunks; the
// load that fills k-rows 4j..4j+3 has lane L fetch k-row 4j + L/16, chunk (L%16) ^ ((k%4)*4).
// Addresses are split into a wave-uniform base (SGPR pair, advanced per load and per step)
// and a per-lane 32-bit offset that is fixed for a whole segment.
template <bool A_KC, bool B_KC>
struct Loader2 {
    const char* a_base; const char* b_base;   // uniform: this wave's first load of the next step
    int64_t a_row_bytes, b_row_bytes;         // uniform: distance between the wave's 4 loads
    int64_t a_step_bytes, b_step_bytes;       // uniform: advance per k-step
    uint32_t a_voff[2], b_voff[2];            // per lane: offsets for even / odd loads
    int seg, kt;                              // cursor: next step to issue
    int total_seg, KT;
    int batch, tile_m, tile_n, wave;
    const Gemm2Params* P;

    template <bool KC>
    __device__ __forceinline__ void point(const void* base, int64_t ld, int64_t bs, int tile,
                                          const char*& ubase, int64_t& row_bytes, int64_t& step_bytes,
                                          uint32_t (&voff)[2]) {
        const int lane = threadIdx.x & 63;
        const char* b = reinterpret_cast<const char*>(base) + (int64_t)batch * bs * 2;
        if constexpr (KC) {
            // rows wave*32 + 8 i + L/8; (row/2)%8 = 4 (i%2) + L/16
            const int chunk0 = (lane & 7) ^ (lane >> 4);
            ubase = b + (int64_t)(tile + wave * 32) * ld * 2;
            row_bytes = 8 * ld * 2;
            step_bytes = kBK2 * 2;
            voff[0] = (uint32_t)(((lane >> 3) * ld + chunk0 * 8) * 2);
            voff[1] = (uint32_t)(((lane >> 3) * ld + (chunk0 ^ 4) * 8) * 2);
        } else {
            // k-rows wave*16 + 4 i + L/16; k%4 = L/16
            const int chunk = (lane & 15) ^ ((lane >> 4) << 2);
            ubase = b + ((int64_t)(wave * 16) * ld + tile) * 2;
            row_bytes = 4 * ld * 2;
            step_bytes = (int64_t)kBK2 * ld * 2;
            voff[0] = voff[1] = (uint32_t)(((lane >> 4) * ld + chunk * 8) * 2);
        }
    }

    __device__ __forceinline__ void point_at_segment() {
        const Seg2& s = P->seg[seg];
        point<A_KC>(s.a, s.a_ld, s.a_bs, tile_m, a_base, a_row_bytes, a_step_bytes, a_voff);
        point<B_KC>(s.b, s.b_ld, s.b_bs, tile_n, b_base, b_row_bytes, b_step_bytes, b_voff);
    }

    __device__ __forceinline__ void issue(uint32_t stage_addr) {
        const uint32_t sa = stage_addr + wave * 4096, sb = sa + kTileBytes2;
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_dma16(a_base + i * a_row_bytes, a_voff[i & 1], sa + i * 1024);
#pragma unroll
        for (int i = 0; i < 4; ++i) lds_dma16(b_base + i * b_row_bytes, b_voff[i & 1], sb + i * 1024);
        a_base += a_step_bytes;
        b_base += b_step_bytes;
        if (++kt == KT) {
            kt = 0;
            if (++seg < total_seg) point_at_segment();
        }
    }

    __device__ __forceinline__ bool done() const { return seg >= total_seg; }
};

// 16 bytes of MFMA operand for sub-tile row block `sub` (multiple of 32), k-group kg of a stage.
template <bool KC>
__device__ __forceinline__ u32x4 read_frag2(const char* tile, int sub, int kg) {
    const int lane = threadIdx.x & 63;
    if constexpr (KC) {
        const int row = sub + (lane & 31);
        const int slot = (kg * 2 + (lane >> 5)) ^ ((lane >> 1) & 7);
        return *reinterpret_cast<const u32x4*>(tile + row * 128 + slot * 16);
    } else {
        const int l16 = lane & 15, grp = lane >> 4;
        const int k = kg * 16 + (grp >> 1) * 8 + (l16 >> 2);
        const int chunk = (sub >> 3) + (grp & 1) * 2 + ((l16 & 3) >> 1);
        const int slot = chunk ^ (((l16 >> 2) & 3) << 2);
        const char* p = tile + k * 256 + slot * 16 + (l16 & 1) * 8;
        s16x4 lo = lds_read_tr16_b64(p);
        s16x4 hi = lds_read_tr16_b64(p + 4 * 256);
        u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
        u32x4 r = {a[0], a[1], b[0], b[1]};
        return r;
    }
}

template <class T, bool A_KC, bool B_KC>
struct Pipe2 {
    Loader2<A_KC, B_KC> ld;
    char* smem;
    int g;             // global step index of the step being computed
    int total;         // total steps over all segments
    int wm, wn;
    u32x4 fa[2][2], fb[2][2];   // [buffer][sub-tile]

    uint32_t smem_addr;   // LDS byte address of smem
    __device__ __forceinline__ char* stage(int step) const { return smem + (step & (kStages - 1)) * kStageBytes2; }
    __device__ __forceinline__ uint32_t stage_addr(int step) const { return smem_addr + (step & (kStages - 1)) * kStageBytes2; }

    __device__ __forceinline__ void read_frags(int buf, int step, int kg) {
        const char* s = stage(step);
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[buf][i] = read_frag2<A_KC>(s, wm + i * 32, kg);
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[buf][j] = read_frag2<B_KC>(s + kTileBytes2, wn + j * 32, kg);
    }

    __device__ __forceinline__ void start() {
        g = 0;
#pragma unroll
        for (int s = 0; s < kStages - 1; ++s)
            if (!ld.done()) ld.issue(stage_addr(s));
        // stage 0 must have landed: at most two younger stages (8 loads each) may be in flight
        wait_vmcnt(total >= 3 ? 16 : (total == 2 ? 8 : 0));
        __syncthreads();
        read_frags(0, 0, 0);
    }

    // One segment: KT steps of 4 k-groups each, accumulating into acc.
    __device__ __forceinline__ void run(Acc& acc, int KT) {
        for (int kt = 0; kt < KT; ++kt, ++g) {
#pragma unroll
            for (int kg = 0; kg < 4; ++kg) {
                if (kg == 2) {
                    // Next stage must be visible to everyone before its fragments are read; this
                    // barrier also retires stage g-1, whose buffer the next load reuses.
                    const int ahead = total - 1 - g;        // steps after this one
                    if (ahead >= 2) wait_vmcnt(8); else wait_vmcnt(0);
                    __syncthreads();
                    if (!ld.done()) ld.issue(stage_addr(g + kStages - 1));
                }
                const int nb = (kg + 1) & 1;
                if (kg < 3) read_frags(nb, g, kg + 1);
                else if (g + 1 < total) read_frags(nb, g + 1, 0);
                const int cb = kg & 1;
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        mfma_step<T>(acc.t[i][j], fa[cb][i], fb[cb][j]);
                    }
            }
        }
    }
};

template <class T>
__device__ __forceinline__ void emit2(const Acc& acc, const Gemm2Params& P, char* Cb, int quad, int tile_m, int tile_n) {
    GemmParams q;
    q.Mh = P.Mh; q.Nh = P.Nh; q.c_rs = P.c_rs; q.c_cs = 1; q.out_f32 = P.out_f32; q.accumulate = P.accumulate;
    q.M = 2 * P.Mh; q.N = 2 * P.Nh;
    store_tile<T, false>(acc, q, Cb, quad, tile_m, tile_n);
}

template <class T, int ALGO, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(kThreads) gemm2_kernel(const Gemm2Params P) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    // tile coordinates: same XCD-aware walk as the first kernel
    GemmParams tp;
    tp.tiles_m = P.tiles_m; tp.tiles_n = P.tiles_n; tp.group_m = P.group_m;
    int tm, tn;
    // The classical kernel can run several independent products of equal shape in one launch
    // (product-major: blockIdx.x = product * tiles + tile), each with its own operand pair
    // (segment) and its own output matrix, c_ps elements apart.
    int prod = 0;
    if constexpr (ALGO == ALGO_CLASSIC) {
        const int tiles = P.tiles_m * P.tiles_n;
        prod = __builtin_amdgcn_readfirstlane((int)blockIdx.x / tiles);
        tile_coords_in(tp, (int)blockIdx.x - prod * tiles, tiles, tm, tn);
    } else {
        tile_coords(tp, tm, tn);
    }
    const int tile_m = tm * 128, tile_n = tn * 128;
    const int batch = blockIdx.y;
    char* Cb = reinterpret_cast<char*>(P.C) + ((int64_t)batch * P.c_bs + (int64_t)prod * P.c_ps) * (P.out_f32 ? 4 : 2);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int NSEG = ALGO == ALGO_CLASSIC ? 1 : 7;
    const int KT = P.Kh / kBK2;

    Pipe2<T, A_KC, B_KC> pipe;
    pipe.smem = smem;
    pipe.smem_addr = (uint32_t)(uintptr_t)(lptr_t)smem;
    pipe.ld.wave = wave;
    pipe.wm = (wave >> 1) * 64;
    pipe.wn = (wave & 1) * 64;
    pipe.total = NSEG * KT;
    pipe.ld.P = &P;
    pipe.ld.seg = prod; pipe.ld.kt = 0; pipe.ld.total_seg = prod + NSEG; pipe.ld.KT = KT;
    pipe.ld.batch = batch; pipe.ld.tile_m = tile_m; pipe.ld.tile_n = tile_n;
    pipe.ld.point_at_segment();
    pipe.start();

#define EMIT2(acc, quad) emit2<T>(acc, P, Cb, quad, tile_m, tile_n)
    enum { Q11 = 0, Q12 = 1, Q21 = 2, Q22 = 3 };
    if constexpr (ALGO == ALGO_CLASSIC) {
        Acc x;
        x.zero();
        pipe.run(x, KT);
        // classic: the "quadrant" is the whole matrix (Mh = M)
        GemmParams q;
        q.Mh = P.Mh; q.Nh = P.Nh; q.c_rs = P.c_rs; q.c_cs = 1; q.out_f32 = P.out_f32; q.accumulate = P.accumulate;
        q.M = P.Mh; q.N = P.Nh;
        store_tile<T, false>(x, q, Cb, 0, tile_m, tile_n);
    } else if constexpr (ALGO == ALGO_STRASSEN) {
        // segment order: M3 M6 M5 M7 M1 M2 M4 (see the first kernel for the chain bookkeeping)
        Acc x, y, z;
        x.zero();
        pipe.run(x, KT);   // M3
        y = x;
        pipe.run(y, KT);   // M6 in place
        z.zero();
        pipe.run(z, KT);   // M5
        x.add(z);
        EMIT2(x, Q12);
        z.negate();
        pipe.run(z, KT);   // M7 in place
        x.zero();
        pipe.run(x, KT);   // M1
        y.add(x);
        z.add(x);
        x.zero();
        pipe.run(x, KT);   // M2
        y.sub(x);
        EMIT2(y, Q22);
        y.zero();
        pipe.run(y, KT);   // M4
        z.add(y);
        EMIT2(z, Q11);
        x.add(y);
        EMIT2(x, Q21);
    } else {
        // segment order: P1 P2 P6 P7 P5 P3 (-P4)
        Acc x, y, z;
        x.zero();
        pipe.run(x, KT);   // P1
        y = x;
        pipe.run(x, KT);   // + P2 -> C11
        EMIT2(x, Q11);
        pipe.run(y, KT);   // + P6 -> U2
        z = y;
        pipe.run(y, KT);   // + P7 -> U3
        x.zero();
        pipe.run(x, KT);   // P5
        z.add(x);          // U4
        x.add(y);          // C22
        EMIT2(x, Q22);
        pipe.run(z, KT);   // + P3 -> C12
        EMIT2(z, Q12);
        pipe.run(y, KT);   // + A22 (-T4) -> C21
        EMIT2(y, Q21);
    }
#undef EMIT2
}

}  // namespace sthip
