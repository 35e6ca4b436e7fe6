// Large-tile pipelined grouped-GEMM kernel for gfx950: 256 x 128 output tile per workgroup,
// four waves (one per SIMD) of 128 x 64 each, 16-bit operands, A contiguous along k.
//
// Why this shape.  A direct-to-LDS load moves 64 bytes per clock per CU; with a 128 x 128
// tile that path saturates exactly at the MFMA rate.  256 x 128 cuts the global->LDS bytes
// per flop by a quarter and the LDS->register bytes per flop by a quarter as well (a
// 128 x 64 wave tile reuses every fragment more).  The price is the register budget: with
// three fp32 accumulator tiles live (the Strassen / Winograd recombination) a wave holds
// 384 of its 512 registers in accumulators, so the main loop stages nothing in registers --
// operand tiles go global -> LDS by DMA, fragments LDS -> MFMA.
//
// Pipeline: k-steps of 64, a ring of three LDS stages (48 KiB each), loads issued two full
// steps ahead of their use, one workgroup barrier per step.  The ring runs across segment
// (product) boundaries without draining.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sthip_kernel2.hpp"

namespace sthip {

constexpr int kThreads3 = 256;
constexpr int kBM3 = 256, kBN3 = 128, kBK3 = 64;
constexpr int kStages3 = 3;
constexpr int kATile3 = kBM3 * kBK3 * 2;                 // 32 KiB
constexpr int kBTile3 = kBN3 * kBK3 * 2;                 // 16 KiB
constexpr int kStageBytes3 = kATile3 + kBTile3;          // 48 KiB
constexpr int kSmemBytes3 = kStages3 * kStageBytes3;     // 144 KiB

template <int N> __device__ __forceinline__ void wait_vmcnt_imm() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

// A tile (k-contiguous): 256 rows x 8 chunks of 16 bytes, i.e. whole 128-byte lines per row
// (half-line requests cost the L2 a quarter of its delivery rate); the load that fills rows
// R..R+7 has lane L fetch row R + L/8, chunk (L%8) ^ ((row/2)%8).  B tile, k-contiguous: the
// same with 128 rows.  B tile, n-contiguous: 64 k-rows x 16 chunks; the load that fills
// k-rows 4j..4j+3 has lane L fetch k-row 4j + L/16, chunk (L%16) ^ ((k%4)*4).
template <bool B_KC>
struct Loader3 {
    const char* a_base; const char* b_base;   // uniform: this wave's first load of the next step
    int64_t a_row_bytes, b_row_bytes;         // uniform: distance between consecutive loads of the wave
    int64_t a_step_bytes, b_step_bytes;       // uniform: advance per k-step
    uint32_t a_voff[2], b_voff[2];            // per lane: offsets for even / odd loads
    int seg, kt, total_seg, KT;
    int batch, tile_m, tile_n, wave;
    const Gemm2Params* P;

    __device__ __forceinline__ void point_at_segment() {
        const Seg2& s = P->seg[seg];
        const int lane = threadIdx.x & 63;
        const char* a = reinterpret_cast<const char*>(s.a) + (int64_t)batch * s.a_bs * 2;
        const char* b = reinterpret_cast<const char*>(s.b) + (int64_t)batch * s.b_bs * 2;
        // k-contiguous tiles: rows 8 i + L/8 of the wave's share; (row/2)%8 = 4 (i%2) + L/16
        const int chunk0 = (lane & 7) ^ (lane >> 4);
        a_base = a + (int64_t)(tile_m + wave * 64) * s.a_ld * 2;     // 8 loads of 8 rows
        a_row_bytes = 8 * s.a_ld * 2;
        a_step_bytes = kBK3 * 2;
        a_voff[0] = (uint32_t)(((lane >> 3) * s.a_ld + chunk0 * 8) * 2);
        a_voff[1] = (uint32_t)(((lane >> 3) * s.a_ld + (chunk0 ^ 4) * 8) * 2);
        if constexpr (B_KC) {                                         // 4 loads of 8 rows
            b_base = b + (int64_t)(tile_n + wave * 32) * s.b_ld * 2;
            b_row_bytes = 8 * s.b_ld * 2;
            b_step_bytes = kBK3 * 2;
            b_voff[0] = (uint32_t)(((lane >> 3) * s.b_ld + chunk0 * 8) * 2);
            b_voff[1] = (uint32_t)(((lane >> 3) * s.b_ld + (chunk0 ^ 4) * 8) * 2);
        } else {                                                      // 4 loads of 4 k-rows; k%4 = L/16
            const int chunk = (lane & 15) ^ ((lane >> 4) << 2);
            b_base = b + ((int64_t)(wave * 16) * s.b_ld + tile_n) * 2;
            b_row_bytes = 4 * s.b_ld * 2;
            b_step_bytes = (int64_t)kBK3 * s.b_ld * 2;
            b_voff[0] = b_voff[1] = (uint32_t)(((lane >> 4) * s.b_ld + chunk * 8) * 2);
        }
    }

    // The twelve loads of one k-step (8 for A, 4 for B), then move the cursor on.
    __device__ __forceinline__ void issue(uint32_t stage_addr) {
        const uint32_t sa = stage_addr + wave * 8192, sb = stage_addr + kATile3 + wave * 4096;
#pragma unroll
        for (int i = 0; i < 8; ++i) lds_dma16(a_base + i * a_row_bytes, a_voff[i & 1], sa + i * 1024);
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

// 16 bytes of MFMA operand: rows sub..sub+31 of a tile, k-group kg (0..3) of a 64-k stage.
template <bool KC>
__device__ __forceinline__ u32x4 read_frag3(const char* tile, int sub, int kg) {
    return read_frag2<KC>(tile, sub, kg);   // same 128-byte-row / 256-byte-k-row layouts as the 128 x 128 kernel
}

struct Acc3 {   // one 128 x 64 wave tile = 4 x 2 MFMA tiles
    f32x16 t[4][2];
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) t[i][j][e] = 0.f;
    }
    __device__ __forceinline__ void add(const Acc3& o) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) t[i][j] += o.t[i][j];
    }
    __device__ __forceinline__ void sub(const Acc3& o) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) t[i][j] -= o.t[i][j];
    }
    __device__ __forceinline__ void negate() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) t[i][j] = -t[i][j];
    }
};

template <class T, bool B_KC>
struct Pipe3 {
    Loader3<B_KC> ld;
    char* smem;
    uint32_t smem_addr;
    int g, total;
    int wm, wn;
    u32x4 fa[2][4], fb[2][2];   // [buffer][sub-tile]

    int slot;          // ring slot of the step being computed

    __device__ __forceinline__ static int next_slot(int x) { return x + 1 == kStages3 ? 0 : x + 1; }
    __device__ __forceinline__ static int prev_slot(int x) { return x == 0 ? kStages3 - 1 : x - 1; }

    __device__ __forceinline__ void read_frags(int buf, int sl, int kg) {
        const char* s = smem + sl * kStageBytes3;
        // B first: both B fragments feed the first two MFMAs of the k-group, A fragment i only
        // MFMAs 2i and 2i+1, so this order gives every read the longest head start.
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[buf][j] = read_frag3<B_KC>(s + kATile3, wn + j * 32, kg);
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[buf][i] = read_frag3<true>(s, wm + i * 32, kg);
    }

    __device__ __forceinline__ void start() {
        g = 0;
        slot = 0;
        int issued = 0;
#pragma unroll
        for (int st = 0; st < kStages3; ++st)
            if (!ld.done()) { ld.issue(smem_addr + st * kStageBytes3); ++issued; }
        // step 0 has landed once at most the younger batches (12 loads each) are in flight
        if (issued >= 3) wait_vmcnt_imm<24>(); else if (issued == 2) wait_vmcnt_imm<12>(); else wait_vmcnt_imm<0>();
        __syncthreads();
        read_frags(0, 0, 0);
    }

    // One segment: KT steps of four k-groups each, accumulating into acc.
    //
    // The one barrier of a step sits just before the first fragments of the next step are
    // read.  By then every wave has read all fragments of the current step out of LDS, so the
    // current slot can be refilled at once with the step three ahead: a ring of three stages
    // gives every load two full steps to arrive.
    __device__ __forceinline__ void run(Acc3& acc, int KT) {
        for (int kt = 0; kt < KT; ++kt, ++g) {
#pragma unroll
            for (int kg = 0; kg < 4; ++kg) {
                const int nb = (kg + 1) & 1, cb = kg & 1;
                if (kg < 3) {
                    read_frags(nb, slot, kg + 1);
                } else {
                    const int ahead = total - 1 - g;   // steps after this one
                    // in flight: step g+1 (needed now) and step g+2
                    if (ahead >= 2) wait_vmcnt_imm<12>(); else wait_vmcnt_imm<0>();
                    __syncthreads();
                    if (!ld.done()) ld.issue(smem_addr + slot * kStageBytes3);
                    if (ahead > 0) read_frags(nb, next_slot(slot), 0);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        mfma_step<T>(acc.t[i][j], fa[cb][i], fb[cb][j]);
                    }
                // Pin the software pipeline: the fragment reads of the next k-group are spread one
                // per MFMA of this k-group, so their LDS latency hides behind matrix-core time
                // instead of being sunk next to their first use.
#pragma unroll
                for (int m = 0; m < 8; ++m) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            slot = next_slot(slot);
        }
    }
};

// Store (or accumulate into) this wave's 128 x 64 part of C block `quad`; (row, col) is the
// wave tile's origin inside the block.  Lane l of MFMA tile (i, j) holds m = l%32 and, in
// registers 4g..4g+3, n = 8g + 4*(l/32) + 0..3, so every store is 8 (or 16) contiguous bytes.
// With PLUS the stored value is acc + plus, formed on the fly (neither tile is modified).
template <class T, bool PLUS = false>
__device__ __forceinline__ void store_tile3(const Acc3& acc, const Gemm2Params& P, char* Cb, int quad, int row, int col,
                                            const Acc3& plus) {
    const int lane = threadIdx.x & 63;
    const int esz = P.out_f32 ? 4 : 2;
    const int m0 = (quad >> 1) * P.Mh + row + (lane & 31);
    const int n0 = (quad & 1) * P.Nh + col + 4 * (lane >> 5);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = PLUS ? acc.t[i][j][4 * g + e] + plus.t[i][j][4 * g + e] : acc.t[i][j][4 * g + e];
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
            }
        }
    }
}

// Parking: with two accumulator tiles in registers (256 AGPRs) the main loops need no
// spills and no register shuffling; the third tile the Strassen recombination needs is
// kept in a private scratch slab (128 KiB per workgroup, written once and read once per
// parking, fully coalesced: lane-major groups of four registers).
__device__ __forceinline__ void park_store(const Acc3& acc, float* slab) {
    f32x4* p = reinterpret_cast<f32x4*>(slab) + threadIdx.x;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 v = {acc.t[i][j][4 * g], acc.t[i][j][4 * g + 1], acc.t[i][j][4 * g + 2], acc.t[i][j][4 * g + 3]};
                p[((i * 2 + j) * 4 + g) * kThreads3] = v;
            }
}
__device__ __forceinline__ void park_add(Acc3& acc, const float* slab) {
    const f32x4* p = reinterpret_cast<const f32x4*>(slab) + threadIdx.x;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 v = p[((i * 2 + j) * 4 + g) * kThreads3];
#pragma unroll
                for (int e = 0; e < 4; ++e) acc.t[i][j][4 * g + e] += v[e];
            }
}

template <class T, int ALGO, bool B_KC>
__global__ void __launch_bounds__(kThreads3) gemm3_kernel(const Gemm2Params P) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    GemmParams tp;
    tp.tiles_m = P.tiles_m; tp.tiles_n = P.tiles_n; tp.group_m = P.group_m;
    int tm, tn;
    tile_coords(tp, tm, tn);
    const int tile_m = tm * kBM3, tile_n = tn * kBN3;
    const int batch = blockIdx.y;
    char* Cb = reinterpret_cast<char*>(P.C) + (int64_t)batch * P.c_bs * (P.out_f32 ? 4 : 2);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int NSEG = ALGO == ALGO_CLASSIC ? 1 : 7;
    const int KT = P.Kh / kBK3;

    Pipe3<T, B_KC> pipe;
    pipe.smem = smem;
    pipe.smem_addr = (uint32_t)(uintptr_t)(lptr_t)smem;
    pipe.wm = (wave >> 1) * 128;
    pipe.wn = (wave & 1) * 64;
    pipe.total = NSEG * KT;
    pipe.ld.P = &P;
    pipe.ld.wave = wave;
    pipe.ld.seg = 0; pipe.ld.kt = 0; pipe.ld.total_seg = NSEG; pipe.ld.KT = KT;
    pipe.ld.batch = batch; pipe.ld.tile_m = tile_m; pipe.ld.tile_n = tile_n;
    pipe.ld.point_at_segment();
    pipe.start();

#define EMIT3(acc, quad) store_tile3<T, false>(acc, P, Cb, quad, tile_m + pipe.wm, tile_n + pipe.wn, acc)
    enum { Q11 = 0, Q12 = 1, Q21 = 2, Q22 = 3 };
    if constexpr (ALGO == ALGO_CLASSIC) {
        Acc3 x;
        x.zero();
        pipe.run(x, KT);
        EMIT3(x, Q11);
    } else if constexpr (ALGO == ALGO_STRASSEN) {
        // segment order M3 M6 M5 M7 M1 M2 M4; two tiles in registers, one parked
        float* slab = P.park + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * (kBM3 * kBN3);
        Acc3 x, y;
        x.zero();
        pipe.run(x, KT);       // M3
        y = x;
        pipe.run(y, KT);       // + M6: y = M3 + M6, the C22 chain
        park_store(y, slab);
        y.zero();
        pipe.run(y, KT);       // M5
        x.add(y);
        EMIT3(x, Q12);         // C12 = M3 + M5
        y.negate();            // C11 chain starts at -M5
        pipe.run(y, KT);       // + M7
        x.zero();
        pipe.run(x, KT);       // M1
        y.add(x);              // C11 chain = M1 - M5 + M7
        park_add(x, slab);     // x = M1 + (M3 + M6), the C22 chain again
        park_store(y, slab);
        y.zero();
        pipe.run(y, KT);       // M2: starts the C21 chain
        x.sub(y);
        EMIT3(x, Q22);         // C22 = M1 - M2 + M3 + M6
        x.zero();
        pipe.run(x, KT);       // M4
        y.add(x);
        EMIT3(y, Q21);         // C21 = M2 + M4
        park_add(x, slab);
        EMIT3(x, Q11);         // C11 = M1 + M4 - M5 + M7
    } else {
        // segment order P1 P2 P6 P7 P5 P3 (-P4); two tiles in registers, U2 parked once
        float* slab = P.park + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * (kBM3 * kBN3);
        Acc3 x, y;
        x.zero();
        pipe.run(x, KT);       // P1
        y = x;
        pipe.run(x, KT);       // + P2
        EMIT3(x, Q11);         // C11 = P1 + P2
        pipe.run(y, KT);       // + P6 -> U2
        park_store(y, slab);
        pipe.run(y, KT);       // + P7 -> U3
        x.zero();
        pipe.run(x, KT);       // P5
        store_tile3<T, true>(x, P, Cb, Q22, tile_m + pipe.wm, tile_n + pipe.wn, y);   // C22 = U3 + P5
        park_add(x, slab);     // U4 = U2 + P5
        pipe.run(x, KT);       // + P3
        EMIT3(x, Q12);         // C12 = U4 + P3
        pipe.run(y, KT);       // + A22 (-T4)
        EMIT3(y, Q21);         // C21 = U3 - P4
    }
#undef EMIT3
}

}  // namespace sthip
