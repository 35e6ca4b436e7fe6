// 256 x 256-tile pipelined grouped-GEMM kernel for gfx950: eight waves (two per SIMD) of
// 128 x 64 each, 16-bit or fp32 operands, A contiguous along k.
//
// The L2 -> LDS path, not the matrix cores, limits the smaller-tile kernels: bytes moved per
// flop go with (1/BM + 1/BN).  A 256 x 256 tile moves two thirds of what 256 x 128 moves, but
// its fp32 accumulators then fill half of the CU's registers, so no Strassen / Winograd chain
// can stay in registers beside them.  (Parking the chains in per-workgroup fp32 slabs was built
// and measured: every CU parks 256 KiB at the same moment, nine to eighteen times per tile,
// and the kernel ran a third slower than the 256 x 128 one.)  So this kernel only ever runs
// plain products: one launch covers `nprod` independent products of equal shape (the seven
// products of a level, each with its own operand pair and its own output matrix), product-major,
// so that the chip works through one product at a time and each behaves like a classical GEMM.
// The recombination of the seven outputs is a separate elementwise pass.
//
// Two waves per SIMD, not one with a 128 x 128 tile: a wave issues in order, and with a single
// wave per SIMD every LDS read and every direct-to-LDS load was measured to cost its own issue
// time on top of the matrix instructions (the costs added up instead of overlapping); the second
// wave fills those gaps (+3.5 % at 8192^3 bf16, +2.5 % fp32) at the price of half as many more
// fragment reads.
//
// Matrix instruction: v_mfma_f32_16x16x32 (a 128 x 64 wave tile is 8 x 4 of them per 32 k); fp32
// operands: v_mfma_f32_16x16x4_f32, four per 16-byte fragment pair.
// Sustained matrix throughput on this card is set by the power limit, and with random operands
// the 16x16x32 form sustains 14 % more than 32x32x16 in a register-only loop (2.08 against 1.82
// PFLOP/s); in this kernel it is worth 1 - 4 %.
//
// Pipeline: k-steps of 64 (whole 128-byte lines per row), two LDS stages of 64 KiB, the
// barrier of a step sits just before the next step's first fragments are read, at which
// point the current stage is free and is refilled with the step two ahead.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sthip_kernel3.hpp"

namespace sthip {

constexpr int kThreads4 = 512;   // eight waves, two per SIMD
constexpr int kBM4 = 256, kBN4 = 256, kBK4 = 64;   // kBK4: 16-bit elements per k-step (128 bytes per row)
constexpr int kRowBytes4 = 128;                     // bytes of one tile row along k, any element type
template <class T> constexpr int es4() { return __is_same(T, float) ? 4 : 2; }     // element size
template <class T> constexpr int bk4() { return kRowBytes4 / es4<T>(); }           // elements per k-step
constexpr int kStages4 = 2;
constexpr int kATile4 = kBM4 * kBK4 * 2;                 // 32 KiB
constexpr int kBTile4 = kBN4 * kBK4 * 2;                 // 32 KiB
constexpr int kStageBytes4 = kATile4 + kBTile4;          // 64 KiB
constexpr int kSmemBytes4 = kStages4 * kStageBytes4;     // 128 KiB
constexpr int kOutStage4 = 4096;                         // per wave: 32 rows x 128 bytes of a 16-bit result on their way out
constexpr int kSmemBytes4p = kSmemBytes4 + 8 * kOutStage4;   // 160 KiB: the stage buffers stay in use while a tile is stored

// Tile `id` of a launch, numbered over (batch entry, product, tile of the product).
// Products of at least 256 tiles: the XCD-aware renumbering works within one product (workgroup x,
// x + 8, ... run on XCD x; ids are renumbered so that an XCD owns a contiguous run of tiles).
// Products of fewer than 256 tiles (several run at once): that numbering would give every XCD eight
// tiles of each of four products.  Instead XCD x takes whole chunks of 32 tiles -- four tile rows
// by eight columns of ONE product, which share their operand panels in that XCD's L2 -- chunk x
// first, then x + 8, ...  Chunks beyond the last full set of eight are numbered the plain way.
__device__ __forceinline__ void map_tile4(const Gemm2Params& P, int id, int& prod, int& batch, int& tm, int& tn) {
    // `z` is zero, but not to the compiler: everything below is then computed where it is needed, once
    // per tile.  Otherwise the dozen values that are the same for every tile are kept in scalar
    // registers across the main loop, which then spills.
    int z = 0;
    asm volatile("" : "+s"(z));
    const int tiles_m = P.tiles_m + z, tiles_n = P.tiles_n + z, tiles = tiles_m * tiles_n;
    const int nprod = (P.nprod > 0 ? P.nprod : 1) + z;
    const int chunks = P.xcd_chunks + z ? (nprod * P.nbatch * tiles / 32) / 8 * 8 : 0;
    int pb;
    if (id < chunks * 32) {
        const int x = id & 7, j = id >> 3;
        const int h = (j >> 5) * 8 + x, per = tiles / 32;
        pb = h / per;
        const int part = h - pb * per, l = j & 31;
        const int t = part * 32 + l;                 // tile of the product, walked four rows at a time
        const int width = 4 * tiles_n, grp = t / width, in = t - grp * width;
        tm = grp * 4 + (in & 3); tn = in >> 2;
    } else {
        const int rest = id - chunks * 32, first = chunks * 32 / tiles;   // whole products before `rest`
        const int pl = rest / tiles;
        GemmParams tp;
        tp.tiles_m = tiles_m; tp.tiles_n = tiles_n; tp.group_m = P.group_m + z;
        tile_coords_in(tp, rest - pl * tiles, tiles, tm, tn);
        pb = first + pl;
    }
    batch = __builtin_amdgcn_readfirstlane(pb / nprod);
    prod = __builtin_amdgcn_readfirstlane(pb - batch * nprod);
    tm = __builtin_amdgcn_readfirstlane(tm);   // uniform by construction; the loader needs its bases in scalar registers
    tn = __builtin_amdgcn_readfirstlane(tn);
}

// A and k-contiguous B: 256 rows x 8 chunks; wave w loads rows 32 w + 8 i + L/8, i = 0..3,
// chunk (L%8) ^ ((row/2)%8).  n-contiguous B: 64 k-rows x 32 chunks (512 bytes); wave w loads
// k-rows 8 w + 2 i + L/32, i = 0..3, chunk (L%32) ^ ((k%4)*4) ^ (((k/8)%2)*2).
// fp32 operands use the same bytes: a k-step is 32 elements, a 16-byte chunk four of them.  The
// n-contiguous fp32 B tile is 32 k-rows x 1024 bytes, one row per load: wave w loads k-rows
// 4 w + i (i = 0..3), and slot s of row k holds chunk s ^ (((k / 4) % 4) * 4), so that the four k-rows a
// fragment read touches (k = 4 g + c, lane group g) fall into different 64-byte bank groups.
// 16-bit operands: the lane offset of load i includes the rows of load i (a_voff[i], b_voff[i]), so that
// issuing a load in the main loop is m0, a wait state and the load (between two writes of the lane mask,
// see Pipe4::run16) and no scalar address arithmetic: a wave issues in order, and a dozen scalar
// instructions and a branch per load held back the matrix instructions behind them (measured: k-step
// 2890 -> 2750 cycles together with the row order of Pipe4::run16).  Lane offsets are 32-bit: 32 rows of
// the operand must span less than 4 GiB (the launcher checks).  fp32 operands keep one offset per load
// parity and add the rows to the base: that kernel has no registers to spare.
template <int ES, bool B_KC>
struct Loader4 {
    static constexpr bool kRowsInLane = ES == 2;
    const char* a_base; const char* b_base;
    int64_t a_row_bytes, b_row_bytes, a_step_bytes, b_step_bytes;
    uint32_t a_voff[kRowsInLane ? 4 : 2], b_voff[kRowsInLane ? 4 : 2];   // load i of the wave (fp32: i % 2)
    int seg, kt, total_seg, KT;
    int batch, tile_m, tile_n, wave;
    int id, stride, total_ids;   // stride > 0: after the KT steps of tile `id` the loader goes on with tile id + stride
    const Gemm2Params* P;

    __device__ __forceinline__ void point_at_segment() {
        const Seg2& s = P->seg[seg];
        const int lane = threadIdx.x & 63;
        const char* a = reinterpret_cast<const char*>(s.a) + (int64_t)batch * s.a_bs * ES;
        const char* b = reinterpret_cast<const char*>(s.b) + (int64_t)batch * s.b_bs * ES;
        const int chunk0 = (lane & 7) ^ (lane >> 4);     // (row/2)%8 = 4 (i%2) + L/16
        a_base = a + (int64_t)(tile_m + wave * 32) * s.a_ld * ES;
        a_row_bytes = 8 * s.a_ld * ES;
        a_step_bytes = kRowBytes4;
        if constexpr (kRowsInLane) {
            const uint32_t row = (uint32_t)(s.a_ld * ES), l8 = (uint32_t)(lane >> 3) * row;
#pragma unroll
            for (int i = 0; i < 4; ++i) a_voff[i] = l8 + 8 * i * row + (chunk0 ^ ((i & 1) << 2)) * 16;
        } else {
            a_voff[0] = (uint32_t)((lane >> 3) * s.a_ld * ES + chunk0 * 16);
            a_voff[1] = (uint32_t)((lane >> 3) * s.a_ld * ES + (chunk0 ^ 4) * 16);
        }
        if constexpr (B_KC) {
            b_base = b + (int64_t)(tile_n + wave * 32) * s.b_ld * ES;
            b_row_bytes = 8 * s.b_ld * ES;
            b_step_bytes = kRowBytes4;
            if constexpr (kRowsInLane) {
                const uint32_t row = (uint32_t)(s.b_ld * ES), l8 = (uint32_t)(lane >> 3) * row;
#pragma unroll
                for (int i = 0; i < 4; ++i) b_voff[i] = l8 + 8 * i * row + (chunk0 ^ ((i & 1) << 2)) * 16;
            } else {
                b_voff[0] = (uint32_t)((lane >> 3) * s.b_ld * ES + chunk0 * 16);
                b_voff[1] = (uint32_t)((lane >> 3) * s.b_ld * ES + (chunk0 ^ 4) * 16);
            }
        } else if constexpr (ES == 4) {
            // k-row of load i: k = 4 w + i, so (k/4)%4 = w % 4
            b_base = b + ((int64_t)(wave * 4) * s.b_ld + tile_n) * 4;
            b_row_bytes = s.b_ld * 4;
            b_step_bytes = (int64_t)kRowBytes4 * s.b_ld;
            b_voff[0] = b_voff[1] = (uint32_t)((lane ^ ((wave & 3) << 2)) * 16);
        } else {
            // k-row of load i: k = 8 w + 2 i + L/32, so k%4 = 2 (i%2) + L/32 and (k/8)%2 = w%2;
            // the chunk stored in slot s of row k is s ^ ((k%4) * 4) ^ (((k/8)%2) * 2)
            const int chunk = (lane & 31) ^ ((lane >> 5) << 2);
            b_base = b + ((int64_t)(wave * 8) * s.b_ld + tile_n) * 2;
            b_row_bytes = 2 * s.b_ld * 2;
            b_step_bytes = (int64_t)kBK4 * s.b_ld * 2;
            const uint32_t row = (uint32_t)(s.b_ld * 2), l32 = (uint32_t)(lane >> 5) * row;
#pragma unroll
            for (int v = 0; v < 4; ++v) b_voff[v] = l32 + 2 * v * row + (chunk ^ ((v & 1) << 3) ^ ((wave & 1) << 1)) * 16;
        }
    }

    // The wave's eight loads of one k-step (4 for A, 4 for B), then move the cursor on.
    __device__ __forceinline__ void issue(uint32_t stage_addr) {
#pragma unroll
        for (int q = 0; q < 8; ++q) issue_one(stage_addr + wave * 4096, q);
        advance();
    }

    // 16-bit main loop: load q under a lane mask (all ones, or zero once the loader has run dry).
    __device__ __forceinline__ void issue_one_masked(uint32_t wave_stage, int q, uint32_t mask) {
        if (q < 4) lds_dma16_km(a_base, a_voff[q], wave_stage, q * 1024, mask);
        else lds_dma16_km(b_base, b_voff[q - 4], wave_stage, kATile4 + (q - 4) * 1024, mask);
    }
    // Load q (0..3 the A tile, 4..7 the B tile) of the next k-step into the stage whose LDS address plus
    // this wave's 4 KiB is wave_stage; advance() after the eighth.
    __device__ __forceinline__ void issue_one(uint32_t wave_stage, int q) {
        if constexpr (kRowsInLane) {
            if (q < 4) lds_dma16_k(a_base, a_voff[q], wave_stage, q * 1024);
            else lds_dma16_k(b_base, b_voff[q - 4], wave_stage, kATile4 + (q - 4) * 1024);
        } else {
            if (q < 4) lds_dma16(a_base + q * a_row_bytes, a_voff[q & 1], wave_stage + q * 1024);
            else {
                const int i = q - 4;
                lds_dma16(b_base + i * b_row_bytes, b_voff[i & 1], wave_stage + kATile4 + i * 1024);
            }
        }
    }
    __device__ __forceinline__ void advance() {
        a_base += a_step_bytes;
        b_base += b_step_bytes;
        if (++kt == KT) {
            kt = 0;
            if (stride > 0) {
                id += stride;
                if (id < total_ids) {
                    int tm, tn;
                    map_tile4(*P, id, seg, batch, tm, tn);
                    tile_m = tm * kBM4; tile_n = tn * kBN4;
                    total_seg = seg + 1;
                    point_at_segment();
                } else seg = total_seg;
            } else if (++seg < total_seg) point_at_segment();
        }
    }

    __device__ __forceinline__ bool done() const { return seg >= total_seg; }
};

// Operand fragments of v_mfma_f32_16x16x32: lane L holds, for row (or column) L % 16 of a
// 16-wide block, the eight k-values 8 (L / 16) .. + 7 of a group of 32.
//
// k-contiguous tile (128-byte rows, 16-byte chunks XOR-swizzled with (row/2)%8): one 16-byte read
// per lane.  A 16-lane group reads 16 rows at one chunk position: rows r, r+1 share a slot but lie
// 128 bytes apart, so the group covers all 64 banks once.
__device__ __forceinline__ u32x4 read_frag16_kc(const char* tile, int sub, int kg) {
    const int lane = threadIdx.x & 63;
    const int row = sub + (lane & 15);
    const int slot = (kg * 4 + (lane >> 4)) ^ ((row >> 1) & 7);
    return *reinterpret_cast<const u32x4*>(tile + row * 128 + slot * 16);
}

// n-contiguous B tile (64 k-rows of 512 bytes): two transposing reads.  In each 16-lane group,
// lane r addresses 4 consecutive n of k-row k0 + r/4 (k0 = 32 kg + 8 group) at n = sub + 4 (r%4);
// the read hands lane i the four k-values k0..k0+3 of column sub + i; the second read does
// k0+4..k0+7.  The slot swizzle flips bit 1 with (k/8)%2 so that groups 0/1 (and 2/3) use
// disjoint banks.
__device__ __forceinline__ u32x4 read_frag16_mc(const char* tile, int sub, int kg) {
    const int lane = threadIdx.x & 63;
    const int l16 = lane & 15, grp = lane >> 4;
    const int k = kg * 32 + grp * 8 + (l16 >> 2);
    const int chunk = (sub >> 3) + ((l16 & 3) >> 1);
    const int slot = chunk ^ (((l16 >> 2) & 3) << 2) ^ ((grp & 1) << 1);
    const char* p = tile + k * 512 + slot * 16 + (l16 & 1) * 8;
    s16x4 lo = lds_read_tr16_b64(p);
    s16x4 hi = lds_read_tr16_b64(p + 4 * 512);
    u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
    u32x4 r = {a[0], a[1], b[0], b[1]};
    return r;
}

// n-contiguous fp32 B tile (32 k-rows of 1024 bytes): component c of the fragment is the element
// at k = 16 kg + 4 g + c (g = lane / 16), column sub + lane % 16 -- the same k a lane's 16-byte
// read of a k-contiguous tile puts into component c.
__device__ __forceinline__ u32x4 read_frag16_mc_f32(const char* tile, int sub, int kg) {
    const int lane = threadIdx.x & 63;
    const int e = sub + (lane & 15), g = lane >> 4;
    const char* p = tile + (kg * 16 + g * 4) * 1024 + (((e >> 2) ^ (g << 2)) * 16) + (e & 3) * 4;
    u32x4 r;
#pragma unroll
    for (int c = 0; c < 4; ++c) r[c] = *reinterpret_cast<const uint32_t*>(p + c * 1024);
    return r;
}

struct Acc4 {   // one 128 x 64 wave tile = 8 x 4 MFMA tiles = 128 registers
    f32x4 t[8][4];
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < 4; ++e) t[i][j][e] = 0.f;
    }
};

template <class T, bool B_KC>
struct Pipe4 {
    Loader4<es4<T>(), B_KC> ld;
    char* smem;
    uint32_t smem_addr;
    int g, total, slot;
    int wm, wn;
    u32x4 fa[2][8], fb[2][4];   // [buffer][16-wide block]: fragments of one group of 32 k

    // The A fragment of 16-wide block r and, for r < 4, the B fragment.
    __device__ __forceinline__ void read_pair(int buf, int sl, int kg, int r) {
        const char* s = smem + sl * kStageBytes4;
        if (r < 4) {
            if constexpr (B_KC) fb[buf][r] = read_frag16_kc(s + kATile4, wn + r * 16, kg);
            else if constexpr (es4<T>() == 4) fb[buf][r] = read_frag16_mc_f32(s + kATile4, wn + r * 16, kg);
            else fb[buf][r] = read_frag16_mc(s + kATile4, wn + r * 16, kg);
        }
        fa[buf][r] = read_frag16_kc(s, wm + r * 16, kg);
    }
    __device__ __forceinline__ void read_frags(int buf, int sl, int kg) {
#pragma unroll
        for (int r = 0; r < 8; ++r) read_pair(buf, sl, kg, r);
    }

    __device__ __forceinline__ void start() {
        g = 0;
        slot = 0;
        ld.issue(smem_addr);
        if (!ld.done()) ld.issue(smem_addr + kStageBytes4);
        if (total >= 2) wait_vmcnt_imm<8>(); else wait_vmcnt_imm<0>();   // step 0 has landed
        __syncthreads();
        read_frags(0, 0, 0);
    }

    __device__ __forceinline__ void run(Acc4& acc, int KT) {
        if constexpr (es4<T>() == 2) run16(acc, KT); else run32(acc, KT);
    }

    // 16-bit operands.  A wave issues in order, and whatever stands between two matrix instructions holds
    // the second one back unless it fits into the 16 cycles the first one occupies the pipe: so the row of
    // four matrix instructions takes its other work in between them, at most three instructions at a time
    // -- the A fragment of the next k-group after the first, the B fragment (first four rows) after the
    // second, one of the wave's eight loads of step g+2 (second k-group only) after the third.  Cycle
    // counters around the rows (timing builds): the rows after the barrier, with the loads, took 185 to 240
    // cycles against 64 of matrix instructions while their scalar address arithmetic and a branch stood in
    // front of the row; a k-step 2890 -> 2750 cycles with this order and the three-instruction loads.
    // What a fragment read costs however it is placed is the return of its data, 1 KiB per read into the
    // register file: about 8 cycles, in which the matrix pipe takes no operands -- 24 reads per wave and
    // k-step, 19 % on top of the matrix instructions for this wave tile.
    // No load has a branch around it: once the loader has run dry (the last two steps of a workgroup's
    // last tile) the loads are issued with no lane enabled, which executes nothing.  More than one load per
    // row costs more than it gains (the memory pipeline takes them slowly: all eight in the first four rows,
    // k-step +3 %); the loop written twice, with and without loads, makes the compiler spill around the
    // tile's store (short tiles 10 % slower).
    __device__ __forceinline__ void run16(Acc4& acc, int KT) {
        for (int kt = 0; kt < KT; ++kt, ++g) {
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) {
                const int nb = kg ^ 1, cb = kg;
                if (kg == 1) {
                    // Every wave has read all fragments of this step: after the barrier its stage is
                    // free for the step two ahead.  Step g+1 (the only load batch in flight) must
                    // have landed before its fragments are read.
                    wait_vmcnt_imm<0>();
                    __syncthreads();
                }
                const uint32_t wave_stage = smem_addr + slot * kStageBytes4 + ld.wave * 4096;
                const uint32_t live = (uint32_t)__builtin_amdgcn_readfirstlane(ld.done() ? 0 : -1);
                // In the last step the "next" fragments are stale data that nobody uses.
                const int nsl = kg == 0 ? slot : slot ^ 1, nkg = kg ^ 1;
                const char* st = smem + nsl * kStageBytes4;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    // boustrophedon: the B fragment carries over between rows
                    auto mm = [&](int jj) { const int j = (i & 1) ? 3 - jj : jj; mfma16_step<T>(acc.t[i][j], fa[cb][i], fb[cb][j]); };
                    mm(0);
                    __builtin_amdgcn_sched_barrier(0);
                    fa[nb][i] = read_frag16_kc(st, wm + i * 16, nkg);
                    __builtin_amdgcn_sched_barrier(0);
                    mm(1);
                    __builtin_amdgcn_sched_barrier(0);
                    if (i < 4) {
                        if constexpr (B_KC) fb[nb][i] = read_frag16_kc(st + kATile4, wn + i * 16, nkg);
                        else fb[nb][i] = read_frag16_mc(st + kATile4, wn + i * 16, nkg);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    mm(2);
                    __builtin_amdgcn_sched_barrier(0);
                    if (kg == 1) {
                        ld.issue_one_masked(wave_stage, i, live);
                        if (i == 7 && !ld.done()) ld.advance();
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    mm(3);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            slot ^= 1;
        }
        // the matrix instructions are opaque to the compiler's hazard checks: let the last results
        // retire before the epilogue reads the accumulators
        asm volatile("s_nop 15\n\ts_nop 15");
    }

    // fp32 operands.
    __device__ __forceinline__ void run32(Acc4& acc, int KT) {
        for (int kt = 0; kt < KT; ++kt, ++g) {
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) {
                const int nb = kg ^ 1, cb = kg;
                if (kg == 1) {
                    wait_vmcnt_imm<0>();
                    __syncthreads();
                }
                // The wave's eight loads of step g+2 go out one per row of matrix instructions.
                const bool issuing = kg == 1 && !ld.done();
                // Fragments of the next k-group come in between the rows of matrix instructions, one
                // A and (first four rows) one B fragment per row: few enough in flight for the LDS
                // counter (4 bits) to tell the old fragments from the new.
                const int nsl = kg == 0 ? slot : slot ^ 1, nkg = kg ^ 1;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (issuing) {
                        ld.issue_one(smem_addr + slot * kStageBytes4 + ld.wave * 4096, i);
                        if (i == 7) ld.advance();
                    }
                    read_pair(nb, nsl, nkg, i);
                    // four matrix instructions per accumulator and k-group: component-major, so
                    // that instructions on one accumulator are four apart
#pragma unroll
                    for (int c = 0; c < 4; ++c)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            mfma16_step_f32(acc.t[i][j], fa[cb][i][c], fb[cb][j][c]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            slot ^= 1;
        }
        asm volatile("s_nop 15\n\ts_nop 15");
    }
};

// The lane index as a value the compiler cannot see through: everything a store routine derives from
// it is then computed where the routine runs.  (Otherwise the per-lane addresses of the stores, being
// the same for every tile a workgroup computes, are hoisted out of the tile loop and held in registers
// across the main loop, which has none to spare: eight spills per k-step.)
__device__ __forceinline__ int opaque_lane4() {
    int lane = threadIdx.x & 63;
    asm volatile("" : "+v"(lane));
    return lane;
}

// Lane l of MFMA tile (i, j) holds m = 16 i + l % 16 and n = 16 j + 4 (l / 16) + 0..3.
template <class T>
__device__ __forceinline__ void store_tile4(const Acc4& acc, const Gemm2Params& P, char* Cb, int quad, int row, int col) {
    const int lane = opaque_lane4();
    const int esz = P.out_f32 ? 4 : 2;
    const int m0 = (quad >> 1) * P.Mh + row + (lane & 15);
    const int n0 = (quad & 1) * P.Nh + col + 4 * (lane >> 4);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc.t[i][j][e];
            char* dst = Cb + ((int64_t)(m0 + i * 16) * P.c_rs + (n0 + j * 16)) * esz;
            if (P.out_f32) {
                f32x4* d = reinterpret_cast<f32x4*>(dst);
                f32x4 o = {v[0], v[1], v[2], v[3]};
                if (P.accumulate) { o += *d; *d = o; }
                else store_hinted(o, d, P.c_stream);
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
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The 16-bit, non-accumulating store, staged through LDS so that every store instruction writes
// eight rows x 128 contiguous bytes (16 bytes per lane) instead of sixteen rows x 32 bytes: with
// all workgroups of a round storing at once, the partial-line pattern of the MFMA layout costs
// about twice the time.  Each wave uses its own 16 KiB of the (now idle) stage buffers: row r of
// its 128 x 64 tile at r * 128, the 8-byte chunk c of a row at (c ^ 2 ((r / 2) % 8)) * 8, which
// spreads the sixteen rows a write instruction touches over all banks and keeps 16-byte chunks
// whole for the read back.  The caller has synchronised the workgroup.
template <class T>
__device__ __forceinline__ void store_tile4_lds(const Acc4& acc, const Gemm2Params& P, char* Cb, char* smem,
                                                int wave, int row, int col) {
    const int lane = opaque_lane4();
    const int l16 = lane & 15, q = lane >> 4;
    char* w = smem + wave * 16384;
    uint32_t waddr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) waddr[j] = l16 * 128 + (((4 * j + q) ^ (2 * (l16 >> 1))) * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u32x2 o;
            if constexpr (__is_same(T, bf16_t)) { o[0] = pack_bf16(acc.t[i][j][0], acc.t[i][j][1]); o[1] = pack_bf16(acc.t[i][j][2], acc.t[i][j][3]); }
            else { o[0] = pack_f16(acc.t[i][j][0], acc.t[i][j][1]); o[1] = pack_f16(acc.t[i][j][2], acc.t[i][j][3]); }
            *reinterpret_cast<u32x2*>(w + i * 2048 + waddr[j]) = o;
        }
    }
    wave_exchange_point();
    // read back: lane -> row 8 r + lane / 8, 16-byte chunk lane % 8; the same wave wrote it, LDS keeps order
    const int r8 = lane >> 3, c16 = lane & 7;
    char* dst = Cb + ((int64_t)(row + r8) * P.c_rs + (col + 8 * c16)) * 2;
    const int64_t step = (int64_t)8 * P.c_rs * 2;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int rr = ((8 * r + r8) >> 1) & 7;
        const u32x4 v = *reinterpret_cast<const u32x4*>(w + (8 * r + r8) * 128 + ((c16 ^ rr) * 16));
        // streaming store on large problems: the tile is not read again by this launch, and a round of
        // tiles is as large as the L2s, which hold the operand panels the neighbours are re-reading
        // (measured: -1 % at 8192^3, -3 % at 16384^2 x 4096); on problems whose products fit the
        // memory-side cache the recombination pass finds them there with a plain store (-3 % at 4096^3)
        store_hinted(v, reinterpret_cast<u32x4*>(dst + r * step), P.c_stream);
    }
}

// The same for an fp32 result, in two halves of 64 rows (a wave's 128 x 64 fp32 tile is twice its
// 16 KiB of LDS): row r of a half at r * 256, the 16-byte chunk c of a row at (c ^ (r % 16)) * 16.
// Every store instruction then writes four rows x 256 contiguous bytes.
__device__ __forceinline__ void store_tile4_lds_f32(const Acc4& acc, const Gemm2Params& P, char* Cb, char* smem,
                                                    int wave, int row, int col) {
    const int lane = opaque_lane4();
    const int l16 = lane & 15, q = lane >> 4;
    char* w = smem + wave * 16384;
    float* dst = reinterpret_cast<float*>(Cb) + (int64_t)(row + q) * P.c_rs + (col + 4 * l16);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int ii = 0; ii < 4; ++ii)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<f32x4*>(w + (16 * ii + l16) * 256 + (((4 * j + q) ^ l16) * 16)) = acc.t[4 * h + ii][j];
        wave_exchange_point();
        // read back: lane -> row 4 r + lane / 16 of the half, chunk lane % 16; same wave, LDS keeps order
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int rl = 4 * r + q;
            const f32x4 v = *reinterpret_cast<const f32x4*>(w + rl * 256 + ((l16 ^ (rl & 15)) * 16));
            store_hinted(v, reinterpret_cast<f32x4*>(dst + (int64_t)(64 * h + 4 * r) * P.c_rs), P.c_stream);
        }
        wave_exchange_point();
    }
}

// The same 16-bit store for a workgroup that goes on to another tile: the stage buffers already
// hold (or are receiving) the next tile's first k-steps, so each wave stages its 128 x 64 tile in
// four passes of 32 rows through 4 KiB of its own beyond the stage buffers.  Row r of a pass at
// r * 128, the 8-byte chunk c of a row at (c ^ 2 ((r / 2) % 8)) * 8 as above; the wave reads back
// what it wrote itself (LDS keeps a wave's accesses in order), so no barrier is involved.
template <class T>
__device__ __forceinline__ void store_tile4_own(const Acc4& acc, const Gemm2Params& P, char* Cb, char* out_stage,
                                                int wave, int row, int col) {
    const int lane = opaque_lane4();
    const int l16 = lane & 15, q = lane >> 4;
    char* w = out_stage + wave * kOutStage4;
    uint32_t waddr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) waddr[j] = l16 * 128 + (((4 * j + q) ^ (2 * (l16 >> 1))) * 8);
    const int r8 = lane >> 3, c16 = lane & 7;
    char* dst = Cb + ((int64_t)(row + r8) * P.c_rs + (col + 8 * c16)) * 2;
    const int64_t step = (int64_t)8 * P.c_rs * 2;
#pragma unroll
    for (int h = 0; h < 4; ++h) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) {
            const int i = 2 * h + ii;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32x2 o;
                if constexpr (__is_same(T, bf16_t)) { o[0] = pack_bf16(acc.t[i][j][0], acc.t[i][j][1]); o[1] = pack_bf16(acc.t[i][j][2], acc.t[i][j][3]); }
                else { o[0] = pack_f16(acc.t[i][j][0], acc.t[i][j][1]); o[1] = pack_f16(acc.t[i][j][2], acc.t[i][j][3]); }
                *reinterpret_cast<u32x2*>(w + ii * 2048 + waddr[j]) = o;
            }
        }
        wave_exchange_point();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int rr = ((8 * r + r8) >> 1) & 7;
            const u32x4 v = *reinterpret_cast<const u32x4*>(w + (8 * r + r8) * 128 + ((c16 ^ rr) * 16));
            store_hinted(v, reinterpret_cast<u32x4*>(dst + (4 * h + r) * step), P.c_stream);
        }
        wave_exchange_point();
    }
}

// Set-up shared by the two kernels below: the pipeline of workgroup blockIdx.x, pointed at its first tile.
template <class T, bool B_KC>
__device__ __forceinline__ void begin4(Pipe4<T, B_KC>& pipe, const Gemm2Params& P, char* smem, int wave, int KT,
                                       int id, int stride, int total, int& prod, int& batch, int& tm, int& tn) {
    map_tile4(P, id, prod, batch, tm, tn);
    pipe.smem = smem;
    pipe.smem_addr = (uint32_t)(uintptr_t)(lptr_t)smem;
    pipe.wm = (wave >> 2) * 128;
    pipe.wn = (wave & 3) * 64;
    pipe.total = KT * ((total - 1 - id) / stride + 1);
    pipe.ld.P = &P;
    pipe.ld.wave = wave;
    pipe.ld.seg = prod; pipe.ld.kt = 0; pipe.ld.total_seg = prod + 1; pipe.ld.KT = KT;
    pipe.ld.batch = batch; pipe.ld.tile_m = tm * kBM4; pipe.ld.tile_n = tn * kBN4;
    pipe.ld.id = id; pipe.ld.stride = stride; pipe.ld.total_ids = total;
    pipe.ld.point_at_segment();
    pipe.start();
}

// One tile per workgroup (blockIdx.x = tile id, see map_tile4), any kind of result.
template <class T, bool B_KC>
__global__ void __launch_bounds__(kThreads4) gemm4_kernel(const Gemm2Params P) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int total = P.tiles_m * P.tiles_n * (P.nprod > 0 ? P.nprod : 1) * P.nbatch;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int KT = P.Kh / bk4<T>();
    const int id = __builtin_amdgcn_readfirstlane((int)blockIdx.x);
    int prod, batch, tm, tn;
    Pipe4<T, B_KC> pipe;
    begin4<T, B_KC>(pipe, P, smem, wave, KT, id, total, total, prod, batch, tm, tn);
    const int tile_m = tm * kBM4, tile_n = tn * kBN4;
    char* Cb = reinterpret_cast<char*>(P.C) + ((int64_t)batch * P.c_bs + (int64_t)prod * P.c_ps) * (P.out_f32 ? 4 : 2);
    Acc4 r;
    r.zero();
    pipe.run(r, KT);
    if (P.c_wide && !P.out_f32 && !P.accumulate) {
        __syncthreads();   // every wave has read its last fragments: the stage buffers are free
        store_tile4_lds<T>(r, P, Cb, smem, wave, tile_m + pipe.wm, tile_n + pipe.wn);
    } else if (P.out_f32 && !P.accumulate) {
        __syncthreads();
        store_tile4_lds_f32(r, P, Cb, smem, wave, tile_m + pipe.wm, tile_n + pipe.wn);
    } else {
        store_tile4<T>(r, P, Cb, 0, tile_m + pipe.wm, tile_n + pipe.wn);
    }
}

// Fewer workgroups than tiles (one per CU): workgroup b computes tiles b, b + gridDim.x, ... as ONE
// software pipeline.  The loader runs on into the next tile, whose first k-steps are in flight
// while this tile's last ones are multiplied and while its result is stored, so that a tile costs
// its k-steps and a store, not a dispatch, a prologue and a drain as well.  16-bit results with
// 16-byte aligned rows, not accumulating (the launcher sees to it).
template <class T, bool B_KC>
__global__ void __launch_bounds__(kThreads4) gemm4p_kernel(const Gemm2Params P) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const int total = P.tiles_m * P.tiles_n * (P.nprod > 0 ? P.nprod : 1) * P.nbatch;
    const int stride = (int)gridDim.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int KT = P.Kh / bk4<T>();
    int id = __builtin_amdgcn_readfirstlane((int)blockIdx.x);
    int prod, batch, tm, tn;
    Pipe4<T, B_KC> pipe;
    begin4<T, B_KC>(pipe, P, smem, wave, KT, id, stride, total, prod, batch, tm, tn);
    for (;;) {
        const int tile_m = tm * kBM4, tile_n = tn * kBN4;
        char* Cb = reinterpret_cast<char*>(P.C) + ((int64_t)batch * P.c_bs + (int64_t)prod * P.c_ps) * 2;
        Acc4 r;
        r.zero();
        pipe.run(r, KT);
        if (id + stride >= total) {
            __syncthreads();   // every wave has read its last fragments: the stage buffers are free
            store_tile4_lds<T>(r, P, Cb, smem, wave, tile_m + pipe.wm, tile_n + pipe.wn);
            break;
        }
        store_tile4_own<T>(r, P, Cb, smem + kSmemBytes4, wave, tile_m + pipe.wm, tile_n + pipe.wn);
        id += stride;
        map_tile4(P, id, prod, batch, tm, tn);
        // The first fragments of the next tile were read before the store; reading them again here
        // means they need not stay in registers across the store.
        pipe.read_frags(0, pipe.slot, 0);
        // Nothing the compiler knows of may be outstanding when the main loop starts again: it guards
        // the data registers of the stores above until they have completed, with vmcnt waits INSIDE
        // the loop, where a wait also counts the direct-to-LDS loads it does not know of and drains
        // them at every k-step (measured: +20 %).  The empty statements keep the stores before the wait.
        asm volatile("" ::: "memory");
        wait_vmcnt_imm<0>();
        asm volatile("" ::: "memory");
    }
}

}  // namespace sthip
