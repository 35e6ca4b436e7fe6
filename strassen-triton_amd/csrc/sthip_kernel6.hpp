// 64 x 64-tile grouped fp32 kernel for gfx950 with the quadrant pre-additions fused into the
// operand loads: the small-matrix form of one Strassen level.
//
// Why.  At 1024^3 .. 2048^3 fp32 the seven half-size products have 16 .. 64 tiles of 128 x 128
// each: too few for 256 CUs, and three launches (sums, products, recombination) of a few
// microseconds each weigh as much as the arithmetic.  Here `nprod` products run side by side on
// 64 x 64 tiles (7 x 64 = 448 workgroups at 1024^3), each operand is either a block read in place
// or the sum / difference of two blocks formed in registers on the way from global memory to LDS
// (one fp32 add per element, formed once per tile -- cheap next to the fp32 matrix instructions,
// unlike the 16-bit case), and the products leave as dense fp32 matrices for the recombination
// pass.  Nothing is rounded that the three-launch form does not round: the sums are the same single
// fp32 additions.
//
// Tile: 64 x 64 x 32, four waves of 32 x 32 (2 x 2 blocks of v_mfma_f32_16x16x4_f32, four
// independent accumulators per wave).  A is contiguous along k; B along n or along k.  Loads are
// 16 bytes per lane into registers two k-steps ahead (two register sets, the k loop is unrolled by
// two), added, and written to a double-buffered LDS stage with the 16-byte XOR swizzles of the
// large-tile kernel, so fragment reads are conflict free.  32 KiB of LDS and few registers: several
// workgroups share a CU.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sthip_kernel3.hpp"

namespace sthip {

constexpr int kThreads6 = 256;
constexpr int kBM6 = 64, kBN6 = 64, kBK6 = 32;
constexpr int kTileBytes6 = kBM6 * kBK6 * 4;       // 8 KiB per operand tile
constexpr int kStageBytes6 = 2 * kTileBytes6;      // 16 KiB
constexpr int kMaxProd6 = 7;

// One operand of a product: block p0, or p0 + sign * p1 (sign = +1 / -1; 0: p0 alone).
struct Op6 {
    const float* p0; const float* p1;
    int64_t ld;        // stride of the non-contiguous index, elements (both blocks)
    int sign, pad;
};

struct Gemm6Params {
    Op6 a[kMaxProd6], b[kMaxProd6];
    float* C;              // product q is written to C + q * c_ps, row-major with row stride c_rs
    int64_t c_rs, c_ps;
    int Kh, tiles_m, tiles_n, nprod;
    int accumulate;        // C += product (plain products only)
};

__device__ __forceinline__ f32x4 combine6(f32x4 x, f32x4 y, int sign) {
    return sign > 0 ? x + y : x - y;
}

// The workgroup's whole job.  A_SUM / B_SUM: the operand is p0 + sign * p1 (else p0 alone); they are
// template parameters, chosen by a workgroup-uniform switch in the kernel, so that the main loop has
// no branch: with a branch around the second load the compiler waits for every load where it is
// issued, and nothing is in flight during the matrix instructions.
template <bool B_KC, bool A_SUM, bool B_SUM>
__device__ __forceinline__ void run6(const Gemm6Params& P, char* smem, int prod, int tile_m, int tile_n) {
    const Op6& oa = P.a[prod];
    const Op6& ob = P.b[prod];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    const int KT = P.Kh / kBK6;

    // this thread's two 16-byte chunks of each operand tile: global element offset and LDS byte offset
    int64_t ga[2], gb[2];
    int la[2], lb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int q = tid + kThreads6 * i;
        {   // A: 64 rows x 8 chunks, chunk c of row r in slot c ^ ((r / 2) % 8)
            const int r = q >> 3, c = q & 7;
            ga[i] = (int64_t)(tile_m + r) * oa.ld + 4 * c;
            la[i] = r * 128 + ((c ^ ((r >> 1) & 7)) << 4);
        }
        if constexpr (B_KC) {
            const int r = q >> 3, c = q & 7;
            gb[i] = (int64_t)(tile_n + r) * ob.ld + 4 * c;
            lb[i] = kTileBytes6 + r * 128 + ((c ^ ((r >> 1) & 7)) << 4);
        } else {
            // B: 32 k-rows x 16 chunks, chunk c of row k in slot c ^ (((k / 4) % 4) * 4)
            const int k = q >> 4, c = q & 15;
            gb[i] = (int64_t)k * ob.ld + tile_n + 4 * c;
            lb[i] = kTileBytes6 + k * 256 + ((c ^ (((k >> 2) & 3) << 2)) << 4);
        }
    }
    const int64_t a_step = kBK6, b_step = B_KC ? (int64_t)kBK6 : (int64_t)kBK6 * ob.ld;
    const int a_sign = oa.sign, b_sign = ob.sign;

    // [register set][chunk]: the first block's values and, for a sum, the second block's; the sum is
    // formed when the set is written to LDS, two k-steps after the loads went out.  The loads are
    // inline assembly with hand-placed waits: left to the compiler, every write to LDS waits for all
    // outstanding loads (vmcnt(0)), the set just issued included.
    constexpr int kLoadsPerSet = 4 + (A_SUM ? 2 : 0) + (B_SUM ? 2 : 0);
    f32x4 ra[2][2], rb[2][2], ra1[2][2], rb1[2][2];
    auto fetch = [&](int set, int step) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int64_t o = ga[i] + step * a_step;
            gload16_6(ra[set][i], oa.p0 + o);
            if constexpr (A_SUM) gload16_6(ra1[set][i], oa.p1 + o);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int64_t o = gb[i] + step * b_step;
            gload16_6(rb[set][i], ob.p0 + o);
            if constexpr (B_SUM) gload16_6(rb1[set][i], ob.p1 + o);
        }
    };
    // the older of the two sets in flight has landed; the ties keep every use of it behind the wait
    auto landed = [&](int set) {
        wait_vmcnt_imm<kLoadsPerSet>();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            tie6(ra[set][i]); tie6(rb[set][i]);
            if constexpr (A_SUM) tie6(ra1[set][i]);
            if constexpr (B_SUM) tie6(rb1[set][i]);
        }
    };
    auto stage = [&](int set, int buf) {
        char* s = smem + buf * kStageBytes6;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            f32x4 x = ra[set][i], y = rb[set][i];
            if constexpr (A_SUM) x = combine6(x, ra1[set][i], a_sign);
            if constexpr (B_SUM) y = combine6(y, rb1[set][i], b_sign);
            *reinterpret_cast<f32x4*>(s + la[i]) = x;
            *reinterpret_cast<f32x4*>(s + lb[i]) = y;
        }
    };

    f32x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int l16 = lane & 15, g = lane >> 4;
    // Fragments of one group of 16 k: component c is the element at k = 16 kg + 4 g + c of this lane's
    // row / column.
    struct Frag6 { f32x4 a[2], b[2]; };
    auto read_frags = [&](Frag6& f, int buf, int kg) {
        const char* s = smem + buf * kStageBytes6;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int r = wm + 16 * i + l16;
            f.a[i] = *reinterpret_cast<const f32x4*>(s + r * 128 + (((kg * 4 + g) ^ ((r >> 1) & 7)) << 4));
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = wn + 16 * j + l16;
            if constexpr (B_KC) {
                f.b[j] = *reinterpret_cast<const f32x4*>(s + kTileBytes6 + n * 128 + (((kg * 4 + g) ^ ((n >> 1) & 7)) << 4));
            } else {
                const char* p = s + kTileBytes6 + (kg * 16 + g * 4) * 256 + (((n >> 2) ^ (g << 2)) << 4) + (n & 3) * 4;
#pragma unroll
                for (int c = 0; c < 4; ++c) f.b[j][c] = *reinterpret_cast<const float*>(p + c * 256);
            }
        }
    };
    // operands swapped (rows of the instruction = n): a lane ends up with four consecutive n of one m
    auto multiply = [&](const Frag6& f) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.b[j][c], f.a[i][c], acc[i][j], 0, 0, 0);
    };

    // KT is even (host-checked): set 0 carries the even steps, set 1 the odd ones, one LDS buffer each.
    // One barrier per k-step, in its middle: while the first half of step g is multiplied its second
    // half's fragments are read and step g + 1 goes from registers to the other LDS buffer; after the
    // barrier the first fragments of step g + 1 are read while the second half of step g is
    // multiplied, so that no fragment read is waited for with nothing to do.  (With the barrier
    // between the steps the wait for the first fragments after it was exposed: 27.8 -> 26.5 us at 1024^3.)
    // The loads of the steps two ahead are unconditional (the last iterations load the last two steps
    // again, unused), so that the number of loads in flight is the same at every wait.  (Two k-steps per
    // barrier on four LDS buffers were measured too: no faster at 1024^3, 8 % slower at 2048^3, where
    // 64 KiB of LDS per workgroup leaves fewer workgroups per CU.)
    Frag6 f0, f1;
    fetch(0, 0);
    fetch(1, 1);
    landed(0);
    stage(0, 0);
    fetch(0, min(2, KT - 2));
    __syncthreads();
    read_frags(f0, 0, 0);
    auto half_steps = [&](int buf, int next_set, int next_step) {
        read_frags(f1, buf, 1);
        multiply(f0);
        landed(next_set);
        stage(next_set, buf ^ 1);
        fetch(next_set, next_step);
        __syncthreads();
        read_frags(f0, buf ^ 1, 0);
        multiply(f1);
    };
    for (int kt = 0; kt < KT; kt += 2) {
        half_steps(0, 1, min(kt + 3, KT - 1));
        half_steps(1, 0, min(kt + 4, KT - 2));
    }
    // The reloads of the last two steps are still in flight.  Their target registers are dead to the
    // compiler, which would hand them to the epilogue (addresses, results) while the loads can still
    // land in them: wait, and keep the registers allocated up to the wait.
    wait_vmcnt_imm<0>();
#pragma unroll
    for (int set = 0; set < 2; ++set)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            tie6(ra[set][i]); tie6(rb[set][i]);
            if constexpr (A_SUM) tie6(ra1[set][i]);
            if constexpr (B_SUM) tie6(rb1[set][i]);
        }

    // lane l of block (i, j) holds m = 16 i + l % 16 and n = 16 j + 4 (l / 16) + 0..3
    float* Cb = P.C + (int64_t)prod * P.c_ps;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            f32x4* d = reinterpret_cast<f32x4*>(Cb + (int64_t)(tile_m + wm + 16 * i + l16) * P.c_rs + (tile_n + wn + 16 * j + 4 * g));
            f32x4 v = acc[i][j];
            if (P.accumulate) v += *d;
            *d = v;
        }
}

template <bool B_KC>
__global__ void __launch_bounds__(kThreads6) gemm6_kernel(const Gemm6Params P) {
    __shared__ __attribute__((aligned(1024))) char smem[2 * kStageBytes6];
    const int tiles = P.tiles_m * P.tiles_n;
    const int prod = __builtin_amdgcn_readfirstlane((int)blockIdx.x / tiles);
    // XCD-aware walk within the product (tile_coords_in): each XCD owns a contiguous run of tiles, taken
    // eight tile rows at a time, so that neighbours share operand panels in that XCD's L2
    GemmParams tp;
    tp.tiles_m = P.tiles_m; tp.tiles_n = P.tiles_n; tp.group_m = 8;
    int tm, tn;
    tile_coords_in(tp, (int)blockIdx.x - prod * tiles, tiles, tm, tn);
    const int tile_m = tm * kBM6, tile_n = tn * kBN6;
    const bool a_sum = P.a[prod].sign != 0, b_sum = P.b[prod].sign != 0;
    if (a_sum && b_sum) run6<B_KC, true, true>(P, smem, prod, tile_m, tile_n);
    else if (a_sum) run6<B_KC, true, false>(P, smem, prod, tile_m, tile_n);
    else if (b_sum) run6<B_KC, false, true>(P, smem, prod, tile_m, tile_n);
    else run6<B_KC, false, false>(P, smem, prod, tile_m, tile_n);
}

}  // namespace sthip
