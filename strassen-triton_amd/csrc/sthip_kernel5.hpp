// One Strassen / Winograd level as ONE launch on gfx950: the quadrant sums, the seven half-size
// products on 256 x 256 tiles and the recombination are all workgroups of the same grid.
//
// Why.  As three launches (sums, grouped products, recombination) the two element-wise passes run
// alone on the chip at HBM speed while the matrix cores idle, and the products run with HBM nearly
// idle.  The product kernel fills every CU's registers and LDS, so no second kernel can share a CU
// with it -- but a workgroup of the SAME kernel can do element-wise work on one CU while the other
// CUs multiply.  The grid is therefore a list of work items in dependency order:
//
//   sums the first product needs (all CUs) | the other sums | tiles of product 1 | tiles of product 2 |
//   ... | recombination of a quadrant of C as soon as its products are complete | ... | the rest
//
// Workgroups are dispatched in blockIdx order, one per CU, so an element-wise item occupies one
// CU for as long as it streams (about 50 GB/s per CU) while the others run tiles; the memory
// traffic of the passes overlaps with matrix work instead of preceding and following it.
//
// Measured at 8192^3 bf16: 1.08 ms per call against 0.92 ms for the three launches (bit-identical
// results).  A probe that streamed 705 MB from workgroups interleaved with the tiles of the grouped
// launch showed the overlap itself works (+0.07 ms against 0.12 ms as a pass of its own); what the
// complete form loses is the L2 write-back every producer needs before it can announce its data
// (about 0.07 ms in all), the sums and the recombination at the two ends, which nothing overlaps
// (0.08 ms), and the ~45 GB/s a single CU streams.  The library therefore runs the three launches
// by default; this form runs when bit 4 of the debug stage mask is set.
//
// Dependencies are counters in device memory: every finished sums unit increments its job's
// counter, every finished tile its product's.  A tile waits until the jobs that form its operands
// are complete, a recombination unit until its products are.  An item only ever waits for items
// that come earlier in the grid, which never wait for later ones, so every wait ends; it is
// bounded all the same (a workgroup that gives up counts itself in flags[kFlagGaveUp] and goes
// on with whatever is in memory: a wrong result, never a hang).
//
// Visibility between XCDs (each has its own L2): a producer writes its XCD's L2 back with a
// release fence at agent scope before it increments the counter; counters are read with
// agent-scope atomics, which do not go through the L2 of the reading XCD.  A consumer needs no
// cache invalidation: what it reads was never read by this launch before it was complete, so
// no XCD can hold an older copy (a launch starts with clean caches).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sthip_kernel4.hpp"

namespace sthip {

constexpr int kMaxItems5 = 20, kMaxJobs5 = 4, kMaxRec5 = 4;
enum { kItemSums = 0, kItemTiles = 1, kItemRecombine = 2 };
constexpr int kFlagJob = 0, kFlagProd = 8, kFlagGaveUp = 15, kFlagWords = 16;
constexpr int kSpinLimit5 = 1 << 19;   // polls of ~0.2 us each: about 0.1 s

// out[o] = sum_q coef[o][q] * quadrant q on a rows x (chunks_per_row * 16 bytes) block in storage
// order, fp32 sums rounded once; `units` workgroups share the rows.
struct SumJob5 {
    const void* q[4];
    void* out[5];
    int64_t ld_in, ld_out;   // elements
    int rows, chunks_per_row, nout, units;
    signed char coef[5][4];
};

// One quadrant of C from up to four 16-bit products, added in fp32 in the order given.
struct RecJob5 {
    const void* m[4];
    void* c;
    int nterms, units;
    signed char sign[4];
};

struct Item5 {
    int first;             // first blockIdx of the item's workgroups
    int kind, arg;         // sums job / product / recombination job
    unsigned need_jobs;    // bit j: sums job j must be complete
    unsigned need_prods;   // bit p: product p must be complete
};

struct Fused5Params {
    Gemm2Params g;         // seg[0..6]: the seven products; C = the product matrices
    SumJob5 job[kMaxJobs5];
    RecJob5 rec[kMaxRec5];
    Item5 item[kMaxItems5];
    int nitems, njobs;
    unsigned* flags;       // kFlagWords counters, zero at launch
    int64_t c_rs;          // row stride of C (elements)
    int rec_rows, rec_chunks;   // half-size result: rows and 16-byte chunks per row
    int tiles;             // tiles of one product
    int streaming;
};

__device__ __forceinline__ unsigned peek_flag(const unsigned* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Thread 0 polls until every needed counter has reached its target; the workgroup then meets at a
// barrier.  Returns with the data of the producers visible to every thread of the workgroup.
__device__ __forceinline__ void wait_for(const Fused5Params& P, unsigned need_jobs, unsigned need_prods) {
    if (threadIdx.x == 0) {
        int spins = 0;
        bool gave_up = false;
        for (int j = 0; j < P.njobs && !gave_up; ++j) {
            if (!((need_jobs >> j) & 1)) continue;
            while (peek_flag(P.flags + kFlagJob + j) < (unsigned)P.job[j].units) {
                __builtin_amdgcn_s_sleep(8);
                if (++spins > kSpinLimit5) { gave_up = true; break; }
            }
        }
        for (int p = 0; p < 7 && !gave_up; ++p) {
            if (!((need_prods >> p) & 1)) continue;
            while (peek_flag(P.flags + kFlagProd + p) < (unsigned)P.tiles) {
                __builtin_amdgcn_s_sleep(8);
                if (++spins > kSpinLimit5) { gave_up = true; break; }
            }
        }
        if (gave_up) __hip_atomic_fetch_add(P.flags + kFlagGaveUp, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    asm volatile("" ::: "memory");
}

// The workgroup's stores have reached its XCD's L2 (the barrier waits for them); one thread then
// writes that L2 back (release at agent scope) and counts the item as done.  One write-back per
// workgroup, not one per wave: with all eight waves fencing, the fences alone cost 0.5 ms per call at
// 8192^3.  Stores that ask for write-through (sc1, or sc0 sc1) in place of the fence were measured
// too and are not enough: about 0.1 % of the elements then came out stale.
__device__ __forceinline__ void signal_done(unsigned* counter) {
    __syncthreads();
    if (threadIdx.x == 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Rows [r0, r1) of a block of `chunks` 16-byte chunks per row are shared by the 512 threads without a
// division per chunk: with at least 512 chunks per row a thread walks one row at a time, otherwise the
// threads form 512 / chunks rows per pass.
struct RowWalk5 {
    int row_step, first_row, first_chunk, chunk_step;
    __device__ __forceinline__ RowWalk5(int chunks) {
        if (chunks >= kThreads4) { row_step = 1; first_row = 0; first_chunk = threadIdx.x; chunk_step = kThreads4; }
        else {
            row_step = kThreads4 / chunks;
            first_row = threadIdx.x / chunks; first_chunk = threadIdx.x % chunks; chunk_step = chunks;
            if (first_row >= row_step) first_row = 1 << 30;   // left-over threads sit out
        }
    }
};

// Sums unit u of a job: the same arithmetic, in the same order, as the one-chunk-per-thread pass.
template <class T>
__device__ __forceinline__ void sums_chunk(const SumJob5& J, int64_t in_off, int64_t out_off, int streaming) {
    u32x4 v[4];
    float x[4][8];
#pragma unroll
    for (int q = 0; q < 4; ++q)
        if (J.q[q]) v[q] = load_hinted(reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(J.q[q]) + in_off), streaming);
        else v[q] = u32x4{0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t word = v[q][w];
            if constexpr (__is_same(T, bf16_t)) { x[q][2 * w] = bf16lo(word); x[q][2 * w + 1] = bf16hi(word); }
            else { const f16x2 h = as_f16x2(word); x[q][2 * w] = (float)h[0]; x[q][2 * w + 1] = (float)h[1]; }
        }
    for (int o = 0; o < J.nout; ++o) {
        u32x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float s[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float acc = 0.f;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int cf = J.coef[o][q];
                    if (cf > 0) acc += x[q][2 * i + h]; else if (cf < 0) acc -= x[q][2 * i + h];
                }
                s[h] = acc;
            }
            if constexpr (__is_same(T, bf16_t)) w[i] = pack_bf16(s[0], s[1]);
            else w[i] = pack_f16(s[0], s[1]);
        }
        *reinterpret_cast<u32x4*>(reinterpret_cast<char*>(J.out[o]) + out_off) = w;
    }
}

template <class T>
__device__ __forceinline__ void sums_unit(const SumJob5& J, int u, int streaming) {
    const int r0 = (int)((int64_t)J.rows * u / J.units), r1 = (int)((int64_t)J.rows * (u + 1) / J.units);
    const RowWalk5 w(J.chunks_per_row);
    for (int r = r0 + w.first_row; r < r1; r += w.row_step)
        for (int c = w.first_chunk; c < J.chunks_per_row; c += w.chunk_step)
            sums_chunk<T>(J, ((int64_t)r * J.ld_in + c * 8) * 2, ((int64_t)r * J.ld_out + c * 8) * 2, streaming);
}

// Recombination unit u: rows [r0, r1) of one half-size quadrant of C.
template <class T>
__device__ __forceinline__ void recombine_unit(const Fused5Params& P, const RecJob5& R, int u) {
    const int r0 = (int)((int64_t)P.rec_rows * u / R.units), r1 = (int)((int64_t)P.rec_rows * (u + 1) / R.units);
    const RowWalk5 wk(P.rec_chunks);
    for (int r = r0 + wk.first_row; r < r1; r += wk.row_step)
        for (int c = wk.first_chunk; c < P.rec_chunks; c += wk.chunk_step) {
            const int64_t src = ((int64_t)r * P.rec_chunks + c) * 16;
            float acc[8], m[8];
            u32x4 v[4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (t < R.nterms) v[t] = load_hinted(reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(R.m[t]) + src), P.streaming);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                if (t >= R.nterms) break;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    if constexpr (__is_same(T, bf16_t)) { m[2 * w] = bf16lo(v[t][w]); m[2 * w + 1] = bf16hi(v[t][w]); }
                    else { const f16x2 h = as_f16x2(v[t][w]); m[2 * w] = (float)h[0]; m[2 * w + 1] = (float)h[1]; }
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (t == 0) acc[e] = m[e];
                    else acc[e] = R.sign[t] > 0 ? acc[e] + m[e] : acc[e] - m[e];
                }
            }
            u32x4 w;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if constexpr (__is_same(T, bf16_t)) w[k] = pack_bf16(acc[2 * k], acc[2 * k + 1]);
                else w[k] = pack_f16(acc[2 * k], acc[2 * k + 1]);
            }
            store_hinted(w, reinterpret_cast<u32x4*>(reinterpret_cast<char*>(R.c) + ((int64_t)r * P.c_rs + c * 8) * 2), P.streaming);
        }
}

template <class T, bool B_KC>
__global__ void __launch_bounds__(kThreads4) fused5_kernel(const Fused5Params P) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    // which item does this workgroup belong to?  (uniform: scalar registers)
    const int bid = (int)blockIdx.x;
    int it = 0;
    for (int i = 1; i < P.nitems; ++i)
        if (bid >= P.item[i].first) it = i;
    it = __builtin_amdgcn_readfirstlane(it);
    const Item5& I = P.item[it];
    const int local = bid - I.first;

    if (I.kind == kItemSums) {
        if (local < P.job[I.arg].units) {
            sums_unit<T>(P.job[I.arg], local, P.streaming);
            signal_done(P.flags + kFlagJob + I.arg);
        }
        return;
    }
    if (I.kind == kItemRecombine) {
        if (local < P.rec[I.arg].units) {
            wait_for(P, 0, I.need_prods);
            recombine_unit<T>(P, P.rec[I.arg], local);
        }
        return;
    }
    if (local >= P.tiles) return;   // padding up to a multiple of eight workgroups

    // a 256 x 256 tile of product I.arg: the main loop of the grouped kernel
    const Gemm2Params& G = P.g;
    const int prod = __builtin_amdgcn_readfirstlane(I.arg);
    GemmParams tp;
    tp.tiles_m = G.tiles_m; tp.tiles_n = G.tiles_n; tp.group_m = G.group_m;
    int tm, tn;
    tile_coords_in(tp, local, P.tiles, tm, tn);
    const int tile_m = tm * kBM4, tile_n = tn * kBN4;
    char* Cb = reinterpret_cast<char*>(G.C) + (int64_t)prod * G.c_ps * 2;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int KT = G.Kh / bk4<T>();

    wait_for(P, I.need_jobs, 0);

    Pipe4<T, B_KC> pipe;
    pipe.smem = smem;
    pipe.smem_addr = (uint32_t)(uintptr_t)(lptr_t)smem;
    pipe.wm = (wave >> 2) * 128;
    pipe.wn = (wave & 3) * 64;
    pipe.total = KT;
    pipe.ld.P = &G;
    pipe.ld.wave = wave;
    pipe.ld.seg = prod; pipe.ld.kt = 0; pipe.ld.total_seg = prod + 1; pipe.ld.KT = KT;
    pipe.ld.batch = 0; pipe.ld.tile_m = tile_m; pipe.ld.tile_n = tile_n;
    pipe.ld.stride = 0; pipe.ld.id = 0; pipe.ld.total_ids = 0;
    pipe.ld.point_at_segment();
    pipe.start();

    Acc4 r;
    r.zero();
    pipe.run(r, KT);
    __syncthreads();   // every wave has read its last fragments: the stage buffers are free
    store_tile4_lds<T>(r, G, Cb, smem, wave, tile_m + pipe.wm, tile_n + pipe.wn);
    signal_done(P.flags + kFlagProd + prod);
}

}  // namespace sthip
