// C-ABI front end of libstrassen_hip.so: argument checking, kernel selection, the host-side
// recursion for two or more Strassen levels, and the small element-wise kernels that
// recursion needs.  See include/strassen_hip.h for the contract of every entry point.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <mutex>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/strassen_hip.h"
#include "../../include/strassen_hip_debug.h"
#include "sthip_launch.hpp"

namespace sthip {

static thread_local char g_err[512] = "";
// Process-wide debug switches (include/strassen_hip_debug.h).  Every public entry point reads them
// once, into its Call; nothing below an entry point looks at them again.
// Stages of the pipelined path that run: bit 0 = quadrant-sum pre-pass, bit 1 = grouped GEMM,
// bit 2 = recombination pass, bit 3 = two levels may run as one 49-product launch, bit 4 = one level
// may run as ONE launch (sums, products and recombination as work items of one grid).
constexpr int kAllStages = 63;
constexpr int kDefaultStages = 15;   // the one-launch form is slower than the three launches (sthip_kernel5.hpp): off unless asked for
static std::atomic<int> g_debug_stages{kDefaultStages};
// Forced tile: 0 = the tile table decides, 2 = 128 x 128, 3 = 256 x 128, 4 = 256 x 256, 5 = 128 x 128 with
// the seven products as separate outputs; -1 = not set yet (the first call reads STHIP_FORCE_TILE).
static std::atomic<int> g_debug_tile{-1};

static int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }
static inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
static inline int elem_size(int dt) { return dt == STHIP_F32 ? 4 : 2; }
// The passes and the product tiles use streaming loads and stores when the sums and products of the
// call exceed the 256 MiB memory-side cache; below that the next kernel of the call finds them cached
// (measured at 4096^3 fp16: the call 4.7 % faster with plain accesses; at 8192^3 bf16: 1 % slower).
static inline int streaming_hint(size_t workspace_traffic_bytes) { return workspace_traffic_bytes > ((size_t)256 << 20) ? 1 : 0; }

// A strided 2-D view of device memory, strides in elements of `dt`.
struct View {
    const char* p;
    int64_t rs, cs;
};

static const LaunchTable* table_for(int dt, int algo) {
    switch (dt * 3 + algo) {
        case 0: return &kLaunch_0_0; case 1: return &kLaunch_0_1; case 2: return &kLaunch_0_2;
        case 3: return &kLaunch_1_0; case 4: return &kLaunch_1_1; case 5: return &kLaunch_1_2;
        case 6: return &kLaunch_2_0; case 7: return &kLaunch_2_1; case 8: return &kLaunch_2_2;
    }
    return nullptr;
}

static const LaunchTable2* table2_for(int dt, int algo) {
    switch (dt * 3 + algo) {
        case 3: return &kLaunch2_1_0; case 4: return &kLaunch2_1_1; case 5: return &kLaunch2_1_2;
        case 6: return &kLaunch2_2_0; case 7: return &kLaunch2_2_1; case 8: return &kLaunch2_2_2;
    }
    return nullptr;
}

static int check_launch(const char* what);

static const LaunchTable3* table3_for(int dt, int algo) {
    switch (dt * 3 + algo) {
        case 3: return &kLaunch3_1_0; case 4: return &kLaunch3_1_1; case 5: return &kLaunch3_1_2;
        case 6: return &kLaunch3_2_0; case 7: return &kLaunch3_2_1; case 8: return &kLaunch3_2_2;
    }
    return nullptr;
}

static const LaunchTable5* table5_for(int dt) {
    return dt == STHIP_F16 ? &kLaunch5_1 : dt == STHIP_BF16 ? &kLaunch5_2 : nullptr;
}

static const LaunchTable3* table4_for(int dt) {
    return dt == STHIP_F32 ? &kLaunch4_0 : dt == STHIP_F16 ? &kLaunch4_1 : dt == STHIP_BF16 ? &kLaunch4_2 : nullptr;
}

// STHIP_FORCE_TILE=128x128 | 128x128g | 256x128 | 256x256 | 64x64 in the environment of the process overrides the
// tile table where the shape allows the forced tile (tuning aid); it is read once, by the first call.
// sthip_debug_force_tile changes the setting later.
static int tile_code(const char* e) {
    if (!e) return 0;
    if (!strcmp(e, "128x128")) return 2;
    if (!strcmp(e, "256x128")) return 3;
    if (!strcmp(e, "256x256")) return 4;
    if (!strcmp(e, "128x128g")) return 5;   // 128 x 128 tiles, seven products as separate outputs
    if (!strcmp(e, "64x64")) return 6;      // fp32: 64 x 64 tiles, seven products side by side, sums formed in the loads
    return 0;
}
static int forced_tile_setting() {
    int t = g_debug_tile.load(std::memory_order_relaxed);
    if (t < 0) {
        t = tile_code(getenv("STHIP_FORCE_TILE"));
        int expected = -1;
        if (!g_debug_tile.compare_exchange_strong(expected, t)) t = expected;
    }
    return t;
}

static bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
// 16-bit C whose rows, product stride and batch stride keep 16-byte alignment (strides in elements)
static int wide_rows(const void* C, int64_t rs, int64_t ps, int64_t bs) {
    return aligned_to(C, 16) && rs % 8 == 0 && ps % 8 == 0 && bs % 8 == 0 ? 1 : 0;
}

// Quadrant sums as coefficients over (X11, X12, X21, X22).  Strassen (fixed_strassen.py:88-97): A side
// S2 S3 S5 S7 S9, B side S1 S4 S6 S8 S10.  Winograd: A side S1 S2 S3 S4; B side T1 T2 T3 -T4.
constexpr int str_coef(int side, int o, int q) {
    constexpr signed char a[5][4] = {{1, 1, 0, 0}, {0, 0, 1, 1}, {1, 0, 0, 1}, {0, 1, 0, -1}, {-1, 0, 1, 0}};
    constexpr signed char b[5][4] = {{0, 1, 0, -1}, {-1, 0, 1, 0}, {1, 0, 0, 1}, {0, 0, 1, 1}, {1, 1, 0, 0}};
    return side == 0 ? a[o][q] : b[o][q];
}
constexpr int win_coef(int side, int o, int q) {
    constexpr signed char a[4][4] = {{0, 0, 1, 1}, {-1, 0, 1, 1}, {1, 0, -1, 0}, {1, 1, -1, -1}};
    constexpr signed char b[4][4] = {{-1, 1, 0, 0}, {1, -1, 0, 1}, {0, -1, 0, 1}, {-1, 1, 1, -1}};
    return side == 0 ? a[o][q] : b[o][q];
}

// ------------------------------------------------------------------ quadrant-sum pre-pass
// out[o] = sum_q coef[o][q] * quadrant q, for up to five outputs at once, on matrices seen
// in storage order (rows x cols, cols contiguous).  Each thread handles one 16-byte chunk
// position: the four quadrant chunks are read once, every output is formed in fp32 and
// rounded once to the operand type.
struct ComboParams {
    const void* q[4];
    void* out[7];
    int64_t ld_in, bs_in, ld_out, bs_out;   // elements
    int nout, rows, chunks_per_row;
    int streaming;   // loads and stores carry the streaming hint (working set larger than the caches)
    int table;       // 16-bit kernels: 0 / 1 = the five Strassen sums of an A / B operand, 2 / 3 = the four Winograd sums
                     // (coefficients compiled in); anything else: coef below
    signed char coef[7][4];
};

// TABLE 0..3: coefficients known at compile time (every term a constant, zero terms vanish); -1: read
// from p.coef.  With run-time coefficients the pass issued 680 VALU instructions per thread and kept the
// vector ALUs busy 72 % of its time; the products only ever need the four fixed tables.
template <class T, int TABLE>
__device__ __forceinline__ void quad_combos_body(const ComboParams& p) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.rows * p.chunks_per_row) return;
    const int r = (int)(idx / p.chunks_per_row), c = (int)(idx % p.chunks_per_row);
    const int64_t in_off = ((int64_t)blockIdx.y * p.bs_in + (int64_t)r * p.ld_in + c * 8) * 2;
    const int64_t out_off = ((int64_t)blockIdx.y * p.bs_out + (int64_t)r * p.ld_out + c * 8) * 2;
    u32x4 v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
        v[q] = load_hinted(reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(p.q[q]) + in_off), p.streaming);
    float x[4][8];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t word = v[q][w];
            if constexpr (__is_same(T, bf16_t)) { x[q][2 * w] = bf16lo(word); x[q][2 * w + 1] = bf16hi(word); }
            else { const f16x2 h = as_f16x2(word); x[q][2 * w] = (float)h[0]; x[q][2 * w + 1] = (float)h[1]; }
        }
    auto emit = [&](int o, const float* s) {
        u32x4 w;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (__is_same(T, bf16_t)) w[i] = pack_bf16(s[2 * i], s[2 * i + 1]);
            else w[i] = pack_f16(s[2 * i], s[2 * i + 1]);
        }
        store_hinted(w, reinterpret_cast<u32x4*>(reinterpret_cast<char*>(p.out[o]) + out_off), p.streaming);
    };
    if constexpr (TABLE >= 0) {
        constexpr int NOUT = TABLE < 2 ? 5 : 4;
#pragma unroll
        for (int o = 0; o < NOUT; ++o) {
            float s[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float acc = 0.f;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int cf = TABLE < 2 ? str_coef(TABLE, o, q) : win_coef(TABLE - 2, o, q);
                    if (cf > 0) acc += x[q][e]; else if (cf < 0) acc -= x[q][e];
                }
                s[e] = acc;
            }
            emit(o, s);
        }
    } else {
        for (int o = 0; o < p.nout; ++o) {
            float s[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float acc = 0.f;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int cf = p.coef[o][q];
                    if (cf > 0) acc += x[q][e]; else if (cf < 0) acc -= x[q][e];
                }
                s[e] = acc;
            }
            emit(o, s);
        }
    }
}
template <class T>
__device__ __forceinline__ void quad_combos_any(const ComboParams& p) {
    const int table = __builtin_amdgcn_readfirstlane(p.table);
    if (table == 0) quad_combos_body<T, 0>(p);
    else if (table == 1) quad_combos_body<T, 1>(p);
    else if (table == 2) quad_combos_body<T, 2>(p);
    else if (table == 3) quad_combos_body<T, 3>(p);
    else quad_combos_body<T, -1>(p);
}

template <class T>
__global__ void __launch_bounds__(256) quad_combos_kernel(const ComboParams p) { quad_combos_any<T>(p); }

// fp32 form: four elements per 16-byte chunk, sums stay fp32 (nothing to round).
__device__ __forceinline__ void quad_combos_f32_body(const ComboParams& p) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.rows * p.chunks_per_row) return;
    const int r = (int)(idx / p.chunks_per_row), c = (int)(idx % p.chunks_per_row);
    const int64_t in_off = (int64_t)r * p.ld_in + c * 4, out_off = (int64_t)r * p.ld_out + c * 4;
    f32x4 x[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) x[q] = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.q[q]) + in_off);
    for (int o = 0; o < p.nout; ++o) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int cf = p.coef[o][q];
            if (cf > 0) acc += x[q]; else if (cf < 0) acc -= x[q];
        }
        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.out[o]) + out_off) = acc;
    }
}

// Both operands of a level in one launch: blockIdx.z picks the side.
struct ComboPair { ComboParams side[2]; };
template <class T>
__global__ void __launch_bounds__(256) quad_combos_pair_kernel(const ComboPair pp) { quad_combos_any<T>(pp.side[blockIdx.z]); }

__global__ void __launch_bounds__(256) quad_combos_pair_f32_kernel(const ComboPair pp) { quad_combos_f32_body(pp.side[blockIdx.z]); }

// Eight 16-bit elements of a 16-byte chunk as floats.
template <class T>
__device__ __forceinline__ void unpack8(const u32x4 v, float* x) {
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        if constexpr (__is_same(T, bf16_t)) { x[2 * w] = bf16lo(v[w]); x[2 * w + 1] = bf16hi(v[w]); }
        else { const f16x2 h = as_f16x2(v[w]); x[2 * w] = (float)h[0]; x[2 * w + 1] = (float)h[1]; }
    }
}

// NW 32-bit words (2 NW 16-bit elements) as floats, and back with one rounding.
template <int NW> struct WordVec;
template <> struct WordVec<2> { typedef u32x2 type; };
template <> struct WordVec<4> { typedef u32x4 type; };
// kEPT2 elements of type T as one vector load / store: 8 bytes of 16-bit elements, 16 bytes of fp32
template <class T> struct ElemVec { typedef u32x2 type; };
template <> struct ElemVec<float> { typedef f32x4 type; };
template <class T, int NW>
__device__ __forceinline__ void unpack_words(const typename WordVec<NW>::type v, float* x) {
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        if constexpr (__is_same(T, bf16_t)) { x[2 * w] = bf16lo(v[w]); x[2 * w + 1] = bf16hi(v[w]); }
        else { const f16x2 h = as_f16x2(v[w]); x[2 * w] = (float)h[0]; x[2 * w + 1] = (float)h[1]; }
    }
}
template <class T, int NW>
__device__ __forceinline__ typename WordVec<NW>::type pack_words(const float* x) {
    typename WordVec<NW>::type w;
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        if constexpr (__is_same(T, bf16_t)) w[i] = pack_bf16(x[2 * i], x[2 * i + 1]);
        else w[i] = pack_f16(x[2 * i], x[2 * i + 1]);
    }
    return w;
}
// Elements per thread of the two-level passes: four (8-byte accesses) keep their register use low
// enough for four or more waves per SIMD; with eight the kernels ran at one or two.
constexpr int kNW2 = 2, kEPT2 = 2 * kNW2;
template <class T>
__device__ __forceinline__ void unpack_elems(const typename ElemVec<T>::type v, float* x) {
    if constexpr (__is_same(T, float)) { x[0] = v[0]; x[1] = v[1]; x[2] = v[2]; x[3] = v[3]; }
    else unpack_words<T, kNW2>(v, x);
}
template <class T>
__device__ __forceinline__ typename ElemVec<T>::type pack_elems(const float* x) {
    if constexpr (__is_same(T, float)) { f32x4 v = {x[0], x[1], x[2], x[3]}; return v; }
    else return pack_words<T, kNW2>(x);
}

// The sums of BOTH levels of a two-level product for one operand in one pass: the sixteen quarter
// blocks are read once; every first-level operand (a quadrant, or a sum of two rounded once to
// the operand type, fixed_strassen_fp32_agg.py:87-96) is formed in registers, the quarters of the
// first-level sums that the second level multiplies directly are stored, and so are the
// second-level sums of all seven first-level operands (fp32 sums of the rounded first-level
// values, rounded once).  The other half of the first-level sums is never written and none is
// re-read.
struct Combo2Params {
    const void* x[16];        // quarter blocks of the operand, logical (R, C) -> x[4 R + C]
    void* s1[5];              // first-level sums: dense half-size blocks in the operand's storage orientation
    void* s2[7];              // second-level sums of first-level operand p: s2[p] + o * s2_stride bytes
    int64_t s2_stride;
    int64_t ld_in, ld1, ld2;  // elements
    int64_t q1_u, q1_v;       // element offset of quarter (u, v) inside a first-level sum: u * q1_u + v * q1_v
    int rows, chunks_per_row; // of one quarter block, storage order
    int side;                 // 0: the tables of the A operand, 1: of the B operand
    int algo2;                // algorithm of the second level (the first is always Strassen)
    int streaming;            // loads and stores carry the streaming hint
};
struct Combo2Pair { Combo2Params side[2]; };

// Coefficient tables of the two-level pass, evaluated at compile time: the loops over operands,
// quarters and terms are unrolled, so every coefficient is a constant and zero terms vanish.  (With the
// tables as kernel arguments the pass issued 3300 VALU instructions per thread and was bound by them,
// not by memory: 4.1 TB/s.)
// First-level operands in the order the 49 products use them: A side A11 S9 S2 S7 S5 S3 A22, B side
// S1 S10 B22 S8 S6 B11 S4.  >= 0: index of the sum among the five; -1 - q: quadrant q as it is.
constexpr int first_code(int side, int p) {
    constexpr signed char a[7] = {-1, 4, 0, 3, 2, 1, -4}, b[7] = {0, 4, -4, 3, 2, -1, 1};
    return side == 0 ? a[p] : b[p];
}
constexpr int first_coef(int side, int p, int q) {
    const int f = first_code(side, p);
    return f >= 0 ? str_coef(side, f, q) : (q == -1 - f ? 1 : 0);
}
constexpr int second_coef(int side, int algo2, int o, int uv) {
    return algo2 == STHIP_STRASSEN ? str_coef(side, o, uv) : win_coef(side, o, uv);
}
// Quarters (bit 2 u + v) of a first-level sum that the second level multiplies as they are: Strassen
// 11 and 22; Winograd 11, 12 and 22 of an A-side operand, 11, 21 and 22 of a B-side one.
constexpr int kept_quarters(int side, int algo2) { return algo2 == STHIP_STRASSEN ? 0x9 : (side == 0 ? 0xB : 0xD); }

template <class T, int SIDE, int ALGO2>
__device__ __forceinline__ void combos2_body(const Combo2Params& p) {
    typedef typename ElemVec<T>::type vec_t;
    constexpr int ES = (int)sizeof(T) == 4 ? 4 : 2;
    constexpr int NOUT2 = ALGO2 == STHIP_STRASSEN ? 5 : 4;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.rows * p.chunks_per_row) return;
    const int r = (int)(idx / p.chunks_per_row), c = (int)(idx % p.chunks_per_row);
    const int64_t in_off = ((int64_t)r * p.ld_in + c * kEPT2) * ES;
    const int64_t o1 = (int64_t)r * p.ld1 + c * kEPT2, o2 = ((int64_t)r * p.ld2 + c * kEPT2) * ES;
    vec_t v[16];
#pragma unroll
    for (int b = 0; b < 16; ++b)
        v[b] = load_hinted(reinterpret_cast<const vec_t*>(reinterpret_cast<const char*>(p.x[b]) + in_off), p.streaming);
#pragma unroll
    for (int q = 0; q < 7; ++q) {
        // quarters (u, v) of first-level operand q, in the operand type and unpacked
        vec_t s[4];
        float x[4][kEPT2];
        const int code = first_code(SIDE, q);
#pragma unroll
        for (int uv = 0; uv < 4; ++uv) {
            if (code < 0) {
                // a quadrant as it is: nothing to add, nothing to round
                const int Q = -1 - code;
                s[uv] = v[(2 * (Q >> 1) + (uv >> 1)) * 4 + 2 * (Q & 1) + (uv & 1)];
                unpack_elems<T>(s[uv], x[uv]);
                continue;
            }
            float acc[kEPT2];
#pragma unroll
            for (int e = 0; e < kEPT2; ++e) acc[e] = 0.f;
#pragma unroll
            for (int Q = 0; Q < 4; ++Q) {
                const int cf = first_coef(SIDE, q, Q);
                if (cf == 0) continue;
                float t[kEPT2];
                unpack_elems<T>(v[(2 * (Q >> 1) + (uv >> 1)) * 4 + 2 * (Q & 1) + (uv & 1)], t);
#pragma unroll
                for (int e = 0; e < kEPT2; ++e) acc[e] = cf > 0 ? acc[e] + t[e] : acc[e] - t[e];
            }
            s[uv] = pack_elems<T>(acc);   // the one rounding of a first-level sum
            unpack_elems<T>(s[uv], x[uv]);
            if ((kept_quarters(SIDE, ALGO2) >> uv) & 1)
                store_hinted(s[uv], reinterpret_cast<vec_t*>(reinterpret_cast<char*>(p.s1[code]) + ((uv >> 1) * p.q1_u + (uv & 1) * p.q1_v + o1) * ES), p.streaming);
        }
#pragma unroll
        for (int o = 0; o < NOUT2; ++o) {
            float acc[kEPT2];
#pragma unroll
            for (int e = 0; e < kEPT2; ++e) {
                float a = 0.f;
#pragma unroll
                for (int uv = 0; uv < 4; ++uv) {
                    const int cf = second_coef(SIDE, ALGO2, o, uv);
                    if (cf > 0) a += x[uv][e]; else if (cf < 0) a -= x[uv][e];
                }
                acc[e] = a;
            }
            store_hinted(pack_elems<T>(acc), reinterpret_cast<vec_t*>(reinterpret_cast<char*>(p.s2[q]) + (int64_t)o * p.s2_stride + o2), p.streaming);
        }
    }
}

template <class T>
__global__ void __launch_bounds__(256) quad_combos2_kernel(const Combo2Pair pp) {
    const Combo2Params& p = pp.side[blockIdx.z];
    const int variant = __builtin_amdgcn_readfirstlane(2 * p.side + (p.algo2 == STHIP_STRASSEN ? 0 : 1));
    if (variant == 0) combos2_body<T, 0, STHIP_STRASSEN>(p);
    else if (variant == 1) combos2_body<T, 0, STHIP_WINOGRAD>(p);
    else if (variant == 2) combos2_body<T, 1, STHIP_STRASSEN>(p);
    else combos2_body<T, 1, STHIP_WINOGRAD>(p);
}

// Quadrant sums each algorithm needs, as coefficients over (X11, X12, X21, X22).
// Strassen (fixed_strassen.py:88-97): A side S2 S3 S5 S7 S9, B side S1 S4 S6 S8 S10.
static const signed char kStrA[5][4] = {{1, 1, 0, 0}, {0, 0, 1, 1}, {1, 0, 0, 1}, {0, 1, 0, -1}, {-1, 0, 1, 0}};
static const signed char kStrB[5][4] = {{0, 1, 0, -1}, {-1, 0, 1, 0}, {1, 0, 0, 1}, {0, 0, 1, 1}, {1, 1, 0, 0}};
// All seven operands of each side in the reference's numbering M1..M7 (single quadrants included),
// for the path that runs the products as a batch of dense matrices.
static const signed char kStr7A[7][4] = {{1, 0, 0, 1}, {0, 0, 1, 1}, {1, 0, 0, 0}, {0, 0, 0, 1}, {1, 1, 0, 0}, {-1, 0, 1, 0}, {0, 1, 0, -1}};
static const signed char kStr7B[7][4] = {{1, 0, 0, 1}, {1, 0, 0, 0}, {0, 1, 0, -1}, {-1, 0, 1, 0}, {0, 0, 0, 1}, {1, 1, 0, 0}, {0, 0, 1, 1}};
// Winograd: A side S1 S2 S3 S4; B side T1 T2 T3 -T4.
static const signed char kWinA[4][4] = {{0, 0, 1, 1}, {-1, 0, 1, 1}, {1, 0, -1, 0}, {1, 1, -1, -1}};
static const signed char kWinB[4][4] = {{-1, 1, 0, 0}, {1, -1, 0, 1}, {0, -1, 0, 1}, {-1, 1, 1, -1}};

// Workspace of the pipelined path per problem: five sums per operand, then a region that is
// either the seven 16-bit products of the 256 x 256 grouped launch or the fp32 slabs in which
// the 256 x 128 kernel parks one accumulator tile per workgroup (at most Mh x Nh floats).
// (prod_es = 4: the seven products kept in fp32, for 16-bit operands with an fp32 result.)
static size_t products_bytes(int64_t Mh, int64_t Nh, int prod_es = 2) { return 7 * align256(Mh * Nh * prod_es); }
// (+ 256 bytes at the end: the dependency counters of the one-launch form)
static size_t prepass_body_bytes(int64_t batch, int64_t Mh, int64_t Nh, int64_t Kh, int prod_es = 2) {
    return (size_t)batch * (5 * (align256(Mh * Kh * 2) + align256(Kh * Nh * 2)) + products_bytes(Mh, Nh, prod_es));
}
static size_t prepass_bytes(int64_t batch, int64_t Mh, int64_t Nh, int64_t Kh, int prod_es = 2) {
    return prepass_body_bytes(batch, Mh, Nh, Kh, prod_es) + 256;
}

// Recombination of the seven 16-bit products of one level (kernel order: Strassen
// M3 M6 M5 M7 M1 M2 M4, Winograd P1 P2 P6 P7 P5 P3 -P4) into the four quadrants of C: upcast,
// add in fp32 in the reference's order (fixed_strassen_fp32_agg.py:44-53), round once.  One
// thread per 16-byte chunk of a half-size row.
struct Recombine16Params {
    const void* prod;     // [batch][7] dense Mh x Nh matrices, p_ps elements apart
    void* C;
    int64_t c_rs, c_bs;   // elements
    int64_t p_ps;
    int Mh, Nh, accumulate;
    int out_f32;          // C is fp32 (no final rounding) instead of the operand type
    int streaming = 1;    // loads and stores carry the streaming hint
    const void* bias = nullptr;   // 16-bit, non-accumulating results: bias[column] is added to the rounded
                                  // result and the sum rounded again, as a separate add would (model/layers.py:271-272)
};

// Bias of a Linear forward: the recombination pass that writes `target` adds it, so that no
// separate pass over the output is needed.
struct BiasEpilogue { const void* bias = nullptr; const void* target = nullptr; bool applied = false; };

// Quadrant sums of a constant B operand formed ahead of the call (sthip_linear_prepare_weight).
// The level -- or the two fused levels -- that find their B operand at `target` with the same
// half extents read these and form the A-side sums only.  Layout: five first-level blocks of
// kh x nh, then (two levels) 35 second-level blocks of kh/2 x nh/2, as in the workspace; for
// three levels and more the five first-level blocks, then one such buffer of levels - 1 for the
// B operand of each of the seven products M1..M7.
struct PreparedSums {
    const char* sums = nullptr; size_t bytes = 0; const void* target = nullptr;
    int levels = 0; int64_t kh = 0, nh = 0;
};

// What a public entry point decides once and everything below it shares: the stream, the debug
// switches as they stood at entry, the bias a Linear forward wants added by its last pass, and
// the weight-side sums formed ahead of the call.
struct Call {
    hipStream_t stream = nullptr;
    int stages = kDefaultStages;
    int force_tile = 0;
    BiasEpilogue bias;
    PreparedSums prep;
    int sched = 0;   // kSchedAuto / kSchedReference / kSchedFast (bits 4-5 of the algo argument)
};

// Where 16-bit problems round below the first level.  The reference's fp32-aggregating recursion
// rounds the first level's operand sums to base_dtype and then recurses with base_dtype left at
// its default, fp32 (fixed_strassen_fp32_agg.py:99-113): every deeper sum, product and
// recombination is fp32 arithmetic.  "Reference" does that: the first level's sums are rounded to
// the operand type, widened to fp32, and the seven half-size products run on the fp32 paths with
// levels - 1 levels.  "Fast" rounds the sums and products of every level to the operand type so
// that every product runs on the 16-bit matrix cores (about 1.2e-2 from the reference at two
// levels, 2.3e-2 at three in bf16).  Automatic: fast at two levels (all 49 products in one 16-bit
// launch), reference from three levels on.
enum { kSchedAuto = 0, kSchedReference = 1, kSchedFast = 2 };
static bool reference_schedule(int dt, int levels, int sched) {
    return dt != STHIP_F32 && levels >= 2 && (sched == kSchedReference || (sched == kSchedAuto && levels >= 3));
}

static const void* take_bias(Call& cx, const void* C, bool accumulate, bool out_f32) {
    if (!cx.bias.bias || C != cx.bias.target || accumulate || out_f32) return nullptr;
    cx.bias.applied = true;
    return cx.bias.bias;
}
static size_t prepared_bytes(int levels, int64_t kh, int64_t nh) {
    const size_t first = 5 * align256(kh * nh * 2);
    if (levels <= 1) return first;
    if (levels == 2) return first + 35 * align256((kh / 2) * (nh / 2) * 2);
    return first + 7 * prepared_bytes(levels - 1, kh / 2, nh / 2);
}
static const char* take_prepared(const Call& cx, const void* B, int levels, int64_t kh, int64_t nh, size_t need) {
    const PreparedSums& ps = cx.prep;
    if (!ps.sums || B != ps.target || levels != ps.levels || kh != ps.kh || nh != ps.nh || ps.bytes < need) return nullptr;
    return ps.sums;
}


// x rounded to T, as a float.
template <class T>
__device__ __forceinline__ float round16(float x) {
    if constexpr (__is_same(T, float)) return x;
    else if constexpr (__is_same(T, bf16_t)) return bf16lo(pack_bf16(x, 0.f));
    else return (float)as_f16x2(pack_f16(x, 0.f))[0];
}

template <class T, int ALGO>
__global__ void __launch_bounds__(256) recombine16_kernel(const Recombine16Params p) {
    const int nq = p.Nh / 8;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.Mh * nq) return;
    const int i = (int)(idx / nq), j = (int)(idx % nq) * 8;
    const int64_t blk = p.p_ps;
    const char* src = reinterpret_cast<const char*>(p.prod) + ((int64_t)blockIdx.y * 7 * blk + (int64_t)i * p.Nh + j) * 2;
    float m[7][8];
#pragma unroll
    for (int q = 0; q < 7; ++q) unpack8<T>(load_hinted(reinterpret_cast<const u32x4*>(src + q * blk * 2), p.streaming), m[q]);
    float out[4][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        if constexpr (ALGO == STHIP_STRASSEN) {
            out[0][e] = ((m[4][e] + m[6][e]) - m[2][e]) + m[3][e];   // C11 = M1 + M4 - M5 + M7
            out[1][e] = m[0][e] + m[2][e];                           // C12 = M3 + M5
            out[2][e] = m[5][e] + m[6][e];                           // C21 = M2 + M4
            out[3][e] = ((m[4][e] - m[5][e]) + m[0][e]) + m[1][e];   // C22 = M1 - M2 + M3 + M6
        } else {
            const float u2 = m[0][e] + m[2][e], u3 = u2 + m[3][e], u4 = u2 + m[4][e];
            out[0][e] = m[0][e] + m[1][e];                           // C11 = P1 + P2
            out[1][e] = u4 + m[5][e];                                // C12 = U4 + P3
            out[2][e] = u3 + m[6][e];                                // C21 = U3 - P4
            out[3][e] = u3 + m[4][e];                                // C22 = U3 + P5
        }
    }
    if (p.out_f32) {
        float* Cf = reinterpret_cast<float*>(p.C) + (int64_t)blockIdx.y * p.c_bs;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            f32x4* d = reinterpret_cast<f32x4*>(Cf + (int64_t)(i + (q >> 1) * p.Mh) * p.c_rs + (j + (q & 1) * p.Nh));
            f32x4 lo = {out[q][0], out[q][1], out[q][2], out[q][3]}, hi = {out[q][4], out[q][5], out[q][6], out[q][7]};
            if (p.accumulate) { lo += d[0]; hi += d[1]; }
            d[0] = lo; d[1] = hi;
        }
        return;
    }
    char* Cb = reinterpret_cast<char*>(p.C) + (int64_t)blockIdx.y * p.c_bs * 2;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        u32x4* d = reinterpret_cast<u32x4*>(Cb + ((int64_t)(i + (q >> 1) * p.Mh) * p.c_rs + (j + (q & 1) * p.Nh)) * 2);
        if (p.accumulate) {
            float old[8];
            unpack8<T>(*d, old);
#pragma unroll
            for (int e = 0; e < 8; ++e) out[q][e] += old[e];
        } else if (p.bias) {
            float bv[8];
            unpack8<T>(*reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(p.bias) + (int64_t)(j + (q & 1) * p.Nh) * 2), bv);
#pragma unroll
            for (int e = 0; e < 8; ++e) out[q][e] = round16<T>(out[q][e]) + bv[e];
        }
        u32x4 w;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if constexpr (__is_same(T, bf16_t)) w[k] = pack_bf16(out[q][2 * k], out[q][2 * k + 1]);
            else w[k] = pack_f16(out[q][2 * k], out[q][2 * k + 1]);
        }
        store_hinted(w, d, p.streaming);
    }
}

// Both recombinations of a two-level product in one pass: from the 49 quarter-size 16-bit products
// (first-level product p, second-level product k at prod + (7 p + k) * p_ps) straight to C.  The
// second-level result of every first-level product stays in fp32 registers (the reference's inner
// call returns fp32 as well, fixed_strassen_fp32_agg.py:99-106) and the first level adds in the
// same order as recombine16_kernel (p visited in the order 4 6 5 2 0 3 1 gives each quadrant its
// terms in that order); the seven half-size products are never written.  One thread per 8-byte
// chunk of a quarter-size row; Mh, Nh are the quarter sizes here.

template <class T, int ALGO2>
__global__ void __launch_bounds__(256) recombine16x2_kernel(const Recombine16Params p) {
    typedef typename ElemVec<T>::type vec_t;
    constexpr int E = kEPT2, ES = (int)sizeof(T) == 4 ? 4 : 2;
    const int nq = p.Nh / E;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.Mh * nq) return;
    const int i = (int)(idx / nq), j = (int)(idx % nq) * E;
    const char* src = reinterpret_cast<const char*>(p.prod) + ((int64_t)i * p.Nh + j) * ES;
    float acc[4][4][E];   // [quadrant of C][quarter block within it][element]
    // second level of first-level product pp -> m[quarter block][element], fp32
    auto second = [&](int pp, float (&m)[4][E]) {
        float x[7][E];
#pragma unroll
        for (int k = 0; k < 7; ++k)
            unpack_elems<T>(load_hinted(reinterpret_cast<const vec_t*>(src + (int64_t)(7 * pp + k) * p.p_ps * ES), p.streaming), x[k]);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            if constexpr (ALGO2 == STHIP_STRASSEN) {
                m[0][e] = ((x[4][e] + x[6][e]) - x[2][e]) + x[3][e];
                m[1][e] = x[0][e] + x[2][e];
                m[2][e] = x[5][e] + x[6][e];
                m[3][e] = ((x[4][e] - x[5][e]) + x[0][e]) + x[1][e];
            } else {
                const float u2 = x[0][e] + x[2][e], u3 = u2 + x[3][e], u4 = u2 + x[4][e];
                m[0][e] = x[0][e] + x[1][e];
                m[1][e] = u4 + x[5][e];
                m[2][e] = u3 + x[6][e];
                m[3][e] = u3 + x[4][e];
            }
        }
    };
    float m[4][E];
#define STHIP_EACH for (int b = 0; b < 4; ++b) for (int e = 0; e < E; ++e)
    second(4, m);   // M1: C11 = M1 ..., C22 = M1 ...
#pragma unroll
    STHIP_EACH { acc[0][b][e] = m[b][e]; acc[3][b][e] = m[b][e]; }
    second(6, m);   // M4: C11 += M4, C21 = M4
#pragma unroll
    STHIP_EACH { acc[0][b][e] += m[b][e]; acc[2][b][e] = m[b][e]; }
    second(5, m);   // M2: C22 -= M2, C21 += M2
#pragma unroll
    STHIP_EACH { acc[3][b][e] -= m[b][e]; acc[2][b][e] += m[b][e]; }
    second(2, m);   // M5: C11 -= M5, C12 = M5
#pragma unroll
    STHIP_EACH { acc[0][b][e] -= m[b][e]; acc[1][b][e] = m[b][e]; }
    second(0, m);   // M3: C22 += M3, C12 += M3
#pragma unroll
    STHIP_EACH { acc[3][b][e] += m[b][e]; acc[1][b][e] += m[b][e]; }
    second(3, m);   // M7: C11 += M7
#pragma unroll
    STHIP_EACH { acc[0][b][e] += m[b][e]; }
    second(1, m);   // M6: C22 += M6
#pragma unroll
    STHIP_EACH { acc[3][b][e] += m[b][e]; }
#undef STHIP_EACH
    const int mh = 2 * p.Mh, nh = 2 * p.Nh;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int64_t row = (int64_t)(q >> 1) * mh + (b >> 1) * p.Mh + i, col = (int64_t)(q & 1) * nh + (b & 1) * p.Nh + j;
            if (p.out_f32 || ES == 4) {
                float* d = reinterpret_cast<float*>(p.C) + row * p.c_rs + col;
#pragma unroll
                for (int e = 0; e < E; e += 4) {
                    f32x4 o = {acc[q][b][e], acc[q][b][e + 1], acc[q][b][e + 2], acc[q][b][e + 3]};
                    f32x4* dd = reinterpret_cast<f32x4*>(d + e);
                    if (p.accumulate) o += *dd;
                    *dd = o;
                }
            } else if constexpr (ES == 2) {
                vec_t* d = reinterpret_cast<vec_t*>(reinterpret_cast<char*>(p.C) + (row * p.c_rs + col) * 2);
                if (p.accumulate) {
                    float old[E];
                    unpack_elems<T>(*d, old);
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[q][b][e] += old[e];
                } else if (p.bias) {
                    float bv[E];
                    unpack_elems<T>(*reinterpret_cast<const vec_t*>(reinterpret_cast<const char*>(p.bias) + col * 2), bv);
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[q][b][e] = round16<T>(acc[q][b][e]) + bv[e];
                }
                store_hinted(pack_elems<T>(acc[q][b]), d, p.streaming);
            }
        }
}

// The same recombination for seven fp32 products (16-bit operands, fp32 result: the products are
// not rounded, as in the reference's Triton kernels, strassen.py:150-190): one thread per four
// consecutive columns of a half-size row.
template <int ALGO>
__global__ void __launch_bounds__(256) recombine32_kernel(const Recombine16Params p) {
    const int nq = p.Nh / 4;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.Mh * nq) return;
    const int i = (int)(idx / nq), j = (int)(idx % nq) * 4;
    const float* src = reinterpret_cast<const float*>(p.prod) + (int64_t)blockIdx.y * 7 * p.p_ps + (int64_t)i * p.Nh + j;
    f32x4 m[7];
#pragma unroll
    for (int q = 0; q < 7; ++q) m[q] = load_hinted(reinterpret_cast<const f32x4*>(src + q * p.p_ps), p.streaming);
    f32x4 out[4];
    if constexpr (ALGO == STHIP_STRASSEN) {
        out[0] = ((m[4] + m[6]) - m[2]) + m[3];   // C11 = M1 + M4 - M5 + M7
        out[1] = m[0] + m[2];                     // C12 = M3 + M5
        out[2] = m[5] + m[6];                     // C21 = M2 + M4
        out[3] = ((m[4] - m[5]) + m[0]) + m[1];   // C22 = M1 - M2 + M3 + M6
    } else {
        const f32x4 u2 = m[0] + m[2], u3 = u2 + m[3], u4 = u2 + m[4];
        out[0] = m[0] + m[1];                     // C11 = P1 + P2
        out[1] = u4 + m[5];                       // C12 = U4 + P3
        out[2] = u3 + m[6];                       // C21 = U3 - P4
        out[3] = u3 + m[4];                       // C22 = U3 + P5
    }
    float* Cf = reinterpret_cast<float*>(p.C) + (int64_t)blockIdx.y * p.c_bs;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        f32x4* d = reinterpret_cast<f32x4*>(Cf + (int64_t)(i + (q >> 1) * p.Mh) * p.c_rs + (j + (q & 1) * p.Nh));
        f32x4 v = out[q];
        if (p.accumulate) v += *d;
        *d = v;
    }
}

static bool fast_shape(int dt, int64_t Mh, int64_t Nh, int64_t Kh) {
    return dt != STHIP_F32 && Mh > 0 && Nh > 0 && Kh > 0 && Mh % 128 == 0 && Nh % 128 == 0 && Kh % kBK2 == 0;
}

__global__ void clear_flags5_kernel(unsigned* flags) {
    if (threadIdx.x < kFlagWords) flags[threadIdx.x] = 0;
}

// One Strassen level as ONE launch (sthip_kernel5.hpp).  Same workspace layout, same arithmetic and
// same bits as the three-launch form: five sums per operand, seven 16-bit products, fp32 recombination.
// Run order of the products: M3 M5 M2 M4 M1 M7 M6, so that C12 and C21 are complete after the second
// and the fourth product and recombine while the later products run; C11 and C22 follow at the end.
static int one_level_fused(View A, View B, char* C, int64_t c_rs, int64_t Mh, int64_t Nh, int64_t Kh, int dt,
                           bool a_kc, bool b_kc, char* ws, Call& cx) {
    const LaunchTable5* t5 = table5_for(dt);
    if (!t5) return 1;
    const int64_t a_ld = a_kc ? A.rs : A.cs, b_ld = b_kc ? B.cs : B.rs;
    const size_t sa_b = align256(Mh * Kh * 2), sb_b = align256(Kh * Nh * 2), pm_b = align256(Mh * Nh * 2);
    char* SA = ws;
    char* SB = ws + 5 * sa_b;
    char* PM = ws + 5 * (sa_b + sb_b);
    unsigned* flags = reinterpret_cast<unsigned*>(ws + prepass_body_bytes(1, Mh, Nh, Kh));
    const int64_t sa_ld = a_kc ? Kh : Mh, sb_ld = b_kc ? Kh : Nh;
    const char* Aq[4]; const char* Bq[4];
    for (int q = 0; q < 4; ++q) {
        Aq[q] = A.p + ((int64_t)(q >> 1) * Mh * A.rs + (int64_t)(q & 1) * Kh * A.cs) * 2;
        Bq[q] = B.p + ((int64_t)(q >> 1) * Kh * B.rs + (int64_t)(q & 1) * Nh * B.cs) * 2;
    }
    Fused5Params P;
    memset(&P, 0, sizeof(P));
    auto SAo = [&](int o) { return (const void*)(SA + (size_t)o * sa_b); };
    auto SBo = [&](int o) { return (const void*)(SB + (size_t)o * sb_b); };
    // products in run order; A sums S2 S3 S5 S7 S9 = SA 0..4, B sums S1 S4 S6 S8 S10 = SB 0..4
    P.g.seg[0] = Seg2{Aq[0], SBo(0), a_ld, sb_ld, 0, 0};     // M3 = A11 S1
    P.g.seg[1] = Seg2{SAo(0), Bq[3], sa_ld, b_ld, 0, 0};     // M5 = S2 B22
    P.g.seg[2] = Seg2{SAo(1), Bq[0], sa_ld, b_ld, 0, 0};     // M2 = S3 B11
    P.g.seg[3] = Seg2{Aq[3], SBo(1), a_ld, sb_ld, 0, 0};     // M4 = A22 S4
    P.g.seg[4] = Seg2{SAo(2), SBo(2), sa_ld, sb_ld, 0, 0};   // M1 = S5 S6
    P.g.seg[5] = Seg2{SAo(3), SBo(3), sa_ld, sb_ld, 0, 0};   // M7 = S7 S8
    P.g.seg[6] = Seg2{SAo(4), SBo(4), sa_ld, sb_ld, 0, 0};   // M6 = S9 S10
    P.g.C = PM; P.g.c_rs = Nh; P.g.c_ps = (int64_t)(pm_b / 2); P.g.c_bs = 0;
    P.g.Mh = (int)Mh; P.g.Nh = (int)Nh; P.g.Kh = (int)Kh;
    P.g.tiles_m = (int)(Mh / kBM4); P.g.tiles_n = (int)(Nh / kBN4);
    P.g.group_m = 4; P.g.nprod = 7; P.g.c_wide = 1;
    const int streaming = streaming_hint(prepass_bytes(1, Mh, Nh, Kh));
    P.g.c_stream = 0; P.streaming = streaming;   // the tiles are read again by the recombination items of this launch
    P.tiles = P.g.tiles_m * P.g.tiles_n;
    P.flags = flags;
    P.c_rs = c_rs; P.rec_rows = (int)Mh; P.rec_chunks = (int)(Nh / 8);

    // element-wise work is cut into units of about 2.5 MB (half the time of a tile at the ~50 GB/s one
    // CU streams); what must be complete before anything else can start runs on every CU at once
    auto units_for = [](double bytes) { return (int)std::max<int64_t>(8, round_up((int64_t)(bytes / 2.5e6), 8)); };
    const int everywhere = 256;
    auto fill_job = [&](SumJob5& J, bool a_side, const int* outs, int nout, int units) {
        const int64_t r_ext = a_side ? (a_kc ? Mh : Kh) : (b_kc ? Nh : Kh);
        const int64_t c_ext = a_side ? (a_kc ? Kh : Mh) : (b_kc ? Kh : Nh);
        J.ld_in = a_side ? a_ld : b_ld; J.ld_out = a_side ? sa_ld : sb_ld;
        J.rows = (int)r_ext; J.chunks_per_row = (int)(c_ext / 8); J.nout = nout;
        J.units = (int)std::min<int64_t>(units, r_ext);
        bool used[4] = {false, false, false, false};
        for (int o = 0; o < nout; ++o) {
            J.out[o] = a_side ? SA + (size_t)outs[o] * sa_b : SB + (size_t)outs[o] * sb_b;
            for (int q = 0; q < 4; ++q) {
                J.coef[o][q] = a_side ? kStrA[outs[o]][q] : kStrB[outs[o]][q];
                if (J.coef[o][q]) used[q] = true;
            }
        }
        for (int q = 0; q < 4; ++q) J.q[q] = used[q] ? (a_side ? Aq[q] : Bq[q]) : nullptr;
    };
    const double a_blk = (double)Mh * Kh * 2, b_blk = (double)Kh * Nh * 2, c_blk = (double)Mh * Nh * 2;
    static const int kS1[1] = {0}, kAall[5] = {0, 1, 2, 3, 4}, kBrest[4] = {1, 2, 3, 4};
    fill_job(P.job[0], false, kS1, 1, everywhere);
    fill_job(P.job[1], true, kAall, 5, units_for(9 * a_blk));
    fill_job(P.job[2], false, kBrest, 4, units_for(8 * b_blk));
    P.njobs = 3;
    auto prod_ptr = [&](int p) { return (const void*)(PM + (size_t)p * pm_b); };
    auto fill_rec = [&](RecJob5& R, int quad, std::initializer_list<int> prods, std::initializer_list<int> signs, int units) {
        int t = 0;
        for (int p : prods) R.m[t++] = prod_ptr(p);
        t = 0;
        for (int sg : signs) R.sign[t++] = (signed char)sg;
        R.nterms = (int)prods.size();
        R.c = C + ((int64_t)(quad >> 1) * Mh * c_rs + (int64_t)(quad & 1) * Nh) * 2;
        R.units = (int)std::min<int64_t>(units, Mh);
    };
    fill_rec(P.rec[0], 1, {0, 1}, {1, 1}, units_for(3 * c_blk));                 // C12 = M3 + M5
    fill_rec(P.rec[1], 2, {2, 3}, {1, 1}, units_for(3 * c_blk));                 // C21 = M2 + M4
    fill_rec(P.rec[2], 0, {4, 3, 1, 5}, {1, 1, -1, 1}, everywhere);              // C11 = M1 + M4 - M5 + M7
    fill_rec(P.rec[3], 3, {4, 2, 0, 6}, {1, -1, 1, 1}, everywhere);              // C22 = M1 - M2 + M3 + M6

    int n = 0, next = 0;
    auto add = [&](int kind, int arg, int count, unsigned need_jobs, unsigned need_prods) {
        P.item[n] = Item5{next, kind, arg, need_jobs, need_prods};
        next += (int)round_up(count, 8);   // the XCD of a workgroup is its index modulo eight: keep items aligned
        ++n;
    };
    add(kItemSums, 0, P.job[0].units, 0, 0);
    add(kItemSums, 1, P.job[1].units, 0, 0);
    add(kItemTiles, 0, P.tiles, 1u << 0, 0);
    add(kItemSums, 2, P.job[2].units, 0, 0);
    add(kItemTiles, 1, P.tiles, 1u << 1, 0);
    add(kItemTiles, 2, P.tiles, 1u << 1, 0);
    add(kItemRecombine, 0, P.rec[0].units, 0, (1u << 0) | (1u << 1));
    add(kItemTiles, 3, P.tiles, 1u << 2, 0);
    add(kItemTiles, 4, P.tiles, (1u << 1) | (1u << 2), 0);
    add(kItemRecombine, 1, P.rec[1].units, 0, (1u << 2) | (1u << 3));
    add(kItemTiles, 5, P.tiles, (1u << 1) | (1u << 2), 0);
    add(kItemTiles, 6, P.tiles, (1u << 1) | (1u << 2), 0);
    add(kItemRecombine, 2, P.rec[2].units, 0, (1u << 4) | (1u << 3) | (1u << 1) | (1u << 5));
    add(kItemRecombine, 3, P.rec[3].units, 0, (1u << 4) | (1u << 2) | (1u << 0) | (1u << 6));
    P.nitems = n;

    hipLaunchKernelGGL(clear_flags5_kernel, dim3(1), dim3(64), 0, cx.stream, flags);
    int rc = check_launch("clear_flags");
    if (rc) return rc;
    hipError_t e = t5->fn[b_kc ? 1 : 0](P, next, cx.stream);
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
    return STHIP_OK;
}

// The pipelined path: optional quadrant-sum pre-pass into `ws`, then one grouped-GEMM launch.
// Returns 1 if the problem does not qualify (the caller then takes the fused kernel).
static int launch_pipelined(View A, View B, char* C, int64_t c_rs, int64_t batch, int64_t a_bs, int64_t b_bs,
                            int64_t c_bs, int64_t Mh, int64_t Nh, int64_t Kh, int dt, bool out_f32, int algo,
                            bool accumulate, bool a_kc, bool b_kc, char* ws, size_t ws_bytes, Call& cx) {
    const bool split = algo != STHIP_CLASSIC;
    if (split && (!ws || !aligned_to(ws, 256) || ws_bytes < prepass_bytes(batch, Mh, Nh, Kh))) return 1;
    const int64_t a_ld = a_kc ? A.rs : A.cs, b_ld = b_kc ? B.cs : B.rs;
    Gemm2Params p;
    memset(&p, 0, sizeof(p));
    p.C = C; p.c_rs = c_rs; p.c_bs = c_bs;
    p.Mh = (int)Mh; p.Nh = (int)Nh; p.Kh = (int)Kh;
    p.tiles_m = (int)(Mh / 128); p.tiles_n = (int)(Nh / 128);
    p.out_f32 = out_f32 ? 1 : 0; p.accumulate = accumulate ? 1 : 0; p.group_m = 8;
    // raw quadrants in place
    const char* Aq[4]; const char* Bq[4];
    for (int q = 0; q < 4; ++q) {
        Aq[q] = A.p + ((int64_t)(q >> 1) * Mh * A.rs + (int64_t)(q & 1) * Kh * A.cs) * 2;
        Bq[q] = B.p + ((int64_t)(q >> 1) * Kh * B.rs + (int64_t)(q & 1) * Nh * B.cs) * 2;
    }
    // Fixed tile table.  Bytes moved L2 -> LDS per flop go with 1/BM + 1/BN, so the largest tile
    // that still gives every CU work wins.  256 x 256 holds one accumulator per wave and nothing
    // else: a classical product runs on it directly, a Strassen / Winograd level runs its seven
    // products on it as one grouped launch into 16-bit product matrices (the reference's own
    // cast schedule) followed by the recombination pass.  256 x 128 (two accumulators in
    // registers, one parked) and 128 x 128 (three in registers) recombine in registers and serve
    // fp32 results and the sizes that are too small for the large tile.  The large tiles need A
    // contiguous along k; the recombination pass needs 16-byte aligned rows of C.
    const LaunchTable3* t3 = table3_for(dt, algo);
    const LaunchTable3* t4 = table4_for(dt);
    const int force = cx.force_tile;
    const bool c_vec = c_rs % 8 == 0 && c_bs % 8 == 0 && aligned_to(C, 16);
    // products as matrices + recombination pass: 16-bit products for a result in the operand type,
    // fp32 products (twice the room) for an fp32 result
    const bool f32_prod = split && out_f32 && c_rs % 4 == 0 && c_bs % 4 == 0 && aligned_to(C, 16) &&
                          ws_bytes >= prepass_bytes(batch, Mh, Nh, Kh, 4);
    const bool grouped_ok = !split || (out_f32 ? f32_prod : c_vec);
    const bool can4 = a_kc && Mh % kBM4 == 0 && Nh % kBN4 == 0 && t4 && grouped_ok;
    const bool can3 = a_kc && Mh % kBM3 == 0 && t3;
    const bool can5 = split && !out_f32 && grouped_ok;
    const int64_t tiles4 = (Mh / kBM4) * (Nh / kBN4) * batch * (split ? 7 : 1);
    const int64_t tiles3 = (Mh / kBM3) * (Nh / kBN3) * batch;
    const int64_t tiles2 = (Mh / 128) * (Nh / 128) * batch;
    // Measured on MI355X (bf16): the 256 x 256 grouped path wins from 4096^3 up when k is long
    // enough to pay for writing the sums and the products (its extra passes cost bytes
    // ~ MK + KN + MN, the products flops ~ MNK); when the 128 x 128 tiles of ONE product cannot
    // fill the 256 CUs (small matrices, weight gradients with short M and N) the seven products
    // side by side can, and that launch is 2 - 4 x faster; otherwise recombining in registers
    // (no product round trip) is as fast or faster.
    int pick = 2;
    if (can4 && tiles4 >= (split ? 400 : 224) && (!split || Kh >= 1024)) pick = 4;
    else if (can5 && tiles2 < 256) pick = 5;
    else if (can3 && tiles3 >= (split ? 256 : 176)) pick = 3;   // classical: 192 tiles of 256 x 128 beat 384 of 128 x 128 (8192 x 768 x 2304: 39.7 against 45.9 us), 128 do not
    if (force == 4 && can4) pick = 4;
    else if (force == 3 && can3) pick = 3;
    else if (force == 5 && can5) pick = 5;
    else if (force == 2) pick = 2;
    // one level on the large tile, plain result in the operand type: everything as work items of one launch
    if (pick == 4 && split && algo == STHIP_STRASSEN && !out_f32 && !accumulate && batch == 1 && (cx.stages & 16) &&
        (cx.stages & 7) == 7 && !(cx.bias.bias && cx.bias.target == C) && !cx.prep.sums && table5_for(dt))
        return one_level_fused(A, B, C, c_rs, Mh, Nh, Kh, dt, a_kc, b_kc, ws, cx);
    hipError_t e = hipSuccess;
    if (!split) {
        p.seg[0] = {A.p, B.p, a_ld, b_ld, a_bs, b_bs};
    } else {
        const size_t sa_b = align256(Mh * Kh * 2), sb_b = align256(Kh * Nh * 2);
        char* SA = ws;                                // [5][batch] blocks of Mh x Kh (storage order of A)
        char* SB = ws + (size_t)batch * 5 * sa_b;
        const char* ready = algo == STHIP_STRASSEN && batch == 1 && b_kc ? take_prepared(cx, B.p, 1, Kh, Nh, 5 * sb_b) : nullptr;
        if (ready) SB = const_cast<char*>(ready);     // B-side sums formed ahead of the call: read, never written
        // region after the sums: parked fp32 tiles (256 x 128 kernel) or the seven 16-bit products (grouped paths)
        p.park = reinterpret_cast<float*>(ws + (size_t)batch * 5 * (sa_b + sb_b));
        const int64_t sa_ld = a_kc ? Kh : Mh, sb_ld = b_kc ? Kh : Nh;
        const int nout = algo == STHIP_STRASSEN ? 5 : 4;
        if (cx.stages & 1) {
            ComboPair pp;
            memset(&pp, 0, sizeof(pp));
            int64_t most = 0;
            const int sides = ready ? 1 : 2;
            for (int side = 0; side < sides; ++side) {
                ComboParams& cp = pp.side[side];
                cp.streaming = streaming_hint(prepass_bytes(batch, Mh, Nh, Kh));
                const int64_t r_ext = side == 0 ? (a_kc ? Mh : Kh) : (b_kc ? Nh : Kh);
                const int64_t c_ext = side == 0 ? (a_kc ? Kh : Mh) : (b_kc ? Kh : Nh);
                for (int q = 0; q < 4; ++q) cp.q[q] = side == 0 ? Aq[q] : Bq[q];
                for (int o = 0; o < nout; ++o) {
                    cp.out[o] = (side == 0 ? SA + (size_t)o * batch * sa_b : SB + (size_t)o * batch * sb_b);
                    for (int q = 0; q < 4; ++q)
                        cp.coef[o][q] = algo == STHIP_STRASSEN ? (side == 0 ? kStrA[o][q] : kStrB[o][q])
                                                               : (side == 0 ? kWinA[o][q] : kWinB[o][q]);
                }
                cp.ld_in = side == 0 ? a_ld : b_ld;
                cp.bs_in = side == 0 ? a_bs : b_bs;
                cp.ld_out = side == 0 ? sa_ld : sb_ld;
                cp.bs_out = (int64_t)((side == 0 ? sa_b : sb_b) / 2);
                cp.nout = nout; cp.rows = (int)r_ext; cp.chunks_per_row = (int)(c_ext / 8);
                cp.table = (algo == STHIP_STRASSEN ? 0 : 2) + side;
                most = std::max(most, r_ext * (c_ext / 8));
            }
            dim3 grid((unsigned)ceil_div(most, 256), (unsigned)batch, (unsigned)sides);
            if (dt == STHIP_BF16) hipLaunchKernelGGL(quad_combos_pair_kernel<bf16_t>, grid, dim3(256), 0, cx.stream, pp);
            else hipLaunchKernelGGL(quad_combos_pair_kernel<f16_t>, grid, dim3(256), 0, cx.stream, pp);
            int rc = check_launch("quad_combos");
            if (rc) return rc;
        }
        const int64_t sa_bs = (int64_t)(sa_b / 2), sb_bs = (int64_t)(sb_b / 2);
        auto SAo = [&](int o) { return (const void*)(SA + (size_t)o * batch * sa_b); };
        auto SBo = [&](int o) { return (const void*)(SB + (size_t)o * batch * sb_b); };
        auto set = [&](int i, const void* a, int64_t ald, int64_t abs_, const void* b, int64_t bld, int64_t bbs) {
            p.seg[i] = {a, b, ald, bld, abs_, bbs};
        };
        if (algo == STHIP_STRASSEN) {
            // kernel order M3 M6 M5 M7 M1 M2 M4; A sums S2 S3 S5 S7 S9 = outputs 0..4, B sums S1 S4 S6 S8 S10
            set(0, Aq[0], a_ld, a_bs, SBo(0), sb_ld, sb_bs);      // M3 = A11 S1
            set(1, SAo(4), sa_ld, sa_bs, SBo(4), sb_ld, sb_bs);   // M6 = S9 S10
            set(2, SAo(0), sa_ld, sa_bs, Bq[3], b_ld, b_bs);      // M5 = S2 B22
            set(3, SAo(3), sa_ld, sa_bs, SBo(3), sb_ld, sb_bs);   // M7 = S7 S8
            set(4, SAo(2), sa_ld, sa_bs, SBo(2), sb_ld, sb_bs);   // M1 = S5 S6
            set(5, SAo(1), sa_ld, sa_bs, Bq[0], b_ld, b_bs);      // M2 = S3 B11
            set(6, Aq[3], a_ld, a_bs, SBo(1), sb_ld, sb_bs);      // M4 = A22 S4
        } else {
            // kernel order P1 P2 P6 P7 P5 P3 -P4; A outputs S1..S4 = 0..3, B outputs T1 T2 T3 -T4 = 0..3
            set(0, Aq[0], a_ld, a_bs, Bq[0], b_ld, b_bs);         // P1 = A11 B11
            set(1, Aq[1], a_ld, a_bs, Bq[2], b_ld, b_bs);         // P2 = A12 B21
            set(2, SAo(1), sa_ld, sa_bs, SBo(1), sb_ld, sb_bs);   // P6 = S2 T2
            set(3, SAo(2), sa_ld, sa_bs, SBo(2), sb_ld, sb_bs);   // P7 = S3 T3
            set(4, SAo(0), sa_ld, sa_bs, SBo(0), sb_ld, sb_bs);   // P5 = S1 T1
            set(5, SAo(3), sa_ld, sa_bs, Bq[3], b_ld, b_bs);      // P3 = S4 B22
            set(6, Aq[3], a_ld, a_bs, SBo(3), sb_ld, sb_bs);      // -P4 = A22 (-T4)
        }
    }
    if ((pick == 4 || pick == 5) && split) {
        Recombine16Params rp;
        rp.prod = p.park; rp.C = C; rp.c_rs = c_rs; rp.c_bs = c_bs;
        rp.Mh = (int)Mh; rp.Nh = (int)Nh; rp.accumulate = accumulate ? 1 : 0; rp.p_ps = Mh * Nh; rp.out_f32 = out_f32 ? 1 : 0;
        rp.streaming = streaming_hint(prepass_bytes(batch, Mh, Nh, Kh, out_f32 ? 4 : 2));
        if (batch == 1 && (cx.stages & 4)) rp.bias = take_bias(cx, C, accumulate, out_f32);
        if (cx.stages & 2) {
            p.C = p.park; p.c_rs = Nh; p.c_ps = Mh * Nh; p.c_bs = 7 * Mh * Nh;
            p.out_f32 = out_f32 ? 1 : 0; p.accumulate = 0; p.nprod = 7;
            p.c_stream = rp.streaming;
            if (pick == 4) {
                p.tiles_m = (int)(Mh / kBM4); p.tiles_n = (int)(Nh / kBN4);
                p.group_m = 4;
                p.c_wide = wide_rows(p.C, p.c_rs, p.c_ps, p.c_bs);
                p.one_tile_per_wg = (cx.stages & 32) ? 1 : 0;
                e = t4->fn[b_kc ? 1 : 0](p, (int)batch, cx.stream);
            } else {
                const LaunchTable2* t = table2_for(dt, STHIP_CLASSIC);
                if (!t) return 1;
                e = t->fn[a_kc ? 1 : 0][b_kc ? 1 : 0](p, (int)batch, cx.stream);
            }
            if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
        }
        if ((cx.stages & 4) && out_f32) {
            dim3 grid((unsigned)ceil_div(Mh * (Nh / 4), 256), (unsigned)batch);
            if (algo == STHIP_STRASSEN) hipLaunchKernelGGL(recombine32_kernel<STHIP_STRASSEN>, grid, dim3(256), 0, cx.stream, rp);
            else hipLaunchKernelGGL(recombine32_kernel<STHIP_WINOGRAD>, grid, dim3(256), 0, cx.stream, rp);
            return check_launch("recombine32");
        }
        if (cx.stages & 4) {
            dim3 grid((unsigned)ceil_div(Mh * (Nh / 8), 256), (unsigned)batch);
#define GO(T, A) hipLaunchKernelGGL((recombine16_kernel<T, A>), grid, dim3(256), 0, cx.stream, rp)
            if (dt == STHIP_BF16) { if (algo == STHIP_STRASSEN) GO(bf16_t, STHIP_STRASSEN); else GO(bf16_t, STHIP_WINOGRAD); }
            else { if (algo == STHIP_STRASSEN) GO(f16_t, STHIP_STRASSEN); else GO(f16_t, STHIP_WINOGRAD); }
#undef GO
            return check_launch("recombine16");
        }
        return STHIP_OK;
    }
    if (!(cx.stages & 2)) return STHIP_OK;
    if (pick == 4) {
        p.tiles_m = (int)(Mh / kBM4); p.tiles_n = (int)(Nh / kBN4);
        p.group_m = 4; p.nprod = 1;
        p.c_stream = 1;   // the final result: not read again by this call
        p.c_wide = wide_rows(p.C, p.c_rs, 0, p.c_bs);
        p.one_tile_per_wg = (cx.stages & 32) ? 1 : 0;
        e = t4->fn[b_kc ? 1 : 0](p, (int)batch, cx.stream);
    } else if (pick == 3) {
        p.tiles_m = (int)(Mh / kBM3);
        p.group_m = 4;
        e = t3->fn[b_kc ? 1 : 0](p, (int)batch, cx.stream);
    } else {
        const LaunchTable2* t = table2_for(dt, algo);
        if (!t) return 1;
        e = t->fn[a_kc ? 1 : 0][b_kc ? 1 : 0](p, (int)batch, cx.stream);
    }
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
    return STHIP_OK;
}

// One fused launch: C (+)= A x B with zero or one Strassen / Winograd level.
// (Mh, Nh, Kh) is the block size used for the split; pass 0 to derive it from the sizes.
static size_t f32_batched_bytes(int64_t Mh, int64_t Nh, int64_t Kh) {
    return 7 * (align256(Mh * Kh * 4) + align256(Kh * Nh * 4) + align256(Mh * Nh * 4));
}
static int one_level_f32_batched(View A, View B, char* C, int64_t c_rs, int64_t Mh, int64_t Nh, int64_t Kh,
                                 bool accumulate, char* ws, Call& cx);
static int one_level_f32_grouped(View A, View B, char* C, int64_t c_rs, int64_t Mh, int64_t Nh, int64_t Kh,
                                 int algo, bool accumulate, char* ws, Call& cx);
static bool f32_small_shape(View A, View B, int64_t Mh, int64_t Nh, int64_t Kh);
static int one_level_f32_small(View A, View B, char* C, int64_t c_rs, int64_t Mh, int64_t Nh, int64_t Kh,
                               bool accumulate, char* ws, Call& cx);

static int launch_fused(View A, View B, char* C, int64_t c_rs, int64_t c_cs,
                        int64_t batch, int64_t a_bs, int64_t b_bs, int64_t c_bs,
                        int64_t M, int64_t N, int64_t K, int64_t Mh, int64_t Nh, int64_t Kh,
                        int dt, bool out_f32, int algo, bool accumulate, char* ws, size_t ws_bytes,
                        Call& cx) {
    if (M == 0 || N == 0 || batch == 0) return STHIP_OK;
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || batch > 65535)
        return fail(STHIP_ERR_SHAPE, "size out of range (M=%lld N=%lld K=%lld batch=%lld)",
                    (long long)M, (long long)N, (long long)K, (long long)batch);
    if (dt == STHIP_F32 && !out_f32) return fail(STHIP_ERR_DTYPE, "fp32 operands need an fp32 result");
    const int es = elem_size(dt), epc = 16 / es, bk = 8 * epc;
    if (algo == STHIP_CLASSIC) { Mh = M; Nh = N; Kh = K; }
    else {
        if (Mh <= 0) Mh = ceil_div(M, 2);
        if (Nh <= 0) Nh = ceil_div(N, 2);
        if (Kh <= 0) Kh = ceil_div(K, 2);
    }
    // operand layouts: contiguous along k, or along m/n
    const bool a_kc = (A.cs == 1), b_kc = (B.rs == 1);
    if (!a_kc && A.rs != 1) return fail(STHIP_ERR_LAYOUT, "A has no unit stride (row %lld, col %lld)", (long long)A.rs, (long long)A.cs);
    if (!b_kc && B.cs != 1) return fail(STHIP_ERR_LAYOUT, "B has no unit stride (row %lld, col %lld)", (long long)B.rs, (long long)B.cs);

    GemmParams p;
    memset(&p, 0, sizeof(p));
    p.A = A.p; p.B = B.p; p.C = C;
    p.a_rs = A.rs; p.a_cs = A.cs; p.a_bs = a_bs;
    p.b_rs = B.rs; p.b_cs = B.cs; p.b_bs = b_bs;
    p.c_rs = c_rs; p.c_cs = c_cs; p.c_bs = c_bs;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    p.Mh = (int)Mh; p.Nh = (int)Nh; p.Kh = (int)Kh;
    p.tiles_m = (int)ceil_div(Mh, kBM);
    p.tiles_n = (int)ceil_div(Nh, kBN);
    p.out_f32 = out_f32 ? 1 : 0;
    p.accumulate = accumulate ? 1 : 0;
    p.group_m = 8;

    // 16-byte loads are legal when the base, the long stride, the batch stride and every
    // block origin along the contiguous index are multiples of one chunk.
    const bool split = algo != STHIP_CLASSIC;
    const int64_t a_long = a_kc ? A.rs : A.cs, b_long = b_kc ? B.cs : B.rs;
    const int64_t a_blk = a_kc ? Kh : Mh, b_blk = b_kc ? Kh : Nh;
    p.a_vec = aligned_to(A.p, 16) && a_long % epc == 0 && (batch == 1 || a_bs % epc == 0) && (!split || a_blk % epc == 0);
    p.b_vec = aligned_to(B.p, 16) && b_long % epc == 0 && (batch == 1 || b_bs % epc == 0) && (!split || b_blk % epc == 0);
    const size_t c_es = out_f32 ? 4 : es;
    p.c_vec = c_cs == 1 && aligned_to(C, 4 * c_es) && c_rs % 4 == 0 && (batch == 1 || c_bs % 4 == 0) && (!split || Nh % 4 == 0);

    const bool whole = !split || (M == 2 * Mh && N == 2 * Nh && K == 2 * Kh);
    const bool fast = whole && Mh % kBM == 0 && Nh % kBN == 0 && Kh % bk == 0 && Kh > 0 && p.a_vec && p.b_vec && p.c_vec;

    if (fast && fast_shape(dt, Mh, Nh, Kh) && a_long % 8 == 0 && b_long % 8 == 0) {
        int rc = launch_pipelined(A, B, C, c_rs, batch, a_bs, b_bs, c_bs, Mh, Nh, Kh, dt, out_f32, algo, accumulate,
                                  a_kc, b_kc, ws, ws_bytes, cx);
        if (rc <= 0) return rc;
    }
    // fp32 on the 256 x 256 pipelined kernel (A contiguous along k, enough tiles to fill the chip):
    // a classical product directly; one Strassen level as sums, ONE grouped launch of the seven
    // products and the recombination pass.  Measured at 8192^3: the classical product runs at
    // 142 TFLOP/s against 85 on the fused kernel.
    if (fast && dt == STHIP_F32 && a_kc && Mh % kBM4 == 0 && Nh % kBN4 == 0 && Kh % 32 == 0 && cx.force_tile != 2) {
        const int64_t tiles4 = (Mh / kBM4) * (Nh / kBN4) * batch;
        if (!split && tiles4 >= 224) {
            Gemm2Params g;
            memset(&g, 0, sizeof(g));
            g.seg[0] = Seg2{A.p, B.p, A.rs, b_kc ? B.cs : B.rs, a_bs, b_bs};
            g.C = C; g.c_rs = c_rs; g.c_bs = c_bs;
            g.Mh = (int)Mh; g.Nh = (int)Nh; g.Kh = (int)Kh;
            g.tiles_m = (int)(Mh / kBM4); g.tiles_n = (int)(Nh / kBN4);
            g.out_f32 = 1; g.accumulate = accumulate ? 1 : 0; g.group_m = 4; g.nprod = 1; g.c_stream = 1;
            hipError_t e = table4_for(dt)->fn[b_kc ? 1 : 0](g, (int)batch, cx.stream);
            if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
            return STHIP_OK;
        }
        if (split && batch == 1 && 7 * tiles4 >= 224 && ws && aligned_to(ws, 256) &&
            ws_bytes >= f32_batched_bytes(Mh, Nh, Kh))
            return one_level_f32_grouped(A, B, C, c_rs, Mh, Nh, Kh, algo, accumulate, ws, cx);
    }
    // fp32 classical product too small for the 256 x 256 kernel: 64 x 64 tiles (sthip_kernel6.hpp, one
    // product, no sums).  Measured against the 128 x 128 fused kernel: 1024^3 0.098 -> 0.03 ms.
    if (fast && dt == STHIP_F32 && !split && batch == 1 && cx.force_tile != 2 && f32_small_shape(A, B, Mh, Nh, Kh)) {
        Gemm6Params g;
        memset(&g, 0, sizeof(g));
        g.a[0] = Op6{reinterpret_cast<const float*>(A.p), nullptr, A.rs, 0, 0};
        g.b[0] = Op6{reinterpret_cast<const float*>(B.p), nullptr, b_kc ? B.cs : B.rs, 0, 0};
        g.C = reinterpret_cast<float*>(C); g.c_rs = c_rs; g.c_ps = 0;
        g.Kh = (int)Kh; g.tiles_m = (int)(Mh / kBM6); g.tiles_n = (int)(Nh / kBN6); g.nprod = 1;
        g.accumulate = accumulate ? 1 : 0;
        hipError_t e = launch_gemm6(g, b_kc, cx.stream);
        if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
        return STHIP_OK;
    }
    // fp32, one Strassen level: run the seven products side by side as a batch (see
    // one_level_f32_batched).  Measured against the fused kernel: 5 x faster at 1024^3 (one product
    // has 16 tiles for 256 CUs), 3 x at 2048^3, equal at 4096^3, 10 % faster at 8192^3.
    if (fast && dt == STHIP_F32 && algo == STHIP_STRASSEN && batch == 1 && ws && aligned_to(ws, 256) &&
        ws_bytes >= f32_batched_bytes(Mh, Nh, Kh) && cx.force_tile != 2) {
        // small products: 64 x 64 tiles with the sums formed in the operand loads (two launches);
        // measured against the batched form below: see one_level_f32_small
        if (f32_small_shape(A, B, Mh, Nh, Kh) && (cx.force_tile == 6 || (cx.force_tile == 0 && Mh * Nh <= (int64_t)1024 * 1024)))
            return one_level_f32_small(A, B, C, c_rs, Mh, Nh, Kh, accumulate, ws, cx);
        return one_level_f32_batched(A, B, C, c_rs, Mh, Nh, Kh, accumulate, ws, cx);
    }
    const LaunchTable* t = table_for(dt, algo);
    if (!t) return fail(STHIP_ERR_ARG, "bad dtype/algo (%d, %d)", dt, algo);
    hipError_t e = t->fn[a_kc ? 1 : 0][b_kc ? 1 : 0][fast ? 0 : 1](p, (int)batch, cx.stream);
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
    return STHIP_OK;
}

// ------------------------------------------------------------------ element-wise kernels
template <class T> __device__ __forceinline__ float ld_elem(const char* p, int64_t i);
template <> __device__ __forceinline__ float ld_elem<float>(const char* p, int64_t i) { return reinterpret_cast<const float*>(p)[i]; }
template <> __device__ __forceinline__ float ld_elem<bf16_t>(const char* p, int64_t i) {
    return __builtin_bit_cast(float, (uint32_t)reinterpret_cast<const uint16_t*>(p)[i] << 16);
}
template <> __device__ __forceinline__ float ld_elem<f16_t>(const char* p, int64_t i) {
    return (float)__builtin_bit_cast(_Float16, reinterpret_cast<const uint16_t*>(p)[i]);
}
template <class T> __device__ __forceinline__ void st_elem(char* p, int64_t i, float v);
template <> __device__ __forceinline__ void st_elem<float>(char* p, int64_t i, float v) { reinterpret_cast<float*>(p)[i] = v; }
template <> __device__ __forceinline__ void st_elem<bf16_t>(char* p, int64_t i, float v) {
    reinterpret_cast<uint16_t*>(p)[i] = (uint16_t)pack_bf16(v, 0.f);
}
template <> __device__ __forceinline__ void st_elem<f16_t>(char* p, int64_t i, float v) {
    reinterpret_cast<uint16_t*>(p)[i] = (uint16_t)pack_f16(v, 0.f);
}

// dst[rows x cols] (dense) = X[block a] + sign * X[block b], each block clipped to the
// logical extent (lim_r, lim_c) of X and read as zero outside it.  sign = 0: copy block a.
// The sum is formed in fp32 and rounded once (fixed_strassen_fp32_agg.py:87-96).
// TO = float with a 16-bit T: the sum is rounded to T all the same and stored widened, exactly.
template <class T, class TO = T>
__global__ void block_sum_kernel(char* dst, const char* X, int64_t rs, int64_t cs,
                                 int ra, int ca, int rb, int cb, int sign,
                                 int rows, int cols, int lim_r, int lim_c) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)rows * cols) return;
    const int i = (int)(idx / cols), j = (int)(idx % cols);
    float v = 0.f;
    if (ra + i < lim_r && ca + j < lim_c) v = ld_elem<T>(X, (int64_t)(ra + i) * rs + (int64_t)(ca + j) * cs);
    if (sign != 0 && rb + i < lim_r && cb + j < lim_c) {
        const float w = ld_elem<T>(X, (int64_t)(rb + i) * rs + (int64_t)(cb + j) * cs);
        v = sign > 0 ? v + w : v - w;
    }
    if constexpr (__is_same(T, TO)) st_elem<T>(dst, idx, v);
    else st_elem<TO>(dst, idx, round16<T>(v));
}

// C blocks from the seven products (dense fp32, mh x nh each):
// C11 = M1+M4-M5+M7, C12 = M3+M5, C21 = M2+M4, C22 = M1-M2+M3+M6 (fixed_strassen.py:116-119),
// clipped to M x N, rounded once to the output type.
template <class TO>
__global__ void recombine_kernel(char* C, int64_t c_rs, int64_t c_cs, const float* Mbuf, int64_t mstride,
                                 int mh, int nh, int M, int N, int accumulate) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)mh * nh) return;
    const int i = (int)(idx / nh), j = (int)(idx % nh);
    float m[7];
#pragma unroll
    for (int q = 0; q < 7; ++q) m[q] = Mbuf[q * mstride + idx];
    const float c11 = m[0] + m[3] - m[4] + m[6];
    const float c12 = m[2] + m[4];
    const float c21 = m[1] + m[3];
    const float c22 = m[0] - m[1] + m[2] + m[5];
    const float out[4] = {c11, c12, c21, c22};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int r = i + (q >> 1) * mh, c = j + (q & 1) * nh;
        if (r >= M || c >= N) continue;
        const int64_t off = (int64_t)r * c_rs + (int64_t)c * c_cs;
        float v = out[q];
        if (accumulate) v += ld_elem<TO>(C, off);
        st_elem<TO>(C, off, v);
    }
}

template <class T>
__global__ void add_bias_kernel(char* y, const char* bias, int64_t rows, int64_t D) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * D) return;
    st_elem<T>(y, idx, ld_elem<T>(y, idx) + ld_elem<T>(bias, idx % D));
}

__global__ void transpose_read_probe_kernel(uint16_t* out) {
    __shared__ __attribute__((aligned(16))) uint16_t lds[256];
    const int lane = threadIdx.x;
    for (int e = 0; e < 4; ++e) lds[lane * 4 + e] = (uint16_t)(lane * 4 + e);
    __syncthreads();
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(lds + lane * 4));
    for (int e = 0; e < 4; ++e) out[lane * 4 + e] = (uint16_t)v[e];
}

static int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "%s launch failed: %s", what, hipGetErrorString(e));
    return STHIP_OK;
}

// All quadrant sums of one operand in one launch (see quad_combos_kernel).  X is the operand,
// (r_blk, c_blk) the block size in its logical (row, col) indexing; outputs are dense blocks in
// the storage orientation of X, `out_stride` bytes apart.
static bool combos_ok(View X, int64_t r_blk, int64_t c_blk, int es = 2) {
    const int epc = 16 / es;
    if (!aligned_to(X.p, 16)) return false;
    if (X.cs == 1) return c_blk % epc == 0 && X.rs % epc == 0;
    if (X.rs == 1) return r_blk % epc == 0 && X.cs % epc == 0;
    return false;
}

static int64_t fill_combo(ComboParams& cp, View X, int64_t r_blk, int64_t c_blk, char* out, size_t out_stride,
                          int nout, const signed char (*coef)[4], int es = 2) {
    memset(&cp, 0, sizeof(cp));
    const bool row_major = X.cs == 1;
    const int epc = 16 / es;   // elements per 16-byte chunk
    for (int q = 0; q < 4; ++q)
        cp.q[q] = X.p + ((int64_t)(q >> 1) * r_blk * X.rs + (int64_t)(q & 1) * c_blk * X.cs) * es;
    for (int o = 0; o < nout; ++o) {
        cp.out[o] = out + (size_t)o * out_stride;
        for (int q = 0; q < 4; ++q) cp.coef[o][q] = coef[o][q];
    }
    const int64_t rows = row_major ? r_blk : c_blk, cols = row_major ? c_blk : r_blk;   // storage order
    cp.ld_in = row_major ? X.rs : X.cs;
    cp.ld_out = cols;
    cp.nout = nout; cp.rows = (int)rows; cp.chunks_per_row = (int)(cols / epc);
    cp.table = coef == kStrA ? 0 : coef == kStrB ? 1 : coef == kWinA ? 2 : coef == kWinB ? 3 : -1;
    return rows * (cols / epc);
}

static int run_combos(int dt, View X, int64_t r_blk, int64_t c_blk, char* out, size_t out_stride, int nout,
                      const signed char (*coef)[4], Call& cx) {
    ComboParams cp;
    const int64_t n = fill_combo(cp, X, r_blk, c_blk, out, out_stride, nout, coef);
    if (n == 0) return STHIP_OK;
    cp.streaming = streaming_hint((size_t)(nout + 4) * out_stride);
    dim3 grid((unsigned)ceil_div(n, 256), 1);
    if (dt == STHIP_BF16) hipLaunchKernelGGL(quad_combos_kernel<bf16_t>, grid, dim3(256), 0, cx.stream, cp);
    else hipLaunchKernelGGL(quad_combos_kernel<f16_t>, grid, dim3(256), 0, cx.stream, cp);
    return check_launch("quad_combos");
}

// Operand pairs of the seven products of one level, in kernel order (Strassen M3 M6 M5 M7 M1 M2 M4,
// Winograd P1 P2 P6 P7 P5 P3 -P4).  X is mh x kh blocks of A, Y is kh x nh blocks of B; a raw
// quadrant is a view into the operand, a sum is dense in the operand's storage orientation at
// S? + index * stride (index = output number of kStr? / kWin?).
static void level_operands(int algo, View A, View B, int64_t mh, int64_t nh, int64_t kh,
                           const char* SA, size_t sa_b, const char* SB, size_t sb_b, View xa[7], View xb[7], int es = 2) {
    auto rawA = [&](int q) { return View{A.p + ((int64_t)(q >> 1) * mh * A.rs + (int64_t)(q & 1) * kh * A.cs) * es, A.rs, A.cs}; };
    auto rawB = [&](int q) { return View{B.p + ((int64_t)(q >> 1) * kh * B.rs + (int64_t)(q & 1) * nh * B.cs) * es, B.rs, B.cs}; };
    auto sumA = [&](int o) { const char* p = SA + (size_t)o * sa_b; return A.cs == 1 ? View{p, kh, 1} : View{p, 1, mh}; };
    auto sumB = [&](int o) { const char* p = SB + (size_t)o * sb_b; return B.cs == 1 ? View{p, nh, 1} : View{p, 1, kh}; };
    if (algo == STHIP_STRASSEN) {
        xa[0] = rawA(0); xb[0] = sumB(0);   // M3 = A11 S1
        xa[1] = sumA(4); xb[1] = sumB(4);   // M6 = S9 S10
        xa[2] = sumA(0); xb[2] = rawB(3);   // M5 = S2 B22
        xa[3] = sumA(3); xb[3] = sumB(3);   // M7 = S7 S8
        xa[4] = sumA(2); xb[4] = sumB(2);   // M1 = S5 S6
        xa[5] = sumA(1); xb[5] = rawB(0);   // M2 = S3 B11
        xa[6] = rawA(3); xb[6] = sumB(1);   // M4 = A22 S4
    } else {
        xa[0] = rawA(0); xb[0] = rawB(0);   // P1 = A11 B11
        xa[1] = rawA(1); xb[1] = rawB(2);   // P2 = A12 B21
        xa[2] = sumA(1); xb[2] = sumB(1);   // P6 = S2 T2
        xa[3] = sumA(2); xb[3] = sumB(2);   // P7 = S3 T3
        xa[4] = sumA(0); xb[4] = sumB(0);   // P5 = S1 T1
        xa[5] = sumA(3); xb[5] = rawB(3);   // P3 = S4 B22
        xa[6] = rawA(3); xb[6] = sumB(3);   // -P4 = A22 (-T4)
    }
}

// One operand of quad_combos2_kernel.  X is the whole operand, (rq, cq) the quarter-block size in
// its logical (row, col) indexing; side 0 = A, 1 = B; first level Strassen, second level `algo2`.
// S1 / S2 are laid out as the two-pass form lays them out (S1: five dense half-size sums s1_b
// bytes apart; S2: for first-level operand p the sums at S2 + (5 p + o) * s2_b).
static int64_t fill_combo2(Combo2Params& cp, View X, int64_t rq, int64_t cq, char* S1, size_t s1_b, char* S2, size_t s2_b,
                           int side, int algo2, int es = 2) {
    memset(&cp, 0, sizeof(cp));
    const bool row_major = X.cs == 1;
    for (int R = 0; R < 4; ++R)
        for (int C = 0; C < 4; ++C) cp.x[4 * R + C] = X.p + ((int64_t)R * rq * X.rs + (int64_t)C * cq * X.cs) * es;
    // the kernel holds the coefficient tables of both levels (str_coef, first_code, ...): first level
    // Strassen in the order of level_operands, second level `algo2`
    for (int p = 0; p < 7; ++p) cp.s2[p] = S2 + (size_t)p * 5 * s2_b;
    for (int o = 0; o < 5; ++o) cp.s1[o] = S1 + (size_t)o * s1_b;
    cp.s2_stride = (int64_t)s2_b;
    cp.side = side; cp.algo2 = algo2;
    const int64_t rows = row_major ? rq : cq, cols = row_major ? cq : rq;   // quarter block, storage order
    cp.ld_in = row_major ? X.rs : X.cs;
    cp.ld1 = 2 * cols;
    cp.ld2 = cols;
    cp.q1_u = row_major ? rq * cp.ld1 : rq;
    cp.q1_v = row_major ? cq : cq * cp.ld1;
    cp.rows = (int)rows; cp.chunks_per_row = (int)(cols / kEPT2);
    return rows * (cols / kEPT2);
}

// Two levels as three launches: the sums of both levels in one pass over the operands, ONE
// grouped GEMM of the 49 quarter-size products (the schedule the reference's two-layer Triton
// kernel runs per tile, strassen.py:373-611, here on whole matrices), both recombinations in one
// pass.  Cast schedule: first-level sums rounded once to the operand type, as the reference rounds
// them (fixed_strassen_fp32_agg.py:87-96); second-level sums formed in fp32 from those and rounded
// once (the reference multiplies them unrounded, in fp32, :99-113 -- here the inner products run
// on the 16-bit matrix cores); the 49 products rounded to the operand type as every product of this
// library is; both recombinations in fp32 with no rounding between them, as the reference's inner
// call returns fp32 (:99-106); one final rounding.  The first level is always Strassen.
// Needs: 16-bit operands, whole aligned problem, C in the operand type with 16-byte aligned rows.
static size_t two_level_bytes(int64_t mh, int64_t nh, int64_t kh) {
    const int64_t mq = mh / 2, nq = nh / 2, kq = kh / 2;
    return 5 * (align256(mh * kh * 2) + align256(kh * nh * 2)) + 35 * (align256(mq * kq * 2) + align256(kq * nq * 2)) +
           49 * align256(mq * nq * 2);
}

static bool two_level_shape(int dt, int64_t mh, int64_t nh, int64_t kh) {
    return mh % 2 == 0 && nh % 2 == 0 && kh % 2 == 0 && fast_shape(dt, mh / 2, nh / 2, kh / 2);
}

static int two_level_flat(View A, View B, char* C, int64_t c_rs, int64_t mh, int64_t nh, int64_t kh,
                          int dt, int algo, bool accumulate, bool out_f32, char* ws, Call& cx) {
    const int64_t mq = mh / 2, nq = nh / 2, kq = kh / 2;
    const size_t sa1 = align256(mh * kh * 2), sb1 = align256(kh * nh * 2);
    const size_t sa2 = align256(mq * kq * 2), sb2 = align256(kq * nq * 2);
    const size_t pb = align256(mq * nq * 2);
    char* SA1 = ws;
    char* SB1 = SA1 + 5 * sa1;
    char* SA2 = SB1 + 5 * sb1;
    char* SB2 = SA2 + 35 * sa2;
    char* P = SB2 + 35 * sb2;
    const bool a_kc = A.cs == 1, b_kc = B.rs == 1;
    const int nout2 = algo == STHIP_STRASSEN ? 5 : 4;
    const int streaming = streaming_hint(two_level_bytes(mh, nh, kh));
    // B-side sums of both levels formed ahead of the call: read, never written
    const char* ready = algo == STHIP_STRASSEN && b_kc ? take_prepared(cx, B.p, 2, kh, nh, 5 * sb1 + 35 * sb2) : nullptr;
    if (ready) { SB1 = const_cast<char*>(ready); SB2 = SB1 + 5 * sb1; }

    // sums of both levels in one pass
    if (cx.stages & 1) {
        Combo2Pair pp;
        const int64_t na = fill_combo2(pp.side[0], A, mq, kq, SA1, sa1, SA2, sa2, 0, algo);
        const int64_t nb = ready ? 0 : fill_combo2(pp.side[1], B, kq, nq, SB1, sb1, SB2, sb2, 1, algo);
        pp.side[0].streaming = pp.side[1].streaming = streaming;
        dim3 grid((unsigned)ceil_div(std::max(na, nb), 256), 1, ready ? 1 : 2);
        if (dt == STHIP_BF16) hipLaunchKernelGGL(quad_combos2_kernel<bf16_t>, grid, dim3(256), 0, cx.stream, pp);
        else hipLaunchKernelGGL(quad_combos2_kernel<f16_t>, grid, dim3(256), 0, cx.stream, pp);
        int rc = check_launch("quad_combos2");
        if (rc) return rc;
    }
    View xa1[7], xb1[7];
    level_operands(STHIP_STRASSEN, A, B, mh, nh, kh, SA1, sa1, SB1, sb1, xa1, xb1);

    // the 49 products, product-major: first-level product p, second-level product j -> P[7 p + j]
    Gemm2Params g;
    memset(&g, 0, sizeof(g));
    for (int p = 0; p < 7; ++p) {
        View xa2[7], xb2[7];
        level_operands(algo, xa1[p], xb1[p], mq, nq, kq, SA2 + (size_t)p * 5 * sa2, sa2, SB2 + (size_t)p * 5 * sb2, sb2, xa2, xb2);
        for (int j = 0; j < 7; ++j)
            g.seg[7 * p + j] = Seg2{xa2[j].p, xb2[j].p, a_kc ? xa2[j].rs : xa2[j].cs, b_kc ? xb2[j].cs : xb2[j].rs, 0, 0};
    }
    g.C = P; g.c_rs = nq; g.c_ps = (int64_t)(pb / 2); g.c_bs = 0;
    g.Mh = (int)mq; g.Nh = (int)nq; g.Kh = (int)kq;
    g.out_f32 = 0; g.accumulate = 0; g.nprod = 49; g.group_m = 4; g.c_stream = streaming;
    const LaunchTable3* t4 = table4_for(dt);
    const bool big = a_kc && t4 && mq % kBM4 == 0 && nq % kBN4 == 0 && kq >= 1024 && cx.force_tile != 5 && cx.force_tile != 2;
    hipError_t e = hipSuccess;
    if (!(cx.stages & 2)) {
    } else if (big) {
        g.tiles_m = (int)(mq / kBM4); g.tiles_n = (int)(nq / kBN4);
        g.c_wide = wide_rows(g.C, g.c_rs, g.c_ps, 0);
        g.one_tile_per_wg = (cx.stages & 32) ? 1 : 0;
        e = t4->fn[b_kc ? 1 : 0](g, 1, cx.stream);
    } else {
        const LaunchTable2* t = table2_for(dt, STHIP_CLASSIC);
        if (!t) return fail(STHIP_ERR_DTYPE, "no 16-bit kernel for dtype %d", dt);
        g.tiles_m = (int)(mq / 128); g.tiles_n = (int)(nq / 128);
        g.group_m = 8;
        e = t->fn[a_kc ? 1 : 0][b_kc ? 1 : 0](g, 1, cx.stream);
    }
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));

    // 49 -> C: both recombinations in one pass
    if (!(cx.stages & 4)) return STHIP_OK;
    Recombine16Params rp;
    rp.prod = P; rp.p_ps = (int64_t)(pb / 2); rp.C = C; rp.c_rs = c_rs; rp.c_bs = 0;
    rp.Mh = (int)mq; rp.Nh = (int)nq; rp.accumulate = accumulate ? 1 : 0; rp.out_f32 = out_f32 ? 1 : 0;
    rp.bias = take_bias(cx, C, accumulate, out_f32);
    rp.streaming = streaming;
    dim3 grid((unsigned)ceil_div(mq * (nq / kEPT2), 256), 1);
#define GO(T, A) hipLaunchKernelGGL((recombine16x2_kernel<T, A>), grid, dim3(256), 0, cx.stream, rp)
    if (dt == STHIP_BF16) { if (algo == STHIP_STRASSEN) GO(bf16_t, STHIP_STRASSEN); else GO(bf16_t, STHIP_WINOGRAD); }
    else { if (algo == STHIP_STRASSEN) GO(f16_t, STHIP_STRASSEN); else GO(f16_t, STHIP_WINOGRAD); }
#undef GO
    return check_launch("recombine16x2");
}

static int launch_recombine32(int algo, const void* prod, int64_t p_ps, char* C, int64_t c_rs, int64_t c_bs,
                              int64_t batch, int64_t Mh, int64_t Nh, bool accumulate, Call& cx) {
    Recombine16Params rp;
    rp.out_f32 = 1;
    rp.prod = prod; rp.p_ps = p_ps; rp.C = C; rp.c_rs = c_rs; rp.c_bs = c_bs;
    rp.Mh = (int)Mh; rp.Nh = (int)Nh; rp.accumulate = accumulate ? 1 : 0;
    rp.streaming = streaming_hint((size_t)batch * 11 * Mh * Nh * 4);
    dim3 grid((unsigned)ceil_div(Mh * (Nh / 4), 256), (unsigned)batch);
    if (algo == STHIP_STRASSEN) hipLaunchKernelGGL(recombine32_kernel<STHIP_STRASSEN>, grid, dim3(256), 0, cx.stream, rp);
    else hipLaunchKernelGGL(recombine32_kernel<STHIP_WINOGRAD>, grid, dim3(256), 0, cx.stream, rp);
    return check_launch("recombine32");
}

// Two levels of fp32 operands in the same three-launch form (two Strassen levels, nothing
// rounded): worth it when
// the 49 quarter-size products fill the chip with 256 x 256 tiles, because the seven children
// of the host recursion would each run their own seven products with a partly empty last round.
static size_t two_level_f32_bytes(int64_t mh, int64_t nh, int64_t kh) {
    const int64_t mq = mh / 2, nq = nh / 2, kq = kh / 2;
    return 5 * (align256(mh * kh * 4) + align256(kh * nh * 4)) + 35 * (align256(mq * kq * 4) + align256(kq * nq * 4)) +
           49 * align256(mq * nq * 4);
}

static bool two_level_f32_shape(int64_t mh, int64_t nh, int64_t kh) {
    if (mh <= 0 || nh <= 0 || kh <= 0 || mh % 2 || nh % 2 || kh % 2) return false;
    const int64_t mq = mh / 2, nq = nh / 2, kq = kh / 2;
    return mq % kBM4 == 0 && nq % kBN4 == 0 && kq % 32 == 0 && 49 * (mq / kBM4) * (nq / kBN4) >= 224;
}

static int two_level_flat_f32(View A, View B, char* C, int64_t c_rs, int64_t mh, int64_t nh, int64_t kh,
                              bool accumulate, char* ws, Call& cx) {
    const int64_t mq = mh / 2, nq = nh / 2, kq = kh / 2;
    const size_t sa1 = align256(mh * kh * 4), sb1 = align256(kh * nh * 4);
    const size_t sa2 = align256(mq * kq * 4), sb2 = align256(kq * nq * 4);
    const size_t pb = align256(mq * nq * 4);
    char* SA1 = ws;
    char* SB1 = SA1 + 5 * sa1;
    char* SA2 = SB1 + 5 * sb1;
    char* SB2 = SA2 + 35 * sa2;
    char* P = SB2 + 35 * sb2;
    const bool b_kc = B.rs == 1;
    {
        Combo2Pair pp;
        const int64_t na = fill_combo2(pp.side[0], A, mq, kq, SA1, sa1, SA2, sa2, 0, STHIP_STRASSEN, 4);
        const int64_t nb = fill_combo2(pp.side[1], B, kq, nq, SB1, sb1, SB2, sb2, 1, STHIP_STRASSEN, 4);
        pp.side[0].streaming = pp.side[1].streaming = 1;   // only large problems come here
        dim3 grid((unsigned)ceil_div(std::max(na, nb), 256), 1, 2);
        hipLaunchKernelGGL(quad_combos2_kernel<float>, grid, dim3(256), 0, cx.stream, pp);
        int rc = check_launch("quad_combos2 (fp32)");
        if (rc) return rc;
    }
    View xa1[7], xb1[7];
    level_operands(STHIP_STRASSEN, A, B, mh, nh, kh, SA1, sa1, SB1, sb1, xa1, xb1, 4);
    Gemm2Params g;
    memset(&g, 0, sizeof(g));
    for (int p = 0; p < 7; ++p) {
        View xa2[7], xb2[7];
        level_operands(STHIP_STRASSEN, xa1[p], xb1[p], mq, nq, kq, SA2 + (size_t)p * 5 * sa2, sa2, SB2 + (size_t)p * 5 * sb2, sb2,
                       xa2, xb2, 4);
        for (int j = 0; j < 7; ++j)
            g.seg[7 * p + j] = Seg2{xa2[j].p, xb2[j].p, xa2[j].rs, b_kc ? xb2[j].cs : xb2[j].rs, 0, 0};
    }
    g.C = P; g.c_rs = nq; g.c_ps = (int64_t)(pb / 4); g.c_bs = 0;
    g.Mh = (int)mq; g.Nh = (int)nq; g.Kh = (int)kq;
    g.tiles_m = (int)(mq / kBM4); g.tiles_n = (int)(nq / kBN4);
    g.out_f32 = 1; g.accumulate = 0; g.nprod = 49; g.group_m = 4; g.c_stream = 1;
    hipError_t e = table4_for(STHIP_F32)->fn[b_kc ? 1 : 0](g, 1, cx.stream);
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
    Recombine16Params rp;
    rp.prod = P; rp.p_ps = (int64_t)(pb / 4); rp.C = C; rp.c_rs = c_rs; rp.c_bs = 0;
    rp.Mh = (int)mq; rp.Nh = (int)nq; rp.accumulate = accumulate ? 1 : 0; rp.out_f32 = 1;
    dim3 grid((unsigned)ceil_div(mq * (nq / kEPT2), 256), 1);
    hipLaunchKernelGGL((recombine16x2_kernel<float, STHIP_STRASSEN>), grid, dim3(256), 0, cx.stream, rp);
    return check_launch("recombine x2 (fp32)");
}

// Vector form of recombine_kernel: four consecutive columns per thread (nh % 4 == 0, C with unit
// column stride, 4-element aligned rows, M = 2 mh, N = 2 nh).
template <class TO>
__global__ void recombine_vec_kernel(char* C, int64_t c_rs, const float* Mbuf, int64_t mstride, int mh, int nh, int accumulate) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int nq = nh / 4;
    if (idx >= (int64_t)mh * nq) return;
    const int i = (int)(idx / nq), j = (int)(idx % nq) * 4;
    f32x4 m[7];
#pragma unroll
    for (int q = 0; q < 7; ++q) m[q] = *reinterpret_cast<const f32x4*>(Mbuf + q * mstride + (int64_t)i * nh + j);
    const f32x4 out[4] = {m[0] + m[3] - m[4] + m[6], m[2] + m[4], m[1] + m[3], m[0] - m[1] + m[2] + m[5]};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int64_t off = (int64_t)(i + (q >> 1) * mh) * c_rs + (j + (q & 1) * nh);
        f32x4 v = out[q];
        if constexpr (sizeof(TO) == 4) {
            f32x4* d = reinterpret_cast<f32x4*>(C) + off / 4;
            if (accumulate) v += *d;
            *d = v;
        } else {
            u32x2* d = reinterpret_cast<u32x2*>(C + off * 2);
            if (accumulate) {
                const u32x2 old = *d;
                const uint32_t w0 = old[0], w1 = old[1];
                if constexpr (__is_same(TO, bf16_t)) { v[0] += bf16lo(w0); v[1] += bf16hi(w0); v[2] += bf16lo(w1); v[3] += bf16hi(w1); }
                else { const f16x2 h0 = as_f16x2(w0), h1 = as_f16x2(w1); v[0] += (float)h0[0]; v[1] += (float)h0[1]; v[2] += (float)h1[0]; v[3] += (float)h1[1]; }
            }
            u32x2 o;
            if constexpr (__is_same(TO, bf16_t)) { o[0] = pack_bf16(v[0], v[1]); o[1] = pack_bf16(v[2], v[3]); }
            else { o[0] = pack_f16(v[0], v[1]); o[1] = pack_f16(v[2], v[3]); }
            *d = o;
        }
    }
}

static int block_sum(int dt, char* dst, View X, int ra, int ca, int rb, int cb, int sign,
                     int64_t rows, int64_t cols, int64_t lim_r, int64_t lim_c, hipStream_t s) {
    const int64_t n = rows * cols;
    if (n == 0) return STHIP_OK;
    const unsigned blocks = (unsigned)ceil_div(n, 256);
#define GO(T) hipLaunchKernelGGL(block_sum_kernel<T>, dim3(blocks), dim3(256), 0, s, dst, X.p, X.rs, X.cs, ra, ca, rb, cb, sign, (int)rows, (int)cols, (int)lim_r, (int)lim_c)
    if (dt == STHIP_F32) GO(float); else if (dt == STHIP_F16) GO(f16_t); else GO(bf16_t);
#undef GO
    return check_launch("block_sum");
}

// block_sum for a 16-bit X with the result stored as fp32 (the operands of the reference schedule's inner products).
static int block_sum_widened(int dt, char* dst, View X, int ra, int ca, int rb, int cb, int sign,
                             int64_t rows, int64_t cols, int64_t lim_r, int64_t lim_c, hipStream_t s) {
    const int64_t n = rows * cols;
    if (n == 0) return STHIP_OK;
    const unsigned blocks = (unsigned)ceil_div(n, 256);
#define GO(T) hipLaunchKernelGGL((block_sum_kernel<T, float>), dim3(blocks), dim3(256), 0, s, dst, X.p, X.rs, X.cs, ra, ca, rb, cb, sign, (int)rows, (int)cols, (int)lim_r, (int)lim_c)
    if (dt == STHIP_F16) GO(f16_t); else GO(bf16_t);
#undef GO
    return check_launch("block_sum (widened)");
}

static int recombine(int out_dt, char* C, int64_t c_rs, int64_t c_cs, const float* Mbuf, int64_t mstride,
                     int64_t mh, int64_t nh, int64_t M, int64_t N, bool accumulate, hipStream_t s) {
    const int64_t n = mh * nh;
    if (n == 0) return STHIP_OK;
    const size_t oes = out_dt == STHIP_F32 ? 4 : 2;
    if (c_cs == 1 && nh % 4 == 0 && c_rs % 4 == 0 && M == 2 * mh && N == 2 * nh && aligned_to(C, 4 * oes) && mstride % 4 == 0) {
        const unsigned vb = (unsigned)ceil_div(n / 4, 256);
        const int acc = accumulate ? 1 : 0;
        if (out_dt == STHIP_F32) hipLaunchKernelGGL(recombine_vec_kernel<float>, dim3(vb), dim3(256), 0, s, C, c_rs, Mbuf, mstride, (int)mh, (int)nh, acc);
        else if (out_dt == STHIP_F16) hipLaunchKernelGGL(recombine_vec_kernel<f16_t>, dim3(vb), dim3(256), 0, s, C, c_rs, Mbuf, mstride, (int)mh, (int)nh, acc);
        else hipLaunchKernelGGL(recombine_vec_kernel<bf16_t>, dim3(vb), dim3(256), 0, s, C, c_rs, Mbuf, mstride, (int)mh, (int)nh, acc);
        return check_launch("recombine_vec");
    }
    const unsigned blocks = (unsigned)ceil_div(n, 256);
#define GO(T) hipLaunchKernelGGL(recombine_kernel<T>, dim3(blocks), dim3(256), 0, s, C, c_rs, c_cs, Mbuf, mstride, (int)mh, (int)nh, (int)M, (int)N, accumulate ? 1 : 0)
    if (out_dt == STHIP_F32) GO(float); else if (out_dt == STHIP_F16) GO(f16_t); else GO(bf16_t);
#undef GO
    return check_launch("recombine");
}

// fp32, one Strassen level: all fourteen operands (sums and single quadrants alike) are written
// as dense matrices by one bandwidth-bound launch, the seven products run as ONE batched launch
// of the classical kernel, and one pass recombines the seven fp32 products into C.  Nothing is
// rounded anywhere, so the result differs from the fused kernel's only by summation order.
static int one_level_f32_batched(View A, View B, char* C, int64_t c_rs, int64_t Mh, int64_t Nh, int64_t Kh,
                                 bool accumulate, char* ws, Call& cx) {
    const size_t sa = align256(Mh * Kh * 4), sb = align256(Kh * Nh * 4), sm = align256(Mh * Nh * 4);
    char* OA = ws;
    char* OB = OA + 7 * sa;
    char* Mbuf = OB + 7 * sb;
    ComboPair pp;
    const int64_t na = fill_combo(pp.side[0], A, Mh, Kh, OA, sa, 7, kStr7A, 4);
    const int64_t nb = fill_combo(pp.side[1], B, Kh, Nh, OB, sb, 7, kStr7B, 4);
    dim3 grid((unsigned)ceil_div(std::max(na, nb), 256), 1, 2);
    hipLaunchKernelGGL(quad_combos_pair_f32_kernel, grid, dim3(256), 0, cx.stream, pp);
    int rc = check_launch("quad_combos (fp32)");
    if (rc) return rc;
    // dense operands keep the storage orientation of their source
    const View a = A.cs == 1 ? View{OA, Kh, 1} : View{OA, 1, Mh};
    const View b = B.cs == 1 ? View{OB, Nh, 1} : View{OB, 1, Kh};
    rc = launch_fused(a, b, Mbuf, Nh, 1, 7, (int64_t)(sa / 4), (int64_t)(sb / 4), (int64_t)(sm / 4), Mh, Nh, Kh, 0, 0, 0,
                      STHIP_F32, true, STHIP_CLASSIC, false, nullptr, 0, cx);
    if (rc) return rc;
    return recombine(STHIP_F32, C, c_rs, 1, reinterpret_cast<const float*>(Mbuf), (int64_t)(sm / 4), Mh, Nh, 2 * Mh, 2 * Nh,
                     accumulate, cx.stream);
}

// Strassen product table in the reference's numbering (fixed_strassen.py:88-114):
// {A block a, A block b, sign} x {B block a, B block b, sign}; block ids 0=11 1=12 2=21 3=22,
// sign 0 = single block.
struct Term { int a, b, sign; };
static const Term kATerms[7] = {{0, 3, +1}, {2, 3, +1}, {0, 0, 0}, {3, 0, 0}, {0, 1, +1}, {2, 0, -1}, {1, 3, -1}};
static const Term kBTerms[7] = {{0, 3, +1}, {0, 0, 0}, {1, 3, -1}, {2, 0, -1}, {3, 0, 0}, {0, 1, +1}, {2, 3, +1}};

// fp32, one Strassen level on small matrices: the seven products side by side on 64 x 64 tiles, every
// operand a quadrant read in place or the sum / difference of two formed in registers on the way
// to LDS (sthip_kernel6.hpp), then the recombination pass.  Two launches instead of three and 7 x
// (Mh / 64) x (Nh / 64) workgroups instead of 7 x (Mh / 128) x (Nh / 128).
static bool f32_small_shape(View A, View B, int64_t Mh, int64_t Nh, int64_t Kh) {
    if (A.cs != 1 || (B.rs != 1 && B.cs != 1)) return false;
    if (Mh % kBM6 || Nh % kBN6 || Kh % (2 * kBK6)) return false;
    const int64_t b_ld = B.rs == 1 ? B.cs : B.rs;
    return aligned_to(A.p, 16) && aligned_to(B.p, 16) && A.rs % 4 == 0 && b_ld % 4 == 0;
}
static int one_level_f32_small(View A, View B, char* C, int64_t c_rs, int64_t Mh, int64_t Nh, int64_t Kh,
                               bool accumulate, char* ws, Call& cx) {
    const size_t sm = align256(Mh * Nh * 4);
    const bool b_kc = B.rs == 1;
    Gemm6Params g;
    memset(&g, 0, sizeof(g));
    const float* Aq[4]; const float* Bq[4];
    for (int q = 0; q < 4; ++q) {
        Aq[q] = reinterpret_cast<const float*>(A.p) + (int64_t)(q >> 1) * Mh * A.rs + (int64_t)(q & 1) * Kh * A.cs;
        Bq[q] = reinterpret_cast<const float*>(B.p) + (int64_t)(q >> 1) * Kh * B.rs + (int64_t)(q & 1) * Nh * B.cs;
    }
    for (int q = 0; q < 7; ++q) {
        g.a[q] = Op6{Aq[kATerms[q].a], Aq[kATerms[q].b], A.rs, kATerms[q].sign, 0};
        g.b[q] = Op6{Bq[kBTerms[q].a], Bq[kBTerms[q].b], b_kc ? B.cs : B.rs, kBTerms[q].sign, 0};
    }
    g.C = reinterpret_cast<float*>(ws); g.c_rs = Nh; g.c_ps = (int64_t)(sm / 4);
    g.Kh = (int)Kh; g.tiles_m = (int)(Mh / kBM6); g.tiles_n = (int)(Nh / kBN6); g.nprod = 7;
    hipError_t e = launch_gemm6(g, b_kc, cx.stream);
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
    return recombine(STHIP_F32, C, c_rs, 1, reinterpret_cast<const float*>(ws), (int64_t)(sm / 4), Mh, Nh, 2 * Mh, 2 * Nh,
                     accumulate, cx.stream);
}

// sums by product M1..M7 as indices into the outputs of kStrA / kStrB (-1 = a raw block)
static const int kSumA[7] = {2, 1, -1, -1, 0, 4, 3};
static const int kSumB[7] = {2, -1, 0, 1, -1, 4, 3};

// fp32, one Strassen or Winograd level on the 256 x 256 kernel: the quadrant sums in one launch,
// the seven products (raw quadrants read in place) as one grouped launch into seven dense fp32
// matrices, one recombination pass.  Nothing is rounded anywhere.
static int one_level_f32_grouped(View A, View B, char* C, int64_t c_rs, int64_t Mh, int64_t Nh, int64_t Kh,
                                 int algo, bool accumulate, char* ws, Call& cx) {
    const size_t sa = align256(Mh * Kh * 4), sb = align256(Kh * Nh * 4), sm = align256(Mh * Nh * 4);
    char* SA = ws;
    char* SB = SA + 5 * sa;
    char* Mbuf = SB + 5 * sb;
    const bool strassen = algo == STHIP_STRASSEN;
    const int nout = strassen ? 5 : 4;
    if (cx.stages & 1) {
        ComboPair pp;
        const int64_t na = fill_combo(pp.side[0], A, Mh, Kh, SA, sa, nout, strassen ? kStrA : kWinA, 4);
        const int64_t nb = fill_combo(pp.side[1], B, Kh, Nh, SB, sb, nout, strassen ? kStrB : kWinB, 4);
        dim3 grid((unsigned)ceil_div(std::max(na, nb), 256), 1, 2);
        hipLaunchKernelGGL(quad_combos_pair_f32_kernel, grid, dim3(256), 0, cx.stream, pp);
        int rc = check_launch("quad_combos (fp32)");
        if (rc) return rc;
    }
    const bool b_kc = B.rs == 1;
    View xa[7], xb[7];
    level_operands(algo, A, B, Mh, Nh, Kh, SA, sa, SB, sb, xa, xb, 4);
    Gemm2Params g;
    memset(&g, 0, sizeof(g));
    for (int q = 0; q < 7; ++q) g.seg[q] = Seg2{xa[q].p, xb[q].p, xa[q].rs, b_kc ? xb[q].cs : xb[q].rs, 0, 0};
    g.C = Mbuf; g.c_rs = Nh; g.c_ps = (int64_t)(sm / 4); g.c_bs = 0;
    g.Mh = (int)Mh; g.Nh = (int)Nh; g.Kh = (int)Kh;
    g.tiles_m = (int)(Mh / kBM4); g.tiles_n = (int)(Nh / kBN4);
    g.out_f32 = 1; g.accumulate = 0; g.group_m = 4; g.nprod = 7; g.c_stream = streaming_hint(f32_batched_bytes(Mh, Nh, Kh));
    if (cx.stages & 2) {
        hipError_t e = table4_for(STHIP_F32)->fn[b_kc ? 1 : 0](g, 1, cx.stream);
        if (e != hipSuccess) return fail(STHIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
    }
    if (!(cx.stages & 4)) return STHIP_OK;
    return launch_recombine32(algo, Mbuf, (int64_t)(sm / 4), C, c_rs, 0, 1, Mh, Nh, accumulate, cx);
}

// inner: the product is one of the seven of an upper level, which takes it in fp32 (16-bit operands
// then keep their seven products in fp32 too: twice the room).
static size_t workspace_for(int64_t Mp, int64_t Np, int64_t Kp, int dt, int levels, bool inner = false, int sched = kSchedAuto) {
    const int64_t mh = Mp / 2, nh = Np / 2, kh = Kp / 2;
    if (levels <= 0) return 0;
    if (reference_schedule(dt, levels, sched))   // one widened operand pair, seven fp32 products, the fp32 child
        return align256(mh * kh * 4) + align256(kh * nh * 4) + 7 * align256(mh * nh * 4) +
               workspace_for(mh, nh, kh, STHIP_F32, levels - 1, true);
    if (levels == 1) {
        if (fast_shape(dt, mh, nh, kh)) return prepass_bytes(1, mh, nh, kh, inner ? 4 : 2);
        if (dt == STHIP_F32 && mh > 0 && nh > 0 && kh > 0 && mh % kBM == 0 && nh % kBN == 0 && kh % 32 == 0)
            return f32_batched_bytes(mh, nh, kh);
        return 0;
    }
    const size_t es = elem_size(dt);
    const size_t recursive = 5 * (align256(mh * kh * es) + align256(kh * nh * es)) + 7 * align256(mh * nh * 4) +
                             workspace_for(mh, nh, kh, dt, levels - 1, true, sched);
    // two levels may run as one 49-product launch (two_level_flat) or, if the call's layout or
    // result type rules that out, as the host recursion: room for either
    if (levels == 2 && two_level_shape(dt, mh, nh, kh)) return std::max(recursive, two_level_bytes(mh, nh, kh));
    if (levels == 2 && dt == STHIP_F32 && two_level_f32_shape(mh, nh, kh)) return std::max(recursive, two_level_f32_bytes(mh, nh, kh));
    return recursive;
}

// C (+)= A x B with `levels` levels.  (Mp, Np, Kp) >= (M, N, K) are the padded sizes the
// split is taken on (multiples of 2^levels); everything outside (M, N, K) reads as zero.
static int multiply(View A, View B, char* C, int64_t c_rs, int64_t c_cs,
                    int64_t M, int64_t N, int64_t K, int64_t Mp, int64_t Np, int64_t Kp,
                    int dt, int out_dt, int algo, int levels, bool accumulate,
                    char* ws, size_t ws_bytes, Call& cx, bool inner = false) {
    // inner: this product is one of the seven of an upper level, which wants it in fp32; it may
    // still be formed from 16-bit sub-products (only the last rounding is skipped).
    const bool out_f32 = out_dt == STHIP_F32;
    if (algo == STHIP_CLASSIC || levels <= 0)
        return launch_fused(A, B, C, c_rs, c_cs, 1, 0, 0, 0, M, N, K, 0, 0, 0, dt, out_f32, STHIP_CLASSIC, accumulate,
                            nullptr, 0, cx);
    const int64_t mh = Mp / 2, nh = Np / 2, kh = Kp / 2;
    if (levels == 1)
        return launch_fused(A, B, C, c_rs, c_cs, 1, 0, 0, 0, M, N, K, mh, nh, kh, dt, out_f32, algo, accumulate,
                            ws, ws_bytes, cx);

    const size_t es = elem_size(dt);
    if (reference_schedule(dt, levels, cx.sched)) {
        // fixed_strassen_fp32_agg.py:87-113: S1..S10 rounded to the operand type, everything below in fp32
        const size_t a_b = align256(mh * kh * 4), b_b = align256(kh * nh * 4), m_b = align256(mh * nh * 4);
        const size_t need = a_b + b_b + 7 * m_b;
        if (!ws || ws_bytes < need) return fail(STHIP_ERR_WORKSPACE, "workspace too small: %zu < %zu", ws_bytes, need);
        char* A32 = ws;
        char* B32 = ws + a_b;
        char* Mbuf = ws + a_b + b_b;
        char* child_ws = ws + need;
        const size_t child_bytes = std::min(ws_bytes - need, workspace_for(mh, nh, kh, STHIP_F32, levels - 1, true));
        for (int q = 0; q < 7; ++q) {
            const Term ta = kATerms[q], tb = kBTerms[q];
            int rc = block_sum_widened(dt, A32, A, (ta.a >> 1) * (int)mh, (ta.a & 1) * (int)kh, (ta.b >> 1) * (int)mh, (ta.b & 1) * (int)kh,
                                       ta.sign, mh, kh, M, K, cx.stream);
            if (rc) return rc;
            rc = block_sum_widened(dt, B32, B, (tb.a >> 1) * (int)kh, (tb.a & 1) * (int)nh, (tb.b >> 1) * (int)kh, (tb.b & 1) * (int)nh,
                                   tb.sign, kh, nh, K, N, cx.stream);
            if (rc) return rc;
            Call child;
            child.stream = cx.stream; child.stages = cx.stages; child.force_tile = cx.force_tile; child.sched = cx.sched;
            rc = multiply(View{A32, kh, 1}, View{B32, nh, 1}, Mbuf + q * m_b, nh, 1, mh, nh, kh, mh, nh, kh, STHIP_F32, STHIP_F32,
                          algo, levels - 1, false, child_ws, child_bytes, child, true);
            if (rc) return rc;
        }
        return recombine(out_dt, C, c_rs, c_cs, reinterpret_cast<const float*>(Mbuf), (int64_t)(m_b / 4), mh, nh, M, N, accumulate, cx.stream);
    }
    if (levels == 2 && (cx.stages & 8) && two_level_shape(dt, mh, nh, kh) && (!out_f32 || inner) && M == Mp && N == Np && K == Kp &&
        c_cs == 1 && c_rs % 8 == 0 && aligned_to(C, 16) && combos_ok(A, mh, kh) && combos_ok(B, kh, nh) &&
        (A.cs == 1 || A.rs == 1) && (B.cs == 1 || B.rs == 1) && ws && aligned_to(ws, 256) &&
        ws_bytes >= two_level_bytes(mh, nh, kh))
        return two_level_flat(A, B, C, c_rs, mh, nh, kh, dt, algo, accumulate, out_f32, ws, cx);
    if (levels == 2 && (cx.stages & 8) && dt == STHIP_F32 && algo == STHIP_STRASSEN && two_level_f32_shape(mh, nh, kh) &&
        M == Mp && N == Np && K == Kp && c_cs == 1 && c_rs % 4 == 0 && aligned_to(C, 16) && A.cs == 1 &&
        combos_ok(A, mh, kh, 4) && combos_ok(B, kh, nh, 4) && ws && aligned_to(ws, 256) &&
        ws_bytes >= two_level_f32_bytes(mh, nh, kh))
        return two_level_flat_f32(A, B, C, c_rs, mh, nh, kh, accumulate, ws, cx);
    // Whole, aligned problems: all five sums of each operand in one bandwidth-bound launch.
    const bool whole = M == Mp && N == Np && K == Kp;
    const bool vec = whole && combos_ok(A, mh, kh, (int)es) && combos_ok(B, kh, nh, (int)es);
    const size_t sa_b = align256(mh * kh * es), sb_b = align256(kh * nh * es);
    const size_t m_b = align256(mh * nh * 4);
    const size_t need = 5 * (sa_b + sb_b) + 7 * m_b;
    if (!ws || ws_bytes < need) return fail(STHIP_ERR_WORKSPACE, "workspace too small: %zu < %zu", ws_bytes, need);
    char* SA = ws;
    char* SB = ws + 5 * sa_b;
    char* Mbuf = ws + 5 * (sa_b + sb_b);
    char* child_ws = ws + need;
    // exactly what the query reserves for a child, however much more the caller passed: the kernels a
    // child picks depend on the room it is given
    const size_t child_bytes = std::min(ws_bytes - need, workspace_for(mh, nh, kh, dt, levels - 1, true, cx.sched));
    // B-side sums of this level and of the levels below formed ahead of the call: read, never written
    const char* ready = vec && es == 2 && algo == STHIP_STRASSEN && levels >= 3 && B.rs == 1
                            ? take_prepared(cx, B.p, levels, kh, nh, prepared_bytes(levels, kh, nh)) : nullptr;
    const size_t child_prep = ready ? prepared_bytes(levels - 1, kh / 2, nh / 2) : 0;
    if (ready) SB = const_cast<char*>(ready);

    if (vec && dt == STHIP_F32) {
        ComboPair pp;
        const int64_t na = fill_combo(pp.side[0], A, mh, kh, SA, sa_b, 5, kStrA, 4);
        const int64_t nb = fill_combo(pp.side[1], B, kh, nh, SB, sb_b, 5, kStrB, 4);
        dim3 grid((unsigned)ceil_div(std::max(na, nb), 256), 1, 2);
        hipLaunchKernelGGL(quad_combos_pair_f32_kernel, grid, dim3(256), 0, cx.stream, pp);
        int rc = check_launch("quad_combos (fp32)");
        if (rc) return rc;
    } else if (vec) {
        int rc = run_combos(dt, A, mh, kh, SA, sa_b, 5, kStrA, cx);
        if (rc) return rc;
        if (!ready) rc = run_combos(dt, B, kh, nh, SB, sb_b, 5, kStrB, cx);
        if (rc) return rc;
    }

    for (int q = 0; q < 7; ++q) {
        const Term ta = kATerms[q], tb = kBTerms[q];
        View a, b;
        // A operand: a single block that lies fully inside A is used in place
        const int ara = (ta.a >> 1) * (int)mh, aca = (ta.a & 1) * (int)kh;
        if (ta.sign == 0 && ara + mh <= M && aca + kh <= K) {
            a = {A.p + ((int64_t)ara * A.rs + (int64_t)aca * A.cs) * (int64_t)es, A.rs, A.cs};
        } else if (vec) {
            const char* p = SA + (size_t)kSumA[q] * sa_b;   // dense, in A's storage orientation
            a = A.cs == 1 ? View{p, kh, 1} : View{p, 1, mh};
        } else {
            int rc = block_sum(dt, SA, A, ara, aca, (ta.b >> 1) * (int)mh, (ta.b & 1) * (int)kh, ta.sign, mh, kh, M, K, cx.stream);
            if (rc) return rc;
            a = {SA, kh, 1};
        }
        const int bra = (tb.a >> 1) * (int)kh, bca = (tb.a & 1) * (int)nh;
        if (tb.sign == 0 && bra + kh <= K && bca + nh <= N) {
            b = {B.p + ((int64_t)bra * B.rs + (int64_t)bca * B.cs) * (int64_t)es, B.rs, B.cs};
        } else if (vec) {
            const char* p = SB + (size_t)kSumB[q] * sb_b;
            b = B.cs == 1 ? View{p, nh, 1} : View{p, 1, kh};
        } else {
            int rc = block_sum(dt, SB, B, bra, bca, (tb.b >> 1) * (int)kh, (tb.b & 1) * (int)nh, tb.sign, kh, nh, K, N, cx.stream);
            if (rc) return rc;
            b = {SB, nh, 1};
        }
        // the child writes an fp32 product, never the caller's C: no bias for it, and only the sums of its own B operand
        Call child;
        child.stream = cx.stream; child.stages = cx.stages; child.force_tile = cx.force_tile; child.sched = cx.sched;
        if (ready) {
            child.prep.sums = ready + 5 * sb_b + (size_t)q * child_prep; child.prep.bytes = child_prep; child.prep.target = b.p;
            child.prep.levels = levels - 1; child.prep.kh = kh / 2; child.prep.nh = nh / 2;
        }
        int rc = multiply(a, b, Mbuf + q * m_b, nh, 1, mh, nh, kh, mh, nh, kh, dt, STHIP_F32, algo, levels - 1,
                          false, child_ws, child_bytes, child, true);
        if (rc) return rc;
    }
    return recombine(out_dt, C, c_rs, c_cs, reinterpret_cast<const float*>(Mbuf), (int64_t)(m_b / 4), mh, nh, M, N, accumulate, cx.stream);
}

static int check_common(const void* A, const void* B, const void* C, int64_t batch, int64_t M, int64_t N, int64_t K,
                        int in_dt, int out_dt, int algo, int levels) {
    if (batch < 0 || M < 0 || N < 0 || K < 0) return fail(STHIP_ERR_SHAPE, "negative size");
    if (in_dt < 0 || in_dt > 2 || out_dt < 0 || out_dt > 2) return fail(STHIP_ERR_DTYPE, "unknown dtype (%d, %d)", in_dt, out_dt);
    if (out_dt != in_dt && out_dt != STHIP_F32) return fail(STHIP_ERR_DTYPE, "out dtype must equal in dtype or be fp32");
    if (algo < 0 || (algo & 15) > 2 || (algo >> 4) > 2) return fail(STHIP_ERR_ARG, "unknown algo %d", algo);
    if (levels < 0 || levels > 8) return fail(STHIP_ERR_ARG, "levels must be in [0, 8], got %d", levels);
    if (batch > 0 && M > 0 && N > 0 && (!C || (K > 0 && (!A || !B)))) return fail(STHIP_ERR_ARG, "null pointer");
    return STHIP_OK;
}

// ------------------------------------------------------------------ static scratch
// Workspace of sthip_gemm_static: part of the device image, so every GPU that loads the library
// holds its own copy at its own address.  `scratch` itself is only a host-side handle for the
// symbol; kernels, and everything else that needs the memory, get the per-device address that
// hipGetSymbolAddress returns with that device current.
static __device__ __align__(256) unsigned char scratch[STHIP_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

static int static_scratch(char** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(STHIP_ERR_HIP, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(STHIP_ERR_HIP, "no address for the static scratch buffer on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = reinterpret_cast<char*>(g_scratch_ptr[dev]);
    return STHIP_OK;
}

static Call begin_call(void* stream) {
    g_err[0] = 0;
    Call cx;
    cx.stream = reinterpret_cast<hipStream_t>(stream);
    cx.stages = g_debug_stages.load(std::memory_order_relaxed);
    cx.force_tile = forced_tile_setting();
    return cx;
}

static int gemm_impl(Call& cx, const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K,
                     const int64_t sA[3], const int64_t sB[3], const int64_t sC[3],
                     int in_dtype, int out_dtype, int algo, int levels, int accumulate,
                     void* workspace, size_t workspace_bytes) {
    int rc = check_common(A, B, C, batch, M, N, K, in_dtype, out_dtype, algo, levels);
    if (rc) return rc;
    if (algo >> 4) cx.sched = algo >> 4;   // STHIP_SCHEDULE_REFERENCE / STHIP_SCHEDULE_FAST
    algo &= 15;
    if (!sA || !sB || !sC) return fail(STHIP_ERR_ARG, "null stride array");
    if (batch == 0 || M == 0 || N == 0) return STHIP_OK;
    const int es = elem_size(in_dtype), ces = elem_size(out_dtype);
    if (algo == STHIP_CLASSIC) levels = 0;
    if (algo != STHIP_CLASSIC && levels == 0) algo = STHIP_CLASSIC;
    const int64_t q = (int64_t)1 << levels;
    const int64_t Mp = round_up(M, q), Np = round_up(N, q), Kp = round_up(K, q);
    if (levels <= 1) {
        View a = {reinterpret_cast<const char*>(A), sA[1], sA[2]};
        View b = {reinterpret_cast<const char*>(B), sB[1], sB[2]};
        return launch_fused(a, b, reinterpret_cast<char*>(C), sC[1], sC[2], batch, sA[0], sB[0], sC[0], M, N, K,
                            Mp / 2, Np / 2, Kp / 2, in_dtype, out_dtype == STHIP_F32, algo, accumulate != 0,
                            reinterpret_cast<char*>(workspace), workspace_bytes, cx);
    }
    for (int64_t bi = 0; bi < batch; ++bi) {
        View a = {reinterpret_cast<const char*>(A) + bi * sA[0] * es, sA[1], sA[2]};
        View b = {reinterpret_cast<const char*>(B) + bi * sB[0] * es, sB[1], sB[2]};
        char* c = reinterpret_cast<char*>(C) + bi * sC[0] * ces;
        rc = multiply(a, b, c, sC[1], sC[2], M, N, K, Mp, Np, Kp, in_dtype, out_dtype, algo, levels, accumulate != 0,
                      reinterpret_cast<char*>(workspace), workspace_bytes, cx);
        if (rc) return rc;
    }
    return STHIP_OK;
}

// The bias of a Linear forward goes into the last pass of the product where that pass can take it
// (16-bit, 16-byte aligned); otherwise a pass of its own adds it afterwards.
static void offer_bias(Call& cx, const void* bias, const void* y, int dtype) {
    cx.bias = BiasEpilogue{};
    if (bias && dtype != STHIP_F32 && aligned_to(bias, 16)) { cx.bias.bias = bias; cx.bias.target = y; }
}
static int finish_bias(Call& cx, const void* bias, void* y, int64_t rows, int64_t cols, int dtype) {
    if (!bias || cx.bias.applied) return STHIP_OK;
    const unsigned blocks = (unsigned)ceil_div(rows * cols, 256);
    char* yy = reinterpret_cast<char*>(y);
    const char* bb = reinterpret_cast<const char*>(bias);
    if (dtype == STHIP_F32) hipLaunchKernelGGL(add_bias_kernel<float>, dim3(blocks), dim3(256), 0, cx.stream, yy, bb, rows, cols);
    else if (dtype == STHIP_F16) hipLaunchKernelGGL(add_bias_kernel<f16_t>, dim3(blocks), dim3(256), 0, cx.stream, yy, bb, rows, cols);
    else hipLaunchKernelGGL(add_bias_kernel<bf16_t>, dim3(blocks), dim3(256), 0, cx.stream, yy, bb, rows, cols);
    return check_launch("add_bias");
}

// Levels that make this shape fastest, from a sweep of M, N, K over 768 .. 16384 (both layouts of
// B) timing the classical kernel, one level and two levels of this library against each other.
static int auto_levels(int64_t M, int64_t N, int64_t K, int dt, int max_levels) {
    if (max_levels <= 0 || M <= 0 || N <= 0 || K <= 0) return 0;
    const int64_t smallest = std::min(M, std::min(N, K));
    const double flops = 2.0 * (double)M * (double)N * (double)K;
    int levels = 0;
    if (dt == STHIP_F32) {
        // the fp32 matrix cores are 16 x slower than the 16-bit ones while the passes only double:
        // one level pays from 5e11 flop (8192 x 8192 x 4096: 1.05 x the classical kernel), a second
        // from 1e12 (8192^3: 1.09 x, 16384^3: 1.23 x), a third from 32768^3 (1.32 x against 1.22 x)
        if (std::min(M, N) >= 4096 && K >= 4096 && flops >= 5e11) levels = 1;
        if (smallest >= 4096 && flops >= 1e12) levels = 2;
        if (smallest >= 32768) levels = 3;
        // fewer than 224 tiles of 256 x 256: the classical product runs on 64 x 64 tiles at 0.8 - 0.9 x
        // hipBLASLt, and a level on top of it is 0.75 - 1.0 x of that up to k = 4096 (1.01 - 1.05 x beyond):
        // classical
    } else {
        // 16-bit: the passes of a level cost about 14 n^2 bytes against n^3 / 4 flop saved: break-even
        // near 16384^3 (0.92 x at 8192^3).  At 16384^3 a level measured 1.02 - 1.05 x before the classical
        // kernel's main loop gained 4 % and a Strassen call 1.3 %: within 2 % either way since, so the rule
        // waits for 20480; a second level from 32768^3.  Never a third: from three levels on the default
        // schedule runs the inner products in fp32 as the reference does, which is not a speed-up.
        if (smallest >= 20480 || (smallest >= 8192 && K >= 20480 && M * N >= (int64_t)8192 * 16384)) levels = 1;
        if (smallest >= 32768) levels = 2;
        // at most 128 output tiles of 128 x 128 and a long k (weight gradients): one classical product
        // leaves most CUs idle, seven half-size ones side by side do not (1.1 - 1.5 x from k = 4096)
        if (levels == 0 && ceil_div(M, 128) * ceil_div(N, 128) <= 128 && K >= 4096 &&
            M % 256 == 0 && N % 256 == 0 && K % 128 == 0) levels = 1;
    }
    return std::min(levels, max_levels);
}

static int linear_forward_impl(Call& cx, const void* x, const void* W, const void* bias, void* y,
                               int64_t rows, int64_t in_features, int64_t out_features, int dtype, int levels,
                               void* workspace, size_t workspace_bytes) {
    if (levels < 0) levels = auto_levels(rows, out_features, in_features, dtype, std::min(-levels, 8));
    // the layers the reference has run one or two levels (model/layers.py:246); a third level and the weight-side
    // sums kept for it are this library's own, and round at every level so that all products are 16-bit ones
    cx.sched = kSchedFast;
    int rc = check_common(x, W, y, 1, rows, out_features, in_features, dtype, dtype, STHIP_STRASSEN, levels);
    if (rc) return rc;
    if (rows == 0 || out_features == 0) return STHIP_OK;
    const int64_t sA[3] = {0, in_features, 1}, sB[3] = {0, 1, in_features}, sC[3] = {0, out_features, 1};   // B = W^T as a view
    offer_bias(cx, bias, y, dtype);
    rc = gemm_impl(cx, x, W, y, 1, rows, out_features, in_features, sA, sB, sC, dtype, dtype,
                   levels > 0 ? STHIP_STRASSEN : STHIP_CLASSIC, levels, 0, workspace, workspace_bytes);
    if (rc) return rc;
    return finish_bias(cx, bias, y, rows, out_features, dtype);
}

// Half extents of W^T (in_features x out_features) for which the weight-side sums can be formed
// ahead of the call: 16-bit operands, one to four levels, innermost blocks that the grouped paths take.
static bool weight_sums_shape(int64_t in_features, int64_t out_features, int dtype, int levels) {
    if (dtype != STHIP_BF16 && dtype != STHIP_F16) return false;
    if (levels < 1 || levels > 4) return false;
    const int64_t q = (int64_t)1 << levels;
    if (in_features <= 0 || out_features <= 0 || in_features % q || out_features % q) return false;
    return fast_shape(dtype, 128, out_features / q, in_features / q);
}

// Sums of the k x n operand B (stored n-major: B.rs == 1) for `levels` levels into `buf`.
static int prepare_b(int dt, View B, int64_t k, int64_t n, int levels, char* buf, Call& cx) {
    const int64_t kh = k / 2, nh = n / 2;
    const size_t sb1 = align256(kh * nh * 2);
    if (levels == 1) return run_combos(dt, B, kh, nh, buf, sb1, 5, kStrB, cx);
    if (levels == 2) {
        const size_t sb2 = align256((kh / 2) * (nh / 2) * 2);
        Combo2Pair pp;
        memset(&pp, 0, sizeof(pp));
        const int64_t nb = fill_combo2(pp.side[0], B, kh / 2, nh / 2, buf, sb1, buf + 5 * sb1, sb2, 1, STHIP_STRASSEN);
        pp.side[0].streaming = 1;   // formed once, read by later calls
        dim3 grid((unsigned)ceil_div(nb, 256), 1, 1);
        if (dt == STHIP_BF16) hipLaunchKernelGGL(quad_combos2_kernel<bf16_t>, grid, dim3(256), 0, cx.stream, pp);
        else hipLaunchKernelGGL(quad_combos2_kernel<f16_t>, grid, dim3(256), 0, cx.stream, pp);
        return check_launch("quad_combos2 (weight)");
    }
    int rc = run_combos(dt, B, kh, nh, buf, sb1, 5, kStrB, cx);
    if (rc) return rc;
    const size_t child = prepared_bytes(levels - 1, kh / 2, nh / 2);
    for (int q = 0; q < 7; ++q) {
        // B operand of product M(q+1) as multiply() forms it: a quadrant in place or a dense sum
        const Term tb = kBTerms[q];
        const View b = tb.sign == 0 ? View{B.p + ((int64_t)(tb.a >> 1) * kh * B.rs + (int64_t)(tb.a & 1) * nh * B.cs) * 2, B.rs, B.cs}
                                    : View{buf + (size_t)kSumB[q] * sb1, 1, kh};
        rc = prepare_b(dt, b, kh, nh, levels - 1, buf + 5 * sb1 + (size_t)q * child, cx);
        if (rc) return rc;
    }
    return STHIP_OK;
}

}  // namespace sthip

using namespace sthip;

extern "C" {

int sthip_gemm(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K,
               const int64_t sA[3], const int64_t sB[3], const int64_t sC[3],
               int in_dtype, int out_dtype, int algo, int levels, int accumulate,
               void* workspace, size_t workspace_bytes, void* stream) {
    Call cx = begin_call(stream);
    return gemm_impl(cx, A, B, C, batch, M, N, K, sA, sB, sC, in_dtype, out_dtype, algo, levels, accumulate,
                     workspace, workspace_bytes);
}

int sthip_gemm_static(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K,
                      const int64_t sA[3], const int64_t sB[3], const int64_t sC[3],
                      int in_dtype, int out_dtype, int algo, int levels, int accumulate, void* stream) {
    Call cx = begin_call(stream);
    int rc = check_common(A, B, C, batch, M, N, K, in_dtype, out_dtype, algo, levels);
    if (rc) return rc;
    const size_t need = sthip_workspace_bytes(batch, M, N, K, in_dtype, out_dtype, algo, levels);
    if (need > STHIP_STATIC_SCRATCH_BYTES)
        return fail(STHIP_ERR_WORKSPACE, "problem too large for the static scratch buffer: it needs %zu bytes of workspace, "
                    "the buffer holds %zu; use sthip_gemm with a workspace of that size", need, (size_t)STHIP_STATIC_SCRATCH_BYTES);
    char* ws = nullptr;
    if (need > 0) {
        rc = static_scratch(&ws);
        if (rc) return rc;
    }
    return gemm_impl(cx, A, B, C, batch, M, N, K, sA, sB, sC, in_dtype, out_dtype, algo, levels, accumulate, ws, need);
}

size_t sthip_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int in_dtype, int out_dtype, int algo, int levels) {
    if (algo < 0 || (algo >> 4) > 2) return 0;
    const int sched = algo >> 4;
    algo &= 15;
    if (algo == STHIP_CLASSIC || levels <= 0 || M <= 0 || N <= 0 || K < 0 || levels > 8 || in_dtype < 0 || in_dtype > 2) return 0;
    const int64_t q = (int64_t)1 << levels;
    const int64_t Mp = round_up(M, q), Np = round_up(N, q), Kp = round_up(K, q);
    // one level: the batch goes into a single launch, so the pre-pass buffers scale with it (and
    // only whole, tile-aligned problems take that path); deeper: batches run one after another
    if (levels == 1) {
        if (Mp != M || Np != N || Kp != K) return 0;
        if (in_dtype == STHIP_F32) return batch == 1 ? workspace_for(Mp, Np, Kp, in_dtype, 1) : 0;   // batched-products path: one problem
        // an fp32 result of 16-bit operands keeps its seven products in fp32
        if (out_dtype == STHIP_F32 && fast_shape(in_dtype, Mp / 2, Np / 2, Kp / 2))
            return prepass_bytes(batch, Mp / 2, Np / 2, Kp / 2, 4);
        return (size_t)batch * workspace_for(Mp, Np, Kp, in_dtype, 1);
    }
    return workspace_for(Mp, Np, Kp, in_dtype, levels, false, sched);
}

int sthip_strassen_matmul_n_layers(const void* A, const void* B, void* C, int64_t n,
                                   int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs,
                                   int dtype, int levels, void* workspace, size_t workspace_bytes, void* stream) {
    Call cx = begin_call(stream);
    const int64_t sA[3] = {0, a_rs, a_cs}, sB[3] = {0, b_rs, b_cs}, sC[3] = {0, n, 1};
    if (levels < 1) return fail(STHIP_ERR_ARG, "levels must be >= 1, got %d", levels);
    return gemm_impl(cx, A, B, C, 1, n, n, n, sA, sB, sC, dtype, dtype, STHIP_STRASSEN, levels, 0, workspace, workspace_bytes);
}

int sthip_run_accumulate(const void* A, const void* B, void* C, int64_t batch, int64_t M, int64_t N, int64_t K,
                         int op_dtype, int c_dtype, int algo, int levels,
                         void* workspace, size_t workspace_bytes, void* stream) {
    Call cx = begin_call(stream);
    const int64_t sA[3] = {M * K, K, 1}, sB[3] = {K * N, N, 1}, sC[3] = {M * N, N, 1};
    return gemm_impl(cx, A, B, C, batch, M, N, K, sA, sB, sC, op_dtype, c_dtype, algo, levels, 1, workspace, workspace_bytes);
}

int sthip_linear_strassen_forward(const void* x, const void* W, const void* bias, void* y,
                                  int64_t rows, int64_t D, int dtype, int levels,
                                  void* workspace, size_t workspace_bytes, void* stream) {
    Call cx = begin_call(stream);
    cx.sched = kSchedFast;   // as sthip_linear_forward
    int rc = check_common(x, W, y, 1, rows, D, D, dtype, dtype, STHIP_STRASSEN, levels);
    if (rc) return rc;
    if (levels < 1) return fail(STHIP_ERR_ARG, "levels must be >= 1, got %d", levels);
    if (rows > D) return fail(STHIP_ERR_SHAPE, "rows (%lld) > D (%lld): the input cannot be padded to D x D", (long long)rows, (long long)D);
    if (rows == 0 || D == 0) return STHIP_OK;
    // The reference pads x to D x D (model/layers.py:261-262): split on the padded size.
    const int64_t q = (int64_t)1 << levels;
    const int64_t Dp = round_up(D, q);
    View a = {reinterpret_cast<const char*>(x), D, 1};
    View b = {reinterpret_cast<const char*>(W), 1, D};   // W^T as a view
    offer_bias(cx, bias, y, dtype);
    rc = multiply(a, b, reinterpret_cast<char*>(y), D, 1, rows, D, D, Dp, Dp, Dp, dtype, dtype, STHIP_STRASSEN, levels, false,
                  reinterpret_cast<char*>(workspace), workspace_bytes, cx);
    if (rc) return rc;
    return finish_bias(cx, bias, y, rows, D, dtype);
}

int sthip_linear_forward(const void* x, const void* W, const void* bias, void* y,
                         int64_t rows, int64_t in_features, int64_t out_features, int dtype, int levels,
                         void* workspace, size_t workspace_bytes, void* stream) {
    Call cx = begin_call(stream);
    return linear_forward_impl(cx, x, W, bias, y, rows, in_features, out_features, dtype, levels, workspace, workspace_bytes);
}

int sthip_auto_levels(int64_t M, int64_t N, int64_t K, int dtype, int max_levels) {
    return auto_levels(M, N, K, dtype, max_levels);
}

size_t sthip_linear_weight_sums_bytes(int64_t in_features, int64_t out_features, int dtype, int levels) {
    if (!weight_sums_shape(in_features, out_features, dtype, levels)) return 0;
    return prepared_bytes(levels, in_features / 2, out_features / 2);
}

int sthip_linear_prepare_weight(const void* W, int64_t in_features, int64_t out_features, int dtype, int levels,
                                void* sums, size_t sums_bytes, void* stream) {
    Call cx = begin_call(stream);
    const size_t need = sthip_linear_weight_sums_bytes(in_features, out_features, dtype, levels);
    if (!need) return fail(STHIP_ERR_SHAPE, "no weight-side sums for in=%lld out=%lld dtype=%d levels=%d (16-bit, 1 to 4 levels, aligned blocks)",
                           (long long)in_features, (long long)out_features, dtype, levels);
    if (!W || !sums) return fail(STHIP_ERR_ARG, "null pointer");
    if (!aligned_to(W, 16)) return fail(STHIP_ERR_ARG, "W must be 16-byte aligned");
    if (!aligned_to(sums, 256)) return fail(STHIP_ERR_ARG, "the sums buffer must be 256-byte aligned");
    if (sums_bytes < need) return fail(STHIP_ERR_WORKSPACE, "sums buffer too small: %zu < %zu bytes", sums_bytes, need);
    const View B = {reinterpret_cast<const char*>(W), 1, in_features};   // W^T as a view
    return prepare_b(dtype, B, in_features, out_features, levels, reinterpret_cast<char*>(sums), cx);
}

int sthip_linear_forward_prepared(const void* x, const void* W, const void* sums, size_t sums_bytes, const void* bias, void* y,
                                  int64_t rows, int64_t in_features, int64_t out_features, int dtype, int levels,
                                  void* workspace, size_t workspace_bytes, void* stream) {
    Call cx = begin_call(stream);
    const size_t need = sthip_linear_weight_sums_bytes(in_features, out_features, dtype, levels);
    if (!need) return fail(STHIP_ERR_SHAPE, "no weight-side sums for in=%lld out=%lld dtype=%d levels=%d",
                           (long long)in_features, (long long)out_features, dtype, levels);
    if (!sums || !aligned_to(sums, 256)) return fail(STHIP_ERR_ARG, "the sums buffer must be non-null and 256-byte aligned");
    if (sums_bytes < need) return fail(STHIP_ERR_WORKSPACE, "sums buffer too small: %zu < %zu bytes", sums_bytes, need);
    cx.prep.sums = reinterpret_cast<const char*>(sums); cx.prep.bytes = sums_bytes; cx.prep.target = W;
    cx.prep.levels = levels; cx.prep.kh = in_features / 2; cx.prep.nh = out_features / 2;
    return linear_forward_impl(cx, x, W, bias, y, rows, in_features, out_features, dtype, levels, workspace, workspace_bytes);
}

const char* sthip_last_error(void) { return g_err; }

int sthip_version(void) { return STHIP_VERSION; }

int sthip_debug_set_stages(int mask) { return g_debug_stages.exchange(mask & kAllStages); }

int sthip_debug_force_tile(const char* tile) {
    forced_tile_setting();   // settle the environment's value first, so that it cannot overwrite this one later
    return g_debug_tile.exchange(tile_code(tile));
}

int sthip_debug_one_launch_counters(const void* workspace, int64_t M, int64_t N, int64_t K, unsigned counters[16], void* stream) {
    g_err[0] = 0;
    if (!workspace || !counters || M <= 0 || N <= 0 || K <= 0 || M % 2 || N % 2 || K % 2)
        return fail(STHIP_ERR_ARG, "one-launch counters: null pointer or sizes that no one-launch call takes");
    hipError_t e = hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "hipStreamSynchronize failed: %s", hipGetErrorString(e));
    const char* flags = reinterpret_cast<const char*>(workspace) + prepass_body_bytes(1, M / 2, N / 2, K / 2);
    e = hipMemcpy(counters, flags, kFlagWords * sizeof(unsigned), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return fail(STHIP_ERR_HIP, "hipMemcpy of the counters failed: %s", hipGetErrorString(e));
    return (int)std::min<unsigned>(counters[kFlagGaveUp], 1u << 30);
}

int sthip_debug_transpose_read(void* out, void* stream) {
    g_err[0] = 0;
    if (!out) return fail(STHIP_ERR_ARG, "null pointer");
    hipLaunchKernelGGL(transpose_read_probe_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream),
                       reinterpret_cast<uint16_t*>(out));
    return check_launch("transpose_read_probe");
}

}  // extern "C"
