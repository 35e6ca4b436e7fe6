// Run-time side of the host build of the library's kernels, one host thread per lane.
//
// What is real: the kernels' own code -- tile numbering, loader cursors and lane offsets, LDS layouts and
// swizzles, fragment reads, the order of loads, waits and barriers, the walking of tiles, the stores.
// What is modelled here (in place of sthip_prims.hpp): a direct-to-LDS load copies 16 bytes per lane,
// either at once or not before the lane's next s_waitcnt lets it (the two extremes of what the hardware
// may do), after checking that source and destination lie inside the operands and the LDS allocation;
// the matrix instructions and the transposing LDS read exchange their operands among the 64 threads of
// a wave.  Inline assembly statements are stripped from the library's sources before they are compiled
// against this (the test does that); they only carry scheduling hints, waits that the builtins repeat,
// and the instructions replaced here.
#include <pthread.h>
#include <deque>
#include <thread>
#include "host_runtime.h"
#include "sthip_kernel.hpp"
#include "sthip_prims.hpp"

thread_local HostDim3 threadIdx, blockIdx, gridDim, blockDim;
namespace sthip { alignas(1024) char smem[160 * 1024]; }

std::vector<HostRange> g_host_global;
static std::vector<HostRange> g_host_symbols;
void host_register_symbol(const void* p, size_t bytes) { g_host_symbols.push_back({(const char*)p, bytes}); }
bool g_host_late = false;
int g_host_compute_units = 4;
int host_compute_units() { return g_host_compute_units; }

namespace {
constexpr int kLanes = 64, kWaves = 8, kThreadsWg = kLanes * kWaves;
pthread_barrier_t g_wg_barrier, g_wave_barrier[kWaves];
struct Pending { const char* src; char* dst; };
thread_local std::deque<Pending> t_pending;
thread_local int t_slot[3] = {0, 0, 0};
sthip::u32x4 g_xa[kWaves][2][kLanes], g_xb[kWaves][2][kLanes];
uint32_t g_fa[kWaves][2][kLanes], g_fb[kWaves][2][kLanes];
const char* g_xp[kWaves][2][kLanes];

[[noreturn]] void die(const char* what, const void* p) {
    fprintf(stderr, "MODEL VIOLATION: %s (address %p, workgroup %u, thread %u)\n", what, p, blockIdx.x, threadIdx.x);
    fflush(stderr);
    _Exit(3);
}
void check_global(const char* p) {
    for (const HostRange& r : g_host_global)
        if (p >= r.p && p + 16 <= r.p + r.n) return;
    for (const HostRange& r : g_host_symbols)
        if (p >= r.p && p + 16 <= r.p + r.n) return;
    die("direct-to-LDS load reads outside the operands", p);
}
void load16(const char* src, char* dst) {
    check_global(src);
    if (g_host_late) t_pending.push_back({src, dst});
    else memcpy(dst, src, 16);
}
void dma(const void* sbase, uint32_t voff, uint32_t lds_addr) {
    const int lane = threadIdx.x & 63;
    const char* src = reinterpret_cast<const char*>(sbase) + voff;
    char* dst = reinterpret_cast<char*>((uintptr_t)lds_addr) + 16 * lane;
    check_global(src);
    if (dst < sthip::smem || dst + 16 > sthip::smem + sizeof(sthip::smem)) die("direct-to-LDS load writes outside LDS", dst);
    if (g_host_late) t_pending.push_back({src, dst});
    else memcpy(dst, src, 16);
}
}  // namespace
float host_as_float(uint32_t v, int idx, bool bf16) {
    const uint16_t h = (uint16_t)(v >> (16 * idx));
    if (bf16) return __builtin_bit_cast(float, (uint32_t)h << 16);
    return (float)__builtin_bit_cast(_Float16, h);
}
namespace {
inline float as_float(uint32_t v, int idx, bool bf16) { return host_as_float(v, idx, bf16); }
}  // namespace

void host_syncthreads() { pthread_barrier_wait(&g_wg_barrier); }
void host_waitcnt(int imm) {
    const size_t n = (size_t)((imm & 0xF) | (((imm >> 14) & 3) << 4));   // vmcnt: this many loads may stay in flight
    while (t_pending.size() > n) {
        memcpy(t_pending.front().dst, t_pending.front().src, 16);
        t_pending.pop_front();
    }
}

namespace sthip {
void lds_dma16(const void* sbase, uint32_t voff, uint32_t lds_addr) { dma(sbase, voff, lds_addr); }
void lds_dma16_k(const void* sbase, uint32_t voff, uint32_t lds_addr, int k) { dma(sbase, voff, lds_addr + (uint32_t)k); }
void lds_dma16_km(const void* sbase, uint32_t voff, uint32_t lds_addr, int k, uint32_t mask) {
    if (mask != 0 && mask != 0xffffffffu) die("lane mask of a load is neither all ones nor zero", sbase);
    if (mask) dma(sbase, voff, lds_addr + (uint32_t)k);
}
void wave_exchange_point() { pthread_barrier_wait(&g_wave_barrier[threadIdx.x >> 6]); }
// Lane i of a 16-lane group receives element i % 4 of lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4.
s16x4 lds_read_tr16_b64(const char* p) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, s = t_slot[0] ^= 1;
    if (p < smem || p + 8 > smem + sizeof(smem)) die("transposing read outside LDS", p);
    g_xp[wave][s][lane] = p;
    pthread_barrier_wait(&g_wave_barrier[wave]);
    const int base = lane & ~15, i = lane & 15;
    s16x4 r;
    for (int e = 0; e < 4; ++e) {
        int16_t v;
        memcpy(&v, g_xp[wave][s][base + 4 * e + i / 4] + 2 * (i % 4), 2);
        r[e] = v;
    }
    return r;
}
// v_mfma_f32_16x16x32 as the kernel uses it: lane L accumulates, for m = L % 16 and n = 4 (L / 16) + e,
// the sum over 32 k of A(m, k) B(n, k); the A fragment of row m holds k = 8 g .. 8 g + 7 in lane m + 16 g,
// the B fragment of column n likewise.
template <class T> void mfma16_step(f32x4& acc, const u32x4& a, const u32x4& b) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, s = t_slot[1] ^= 1;
    g_xa[wave][s][lane] = a;
    g_xb[wave][s][lane] = b;
    pthread_barrier_wait(&g_wave_barrier[wave]);
    constexpr bool bf = __is_same(T, bf16_t);
    const int m = lane & 15;
    for (int e = 0; e < 4; ++e) {
        const int n = 4 * (lane >> 4) + e;
        float sum = 0.f;
        for (int k = 0; k < 32; ++k) {
            const u32x4& av = g_xa[wave][s][m + 16 * (k / 8)];
            const u32x4& bv = g_xb[wave][s][n + 16 * (k / 8)];
            sum += as_float(av[(k % 8) / 2], k % 2, bf) * as_float(bv[(k % 8) / 2], k % 2, bf);
        }
        acc[e] += sum;
    }
}
template void mfma16_step<bf16_t>(f32x4&, const u32x4&, const u32x4&);
template void mfma16_step<f16_t>(f32x4&, const u32x4&, const u32x4&);
void gload16_6(f32x4& dst, const float* p) { load16(reinterpret_cast<const char*>(p), reinterpret_cast<char*>(&dst)); }
// v_mfma_f32_16x16x4_f32: k = lane group g; A(m, g) is the operand of lane m + 16 g.
void mfma16_step_f32(f32x4& acc, uint32_t a, uint32_t b) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, s = t_slot[2] ^= 1;
    g_fa[wave][s][lane] = a;
    g_fb[wave][s][lane] = b;
    pthread_barrier_wait(&g_wave_barrier[wave]);
    const int m = lane & 15;
    for (int e = 0; e < 4; ++e) {
        const int n = 4 * (lane >> 4) + e;
        float sum = 0.f;
        for (int g = 0; g < 4; ++g)
            sum += __builtin_bit_cast(float, g_fa[wave][s][m + 16 * g]) * __builtin_bit_cast(float, g_fb[wave][s][n + 16 * g]);
        acc[e] += sum;
    }
}
}  // namespace sthip

// The builtin form (64 x 64 kernel): the instruction's first operand indexes the result's rows, which the
// kernel uses for n, its second the columns (m): the same exchange as mfma16_step_f32 with a = second, b = first.
void host_mfma_16x16x4(float a_inst, float b_inst, float* acc4) {
    sthip::f32x4 acc = {acc4[0], acc4[1], acc4[2], acc4[3]};
    sthip::mfma16_step_f32(acc, __builtin_bit_cast(uint32_t, b_inst), __builtin_bit_cast(uint32_t, a_inst));
    for (int e = 0; e < 4; ++e) acc4[e] = acc[e];
}

// v_mfma_f32_32x32x16: the first operand's lane L holds row L % 32 of a 32 x 16 block, k = 8 (L / 32) .. + 7,
// the second's column L % 32 likewise; lane L receives, in element e, row 8 (e / 4) + 4 (L / 32) + e % 4 of
// column L % 32.
uint16_t g_ha[kWaves][2][kLanes][8], g_hb[kWaves][2][kLanes][8];
float g_sa[kWaves][2][kLanes], g_sb[kWaves][2][kLanes];
thread_local int t_slot32[2] = {0, 0};
void host_mfma_32x32x16(const uint16_t a_inst[8], const uint16_t b_inst[8], float acc16[16], bool bf16) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, s = t_slot32[0] ^= 1;
    memcpy(g_ha[wave][s][lane], a_inst, 16);
    memcpy(g_hb[wave][s][lane], b_inst, 16);
    pthread_barrier_wait(&g_wave_barrier[wave]);
    const int col = lane & 31;
    for (int e = 0; e < 16; ++e) {
        const int row = 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
        float sum = 0.f;
        for (int k = 0; k < 16; ++k)
            sum += as_float(g_ha[wave][s][row + 32 * (k / 8)][k % 8], 0, bf16) * as_float(g_hb[wave][s][col + 32 * (k / 8)][k % 8], 0, bf16);
        acc16[e] += sum;
    }
}
void host_mfma_32x32x2(float a_inst, float b_inst, float acc16[16]) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, s = t_slot32[1] ^= 1;
    g_sa[wave][s][lane] = a_inst;
    g_sb[wave][s][lane] = b_inst;
    pthread_barrier_wait(&g_wave_barrier[wave]);
    const int col = lane & 31;
    for (int e = 0; e < 16; ++e) {
        const int row = 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
        acc16[e] += g_sa[wave][s][row] * g_sb[wave][s][col] + g_sa[wave][s][row + 32] * g_sb[wave][s][col + 32];
    }
}


// One workgroup at a time, one thread per lane; the workgroup barrier is sized to the block.
void host_launch(dim3 grid, dim3 block, const std::function<void()>& body) {
    static bool init = false;
    if (!init) {
        for (auto& b : g_wave_barrier) pthread_barrier_init(&b, nullptr, kLanes);
        pthread_barrier_init(&g_wg_barrier, nullptr, kThreadsWg);
        init = true;
        if ((uintptr_t)sthip::smem + sizeof(sthip::smem) > 0xffffffffull) { fprintf(stderr, "LDS stand-in above 4 GiB: link with -no-pie\n"); _Exit(2); }
    }
    const int threads = (int)(block.x * block.y * block.z);
    if (threads % kLanes != 0 || threads > kThreadsWg) { fprintf(stderr, "host_launch: block of %d threads\n", threads); _Exit(2); }
    pthread_barrier_destroy(&g_wg_barrier);
    pthread_barrier_init(&g_wg_barrier, nullptr, threads);
    for (unsigned bz = 0; bz < grid.z; ++bz)
    for (unsigned by = 0; by < grid.y; ++by)
        for (unsigned bx = 0; bx < grid.x; ++bx) {
            std::vector<std::thread> th;
            th.reserve(threads);
            for (int t = 0; t < threads; ++t)
                th.emplace_back([&, t, bx, by, bz] {
                    threadIdx = {(unsigned)t, 0, 0};
                    blockIdx = {bx, by, bz};
                    gridDim = {grid.x, grid.y, grid.z};
                    blockDim = {(unsigned)threads, 1, 1};
                    t_pending.clear();
                    body();
                    if (!t_pending.empty()) die("a lane ends with direct-to-LDS loads in flight", nullptr);
                });
            for (auto& x : th) x.join();
        }
}
