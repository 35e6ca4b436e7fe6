// The whole library on the CPU: its host code (path selection, workspace layout, launch parameters) compiled
// against the stand-in HIP runtime of hip/hip_runtime.h, its kernels run by host_runtime.cpp.  Calls go through
// the C ABI of include/strassen_hip.h with host memory as "device" memory.  Inputs are small integers, so every
// product and sum is exact in fp32 and the expected bits follow from the cast schedule alone: a level's seven
// products are rounded to the operand type on the paths that keep them in 16-bit, the recombination is fp32.
#include <math.h>
#include "host_runtime.h"
#include "strassen_hip.h"
#include "strassen_hip_debug.h"

namespace {
typedef std::vector<float> Mat;   // row-major, integer-valued

uint16_t bf16_bits(float v) {   // round to nearest even
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float round_to(float v, int dt) {
    if (dt == STHIP_F32) return v;
    if (dt == STHIP_BF16) return __builtin_bit_cast(float, (uint32_t)bf16_bits(v) << 16);
    return (float)(_Float16)v;
}
int small_int(uint32_t& state) {
    state = state * 1664525u + 1013904223u;
    return (int)((state >> 16) % 3) - 1;
}
Mat matmul(const Mat& A, const Mat& B, int M, int N, int K) {
    Mat C((size_t)M * N, 0.f);
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            const float a = A[(size_t)m * K + k];
            if (a == 0.f) continue;
            for (int n = 0; n < N; ++n) C[(size_t)m * N + n] += a * B[(size_t)k * N + n];
        }
    return C;
}
Mat quad(const Mat& X, int R, int Cc, int q) {   // quadrant q = 2 * row half + column half
    const int r2 = R / 2, c2 = Cc / 2;
    Mat o((size_t)r2 * c2);
    for (int r = 0; r < r2; ++r)
        for (int c = 0; c < c2; ++c) o[(size_t)r * c2 + c] = X[(size_t)(r + (q >> 1) * r2) * Cc + c + (q & 1) * c2];
    return o;
}
Mat lin(const Mat& X, float s, const Mat& Y) {
    Mat o(X.size());
    for (size_t i = 0; i < X.size(); ++i) o[i] = X[i] + s * Y[i];
    return o;
}
// Strassen with the products of every level rounded to dt (the sums are exact here), recombined in fp32.
Mat strassen_rounded(const Mat& A, const Mat& B, int M, int N, int K, int levels, int dt) {
    if (levels == 0) {
        Mat C = matmul(A, B, M, N, K);
        for (auto& v : C) v = round_to(v, dt);
        return C;
    }
    const Mat A11 = quad(A, M, K, 0), A12 = quad(A, M, K, 1), A21 = quad(A, M, K, 2), A22 = quad(A, M, K, 3);
    const Mat B11 = quad(B, K, N, 0), B12 = quad(B, K, N, 1), B21 = quad(B, K, N, 2), B22 = quad(B, K, N, 3);
    const int m = M / 2, n = N / 2, k = K / 2;
    auto P = [&](const Mat& X, const Mat& Y) { return strassen_rounded(X, Y, m, n, k, levels - 1, dt); };
    const Mat M1 = P(lin(A11, 1, A22), lin(B11, 1, B22)), M2 = P(lin(A21, 1, A22), B11), M3 = P(A11, lin(B12, -1, B22)),
              M4 = P(A22, lin(B21, -1, B11)), M5 = P(lin(A11, 1, A12), B22), M6 = P(lin(A21, -1, A11), lin(B11, 1, B12)),
              M7 = P(lin(A12, -1, A22), lin(B21, 1, B22));
    Mat C((size_t)M * N);
    for (int r = 0; r < m; ++r)
        for (int c = 0; c < n; ++c) {
            const size_t i = (size_t)r * n + c;
            C[(size_t)r * N + c] = round_to(M1[i] + M4[i] - M5[i] + M7[i], dt);
            C[(size_t)r * N + c + n] = round_to(M3[i] + M5[i], dt);
            C[(size_t)(r + m) * N + c] = round_to(M2[i] + M4[i], dt);
            C[(size_t)(r + m) * N + c + n] = round_to(M1[i] - M2[i] + M3[i] + M6[i], dt);
        }
    return C;
}

struct Dev {   // "device" buffers of one call
    std::vector<char> a, b, c, ws;
};
void store(std::vector<char>& buf, size_t i, float v, int dt) {
    if (dt == STHIP_F32) memcpy(&buf[i * 4], &v, 4);
    else if (dt == STHIP_BF16) { const uint16_t h = bf16_bits(v); memcpy(&buf[i * 2], &h, 2); }
    else { const uint16_t h = __builtin_bit_cast(uint16_t, (_Float16)v); memcpy(&buf[i * 2], &h, 2); }
}
float load(const std::vector<char>& buf, size_t i, int dt) {
    if (dt == STHIP_F32) { float v; memcpy(&v, &buf[i * 4], 4); return v; }
    uint16_t h; memcpy(&h, &buf[i * 2], 2);
    return host_as_float(h, 0, dt == STHIP_BF16);
}
int esize(int dt) { return dt == STHIP_F32 ? 4 : 2; }

// One call of sthip_gemm on M x N x K, row-major operands (B optionally stored n x k), compared bit for bit with
// `expected` (already in the result type's values).  rounded_products: the expectation rounds each level's products.
long run_gemm(const char* name, int M, int N, int K, int dt, int out_dt, int algo, int levels, bool accumulate, bool with_ws,
              bool b_kc, const char* tile, bool rounded_products) {
    uint32_t seed = 2024u + (uint32_t)(M + 3 * N + 5 * K + 7 * levels + algo);
    Mat A((size_t)M * K), B((size_t)K * N), C0((size_t)M * N, 0.f);
    for (auto& v : A) v = (float)small_int(seed);
    for (auto& v : B) v = (float)small_int(seed);
    if (accumulate) for (auto& v : C0) v = (float)small_int(seed);
    Dev d;
    d.a.resize(A.size() * esize(dt)); d.b.resize(B.size() * esize(dt)); d.c.resize(C0.size() * esize(out_dt));
    for (size_t i = 0; i < A.size(); ++i) store(d.a, i, A[i], dt);
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n) store(d.b, b_kc ? (size_t)n * K + k : (size_t)k * N + n, B[(size_t)k * N + n], dt);
    for (size_t i = 0; i < C0.size(); ++i) store(d.c, i, accumulate ? C0[i] : 99.f, out_dt);
    sthip_debug_force_tile(tile);
    const size_t need = with_ws ? sthip_workspace_bytes(1, M, N, K, dt, out_dt, algo, levels) : 0;
    d.ws.resize(need + 512);
    char* ws = need ? (char*)(((uintptr_t)d.ws.data() + 255) & ~(uintptr_t)255) : nullptr;
    g_host_global = {{d.a.data(), d.a.size()}, {d.b.data(), d.b.size()}, {d.ws.data(), d.ws.size()}, {d.c.data(), d.c.size()}};
    const int64_t sA[3] = {0, K, 1}, sB[3] = {0, b_kc ? 1 : N, b_kc ? K : 1}, sC[3] = {0, N, 1};
    const int rc = sthip_gemm(d.a.data(), d.b.data(), d.c.data(), 1, M, N, K, sA, sB, sC, dt, out_dt, algo, levels, accumulate ? 1 : 0,
                              ws, need, nullptr);
    sthip_debug_force_tile(nullptr);
    if (rc != STHIP_OK) { printf("%s: sthip_gemm returned %d (%s)\n", name, rc, sthip_last_error()); return 1; }
    Mat want;
    if (rounded_products) want = strassen_rounded(A, B, M, N, K, levels, dt);
    else want = matmul(A, B, M, N, K);
    long bad = 0;
    for (size_t i = 0; i < want.size(); ++i) {
        const float w = round_to(want[i] + C0[i], out_dt), got = load(d.c, i, out_dt);
        if (got != w && bad++ < 5) fprintf(stderr, "  %s: C[%zu][%zu] = %g, expected %g\n", name, i / N, i % N, got, w);
    }
    printf("%s (workspace %zu bytes): %ld wrong of %zu\n", name, need, bad, want.size());
    fflush(stdout);
    return bad;
}
}  // namespace

int main(int argc, char** argv) try {
    // no argument: every case; "5": case 5 alone; "1/3": the cases whose number leaves 1 when divided by 3
    const int which = argc > 1 ? atoi(argv[1]) : -1;
    const int shares = argc > 1 && strchr(argv[1], '/') ? atoi(strchr(argv[1], '/') + 1) : 0;
    int id = 0;
    auto want = [&]() { const int i = id++; return shares ? i % shares == which : which < 0 || which == i; };
    long bad = 0;
    g_host_compute_units = 4;   // seven tiles on four "CUs": the grouped launch walks its tiles
    if (want()) bad += run_gemm("one level bf16, sums / grouped 256x256 products / recombination, 512x512x256", 512, 512, 256, STHIP_BF16, STHIP_BF16,
                                STHIP_STRASSEN, 1, false, true, false, "256x256", true);
    if (want()) bad += run_gemm("one level fp16, B k-contiguous, fp32 result (products kept in fp32), 512x512x256", 512, 512, 256, STHIP_F16, STHIP_F32,
                                STHIP_STRASSEN, 1, false, true, true, "256x256", false);
    if (want()) bad += run_gemm("two levels bf16 as three launches (49 products), 1024x1024x512", 1024, 1024, 512, STHIP_BF16, STHIP_BF16,
                                STHIP_STRASSEN, 2, false, true, false, "256x256", true);
    if (want()) bad += run_gemm("classical bf16 on the walking 256x256 kernel, 512x768x128", 512, 768, 128, STHIP_BF16, STHIP_BF16,
                                STHIP_CLASSIC, 0, false, false, false, "256x256", false);
    if (want()) bad += run_gemm("one level fp32 on 64x64 tiles, sums formed in the loads, 256x256x128", 256, 256, 128, STHIP_F32, STHIP_F32,
                                STHIP_STRASSEN, 1, false, true, false, "64x64", false);
    if (want()) bad += run_gemm("one level bf16, no workspace (fused kernel), odd sizes 201x137x99", 201, 137, 99, STHIP_BF16, STHIP_BF16,
                                STHIP_STRASSEN, 1, false, false, false, nullptr, false);
    if (want()) bad += run_gemm("one level fp16 Winograd, 128x128 grouped products, accumulating into fp32, 256x256x256", 256, 256, 256, STHIP_F16, STHIP_F32,
                                STHIP_WINOGRAD, 1, true, true, false, "128x128g", false);
    printf("%s\n", bad ? "FAILED" : "ALL EXACT");
    return bad ? 1 : 0;
} catch (const std::exception& e) {
    fprintf(stderr, "exception: %s\n", e.what());
    return 4;
}
