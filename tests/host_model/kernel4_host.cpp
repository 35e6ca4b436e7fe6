// The library's GEMM kernels run on the CPU against exact integer products (run-time side: host_runtime.cpp).
#include "host_runtime.h"
#include "sthip_kernel4.hpp"
#include "sthip_kernel6.hpp"

namespace {
using namespace sthip;

template <class Kernel, class Params> void launch(Kernel kernel, const Params& P, unsigned grid, int threads = 512) {
    host_launch(dim3(grid), dim3((unsigned)threads), [&] { kernel(P); });
}

uint16_t to_half(float v, bool bf) {
    if (bf) return (uint16_t)(__builtin_bit_cast(uint32_t, v) >> 16);
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}
float from_half(uint16_t h, bool bf) { return host_as_float(h, 0, bf); }
int small_int(uint32_t& state) {   // -1, 0, 1
    state = state * 1664525u + 1013904223u;
    return (int)((state >> 16) % 3) - 1;
}

// One configuration: `nprod` products C_p = A_p B_p of M x N x K each (M, N multiples of 256, K of the
// k-step), on `grid` workgroups.  T: bf16_t, f16_t or float.  Returns the number of wrong elements.
template <class T, bool B_KC>
long run_case(const char* name, int nprod, int M, int N, int K, unsigned grid, bool walking, bool out_f32, bool accumulate, bool as_batch = false, bool c_wide = true) {
    constexpr bool f32 = __is_same(T, float), bf = __is_same(T, bf16_t);
    constexpr int ES = f32 ? 4 : 2;
    const int es_out = (f32 || out_f32) ? 4 : 2;
    const size_t a_elems = (size_t)M * K, b_elems = (size_t)K * N, c_elems = (size_t)M * N;
    std::vector<char> A(nprod * a_elems * ES), B(nprod * b_elems * ES), C(nprod * c_elems * es_out);
    std::vector<float> Af(nprod * a_elems), Bf(nprod * b_elems), C0(nprod * c_elems);
    uint32_t seed = 12345u + (uint32_t)(M * 7 + N * 3 + K);
    auto put = [&](std::vector<char>& buf, size_t i, float v) {
        if (f32) memcpy(&buf[i * 4], &v, 4);
        else { const uint16_t h = to_half(v, bf); memcpy(&buf[i * 2], &h, 2); }
    };
    for (size_t i = 0; i < Af.size(); ++i) { Af[i] = (float)small_int(seed); put(A, i, Af[i]); }
    // B is stored k x n (n-contiguous) or n x k (k-contiguous); Bf is always indexed [p][k][n]
    for (int p = 0; p < nprod; ++p)
        for (int k = 0; k < K; ++k)
            for (int n = 0; n < N; ++n) {
                const float v = (float)small_int(seed);
                Bf[p * b_elems + (size_t)k * N + n] = v;
                put(B, p * b_elems + (B_KC ? (size_t)n * K + k : (size_t)k * N + n), v);
            }
    for (size_t i = 0; i < C0.size(); ++i) {
        C0[i] = accumulate ? (float)small_int(seed) : 0.f;
        if (es_out == 4) memcpy(&C[i * 4], &C0[i], 4);
        else { const uint16_t h = to_half(accumulate ? C0[i] : 77.f, bf); memcpy(&C[i * 2], &h, 2); }
    }
    g_host_global = {{A.data(), A.size()}, {B.data(), B.size()}};

    Gemm2Params P;
    memset(&P, 0, sizeof(P));
    for (int p = 0; p < nprod; ++p)
        P.seg[p] = Seg2{A.data() + p * a_elems * ES, B.data() + p * b_elems * ES, K, B_KC ? K : N, 0, 0};
    P.C = C.data(); P.c_rs = N; P.c_ps = (int64_t)c_elems; P.nprod = nprod;
    if (as_batch) {   // the same operands addressed as batch entries of one product
        P.seg[0].a_bs = (int64_t)a_elems; P.seg[0].b_bs = (int64_t)b_elems;
        P.c_bs = (int64_t)c_elems; P.c_ps = 0; P.nprod = 1;
    }
    P.Mh = M; P.Nh = N; P.Kh = K; P.tiles_m = M / 256; P.tiles_n = N / 256;
    P.out_f32 = es_out == 4; P.accumulate = accumulate; P.group_m = 4; P.c_wide = c_wide ? 1 : 0; P.nbatch = as_batch ? nprod : 1;
    P.xcd_chunks = 0;

    long bad_total = 0;
    for (int late = 0; late < 2; ++late) {
        g_host_late = late != 0;
        std::vector<char> Cw = C;
        P.C = Cw.data();
        memset(sthip::smem, 0xEE, sizeof(sthip::smem));
        if (walking) launch(gemm4p_kernel<T, B_KC>, P, grid);
        else launch(gemm4_kernel<T, B_KC>, P, (unsigned)(nprod * P.tiles_m * P.tiles_n));
        long bad = 0;
        for (int p = 0; p < nprod; ++p)
            for (int m = 0; m < M; ++m)
                for (int n = 0; n < N; ++n) {
                    float want = C0[p * c_elems + (size_t)m * N + n];
                    for (int k = 0; k < K; ++k) want += Af[p * a_elems + (size_t)m * K + k] * Bf[p * b_elems + (size_t)k * N + n];
                    float got;
                    const size_t i = p * c_elems + (size_t)m * N + n;
                    if (es_out == 4) memcpy(&got, &Cw[i * 4], 4);
                    else { uint16_t h; memcpy(&h, &Cw[i * 2], 2); got = from_half(h, bf); }
                    if (got != want && bad++ < 5) fprintf(stderr, "  %s: C[%d][%d][%d] = %g, expected %g\n", name, p, m, n, got, want);
                }
        printf("%s  loads %s: %ld wrong of %zu\n", name, late ? "at the last moment" : "at once", bad, (size_t)nprod * c_elems);
        fflush(stdout);
        bad_total += bad;
    }
    return bad_total;
}
}  // namespace

// 64 x 64 fp32 kernel: `nprod` products C_q = (A0 +- A1)(B0 +- B1) (or single blocks) of M x N x K.
template <bool B_KC>
long run_case6(const char* name, int nprod, int M, int N, int K, bool sums, bool accumulate) {
    const size_t a_elems = (size_t)M * K, b_elems = (size_t)K * N, c_elems = (size_t)M * N;
    std::vector<float> A(2 * nprod * a_elems), Bs(2 * nprod * b_elems), Bf(2 * nprod * b_elems), C0(nprod * c_elems);
    uint32_t seed = 999u + (uint32_t)(M + 3 * N + 7 * K);
    for (auto& v : A) v = (float)small_int(seed);
    for (int p = 0; p < 2 * nprod; ++p)
        for (int k = 0; k < K; ++k)
            for (int n = 0; n < N; ++n) {
                const float v = (float)small_int(seed);
                Bf[p * b_elems + (size_t)k * N + n] = v;
                Bs[p * b_elems + (B_KC ? (size_t)n * K + k : (size_t)k * N + n)] = v;
            }
    for (auto& v : C0) v = accumulate ? (float)small_int(seed) : 55.f;
    g_host_global = {{reinterpret_cast<const char*>(A.data()), A.size() * 4}, {reinterpret_cast<const char*>(Bs.data()), Bs.size() * 4}};
    Gemm6Params P;
    memset(&P, 0, sizeof(P));
    std::vector<int> sa(nprod), sb(nprod);
    for (int q = 0; q < nprod; ++q) {
        sa[q] = sums ? (q % 3 == 0 ? 1 : q % 3 == 1 ? -1 : 0) : 0;
        sb[q] = sums ? (q % 4 == 0 ? -1 : q % 4 == 1 ? 0 : 1) : 0;
        P.a[q] = Op6{A.data() + (2 * q) * a_elems, A.data() + (2 * q + 1) * a_elems, K, sa[q], 0};
        P.b[q] = Op6{Bs.data() + (2 * q) * b_elems, Bs.data() + (2 * q + 1) * b_elems, B_KC ? K : N, sb[q], 0};
    }
    P.c_rs = N; P.c_ps = (int64_t)c_elems; P.Kh = K; P.tiles_m = M / 64; P.tiles_n = N / 64; P.nprod = nprod; P.accumulate = accumulate;
    long bad_total = 0;
    for (int late = 0; late < 2; ++late) {
        g_host_late = late != 0;
        std::vector<float> Cw = C0;
        P.C = Cw.data();
        launch(gemm6_kernel<B_KC>, P, (unsigned)(nprod * P.tiles_m * P.tiles_n), 256);
        long bad = 0;
        for (int q = 0; q < nprod; ++q)
            for (int m = 0; m < M; ++m)
                for (int n = 0; n < N; ++n) {
                    float want = accumulate ? C0[q * c_elems + (size_t)m * N + n] : 0.f;
                    for (int k = 0; k < K; ++k) {
                        const float a = A[(2 * q) * a_elems + (size_t)m * K + k] + sa[q] * A[(2 * q + 1) * a_elems + (size_t)m * K + k];
                        const float b = Bf[(2 * q) * b_elems + (size_t)k * N + n] + sb[q] * Bf[(2 * q + 1) * b_elems + (size_t)k * N + n];
                        want += a * b;
                    }
                    const float got = Cw[q * c_elems + (size_t)m * N + n];
                    if (got != want && bad++ < 5) fprintf(stderr, "  %s: C[%d][%d][%d] = %g, expected %g\n", name, q, m, n, got, want);
                }
        printf("%s  loads %s: %ld wrong of %zu\n", name, late ? "at the last moment" : "at once", bad, (size_t)nprod * c_elems);
        fflush(stdout);
        bad_total += bad;
    }
    return bad_total;
}

// 256 x 128 kernel: classical (one segment, C = A B of M x N x K) or the seven segment products S_0..S_6 of
// Mh x Nh x Kh recombined in registers into the four quadrants of C (2 Mh x 2 Nh), one accumulator tile parked
// in global memory: Strassen order M3 M6 M5 M7 M1 M2 M4, Winograd order P1 P2 P6 P7 P5 P3 (-P4).
template <class T, int ALGO, bool B_KC>
long run_case3(const char* name, int Mh, int Nh, int Kh, bool out_f32, bool accumulate) {
    constexpr bool bf = __is_same(T, bf16_t);
    constexpr int NSEG = ALGO == ALGO_CLASSIC ? 1 : 7;
    const int Q = ALGO == ALGO_CLASSIC ? 1 : 2;
    const int es_out = out_f32 ? 4 : 2;
    const size_t a_elems = (size_t)Mh * Kh, b_elems = (size_t)Kh * Nh, c_elems = (size_t)Q * Mh * Q * Nh;
    const int ldc = Q * Nh;
    std::vector<uint16_t> A(NSEG * a_elems), B(NSEG * b_elems);
    std::vector<float> Af(NSEG * a_elems), Bf(NSEG * b_elems), C0(c_elems);
    std::vector<char> C(c_elems * es_out);
    uint32_t seed = 4242u + (uint32_t)(Mh + 5 * Nh + 11 * Kh + ALGO);
    for (size_t i = 0; i < Af.size(); ++i) { Af[i] = (float)small_int(seed); A[i] = to_half(Af[i], bf); }
    for (int p = 0; p < NSEG; ++p)
        for (int k = 0; k < Kh; ++k)
            for (int n = 0; n < Nh; ++n) {
                const float v = (float)small_int(seed);
                Bf[p * b_elems + (size_t)k * Nh + n] = v;
                B[p * b_elems + (B_KC ? (size_t)n * Kh + k : (size_t)k * Nh + n)] = to_half(v, bf);
            }
    for (size_t i = 0; i < c_elems; ++i) {
        C0[i] = accumulate ? (float)small_int(seed) : 0.f;
        if (es_out == 4) memcpy(&C[i * 4], &C0[i], 4);
        else { const uint16_t h = to_half(accumulate ? C0[i] : 77.f, bf); memcpy(&C[i * 2], &h, 2); }
    }
    g_host_global = {{reinterpret_cast<const char*>(A.data()), A.size() * 2}, {reinterpret_cast<const char*>(B.data()), B.size() * 2}};
    Gemm2Params P;
    memset(&P, 0, sizeof(P));
    for (int p = 0; p < NSEG; ++p) P.seg[p] = Seg2{A.data() + p * a_elems, B.data() + p * b_elems, Kh, B_KC ? Kh : Nh, 0, 0};
    P.c_rs = ldc; P.Mh = Mh; P.Nh = Nh; P.Kh = Kh; P.tiles_m = Mh / 256; P.tiles_n = Nh / 128; P.group_m = 4;
    P.out_f32 = out_f32; P.accumulate = accumulate;
    const unsigned grid = (unsigned)(P.tiles_m * P.tiles_n);
    std::vector<float> park((size_t)grid * 256 * 128);
    P.park = park.data();
    // the segment products
    std::vector<float> S(NSEG * (size_t)Mh * Nh, 0.f);
    for (int p = 0; p < NSEG; ++p)
        for (int m = 0; m < Mh; ++m)
            for (int k = 0; k < Kh; ++k) {
                const float a = Af[p * a_elems + (size_t)m * Kh + k];
                if (a == 0.f) continue;
                for (int n = 0; n < Nh; ++n) S[(p * (size_t)Mh + m) * Nh + n] += a * Bf[p * b_elems + (size_t)k * Nh + n];
            }
    auto seg = [&](int p, int m, int n) { return S[(p * (size_t)Mh + m) * Nh + n]; };
    long bad_total = 0;
    for (int late = 0; late < 2; ++late) {
        g_host_late = late != 0;
        std::vector<char> Cw = C;
        P.C = Cw.data();
        launch(gemm3_kernel<T, ALGO, B_KC>, P, grid, 256);
        long bad = 0;
        for (int m = 0; m < Q * Mh; ++m)
            for (int n = 0; n < Q * Nh; ++n) {
                const int qm = m / Mh, qn = n / Nh, mm = m % Mh, nn = n % Nh;
                float want = C0[(size_t)m * ldc + n];
                if (ALGO == ALGO_CLASSIC) want += seg(0, mm, nn);
                else if (ALGO == ALGO_STRASSEN) {   // segments: 0 M3, 1 M6, 2 M5, 3 M7, 4 M1, 5 M2, 6 M4
                    if (qm == 0 && qn == 0) want += seg(4, mm, nn) + seg(6, mm, nn) - seg(2, mm, nn) + seg(3, mm, nn);
                    else if (qm == 0) want += seg(0, mm, nn) + seg(2, mm, nn);
                    else if (qn == 0) want += seg(5, mm, nn) + seg(6, mm, nn);
                    else want += seg(4, mm, nn) - seg(5, mm, nn) + seg(0, mm, nn) + seg(1, mm, nn);
                } else {                            // segments: 0 P1, 1 P2, 2 P6, 3 P7, 4 P5, 5 P3, 6 -P4
                    const float u2 = seg(0, mm, nn) + seg(2, mm, nn), u3 = u2 + seg(3, mm, nn);
                    if (qm == 0 && qn == 0) want += seg(0, mm, nn) + seg(1, mm, nn);
                    else if (qm == 0) want += u2 + seg(4, mm, nn) + seg(5, mm, nn);
                    else if (qn == 0) want += u3 + seg(6, mm, nn);
                    else want += u3 + seg(4, mm, nn);
                }
                float got;
                const size_t i = (size_t)m * ldc + n;
                if (es_out == 4) memcpy(&got, &Cw[i * 4], 4);
                else { uint16_t h; memcpy(&h, &Cw[i * 2], 2); got = from_half(h, bf); }
                if (got != want && bad++ < 5) fprintf(stderr, "  %s: C[%d][%d] = %g, expected %g\n", name, m, n, got, want);
            }
        printf("%s  loads %s: %ld wrong of %zu\n", name, late ? "at the last moment" : "at once", bad, c_elems);
        fflush(stdout);
        bad_total += bad;
    }
    return bad_total;
}

// 128 x 128 pipelined kernel: `nprod` classical products side by side, or the seven segment products recombined in
// registers (three accumulator tiles, nothing parked).  A may be stored k x m (m-contiguous).
template <class T, int ALGO, bool A_KC, bool B_KC>
long run_case2(const char* name, int nprod, int Mh, int Nh, int Kh, bool out_f32, bool accumulate) {
    constexpr bool bf = __is_same(T, bf16_t);
    const int NSEG = ALGO == ALGO_CLASSIC ? nprod : 7;
    const int Q = ALGO == ALGO_CLASSIC ? 1 : 2;
    const int es_out = out_f32 ? 4 : 2;
    const size_t a_elems = (size_t)Mh * Kh, b_elems = (size_t)Kh * Nh, c_one = (size_t)Q * Mh * Q * Nh;
    const size_t c_elems = (ALGO == ALGO_CLASSIC ? nprod : 1) * c_one;
    const int ldc = Q * Nh;
    std::vector<uint16_t> A(NSEG * a_elems), B(NSEG * b_elems);
    std::vector<float> Af(NSEG * a_elems), Bf(NSEG * b_elems), C0(c_elems);
    std::vector<char> C(c_elems * es_out);
    uint32_t seed = 777u + (uint32_t)(Mh + 5 * Nh + 11 * Kh + ALGO + 2 * A_KC + B_KC);
    for (int p = 0; p < NSEG; ++p) {
        for (int m = 0; m < Mh; ++m)
            for (int k = 0; k < Kh; ++k) {
                const float v = (float)small_int(seed);
                Af[p * a_elems + (size_t)m * Kh + k] = v;
                A[p * a_elems + (A_KC ? (size_t)m * Kh + k : (size_t)k * Mh + m)] = to_half(v, bf);
            }
        for (int k = 0; k < Kh; ++k)
            for (int n = 0; n < Nh; ++n) {
                const float v = (float)small_int(seed);
                Bf[p * b_elems + (size_t)k * Nh + n] = v;
                B[p * b_elems + (B_KC ? (size_t)n * Kh + k : (size_t)k * Nh + n)] = to_half(v, bf);
            }
    }
    for (size_t i = 0; i < c_elems; ++i) {
        C0[i] = accumulate ? (float)small_int(seed) : 0.f;
        if (es_out == 4) memcpy(&C[i * 4], &C0[i], 4);
        else { const uint16_t h = to_half(accumulate ? C0[i] : 77.f, bf); memcpy(&C[i * 2], &h, 2); }
    }
    g_host_global = {{reinterpret_cast<const char*>(A.data()), A.size() * 2}, {reinterpret_cast<const char*>(B.data()), B.size() * 2}};
    Gemm2Params P;
    memset(&P, 0, sizeof(P));
    for (int p = 0; p < NSEG; ++p) P.seg[p] = Seg2{A.data() + p * a_elems, B.data() + p * b_elems, A_KC ? Kh : Mh, B_KC ? Kh : Nh, 0, 0};
    P.c_rs = ldc; P.c_ps = (int64_t)c_one; P.nprod = ALGO == ALGO_CLASSIC ? nprod : 0;
    P.Mh = Mh; P.Nh = Nh; P.Kh = Kh; P.tiles_m = Mh / 128; P.tiles_n = Nh / 128; P.group_m = 4;
    P.out_f32 = out_f32; P.accumulate = accumulate;
    const unsigned grid = (unsigned)(P.tiles_m * P.tiles_n * (ALGO == ALGO_CLASSIC ? nprod : 1));
    std::vector<float> S(NSEG * (size_t)Mh * Nh, 0.f);
    for (int p = 0; p < NSEG; ++p)
        for (int m = 0; m < Mh; ++m)
            for (int k = 0; k < Kh; ++k) {
                const float a = Af[p * a_elems + (size_t)m * Kh + k];
                if (a == 0.f) continue;
                for (int n = 0; n < Nh; ++n) S[(p * (size_t)Mh + m) * Nh + n] += a * Bf[p * b_elems + (size_t)k * Nh + n];
            }
    auto seg = [&](int p, int m, int n) { return S[(p * (size_t)Mh + m) * Nh + n]; };
    long bad_total = 0;
    for (int late = 0; late < 2; ++late) {
        g_host_late = late != 0;
        std::vector<char> Cw = C;
        P.C = Cw.data();
        launch(gemm2_kernel<T, ALGO, A_KC, B_KC>, P, grid, 256);
        long bad = 0;
        for (int q = 0; q < (ALGO == ALGO_CLASSIC ? nprod : 1); ++q)
            for (int m = 0; m < Q * Mh; ++m)
                for (int n = 0; n < Q * Nh; ++n) {
                    const int qm = m / Mh, qn = n / Nh, mm = m % Mh, nn = n % Nh;
                    const size_t i = q * c_one + (size_t)m * ldc + n;
                    float want = C0[i];
                    if (ALGO == ALGO_CLASSIC) want += seg(q, mm, nn);
                    else if (ALGO == ALGO_STRASSEN) {
                        if (qm == 0 && qn == 0) want += seg(4, mm, nn) + seg(6, mm, nn) - seg(2, mm, nn) + seg(3, mm, nn);
                        else if (qm == 0) want += seg(0, mm, nn) + seg(2, mm, nn);
                        else if (qn == 0) want += seg(5, mm, nn) + seg(6, mm, nn);
                        else want += seg(4, mm, nn) - seg(5, mm, nn) + seg(0, mm, nn) + seg(1, mm, nn);
                    } else {
                        const float u2 = seg(0, mm, nn) + seg(2, mm, nn), u3 = u2 + seg(3, mm, nn);
                        if (qm == 0 && qn == 0) want += seg(0, mm, nn) + seg(1, mm, nn);
                        else if (qm == 0) want += u2 + seg(4, mm, nn) + seg(5, mm, nn);
                        else if (qn == 0) want += u3 + seg(6, mm, nn);
                        else want += u3 + seg(4, mm, nn);
                    }
                    float got;
                    if (es_out == 4) memcpy(&got, &Cw[i * 4], 4);
                    else { uint16_t h; memcpy(&h, &Cw[i * 2], 2); got = from_half(h, bf); }
                    if (got != want && bad++ < 5) fprintf(stderr, "  %s: C[%d][%d][%d] = %g, expected %g\n", name, q, m, n, got, want);
                }
        printf("%s  loads %s: %ld wrong of %zu\n", name, late ? "at the last moment" : "at once", bad, c_elems);
        fflush(stdout);
        bad_total += bad;
    }
    return bad_total;
}

// The fused 128 x 128 kernel (operands straight from A and B, quadrant sums formed in registers, seven products
// recombined in registers): C = A B over the whole M x N x K problem, any sizes with EDGE (virtual zero padding).
template <class T, int ALGO, bool A_KC, bool B_KC, bool EDGE>
long run_case_fused(const char* name, int M, int N, int K, bool out_f32, bool accumulate) {
    constexpr bool f32 = __is_same(T, float), bf = __is_same(T, bf16_t);
    constexpr int ES = f32 ? 4 : 2, EPC = 16 / ES;
    const int es_out = (f32 || out_f32) ? 4 : 2;
    std::vector<char> A((size_t)M * K * ES), B((size_t)K * N * ES), C((size_t)M * N * es_out);
    std::vector<float> Af((size_t)M * K), Bf((size_t)K * N), C0((size_t)M * N);
    uint32_t seed = 31337u + (uint32_t)(M + 5 * N + 11 * K + ALGO + 2 * A_KC + B_KC);
    auto put = [&](std::vector<char>& buf, size_t i, float v) {
        if (f32) memcpy(&buf[i * 4], &v, 4);
        else { const uint16_t h = to_half(v, bf); memcpy(&buf[i * 2], &h, 2); }
    };
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            const float v = (float)small_int(seed);
            Af[(size_t)m * K + k] = v;
            put(A, A_KC ? (size_t)m * K + k : (size_t)k * M + m, v);
        }
    for (int k = 0; k < K; ++k)
        for (int n = 0; n < N; ++n) {
            const float v = (float)small_int(seed);
            Bf[(size_t)k * N + n] = v;
            put(B, B_KC ? (size_t)n * K + k : (size_t)k * N + n, v);
        }
    for (size_t i = 0; i < C0.size(); ++i) {
        C0[i] = accumulate ? (float)small_int(seed) : 0.f;
        if (es_out == 4) memcpy(&C[i * 4], &C0[i], 4);
        else { const uint16_t h = to_half(accumulate ? C0[i] : 77.f, bf); memcpy(&C[i * 2], &h, 2); }
    }
    const bool split = ALGO != ALGO_CLASSIC;
    GemmParams P;
    memset(&P, 0, sizeof(P));
    P.A = A.data(); P.B = B.data();
    P.a_rs = A_KC ? K : 1; P.a_cs = A_KC ? 1 : M;
    P.b_rs = B_KC ? 1 : N; P.b_cs = B_KC ? K : 1;
    P.c_rs = N; P.c_cs = 1;
    P.M = M; P.N = N; P.K = K;
    P.Mh = split ? (M + 1) / 2 : M; P.Nh = split ? (N + 1) / 2 : N; P.Kh = split ? (K + 1) / 2 : K;
    P.tiles_m = (P.Mh + 127) / 128; P.tiles_n = (P.Nh + 127) / 128;
    P.out_f32 = es_out == 4 && !f32 ? 1 : (f32 ? 1 : 0); P.accumulate = accumulate; P.group_m = 8;
    const int a_long = A_KC ? K : M, b_long = B_KC ? K : N, a_blk = A_KC ? P.Kh : P.Mh, b_blk = B_KC ? P.Kh : P.Nh;
    P.a_vec = a_long % EPC == 0 && (!split || a_blk % EPC == 0);
    P.b_vec = b_long % EPC == 0 && (!split || b_blk % EPC == 0);
    P.c_vec = N % 4 == 0 && (!split || P.Nh % 4 == 0);
    long bad_total = 0;
    g_host_global.clear();
    for (int late = 0; late < 1; ++late) {   // this kernel loads through registers with plain loads: one timing
        g_host_late = false;
        std::vector<char> Cw = C;
        P.C = Cw.data();
        launch(gemm_kernel<T, ALGO, A_KC, B_KC, EDGE>, P, (unsigned)(P.tiles_m * P.tiles_n), 256);
        long bad = 0;
        for (int m = 0; m < M; ++m)
            for (int n = 0; n < N; ++n) {
                float want = C0[(size_t)m * N + n];
                for (int k = 0; k < K; ++k) want += Af[(size_t)m * K + k] * Bf[(size_t)k * N + n];
                float got;
                const size_t i = (size_t)m * N + n;
                if (es_out == 4) memcpy(&got, &Cw[i * 4], 4);
                else { uint16_t h; memcpy(&h, &Cw[i * 2], 2); got = from_half(h, bf); }
                if (got != want && bad++ < 5) fprintf(stderr, "  %s: C[%d][%d] = %g, expected %g\n", name, m, n, got, want);
            }
        printf("%s: %ld wrong of %zu\n", name, bad, (size_t)M * N);
        fflush(stdout);
        bad_total += bad;
    }
    return bad_total;
}

// Every tile id of a launch must map to a different (batch, product, tile row, tile column), all of them in range.
long check_tile_numbering(int tiles_m, int tiles_n, int nprod, int nbatch, int xcd_chunks, int group_m) {
    Gemm2Params P;
    memset(&P, 0, sizeof(P));
    P.tiles_m = tiles_m; P.tiles_n = tiles_n; P.nprod = nprod; P.nbatch = nbatch; P.xcd_chunks = xcd_chunks; P.group_m = group_m;
    const int total = tiles_m * tiles_n * nprod * nbatch;
    std::vector<char> seen((size_t)total, 0);
    long bad = 0;
    for (int id = 0; id < total; ++id) {
        int prod, batch, tm, tn;
        map_tile4(P, id, prod, batch, tm, tn);
        if (prod < 0 || prod >= nprod || batch < 0 || batch >= nbatch || tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) { ++bad; continue; }
        const size_t key = (((size_t)batch * nprod + prod) * tiles_m + tm) * tiles_n + tn;
        if (seen[key]++) ++bad;
    }
    printf("tile numbering %d x %d tiles, %d products, batch %d, chunks %d, group %d: %ld wrong of %d\n", tiles_m, tiles_n, nprod, nbatch, xcd_chunks, group_m, bad, total);
    return bad;
}

int main(int argc, char** argv) {
    // no argument: every case; "5": case 5 alone; "1/3": the cases whose number leaves 1 when divided by 3
    const int which = argc > 1 ? atoi(argv[1]) : -1;
    const int shares = argc > 1 && strchr(argv[1], '/') ? atoi(strchr(argv[1], '/') + 1) : 0;
    int id = 0;
    auto want = [&]() { const int i = id++; return shares ? i % shares == which : which < 0 || which == i; };
    long bad = 0;
    // workgroups that walk their tiles: 4 tiles on 2 workgroups, odd number of k-steps
    if (want()) bad += run_case<bf16_t, false>("walking bf16, B n-contiguous, 512x512x192, 2 workgroups", 1, 512, 512, 192, 2, true, false, false);
    if (want()) bad += run_case<bf16_t, true>("walking bf16, B k-contiguous, 512x512x192, 2 workgroups", 1, 512, 512, 192, 2, true, false, false);
    // two products side by side, 4 tiles on 3 workgroups (one walks two, tiles of different products)
    if (want()) bad += run_case<f16_t, false>("walking fp16, two products of 256x512x128, 3 workgroups", 2, 256, 512, 128, 3, true, false, false);
    if (want()) bad += run_case<bf16_t, true>("walking bf16, batch of three 256x256x128, 2 workgroups", 3, 256, 256, 128, 2, true, false, false, true);
    // one tile per workgroup: plain, fp32 result, accumulating
    if (want()) bad += run_case<bf16_t, true>("one tile per workgroup bf16, 256x512x64 (one k-step)", 1, 256, 512, 64, 0, false, false, false);
    if (want()) bad += run_case<bf16_t, false>("one tile per workgroup bf16 -> fp32, 256x256x128", 1, 256, 256, 128, 0, false, true, false);
    if (want()) bad += run_case<f16_t, true>("one tile per workgroup fp16, accumulating, 256x256x128", 1, 256, 256, 128, 0, false, false, true);
    if (want()) bad += run_case<bf16_t, false>("one tile per workgroup bf16, store straight from the accumulators, 256x256x64", 1, 256, 256, 64, 0, false, false, false, false, false);
    if (want()) bad += run_case<bf16_t, true>("one tile per workgroup bf16 -> fp32, accumulating, 256x256x64", 1, 256, 256, 64, 0, false, true, true);
    if (want()) bad += run_case<f16_t, true>("walking fp16, three tiles of two k-steps on 2 workgroups, 768x256x128", 1, 768, 256, 128, 2, true, false, false);
    // the 64 x 64 fp32 kernel: one product, and seven with operand sums formed in the loads
    if (want()) bad += run_case6<false>("64x64 fp32, one product 128x192x128, B n-contiguous", 1, 128, 192, 128, false, false);
    if (want()) bad += run_case6<true>("64x64 fp32, one product 128x128x64, B k-contiguous, accumulating", 1, 128, 128, 64, false, true);
    if (want()) bad += run_case6<false>("64x64 fp32, seven products 128x128x128 of operand sums, B n-contiguous", 7, 128, 128, 128, true, false);
    if (want()) bad += run_case6<true>("64x64 fp32, seven products 64x128x64 of operand sums, B k-contiguous", 7, 64, 128, 64, true, false);
    // the 256 x 128 kernel: classical, and the seven products recombined in registers
    if (want()) bad += run_case3<bf16_t, ALGO_CLASSIC, false>("256x128 bf16 classical, 256x256x192, B n-contiguous", 256, 256, 192, false, false);
    if (want()) bad += run_case3<f16_t, ALGO_STRASSEN, false>("256x128 fp16 Strassen in registers, halves 256x128x128 -> fp32", 256, 128, 128, true, false);
    if (want()) bad += run_case3<bf16_t, ALGO_STRASSEN, true>("256x128 bf16 Strassen in registers, halves 256x256x64, B k-contiguous, accumulating fp32", 256, 256, 64, true, true);
    if (want()) bad += run_case3<bf16_t, ALGO_WINOGRAD, false>("256x128 bf16 Winograd in registers, halves 256x128x128 -> fp32", 256, 128, 128, true, false);
    // the 128 x 128 pipelined kernel
    if (want()) bad += run_case2<bf16_t, ALGO_CLASSIC, true, false>("128x128 bf16, three products of 128x256x128 side by side", 3, 128, 256, 128, false, false);
    if (want()) bad += run_case2<f16_t, ALGO_CLASSIC, false, true>("128x128 fp16, A m-contiguous, B k-contiguous, 256x128x192, accumulating", 1, 256, 128, 192, false, true);
    if (want()) bad += run_case2<bf16_t, ALGO_STRASSEN, true, false>("128x128 bf16 Strassen in registers, halves 128x128x64, 16-bit result", 1, 128, 128, 64, false, false);
    if (want()) bad += run_case2<f16_t, ALGO_WINOGRAD, false, false>("128x128 fp16 Winograd in registers, A m-contiguous, halves 128x256x128 -> fp32, accumulating", 1, 128, 256, 128, true, true);
    // the fused kernel: whole problems, quadrant sums in registers; odd sizes through the EDGE form
    if (want()) bad += run_case_fused<bf16_t, ALGO_STRASSEN, true, false, false>("fused bf16 Strassen, 256x256x128", 256, 256, 128, false, false);
    if (want()) bad += run_case_fused<f16_t, ALGO_WINOGRAD, true, true, false>("fused fp16 Winograd, B k-contiguous, 256x512x128 -> fp32, accumulating", 256, 512, 128, true, true);
    if (want()) bad += run_case_fused<bf16_t, ALGO_STRASSEN, true, false, true>("fused bf16 Strassen, odd sizes 201x137x99", 201, 137, 99, false, false);
    if (want()) bad += run_case_fused<f16_t, ALGO_WINOGRAD, false, true, true>("fused fp16 Winograd, A m-contiguous, B k-contiguous, odd sizes 130x260x77 -> fp32", 130, 260, 77, true, false);
    if (want()) bad += run_case_fused<float, ALGO_STRASSEN, true, false, true>("fused fp32 Strassen, odd sizes 150x131x45, accumulating", 150, 131, 45, true, true);
    if (want()) bad += run_case_fused<bf16_t, ALGO_CLASSIC, false, false, true>("fused bf16 classical, A m-contiguous, 129x257x65", 129, 257, 65, false, false);
    // fp32 operands (k-steps of 32)
    if (want()) bad += run_case<float, false>("one tile per workgroup fp32, B n-contiguous, 256x256x96", 1, 256, 256, 96, 0, false, true, false);
    if (want()) bad += run_case<float, true>("one tile per workgroup fp32, B k-contiguous, accumulating, 256x256x64", 1, 256, 256, 64, 0, false, true, true);
    if (which < 0 || (shares && which == 0)) {
        // the launcher's choices: chunks for products of 32 / 64 / 128 tiles with tiles_m % 4 == 0 and >= 256 tiles in all
        bad += check_tile_numbering(16, 16, 7, 1, 0, 4);
        bad += check_tile_numbering(32, 32, 1, 1, 0, 8);
        bad += check_tile_numbering(8, 8, 49, 1, 1, 4);
        bad += check_tile_numbering(8, 16, 7, 1, 1, 4);
        bad += check_tile_numbering(4, 8, 7, 8, 1, 4);
        bad += check_tile_numbering(8, 4, 9, 1, 1, 4);     // 288 tiles: one chunk set of 256, the rest numbered plainly
        bad += check_tile_numbering(3, 5, 7, 2, 0, 4);
        bad += check_tile_numbering(32, 9, 1, 1, 0, 8);
        bad += check_tile_numbering(5, 3, 1, 1, 0, 4);
    }
    printf("%s\n", bad ? "FAILED" : "ALL EXACT");
    return bad ? 1 : 0;
}
