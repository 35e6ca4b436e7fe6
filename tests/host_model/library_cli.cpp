// One sthip_gemm call on the CPU build of the library, driven from a file (tests/test_host_parity.py writes it):
// header, then the storage of A, of B and of C as the caller holds them; the storage of C is written back.
#include "host_runtime.h"
#include "strassen_hip.h"
#include "strassen_hip_debug.h"

struct Job {
    int64_t batch, M, N, K;
    int64_t sA[3], sB[3], sC[3];
    int64_t a_bytes, b_bytes, c_bytes;
    int32_t dt, out_dt, algo, levels, accumulate, use_ws, tile, cus;
};

int main(int argc, char** argv) {
    if (argc < 3) return 2;
    FILE* f = fopen(argv[1], "rb");
    if (!f) return 2;
    Job j;
    if (fread(&j, sizeof(j), 1, f) != 1) return 2;
    std::vector<char> a(j.a_bytes + 64), b(j.b_bytes + 64), c(j.c_bytes + 64);
    if (fread(a.data(), 1, j.a_bytes, f) != (size_t)j.a_bytes || fread(b.data(), 1, j.b_bytes, f) != (size_t)j.b_bytes ||
        fread(c.data(), 1, j.c_bytes, f) != (size_t)j.c_bytes) return 2;
    fclose(f);
    static const char* tiles[] = {nullptr, "128x128", "256x128", "128x128g", "256x256", "64x64"};
    g_host_compute_units = j.cus > 0 ? j.cus : 4;
    sthip_debug_force_tile(tiles[j.tile]);
    const size_t need = j.use_ws ? sthip_workspace_bytes(j.batch, j.M, j.N, j.K, j.dt, j.out_dt, j.algo, j.levels) : 0;
    std::vector<char> wsbuf(need + 512);
    char* ws = need ? (char*)(((uintptr_t)wsbuf.data() + 255) & ~(uintptr_t)255) : nullptr;
    g_host_global = {{a.data(), a.size()}, {b.data(), b.size()}, {c.data(), c.size()}, {wsbuf.data(), wsbuf.size()}};
    const int rc = sthip_gemm(a.data(), b.data(), c.data(), j.batch, j.M, j.N, j.K, j.sA, j.sB, j.sC, j.dt, j.out_dt, j.algo, j.levels,
                              j.accumulate, ws, need, nullptr);
    if (rc != STHIP_OK) { fprintf(stderr, "sthip_gemm: %d %s\n", rc, sthip_last_error()); return 1; }
    f = fopen(argv[2], "wb");
    if (!f || fwrite(c.data(), 1, j.c_bytes, f) != (size_t)j.c_bytes) return 2;
    fclose(f);
    return 0;
}
