// Calls into the CPU build of the library, driven by a script (tests/test_host_parity.py writes it).  One statement per line:
//   buf NAME BYTES [FILE]     a 256-byte aligned buffer of BYTES bytes, zero or read from FILE ("device" memory)
//   wsbuf NAME batch M N K in_dtype out_dtype algo levels      a buffer of sthip_workspace_bytes(...) bytes
//   sumsbuf NAME in_features out_features dtype levels          a buffer of sthip_linear_weight_sums_bytes(...) bytes
//   save NAME FILE            write a buffer to FILE
//   units N                   compute units the "device" reports        tile NAME|-    force a tile of the pipelined paths
//   stages MASK               sthip_debug_set_stages(MASK)
//   one_launch_counters WS M N K TILES   sthip_debug_one_launch_counters: nobody gave up, every product counted TILES tiles
//   expect CODE               the following call must return CODE (default 0)
//   gemm / gemm_static / n_layers / run_accumulate / linear_strassen / linear / prepare / linear_prepared ARGS...
//                             the entry point of include/strassen_hip.h of that name, arguments in its order, buffers by
//                             name ("-" = null, NAME+BYTES = a view that starts BYTES into the buffer), a workspace as one buffer name standing for pointer and size
#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include "host_runtime.h"
#include "strassen_hip.h"
#include "strassen_hip_debug.h"

struct Buf { std::vector<char> raw; char* p = nullptr; size_t n = 0; };
static std::map<std::string, Buf> g_bufs;

static Buf* buf(std::istringstream& in) {
    std::string name;
    in >> name;
    if (name == "-") return nullptr;
    if (!g_bufs.count(name)) { fprintf(stderr, "no buffer %s\n", name.c_str()); exit(2); }
    return &g_bufs[name];
}
static void* ptr(std::istringstream& in) {   // NAME or NAME+BYTES (a view that starts inside the buffer)
    std::string name;
    in >> name;
    if (name == "-") return nullptr;
    const size_t plus = name.find('+');
    const size_t off = plus == std::string::npos ? 0 : std::stoull(name.substr(plus + 1));
    name = name.substr(0, plus);
    if (!g_bufs.count(name)) { fprintf(stderr, "no buffer %s\n", name.c_str()); exit(2); }
    return g_bufs[name].p + off;
}
static int64_t num(std::istringstream& in) { long long v; if (!(in >> v)) { fprintf(stderr, "number expected\n"); exit(2); } return v; }
static void strides(std::istringstream& in, int64_t s[3]) { for (int i = 0; i < 3; ++i) s[i] = num(in); }

int main(int argc, char** argv) {
    if (argc < 2) return 2;
    std::ifstream script(argv[1]);
    std::string line;
    int expect = 0;
    while (std::getline(script, line)) {
        std::istringstream in(line);
        std::string op;
        if (!(in >> op) || op[0] == '#') continue;
        int rc = 0;
        bool call = true;
        g_host_global.clear();
        for (auto& kv : g_bufs) g_host_global.push_back({kv.second.p, kv.second.n + 64});
        if (op == "buf" || op == "wsbuf" || op == "sumsbuf") {
            std::string name, file;
            in >> name;
            size_t n;
            if (op == "buf") {
                n = num(in);
            } else if (op == "wsbuf") {
                const int64_t batch = num(in), M = num(in), N = num(in), K = num(in);
                const int dt = num(in), odt = num(in), algo = num(in), levels = num(in);
                n = sthip_workspace_bytes(batch, M, N, K, dt, odt, algo, levels);
            } else {
                const int64_t fin = num(in), fout = num(in);
                const int dt = num(in), levels = num(in);
                n = sthip_linear_weight_sums_bytes(fin, fout, dt, levels);
                if (!n) { fprintf(stderr, "no sums can be kept for this layer\n"); return 1; }
            }
            Buf& b = g_bufs[name];
            b.raw.assign(n + 512, 0);
            b.p = (char*)(((uintptr_t)b.raw.data() + 255) & ~(uintptr_t)255);
            b.n = n;
            if (in >> file) {
                FILE* f = fopen(file.c_str(), "rb");
                if (!f || fread(b.p, 1, n, f) != n) { fprintf(stderr, "cannot read %s\n", file.c_str()); return 2; }
                fclose(f);
            }
            call = false;
        } else if (op == "save") {
            Buf* b = buf(in);
            std::string file;
            in >> file;
            FILE* f = fopen(file.c_str(), "wb");
            if (!f || fwrite(b->p, 1, b->n, f) != b->n) return 2;
            fclose(f);
            call = false;
        } else if (op == "units") {
            g_host_compute_units = (int)num(in);
            call = false;
        } else if (op == "tile") {
            std::string t;
            in >> t;
            sthip_debug_force_tile(t == "-" ? nullptr : t.c_str());
            call = false;
        } else if (op == "stages") {
            sthip_debug_set_stages((int)num(in));
            call = false;
        } else if (op == "expect") {
            expect = (int)num(in);
            call = false;
        } else if (op == "gemm" || op == "gemm_static") {
            void *A = ptr(in), *B = ptr(in), *C = ptr(in);
            const int64_t batch = num(in), M = num(in), N = num(in), K = num(in);
            int64_t sA[3], sB[3], sC[3];
            strides(in, sA), strides(in, sB), strides(in, sC);
            const int dt = num(in), odt = num(in), algo = num(in), levels = num(in), acc = num(in);
            if (op == "gemm") {
                Buf* ws = buf(in);
                rc = sthip_gemm(A, B, C, batch, M, N, K, sA, sB, sC, dt, odt, algo, levels, acc, ws ? ws->p : nullptr, ws ? ws->n : 0, nullptr);
            } else {
                rc = sthip_gemm_static(A, B, C, batch, M, N, K, sA, sB, sC, dt, odt, algo, levels, acc, nullptr);
            }
        } else if (op == "one_launch_counters") {
            Buf* ws = buf(in);
            const int64_t M = num(in), N = num(in), K = num(in), tiles = num(in);
            unsigned c[16];
            rc = sthip_debug_one_launch_counters(ws->p, M, N, K, c, nullptr);
            for (int p = 8; p < 15 && rc == 0; ++p)
                if (c[p] != (unsigned)tiles) { fprintf(stderr, "product %d counted %u tiles, expected %lld\n", p - 8, c[p], (long long)tiles); return 1; }
        } else if (op == "n_layers") {
            void *A = ptr(in), *B = ptr(in), *C = ptr(in);
            const int64_t n = num(in), ar = num(in), ac = num(in), br = num(in), bc = num(in);
            const int dt = num(in), levels = num(in);
            Buf* ws = buf(in);
            rc = sthip_strassen_matmul_n_layers(A, B, C, n, ar, ac, br, bc, dt, levels, ws ? ws->p : nullptr, ws ? ws->n : 0, nullptr);
        } else if (op == "run_accumulate") {
            void *A = ptr(in), *B = ptr(in), *C = ptr(in);
            const int64_t batch = num(in), M = num(in), N = num(in), K = num(in);
            const int dt = num(in), cdt = num(in), algo = num(in), levels = num(in);
            Buf* ws = buf(in);
            rc = sthip_run_accumulate(A, B, C, batch, M, N, K, dt, cdt, algo, levels, ws ? ws->p : nullptr, ws ? ws->n : 0, nullptr);
        } else if (op == "linear_strassen") {
            void *x = ptr(in), *W = ptr(in), *bias = ptr(in), *y = ptr(in);
            const int64_t rows = num(in), D = num(in);
            const int dt = num(in), levels = num(in);
            Buf* ws = buf(in);
            rc = sthip_linear_strassen_forward(x, W, bias, y, rows, D, dt, levels, ws ? ws->p : nullptr, ws ? ws->n : 0, nullptr);
        } else if (op == "linear") {
            void *x = ptr(in), *W = ptr(in), *bias = ptr(in), *y = ptr(in);
            const int64_t rows = num(in), fin = num(in), fout = num(in);
            const int dt = num(in), levels = num(in);
            Buf* ws = buf(in);
            rc = sthip_linear_forward(x, W, bias, y, rows, fin, fout, dt, levels, ws ? ws->p : nullptr, ws ? ws->n : 0, nullptr);
        } else if (op == "prepare") {
            void* W = ptr(in);
            const int64_t fin = num(in), fout = num(in);
            const int dt = num(in), levels = num(in);
            Buf* sums = buf(in);
            rc = sthip_linear_prepare_weight(W, fin, fout, dt, levels, sums->p, sums->n, nullptr);
        } else if (op == "linear_prepared") {
            void *x = ptr(in), *W = ptr(in);
            Buf* sums = buf(in);
            void *bias = ptr(in), *y = ptr(in);
            const int64_t rows = num(in), fin = num(in), fout = num(in);
            const int dt = num(in), levels = num(in);
            Buf* ws = buf(in);
            rc = sthip_linear_forward_prepared(x, W, sums ? sums->p : nullptr, sums ? sums->n : 0, bias, y, rows, fin, fout, dt, levels,
                                               ws ? ws->p : nullptr, ws ? ws->n : 0, nullptr);
        } else {
            fprintf(stderr, "unknown statement %s\n", op.c_str());
            return 2;
        }
        if (call) {
            if (rc != expect) { fprintf(stderr, "%s: returned %d, expected %d: %s\n", op.c_str(), rc, expect, sthip_last_error()); return 1; }
            expect = 0;
        }
    }
    return 0;
}
