// Fused Strassen / Strassen-Winograd / classical GEMM kernel for gfx950 (CDNA4, wave64).
//
// One workgroup owns one BM x BN tile position (i, j) of the *half-size* output grid and
// computes all seven sub-products for that position back to back.  Each product's
// operand tiles are read straight from the caller's A and B: the quadrant pre-additions
// (A11+A22, B12-B22, ...) happen in registers between the 128-bit global load and the LDS
// store, so no S or M matrix ever exists in HBM.  The recombination C11 = M1+M4-M5+M7 ...
// is done on the fp32 MFMA accumulators with at most three accumulator tiles live
// (product order M3 M6 M5 M7 M1 M2 M4; M6 and M7 accumulate in place), and every C
// quadrant tile is written exactly once.
//
// The formulas are those of the reference's one-level routine (fixed_strassen.py:39-51,
// fixed_strassen_fp32_agg.py:38-50); the Winograd schedule is the textbook 7-product /
// 15-addition form (the reference has no correct one).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sthip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

struct bf16_t { uint16_t v; };   // tag types: storage is 2 bytes, arithmetic is explicit
struct f16_t { uint16_t v; };

__device__ s16x4 lds_read_tr16_b64(const char* p);   // the transposing LDS read, defined in sthip_prims.hpp

enum { ALGO_CLASSIC = 0, ALGO_STRASSEN = 1, ALGO_WINOGRAD = 2 };

// Everything the kernel needs, passed by value.  Strides are in elements.
struct GemmParams {
    const void* A; const void* B; void* C;
    int64_t a_rs, a_cs, a_bs;   // A[m][k]
    int64_t b_rs, b_cs, b_bs;   // B[k][n]
    int64_t c_rs, c_cs, c_bs;   // C[m][n]
    int M, N, K;                // logical problem size
    int Mh, Nh, Kh;             // size of one operand block (M,N,K when classical, ceil(x/2) else)
    int tiles_m, tiles_n;       // tile grid over Mh x Nh
    int out_f32;                // C holds float (else the operand type)
    int accumulate;             // C += product instead of C = product
    int group_m;                // tile-rows per rasterisation group
    int a_vec, b_vec, c_vec;    // EDGE kernels only: 16-byte (A,B) / 4-element (C) accesses are legal
};

constexpr int kThreads = 256;
constexpr int kBM = 128, kBN = 128;

template <class T> struct ElemTraits;
template <> struct ElemTraits<float> { static constexpr int EPC = 4; };
template <> struct ElemTraits<bf16_t> { static constexpr int EPC = 8; };
template <> struct ElemTraits<f16_t> { static constexpr int EPC = 8; };

// Geometry of one operand tile in LDS.  KC = the operand is contiguous along k in memory
// (LDS rows are m/n indices, 128 bytes of k each); otherwise it is contiguous along m/n
// (LDS rows are k indices).  A row is padded so that the fragment reads spread over banks.
template <class T, bool KC>
struct TileGeom {
    static constexpr int EPC = ElemTraits<T>::EPC;        // elements per 16-byte chunk
    static constexpr int BK = 8 * EPC;                    // 128 bytes of k per step
    static constexpr int CPR = KC ? 8 : kBM / EPC;        // chunks per memory row
    static constexpr int RPP = kThreads / CPR;            // memory rows covered per pass
    static constexpr int NROWS = KC ? kBM : BK;
    static constexpr int PASSES = NROWS / RPP;
    static constexpr int ROWB = KC ? 144 : kBM * (int)sizeof(T) + (sizeof(T) == 2 ? 64 : 32);
    static constexpr int BYTES = ROWB * NROWS;
    static_assert(PASSES == 4, "four 16-byte chunks per thread per term");
};

// ------------------------------------------------------------------ element arithmetic
// A load / store with a streaming (nontemporal) hint when `streaming` is set: data that is touched once
// and is larger than the caches should not push the operand panels out of them; data that the next kernel
// of the same call reads again and that fits should stay.
template <class V> __device__ __forceinline__ V load_hinted(const V* p, int streaming) {
    return streaming ? __builtin_nontemporal_load(p) : *p;
}
template <class V> __device__ __forceinline__ void store_hinted(V v, V* p, int streaming) {
    if (streaming) __builtin_nontemporal_store(v, p); else *p = v;
}

__device__ __forceinline__ float bf16lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
// Taking the argument by value matters: __builtin_bit_cast applied directly to a vector
// element expression reads element 0 whatever the index is.
__device__ __forceinline__ f16x2 as_f16x2(uint32_t w) { return __builtin_bit_cast(f16x2, w); }
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
    f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
}

// Signed sum of NT 16-byte chunks.  The sum is formed in fp32 and rounded once to the
// operand type (fixed_strassen_fp32_agg.py:38-44); a two-term fp16 sum uses the packed
// fp16 adder, which rounds the same exact sum.
template <class T, int NT, unsigned NEG>
__device__ __forceinline__ u32x4 combine(const u32x4 (&v)[NT]) {
    if constexpr (NT == 1) {
        static_assert(NEG == 0, "a single term is never negated");
        return v[0];
    } else if constexpr (sizeof(T) == 4) {
        f32x4 s = __builtin_bit_cast(f32x4, v[0]);
        if (NEG & 1u) s = -s;
#pragma unroll
        for (int t = 1; t < NT; ++t) {
            f32x4 x = __builtin_bit_cast(f32x4, v[t]);
            s = ((NEG >> t) & 1u) ? s - x : s + x;
        }
        return __builtin_bit_cast(u32x4, s);
    } else if constexpr (__is_same(T, f16_t) && NT == 2 && (NEG & 1u) == 0) {
        u32x4 r;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const f16x2 a = as_f16x2(v[0][w]), b = as_f16x2(v[1][w]);
            f16x2 c;
            if constexpr ((NEG & 2u) != 0) c = a - b; else c = a + b;
            r[w] = __builtin_bit_cast(uint32_t, c);
        }
        return r;
    } else {
        u32x4 r;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            float lo = 0.f, hi = 0.f;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                float xl, xh;
                if constexpr (__is_same(T, bf16_t)) {
                    xl = bf16lo(v[t][w]);
                    xh = bf16hi(v[t][w]);
                } else {
                    const f16x2 h = as_f16x2(v[t][w]);
                    xl = (float)h[0];
                    xh = (float)h[1];
                }
                if (t == 0) {
                    lo = ((NEG >> t) & 1u) ? -xl : xl;
                    hi = ((NEG >> t) & 1u) ? -xh : xh;
                } else if ((NEG >> t) & 1u) {
                    lo -= xl; hi -= xh;
                } else {
                    lo += xl; hi += xh;
                }
            }
            if constexpr (__is_same(T, bf16_t)) r[w] = pack_bf16(lo, hi);
            else r[w] = pack_f16(lo, hi);
        }
        return r;
    }
}

// ------------------------------------------------------------------------- operand loader
// One of these per operand per product.  Thread (row r, chunk c) of the tile owns PASSES
// chunks, RPP rows apart.  For KC operands rows are m/n and chunks run along k; for the
// other layout rows are k and chunks run along m/n.
template <class T, bool KC, bool EDGE, int NT, unsigned NEG>
struct OperandLoader {
    using G = TileGeom<T, KC>;
    const T* ptr[NT];
    int64_t pass_stride;   // elements between this thread's passes
    int64_t step_stride;   // elements per k step
    int lds_off;           // byte offset of this thread's pass-0 chunk inside the tile
    // EDGE only: how many valid m/n and k positions remain counted from this thread's first element
    int mn_rem[NT];
    int k_rem[NT];
    bool vec;

    // base: operand base for this batch; (rs, cs): strides of the (m|n) index and of k
    // blk_mn[t], blk_k[t]: first m/n and k index of term t's block; lim_mn, lim_k: logical sizes
    // tile_mn: first m/n index of the tile inside the block; ext_mn/ext_k: block extents
    __device__ __forceinline__ void init(const T* base, int64_t s_mn, int64_t s_k,
                                         const int (&blk_mn)[NT], const int (&blk_k)[NT],
                                         int lim_mn, int lim_k, int ext_mn, int ext_k,
                                         int tile_mn, bool vec_ok) {
        const int tid = threadIdx.x;
        const int c = tid % G::CPR, r = tid / G::CPR;
        lds_off = r * G::ROWB + c * 16;
        const int my_mn = KC ? r : c * G::EPC;
        const int my_k = KC ? c * G::EPC : r;
        pass_stride = (int64_t)G::RPP * (KC ? s_mn : s_k);
        step_stride = (int64_t)G::BK * s_k;
        vec = vec_ok;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            ptr[t] = base + (int64_t)(blk_mn[t] + tile_mn + my_mn) * s_mn + (int64_t)(blk_k[t] + my_k) * s_k;
            if constexpr (EDGE) {
                int vmn = min(ext_mn, lim_mn - blk_mn[t]);   // valid extent of this block
                int vk = min(ext_k, lim_k - blk_k[t]);
                mn_rem[t] = vmn - tile_mn - my_mn;
                k_rem[t] = vk - my_k;
            }
        }
    }

    __device__ __forceinline__ void advance() {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            ptr[t] += step_stride;
            if constexpr (EDGE) k_rem[t] -= G::BK;
        }
    }

    __device__ __forceinline__ u32x4 load_one(int t, int p) const {
        const T* q = ptr[t] + p * pass_stride;
        if constexpr (!EDGE) {
            return *reinterpret_cast<const u32x4*>(q);
        } else {
            // rows advance by RPP per pass; the chunk runs along the other index
            const int row_rem = (KC ? mn_rem[t] : k_rem[t]) - p * G::RPP;
            const int col_rem = KC ? k_rem[t] : mn_rem[t];
            u32x4 z = {0u, 0u, 0u, 0u};
            if (row_rem <= 0 || col_rem <= 0) return z;
            if (vec && col_rem >= G::EPC) return *reinterpret_cast<const u32x4*>(q);
            if constexpr (sizeof(T) == 4) {
                const uint32_t* s = reinterpret_cast<const uint32_t*>(q);
#pragma unroll
                for (int e = 0; e < 4; ++e) if (e < col_rem) z[e] = s[e];
            } else {
                const uint16_t* s = reinterpret_cast<const uint16_t*>(q);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (e < col_rem) z[e >> 1] |= (uint32_t)s[e] << ((e & 1) * 16);
            }
            return z;
        }
    }

    __device__ __forceinline__ void load(u32x4 (&out)[4]) const {
        u32x4 v[4][NT];
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
            for (int t = 0; t < NT; ++t) v[p][t] = load_one(t, p);
#pragma unroll
        for (int p = 0; p < 4; ++p) out[p] = combine<T, NT, NEG>(v[p]);
    }

    __device__ __forceinline__ void store(char* tile, const u32x4 (&r)[4]) const {
#pragma unroll
        for (int p = 0; p < 4; ++p)
            *reinterpret_cast<u32x4*>(tile + lds_off + p * G::RPP * G::ROWB) = r[p];
    }
};

// ---------------------------------------------------------------------- fragment reads
// Returns, for MFMA 32x32 sub-tile starting at row `sub` of the tile and k-group kg
// (16 k for 16-bit types, 8 k for fp32), the 16 bytes this lane feeds to the matrix core:
// lane l holds row sub + l%32 and k = kg*KG + (l/32)*KG/2 + [0, KG/2).
template <class T, bool KC>
__device__ __forceinline__ u32x4 read_frag(const char* tile, int sub, int kg) {
    using G = TileGeom<T, KC>;
    const int lane = threadIdx.x & 63;
    if constexpr (KC) {
        return *reinterpret_cast<const u32x4*>(tile + (sub + (lane & 31)) * G::ROWB + (kg * 2 + (lane >> 5)) * 16);
    } else if constexpr (sizeof(T) == 4) {
        const int k0 = kg * 8 + (lane >> 5) * 4;
        const char* p = tile + k0 * G::ROWB + (sub + (lane & 31)) * 4;
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = *reinterpret_cast<const uint32_t*>(p + j * G::ROWB);
        return r;
    } else {
        // Transposing LDS read: within each group of 16 lanes, lane (a, b) = (l16/4, l16%4)
        // points at row a, columns 4b..4b+3 of a 4 x 16 block; lane i receives column i, rows 0..3.
        const int l16 = lane & 15, grp = lane >> 4;
        const int k0 = kg * 16 + (grp >> 1) * 8 + (l16 >> 2);
        const int col = sub + (grp & 1) * 16 + (l16 & 3) * 4;
        const char* p = tile + k0 * G::ROWB + col * 2;
        s16x4 lo = lds_read_tr16_b64(p);
        s16x4 hi = lds_read_tr16_b64(p + 4 * G::ROWB);
        u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
        u32x4 r = {a[0], a[1], b[0], b[1]};
        return r;
    }
}

// acc(32 n-rows x 32 m-cols) += Bfrag^T-as-rows * Afrag.  The operands are swapped on purpose:
// the accumulator then holds, per lane, runs of four consecutive n for one m, which the
// epilogue stores as one 8- or 16-byte access.
template <class T>
__device__ __forceinline__ void mfma_step(f32x16& acc, const u32x4& a, const u32x4& b) {
    if constexpr (__is_same(T, bf16_t)) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b), __builtin_bit_cast(bf16x8, a), acc, 0, 0, 0);
    } else if constexpr (__is_same(T, f16_t)) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, b), __builtin_bit_cast(f16x8, a), acc, 0, 0, 0);
    } else {
        f32x4 fa = __builtin_bit_cast(f32x4, a), fb = __builtin_bit_cast(f32x4, b);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j], fa[j], acc, 0, 0, 0);
    }
}

struct Acc {   // one 64 x 64 wave tile = 2 x 2 MFMA tiles
    f32x16 t[2][2];
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) t[i][j][e] = 0.f;
    }
    __device__ __forceinline__ void add(const Acc& o) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) t[i][j] += o.t[i][j];
    }
    __device__ __forceinline__ void sub(const Acc& o) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) t[i][j] -= o.t[i][j];
    }
    __device__ __forceinline__ void negate() {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) t[i][j] = -t[i][j];
    }
};

// Block context shared by the products of one tile.
template <class T, bool A_KC, bool B_KC>
struct Ctx {
    using GA = TileGeom<T, A_KC>;
    using GB = TileGeom<T, B_KC>;
    static constexpr int SMEM_BYTES = 2 * (GA::BYTES + GB::BYTES);
    const GemmParams* p;
    const T* A; const T* B; char* C;   // batch-offset bases
    char* smem;
    int tile_m, tile_n;                // first row / column of this tile inside a block
    int kt;                            // k steps per product
};

// One product: acc += (sum of A blocks) x (sum of B blocks) over the block's k extent.
// QA / QB list the quadrant ids (0=11, 1=12, 2=21, 3=22) of the terms; NEGA / NEGB their signs.
template <class T, bool A_KC, bool B_KC, bool EDGE, int NTA, unsigned NEGA, int NTB, unsigned NEGB>
__device__ __forceinline__ void product(Acc& acc, const Ctx<T, A_KC, B_KC>& cx,
                                        const int (&qa)[NTA], const int (&qb)[NTB]) {
    using C = Ctx<T, A_KC, B_KC>;
    using GA = typename C::GA;
    using GB = typename C::GB;
    const GemmParams& P = *cx.p;
    OperandLoader<T, A_KC, EDGE, NTA, NEGA> la;
    OperandLoader<T, B_KC, EDGE, NTB, NEGB> lb;
    {
        int bm[NTA], bk[NTA];
#pragma unroll
        for (int t = 0; t < NTA; ++t) { bm[t] = (qa[t] >> 1) * P.Mh; bk[t] = (qa[t] & 1) * P.Kh; }
        la.init(cx.A, P.a_rs, P.a_cs, bm, bk, P.M, P.K, P.Mh, P.Kh, cx.tile_m, P.a_vec != 0);
        int bn[NTB], bk2[NTB];
#pragma unroll
        for (int t = 0; t < NTB; ++t) { bk2[t] = (qb[t] >> 1) * P.Kh; bn[t] = (qb[t] & 1) * P.Nh; }
        lb.init(cx.B, P.b_cs, P.b_rs, bn, bk2, P.N, P.K, P.Nh, P.Kh, cx.tile_n, P.b_vec != 0);
    }
    char* sA[2] = {cx.smem, cx.smem + GA::BYTES + GB::BYTES};
    char* sB[2] = {cx.smem + GA::BYTES, cx.smem + 2 * GA::BYTES + GB::BYTES};
    const int wave = threadIdx.x >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    u32x4 ra[4], rb[4];
    la.load(ra);
    lb.load(rb);
    la.store(sA[0], ra);
    lb.store(sB[0], rb);
    __syncthreads();
    for (int kt = 0; kt < cx.kt; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < cx.kt;
        if (more) {
            la.advance();
            lb.advance();
            la.load(ra);
            lb.load(rb);
        }
#pragma unroll
        for (int kg = 0; kg < 4; ++kg) {
            u32x4 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[i] = read_frag<T, A_KC>(sA[cur], wm + i * 32, kg);
#pragma unroll
            for (int j = 0; j < 2; ++j) fb[j] = read_frag<T, B_KC>(sB[cur], wn + j * 32, kg);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) mfma_step<T>(acc.t[i][j], fa[i], fb[j]);
        }
        if (more) {
            la.store(sA[cur ^ 1], ra);
            lb.store(sB[cur ^ 1], rb);
        }
        __syncthreads();
    }
}

// Store (or accumulate into) the C block `quad` at this tile.  Lane l of sub-tile (i, j)
// holds m = l%32 and, in registers 4g..4g+3, n = 8g + 4*(l/32) + 0..3.
template <class T, bool EDGE>
__device__ __forceinline__ void store_tile(const Acc& acc, const GemmParams& P, char* Cb, int quad,
                                           int tile_m, int tile_n) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int row0 = (quad >> 1) * P.Mh, col0 = (quad & 1) * P.Nh;
    const int esz = P.out_f32 ? 4 : (int)sizeof(T);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int mloc = tile_m + wm + i * 32 + (lane & 31);
        const int m = row0 + mloc;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int nloc = tile_n + wn + j * 32 + 8 * g + 4 * (lane >> 5);
                const int n = col0 + nloc;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc.t[i][j][4 * g + e];
                char* dst = Cb + ((int64_t)m * P.c_rs + (int64_t)n * P.c_cs) * esz;
                if constexpr (!EDGE) {
                    if (P.out_f32) {
                        f32x4* d = reinterpret_cast<f32x4*>(dst);
                        f32x4 o = {v[0], v[1], v[2], v[3]};
                        if (P.accumulate) o += *d;
                        *d = o;
                    } else {
                        u32x2* d = reinterpret_cast<u32x2*>(dst);
                        if (P.accumulate) {
                            u32x2 old = *d;
                            if constexpr (__is_same(T, bf16_t)) {
                                v[0] += bf16lo(old[0]); v[1] += bf16hi(old[0]);
                                v[2] += bf16lo(old[1]); v[3] += bf16hi(old[1]);
                            } else if constexpr (__is_same(T, f16_t)) {
                                const f16x2 h0 = as_f16x2(old[0]), h1 = as_f16x2(old[1]);
                                v[0] += (float)h0[0]; v[1] += (float)h0[1];
                                v[2] += (float)h1[0]; v[3] += (float)h1[1];
                            }
                        }
                        u32x2 o;
                        if constexpr (__is_same(T, bf16_t)) { o[0] = pack_bf16(v[0], v[1]); o[1] = pack_bf16(v[2], v[3]); }
                        else if constexpr (__is_same(T, f16_t)) { o[0] = pack_f16(v[0], v[1]); o[1] = pack_f16(v[2], v[3]); }
                        else { o[0] = 0; o[1] = 0; }
                        *d = o;
                    }
                } else {
                    if (mloc >= P.Mh || m >= P.M) continue;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (nloc + e >= P.Nh || n + e >= P.N) continue;
                        char* de = dst + (int64_t)e * P.c_cs * esz;
                        float x = v[e];
                        if (P.out_f32) {
                            float* d = reinterpret_cast<float*>(de);
                            if (P.accumulate) x += *d;
                            *d = x;
                        } else if constexpr (__is_same(T, bf16_t)) {
                            uint16_t* d = reinterpret_cast<uint16_t*>(de);
                            if (P.accumulate) x += bf16lo(*d);
                            *d = (uint16_t)pack_bf16(x, 0.f);
                        } else if constexpr (__is_same(T, f16_t)) {
                            uint16_t* d = reinterpret_cast<uint16_t*>(de);
                            if (P.accumulate) x += (float)__builtin_bit_cast(_Float16, *d);
                            *d = (uint16_t)pack_f16(x, 0.f);
                        }
                    }
                }
            }
        }
    }
}

// fp32 operands always write fp32: route them through the out_f32 branch.
template <class T, bool EDGE>
__device__ __forceinline__ void emit(const Acc& acc, const GemmParams& P, char* Cb, int quad, int tm, int tn) {
    store_tile<T, EDGE>(acc, P, Cb, quad, tm, tn);
}

// Tile id -> (tile_m, tile_n).  Workgroups are dealt round-robin to the 8 XCDs, each with
// its own L2; renumber so that one XCD works on a contiguous run of tiles, then walk the
// tile grid in groups of group_m tile-rows so that the run reuses A row-panels and B
// column-panels out of that L2.
__device__ __forceinline__ void tile_coords_in(const GemmParams& P, int bid, int nb, int& tm, int& tn) {
    const int per = nb / 8, rem = nb % 8;
    const int xcd = bid % 8, idx = bid / 8;
    const int logical = idx + (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per);
    const int width = P.group_m * P.tiles_n;
    const int grp = logical / width, in = logical % width;
    const int first = grp * P.group_m;
    const int gsz = min(P.tiles_m - first, P.group_m);
    tm = first + in % gsz;
    tn = in / gsz;
}
__device__ __forceinline__ void tile_coords(const GemmParams& P, int& tm, int& tn) {
    tile_coords_in(P, (int)blockIdx.x, (int)gridDim.x, tm, tn);
}

template <class T, int ALGO, bool A_KC, bool B_KC, bool EDGE>
__global__ void __launch_bounds__(kThreads) gemm_kernel(const GemmParams P) {
    using C = Ctx<T, A_KC, B_KC>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    C cx;
    cx.p = &P;
    const int batch = blockIdx.y;
    cx.A = reinterpret_cast<const T*>(P.A) + (int64_t)batch * P.a_bs;
    cx.B = reinterpret_cast<const T*>(P.B) + (int64_t)batch * P.b_bs;
    cx.C = reinterpret_cast<char*>(P.C) + (int64_t)batch * P.c_bs * (P.out_f32 ? 4 : (int)sizeof(T));
    cx.smem = smem;
    int tm, tn;
    tile_coords(P, tm, tn);
    cx.tile_m = tm * kBM;
    cx.tile_n = tn * kBN;
    cx.kt = (P.Kh + C::GA::BK - 1) / C::GA::BK;
    if constexpr (EDGE) {
        // tiles that lie entirely in the zero padding have nothing to store
        if (cx.tile_m >= P.M || cx.tile_n >= P.N) return;
    }

#define PRODUCT(acc, NTA, NEGA, NTB, NEGB, ...) product<T, A_KC, B_KC, EDGE, NTA, NEGA, NTB, NEGB>(acc, cx, __VA_ARGS__)
#define EMIT(acc, quad) emit<T, EDGE>(acc, P, cx.C, quad, cx.tile_m, cx.tile_n)
    enum { Q11 = 0, Q12 = 1, Q21 = 2, Q22 = 3 };

    if constexpr (ALGO == ALGO_CLASSIC) {
        Acc x;
        x.zero();
        PRODUCT(x, 1, 0u, 1, 0u, {Q11}, {Q11});
        EMIT(x, Q11);
    } else if constexpr (ALGO == ALGO_STRASSEN) {
        Acc x, y, z;
        // M3 = A11 (B12 - B22): starts the C12 chain (x) and the C22 chain (y)
        x.zero();
        PRODUCT(x, 1, 0u, 2, 2u, {Q11}, {Q12, Q22});
        y = x;
        // M6 = (A21 - A11)(B11 + B12): only C22 needs it -> accumulate in place
        PRODUCT(y, 2, 2u, 2, 0u, {Q21, Q11}, {Q11, Q12});
        // M5 = (A11 + A12) B22: C12 = M3 + M5 is complete; C11 chain starts at -M5
        z.zero();
        PRODUCT(z, 2, 0u, 1, 0u, {Q11, Q12}, {Q22});
        x.add(z);
        EMIT(x, Q12);
        z.negate();
        // M7 = (A12 - A22)(B21 + B22): only C11 needs it
        PRODUCT(z, 2, 2u, 2, 0u, {Q12, Q22}, {Q21, Q22});
        // M1 = (A11 + A22)(B11 + B22): into C11 and C22
        x.zero();
        PRODUCT(x, 2, 0u, 2, 0u, {Q11, Q22}, {Q11, Q22});
        y.add(x);
        z.add(x);
        // M2 = (A21 + A22) B11: C22 = M1 - M2 + M3 + M6 is complete; C21 chain starts at M2
        x.zero();
        PRODUCT(x, 2, 0u, 1, 0u, {Q21, Q22}, {Q11});
        y.sub(x);
        EMIT(y, Q22);
        // M4 = A22 (B21 - B11): completes C11 and C21
        y.zero();
        PRODUCT(y, 1, 0u, 2, 2u, {Q22}, {Q21, Q11});
        z.add(y);
        EMIT(z, Q11);
        x.add(y);
        EMIT(x, Q21);
    } else {
        // Strassen-Winograd.  S1=A21+A22 S2=S1-A11 S3=A11-A21 S4=A12-S2, T1=B12-B11 T2=B22-T1
        // T3=B22-B12 T4=T2-B21; every S/T is expanded over raw quadrants so it can be formed
        // at load time.  U-chain: C11=P1+P2, U2=P1+P6, U3=U2+P7, U4=U2+P5, C12=U4+P3,
        // C21=U3-P4, C22=U3+P5.  Only P5 needs an accumulator of its own.
        Acc x, y, z;
        x.zero();
        PRODUCT(x, 1, 0u, 1, 0u, {Q11}, {Q11});                      // P1 = A11 B11
        y = x;
        PRODUCT(x, 1, 0u, 1, 0u, {Q12}, {Q21});                      // + P2 = A12 B21 -> C11
        EMIT(x, Q11);
        // + P6 = S2 T2 = (A21 + A22 - A11)(B22 - B12 + B11) -> U2
        PRODUCT(y, 3, 4u, 3, 2u, {Q21, Q22, Q11}, {Q22, Q12, Q11});
        z = y;
        // + P7 = S3 T3 = (A11 - A21)(B22 - B12) -> U3
        PRODUCT(y, 2, 2u, 2, 2u, {Q11, Q21}, {Q22, Q12});
        // P5 = S1 T1 = (A21 + A22)(B12 - B11)
        x.zero();
        PRODUCT(x, 2, 0u, 2, 2u, {Q21, Q22}, {Q12, Q11});
        z.add(x);                                                    // U4 = U2 + P5
        x.add(y);                                                    // C22 = U3 + P5
        EMIT(x, Q22);
        // + P3 = S4 B22 = (A12 - A21 - A22 + A11) B22 -> C12
        PRODUCT(z, 4, 6u, 1, 0u, {Q12, Q21, Q22, Q11}, {Q22});
        EMIT(z, Q12);
        // - P4 = A22 T4, T4 = B22 - B12 + B11 - B21: accumulate A22 (-T4) in place -> C21
        PRODUCT(y, 1, 0u, 4, 5u, {Q22}, {Q22, Q12, Q11, Q21});
        EMIT(y, Q21);
    }
#undef PRODUCT
#undef EMIT
}

}  // namespace sthip
