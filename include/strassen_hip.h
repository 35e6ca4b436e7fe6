/* strassen_hip.h -- C ABI of libstrassen_hip.so (gfx950 / MI355X).
 *
 * Every entry point takes plain device pointers, sizes and element strides; nothing here
 * knows about torch.  All work is enqueued on the HIP stream passed in (NULL = the default
 * stream) and nothing synchronises.  The library never allocates or frees device memory:
 * the multi-level paths take a caller-provided workspace (sthip_workspace_bytes).
 * Test and profiling hooks live in strassen_hip_debug.h, not here.
 *
 * Return value: 0 on success, a negative sthip_status otherwise; sthip_last_error() then
 * describes the failure (thread local).
 *
 * The reference (vmad18/strassen-triton) is pure Python and has no FFI of its own; each
 * entry point below names the Python function whose arithmetic it replaces
 * (paths relative to the reference checkout).
 */
#ifndef STRASSEN_HIP_H
#define STRASSEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define STHIP_VERSION 100

enum sthip_status {
    STHIP_OK = 0,
    STHIP_ERR_SHAPE = -1,     /* negative size, mismatched inner dimension, not square where required */
    STHIP_ERR_DTYPE = -2,     /* unknown dtype / unsupported in-out combination */
    STHIP_ERR_LAYOUT = -3,    /* an operand has no unit stride, or C is not writable as given */
    STHIP_ERR_WORKSPACE = -4, /* workspace missing or too small */
    STHIP_ERR_ARG = -5,       /* null pointer, bad algo / levels */
    STHIP_ERR_HIP = -6        /* a HIP runtime call failed */
};

enum sthip_dtype { STHIP_F32 = 0, STHIP_F16 = 1, STHIP_BF16 = 2 };

enum sthip_algo {
    STHIP_CLASSIC = 0,  /* plain tiled MFMA GEMM (levels is ignored) */
    STHIP_STRASSEN = 1, /* 7 products, 18 add/sub */
    STHIP_WINOGRAD = 2  /* 7 products, 15 add/sub (leaf level only; upper levels use Strassen) */
};

/* Optional, OR-ed into an `algo` argument: where a 16-bit problem of two or more levels rounds
 * below its first level.  The reference's fp32-aggregating recursion rounds the first level's
 * operand sums to base_dtype and recurses with base_dtype back at its default, fp32
 * (fixed_strassen_fp32_agg.py:87-113), so everything deeper is fp32 arithmetic.
 *   STHIP_SCHEDULE_REFERENCE  exactly that: first-level sums rounded to the operand type, then
 *       widened; the seven half-size products run on the fp32 paths with levels - 1 levels
 *       (fp32 matrix cores: 16 x slower than 16-bit ones).  Differs from the reference by fp32
 *       summation order only.
 *   STHIP_SCHEDULE_FAST       sums and products of every level rounded to the operand type, every
 *       product on the 16-bit matrix cores.  Relative Frobenius distance from the reference in
 *       bf16: 1.2e-2 at two levels, 2.3e-2 at three (fp16, with three more bits: below 5e-3).
 * Neither flag: fast at two levels (the 49 products as one 16-bit launch), reference from three
 * levels on, so that every default stays within 2e-2 of the reference.  fp32 problems and
 * one-level calls ignore the flags.  Pass the same algo value to sthip_workspace_bytes. */
enum sthip_schedule { STHIP_SCHEDULE_REFERENCE = 1 << 4, STHIP_SCHEDULE_FAST = 2 << 4 };

/* General entry: C[b] (+)= A[b] x B[b] for b < batch, A is M x K, B is K x N, C is M x N.
 * stride*[3] = {batch, row, col} in elements; A and B need one unit stride among (row, col)
 * each (so NN / NT / TN / TT all work without copies; the other stride must stay below 2^26
 * elements, or the call fails with STHIP_ERR_HIP).  in_dtype is the element type of A
 * and B; out_dtype is that of C and must equal in_dtype or be STHIP_F32.  Products
 * accumulate in fp32, operand sums are formed in fp32 and rounded once to in_dtype, the
 * recombination is done in fp32.  Sizes that are not multiples of 2^levels behave as if
 * zero padded.
 *
 * levels = 1 needs no workspace: one fused launch forms the quadrant sums in registers on
 * the way from global memory to LDS.  Given sthip_workspace_bytes() of workspace, 16-bit
 * problems whose half-size blocks are multiples of the tile (128 x 128 x 64) take the faster
 * pipelined path instead: the quadrant sums are written once, then one grouped-GEMM launch
 * runs the seven products.  Large problems (half-size blocks multiples of 256, result in the
 * operand type) use 256 x 256 tiles, round each product once to the operand type as the
 * reference's mm does, and recombine in a third pass in fp32; with an fp32 result the seven
 * products are kept in fp32 instead (never rounded, as in the reference's Triton kernels; the
 * workspace query then asks for twice the product room); the others recombine in registers.  fp32 problems with tile-aligned half-size blocks (128 x 128
 * x 32) and workspace write their sums once and run the seven products as one launch (grouped on
 * 256 x 256 tiles when A is contiguous along k and the blocks are multiples of 256 and large
 * enough to fill the chip, else batched over dense operand copies); nothing is rounded.  Plain
 * products (STHIP_CLASSIC) of all three types take the 256 x 256 kernel under the same conditions.
 * levels = 2 on tile-aligned 16-bit problems runs as three launches (the sums of both levels,
 * ONE grouped GEMM of the 49 quarter-size products, both recombinations; every level returns
 * its products in the operand type, the first level is always Strassen); large fp32 Strassen
 * problems run as five (sums, sums, the 49 products, two recombinations) with nothing rounded.  Otherwise levels >= 2 recurses on the host
 * (sums and products of the upper levels in workspace) and requires the workspace.
 *
 * Replaces: _strassen_base (fixed_strassen.py:11-57, fixed_strassen_fp32_agg.py:12-56),
 * strassen_matmul_n_layers (fixed_strassen.py:59-126, fixed_strassen_fp32_agg.py:58-125),
 * strassen_matmul_two_layers (strassen.py:742-812) and, with accumulate = 1, the Triton
 * launchers run_strassen (strassen.py:195-213), run_strassen2 (:674-693),
 * run_matmul_fp32_accum (:66-88), run_strassen_2_layer_fp32_accum (strassen_2_layer.py:7-15). */
int sthip_gemm(const void* A, const void* B, void* C,
               int64_t batch, int64_t M, int64_t N, int64_t K,
               const int64_t strideA[3], const int64_t strideB[3], const int64_t strideC[3],
               int in_dtype, int out_dtype, int algo, int levels, int accumulate,
               void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of device workspace sthip_gemm can use for this problem: optional for levels = 1 (0 if
 * the pipelined path does not apply), required for levels >= 2.  Must be 256-byte aligned. */
size_t sthip_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K,
                             int in_dtype, int out_dtype, int algo, int levels);

/* sthip_gemm for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same arguments without the
 * workspace, which is replaced by a buffer of STHIP_STATIC_SCRATCH_BYTES that is part of the
 * library's device image (every GPU the library runs on holds its own copy until the process
 * ends).  The call itself allocates and frees nothing.  Same kernels and same bits as
 * sthip_gemm given sthip_workspace_bytes() of workspace.  A problem whose workspace query
 * exceeds the buffer is refused with STHIP_ERR_WORKSPACE before anything is launched (the
 * buffer covers, for example, one level at 4096^3 and two levels at 2048^3 with 16-bit
 * operands).  The first call on a device looks up the buffer's address on that device; make
 * it outside graph capture.  All calls on one GPU share that GPU's buffer: calls that overlap
 * on one GPU (two streams, two host threads) race on it; calls ordered on one stream do not.
 * Nothing in the buffer has to start at zero: every path writes what it later reads.
 * No counterpart in the reference (its torch ops allocate freely). */
#define STHIP_STATIC_SCRATCH_BYTES ((size_t)144 << 20)
int sthip_gemm_static(const void* A, const void* B, void* C,
                      int64_t batch, int64_t M, int64_t N, int64_t K,
                      const int64_t strideA[3], const int64_t strideB[3], const int64_t strideC[3],
                      int in_dtype, int out_dtype, int algo, int levels, int accumulate,
                      void* stream);

/* C = A x B for square n x n operands, `levels` Strassen levels; B may be a transposed view
 * (strides in elements).  Replaces strassen_matmul_n_layers(A, B, n_depth, base_dtype)
 * (fixed_strassen.py:59-126, fixed_strassen_fp32_agg.py:58-125) and, for levels = 1,
 * _strassen_base (fixed_strassen.py:11-57).  C is contiguous row-major in `dtype`. */
int sthip_strassen_matmul_n_layers(const void* A, const void* B, void* C, int64_t n,
                                   int64_t a_row_stride, int64_t a_col_stride,
                                   int64_t b_row_stride, int64_t b_col_stride,
                                   int dtype, int levels,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* C += A x B, the contract of the reference's Triton launchers: run_strassen
 * (strassen.py:195-213; levels = 1), run_strassen2 (strassen.py:674-693; levels = 2),
 * run_strassen_2_layer_fp32_accum (strassen_2_layer.py:7-15; levels = 2) and
 * run_matmul_fp32_accum (strassen.py:66-88; algo = STHIP_CLASSIC).  Operands are in
 * op_dtype (the reference casts tiles to fp16, strassen.py:150-163), C is in c_dtype.
 * batch = 1 for 2-D inputs.  All tensors contiguous row-major. */
int sthip_run_accumulate(const void* A, const void* B, void* C,
                         int64_t batch, int64_t M, int64_t N, int64_t K,
                         int op_dtype, int c_dtype, int algo, int levels,
                         void* workspace, size_t workspace_bytes, void* stream);

/* y[rows x D] = x[rows x D] x W^T (+ bias), W is D x D row-major, rows <= D.  The reference
 * pads x with zero rows up to D x D and slices afterwards (model/layers.py:246-274); here
 * the missing rows are simply never loaded or stored.  bias may be NULL; it is added to the
 * rounded product and the sum rounded again, as the reference's `+ bias` does -- inside the
 * recombination pass where the call runs as sums / grouped products / recombination, else by
 * a pass of its own.  Rounds at every level (see sthip_linear_forward); workspace as
 * sthip_workspace_bytes(1, D, D, D, dtype, dtype, STHIP_STRASSEN | STHIP_SCHEDULE_FAST, levels). */
int sthip_linear_strassen_forward(const void* x, const void* W, const void* bias, void* y,
                                  int64_t rows, int64_t D, int dtype, int levels,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* y[rows x out] = x[rows x in] x W^T (+ bias) for a Linear layer of any shape, W is out x in
 * row-major, all tensors contiguous; bias as in sthip_linear_strassen_forward.  The reference's
 * layer is square, a power of two and pads its input to D x D (model/layers.py:240, :255-262);
 * this is the same forward with those constraints lifted (no padding: sizes that are not tile
 * multiples take the kernels' edge tiles).  levels = 0 runs the classical product; levels < 0 runs
 * sthip_auto_levels(rows, out_features, in_features, dtype, -levels) levels, so that the layer never
 * takes a Strassen path that is slower than the library's classical kernel on that shape.
 * From three levels on (no counterpart: the reference's layers run one or two) every level rounds to the
 * operand type, as with STHIP_SCHEDULE_FAST; sthip_linear_strassen_forward does the same.
 * Workspace as sthip_workspace_bytes(1, rows, out, in, dtype, dtype, STHIP_STRASSEN | STHIP_SCHEDULE_FAST, levels). */
int sthip_linear_forward(const void* x, const void* W, const void* bias, void* y,
                         int64_t rows, int64_t in_features, int64_t out_features, int dtype, int levels,
                         void* workspace, size_t workspace_bytes, void* stream);

/* How many Strassen levels (0 = the classical product, at most max_levels) make C = A x B of this
 * shape fastest on MI355X, from measurements of this library's own kernels against each other
 * (sweep of M, N, K in 768 .. 16384, both layouts of B).  16-bit: one level where the classical
 * product cannot fill the chip but the seven half-size products side by side can (at most 128
 * output tiles of 128 x 128 and k >= 4096: weight gradients), and from 20480^3 up (at 16384^3 a level
 * and the classical kernel are within 2 % of each other); a second level from 32768^3; never a
 * third, which by default runs its inner products in fp32 (STHIP_SCHEDULE_REFERENCE).  fp32: one level from 5e11 flop (8192 x 8192 x 4096), two
 * from 1e12 (8192^3), three from 32768^3, and one level for products too small for the large-tile
 * kernel.  sthip_linear_forward applies this rule when its `levels` argument is negative.  No
 * counterpart in the reference, whose only cutoff is the min_size of replace_linear_with_strassen
 * (model/layers.py:279-300). */
int sthip_auto_levels(int64_t M, int64_t N, int64_t K, int dtype, int max_levels);

/* A Linear layer whose weight stays put between calls (inference, or the reference's benchmark
 * main_profiling.py:94-245, which times repeated forwards of one layer): the quadrant sums of
 * W^T -- the five first-level sums, for two levels the 35 second-level ones, and so on down -- depend on W
 * alone, so they can be formed once and kept in device memory; every forward then forms the
 * input-side sums only.  The reference's LinearStrassen (model/layers.py:246-274) re-forms them
 * on every call.  Results are bit-identical to sthip_linear_forward.
 *
 * sthip_linear_weight_sums_bytes: size of the buffer, or 0 where no sums can be kept (fp32,
 * levels outside 1..4, in_features / 2^levels not a multiple of 64 or out_features / 2^levels
 * not a multiple of 128).  1.25 x the bytes of W for one level, 3.4 x for two, 7.3 x for three, 14 x for four:
 * from three levels on every first-level product keeps the sums of its own weight-side operand.
 * sthip_linear_prepare_weight: forms the sums of W (out x in row-major, 16-byte aligned) into
 * `sums` (256-byte aligned).  Call again whenever W's contents change.
 * sthip_linear_forward_prepared: sthip_linear_forward reading those sums.  A call that does not
 * take the sums / grouped products / recombination form (too few rows, odd rows) ignores them. */
size_t sthip_linear_weight_sums_bytes(int64_t in_features, int64_t out_features, int dtype, int levels);
int sthip_linear_prepare_weight(const void* W, int64_t in_features, int64_t out_features, int dtype, int levels,
                                void* sums, size_t sums_bytes, void* stream);
int sthip_linear_forward_prepared(const void* x, const void* W, const void* sums, size_t sums_bytes,
                                  const void* bias, void* y,
                                  int64_t rows, int64_t in_features, int64_t out_features, int dtype, int levels,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* Description of the most recent failure on this thread ("" if none). */
const char* sthip_last_error(void);

/* STHIP_VERSION the library was built with. */
int sthip_version(void);

#ifdef __cplusplus
}
#endif
#endif /* STRASSEN_HIP_H */
