"""CPU oracle for the Strassen / Strassen-Winograd matmul path.

TEST INFRASTRUCTURE ONLY.  Nothing that ships (the package, its C-ABI library, its host
modules) may import this file; only tests/, __graft_entry__.smoke() and the cpu_baseline
leg of bench.py use it, and only as the checker / reported CPU baseline.

It restates, in eager torch on CPU tensors, the arithmetic of the reference's
matrix-level Strassen recursion.  Every function names the reference lines it follows
(paths relative to the reference checkout):

  strassen_base                fixed_strassen.py:11-57   (one level, all math in input dtype)
  strassen_base_fp32_agg       fixed_strassen_fp32_agg.py:12-56 (sums + recombination in fp32)
  strassen_matmul_n_layers     fixed_strassen.py:59-126 / fixed_strassen_fp32_agg.py:58-125
  strassen_matmul_two_layers   strassen.py:742-812 (+ its _strassen_base :697-740)
  strassen2_zorder_49          strassen.py:373-611 (the 49-product schedule, Z-order naming)
  tile_kernel_semantics        strassen.py:115-192 / :237-672 / strassen_2_layer.py:33-322
                               (C += A@B with fp16-cast operands and fp32 accumulation)
  linear_strassen_forward      model/layers.py:246-274
  winograd_base                textbook Strassen-Winograd (7 products, 15 add/sub); the
                               reference holds no correct Winograd variant
                               (strassen_deprecated_winograd.py:461-472 only gets C11 right),
                               so this one is pinned by the identity C = A @ B alone.

Pinning.  The reference ships no golden vectors or tests of its own, so the oracle is
pinned twice over:
  * formulas -- in exact arithmetic every function here equals A @ B, so tests/test_oracle.py
    runs them on small-integer matrices (every partial sum exactly representable) and
    demands bit-equality with an fp64 classical product; on tiny sizes against a triple
    loop; on identity, zero, one-hot and block-diagonal inputs; and through transposition /
    linearity invariants.  A dropped term, wrong sign, swapped quadrant or transposed
    operand fails at least one of those.
  * cast schedule (where the reference rounds to bf16 / fp16 / fp32) -- mathematics cannot
    fix that, so tests/golden/reference_cast_schedule.npz holds outputs of the reference's own
    fixed_strassen.py / fixed_strassen_fp32_agg.py functions (run eagerly on CPU by
    tests/golden/make_reference_vectors.py) and tests/test_golden_reference.py demands that
    strassen_base, strassen_base_fp32_agg and strassen_matmul_n_layers reproduce them bit
    for bit (fp32, bf16, fp16; depth 1-3; n = 32, 64, 128).
Not covered by reference vectors, because the reference has no counterpart: winograd_base and
strassen_general (rectangular / batched / odd sizes).  Their formulas are pinned by the
identity tests above; their cast schedule is this file's own choice (the fp32_agg schedule
applied to the new shapes) -- "parity unpinned" at the bit level, compared by tolerance
(rel. Frobenius <= 1e-5 fp32, <= 2e-2 bf16/fp16).
"""
from __future__ import annotations

import torch

AGG_DTYPE = torch.float32  # fixed_strassen_fp32_agg.py:10

# Below this size the reference falls back to a classical product
# (fixed_strassen.py:20-21, fixed_strassen_fp32_agg.py:19-20, strassen.py:703-704).
LEAF = 16


def mm_fp32_upcast(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """x @ y for 16-bit operands computed as an fp32 product of the upcast operands, rounded
    once to the operand dtype.  Same arithmetic contract as a half-precision GEMM with fp32
    accumulation, but it runs through sgemm: torch's CPU fp16 matmul is hundreds of times
    slower, which matters for the 4096 / 8192 test sizes.  Not bit-identical to torch.mm on
    16-bit tensors (summation order differs); use it for tolerance comparisons only."""
    if x.dtype == torch.float32 and y.dtype == torch.float32:
        return torch.matmul(x, y)
    return torch.matmul(x.float(), y.float()).to(x.dtype)


def _quadrants(X: torch.Tensor, mid_r: int, mid_c: int):
    return (X[..., :mid_r, :mid_c], X[..., :mid_r, mid_c:],
            X[..., mid_r:, :mid_c], X[..., mid_r:, mid_c:])


def _assemble(C11, C12, C21, C22):
    # fixed_strassen.py:54-57 (vstack of two hstacks)
    return torch.cat([torch.cat([C11, C12], dim=-1), torch.cat([C21, C22], dim=-1)], dim=-2)


def strassen_base(A: torch.Tensor, B: torch.Tensor, mm=torch.mm) -> torch.Tensor:
    """One Strassen level, every add and product in the dtype of the inputs.

    Follows fixed_strassen.py:11-57: n = A.shape[0]; n <= 16 -> plain product (:20-21);
    both matrices are cut at n // 2 in both dimensions (:23-36); products M1..M7 (:39-45);
    C11 = M1+M4-M5+M7, C12 = M3+M5, C21 = M2+M4, C22 = M1-M2+M3+M6 (:48-51).
    """
    if A.shape[0] <= LEAF:
        return mm(A, B)
    mid = A.shape[0] // 2
    A11, A12, A21, A22 = _quadrants(A, mid, mid)
    B11, B12, B21, B22 = _quadrants(B, mid, mid)
    M1 = mm(A11 + A22, B11 + B22)
    M2 = mm(A21 + A22, B11)
    M3 = mm(A11, B12 - B22)
    M4 = mm(A22, B21 - B11)
    M5 = mm(A11 + A12, B22)
    M6 = mm(A21 - A11, B11 + B12)
    M7 = mm(A12 - A22, B21 + B22)
    C11 = M1 + M4 - M5 + M7
    C12 = M3 + M5
    C21 = M2 + M4
    C22 = M1 - M2 + M3 + M6
    return _assemble(C11, C12, C21, C22)


def strassen_base_fp32_agg(A: torch.Tensor, B: torch.Tensor,
                           base_dtype: torch.dtype = torch.float32, mm=torch.mm) -> torch.Tensor:
    """One Strassen level with fp32 sums and fp32 recombination.

    Follows fixed_strassen_fp32_agg.py:12-56: quadrants upcast to fp32 (:26-35); each
    operand sum rounded once to base_dtype before the product, product result (in
    base_dtype) upcast again (:38-44); recombination in fp32, one final rounding (:47-50).
    """
    if A.shape[0] <= LEAF:
        return mm(A, B)
    mid = A.shape[0] // 2
    A11, A12, A21, A22 = (q.to(AGG_DTYPE) for q in _quadrants(A, mid, mid))
    B11, B12, B21, B22 = (q.to(AGG_DTYPE) for q in _quadrants(B, mid, mid))

    def prod(x, y):
        return mm(x.to(base_dtype), y.to(base_dtype)).to(AGG_DTYPE)

    M1 = prod(A11 + A22, B11 + B22)
    M2 = prod(A21 + A22, B11)
    M3 = prod(A11, B12 - B22)
    M4 = prod(A22, B21 - B11)
    M5 = prod(A11 + A12, B22)
    M6 = prod(A21 - A11, B11 + B12)
    M7 = prod(A12 - A22, B21 + B22)
    C11 = (M1 + M4 - M5 + M7).to(base_dtype)
    C12 = (M3 + M5).to(base_dtype)
    C21 = (M2 + M4).to(base_dtype)
    C22 = (M1 - M2 + M3 + M6).to(base_dtype)
    return _assemble(C11, C12, C21, C22)


def strassen_matmul_n_layers(A: torch.Tensor, B: torch.Tensor, n_depth: int = 2,
                             base_dtype: torch.dtype = torch.float32, *,
                             fp32_agg: bool = False,
                             inner_keeps_base_dtype: bool = False, mm=torch.mm) -> torch.Tensor:
    """n_depth-level recursion.

    fp32_agg=False follows fixed_strassen.py:59-126 (base_dtype ignored, math in the
    input dtype); fp32_agg=True follows fixed_strassen_fp32_agg.py:58-125.  Termination:
    depth 1 -> one level (:71-72); otherwise S1..S10 (:88-97), then the one-level routine
    when mid == 2 or n_depth == 2 (:99-106), else recursion with n_depth-1 (:107-114).

    In the fp32_agg file the inner calls do not forward base_dtype (:99-113), so below
    the first level the products run with the default base_dtype=float32 and come back as
    fp32.  inner_keeps_base_dtype=False reproduces that; True is the evident intent
    (every level's products in base_dtype).
    """
    if not fp32_agg:
        if n_depth == 1:
            return strassen_base(A, B, mm)
        mid = A.shape[0] // 2
        A11, A12, A21, A22 = _quadrants(A, mid, mid)
        B11, B12, B21, B22 = _quadrants(B, mid, mid)
        S1, S2, S3, S4, S5 = B12 - B22, A11 + A12, A21 + A22, B21 - B11, A11 + A22
        S6, S7, S8, S9, S10 = B11 + B22, A12 - A22, B21 + B22, A21 - A11, B11 + B12
        if mid == 2 or n_depth == 2:
            def f(x, y):
                return strassen_base(x, y, mm)
        else:
            def f(x, y):
                return strassen_matmul_n_layers(x, y, n_depth - 1, mm=mm)
        M1, M2, M3, M4 = f(S5, S6), f(S3, B11), f(A11, S1), f(A22, S4)
        M5, M6, M7 = f(S2, B22), f(S9, S10), f(S7, S8)
        return _assemble(M1 + M4 - M5 + M7, M3 + M5, M2 + M4, M1 - M2 + M3 + M6)

    if n_depth == 1:
        return strassen_base_fp32_agg(A, B, base_dtype, mm)
    mid = A.shape[0] // 2
    A11, A12, A21, A22 = (q.to(AGG_DTYPE) for q in _quadrants(A, mid, mid))
    B11, B12, B21, B22 = (q.to(AGG_DTYPE) for q in _quadrants(B, mid, mid))
    r = lambda t: t.to(base_dtype)
    S1, S2, S3, S4, S5 = r(B12 - B22), r(A11 + A12), r(A21 + A22), r(B21 - B11), r(A11 + A22)
    S6, S7, S8, S9, S10 = r(B11 + B22), r(A12 - A22), r(B21 + B22), r(A21 - A11), r(B11 + B12)
    inner_dtype = base_dtype if inner_keeps_base_dtype else torch.float32
    if mid == 2 or n_depth == 2:
        def f(x, y):
            return strassen_base_fp32_agg(x, y, inner_dtype, mm).to(AGG_DTYPE)
    else:
        def f(x, y):
            return strassen_matmul_n_layers(
                x, y, n_depth - 1, inner_dtype, fp32_agg=True,
                inner_keeps_base_dtype=inner_keeps_base_dtype, mm=mm).to(AGG_DTYPE)
    M1, M2, M3, M4 = f(S5, S6), f(S3, r(B11)), f(r(A11), S1), f(r(A22), S4)
    M5, M6, M7 = f(S2, r(B22)), f(S9, S10), f(S7, S8)
    return _assemble(r(M1 + M4 - M5 + M7), r(M3 + M5), r(M2 + M4), r(M1 - M2 + M3 + M6))


def strassen_matmul_two_layers(A: torch.Tensor, B: torch.Tensor, mm=torch.mm) -> torch.Tensor:
    """Fixed two-level recursion with the reference's validation (strassen.py:742-812).

    Raises ValueError with the reference's messages for non-square / n % 4 / n <= 0
    (:757-762).  Arithmetic in the input dtype (its _strassen_base, :697-740).
    """
    n = A.shape[0]
    if n != B.shape[0] or A.shape[1] != B.shape[0] or A.shape[0] != A.shape[1]:
        raise ValueError("Input matrices must be square and have the same dimensions.")
    if n % 4 != 0:
        raise ValueError("Matrix size must be divisible by 4 for two Strassen layers.")
    if not n > 0:
        raise ValueError("Matrix size must be positive.")
    return strassen_matmul_n_layers(A, B, n_depth=2, fp32_agg=False, mm=mm)


# ---------------------------------------------------------------------------------------
# 49-product two-level schedule (strassen.py:373-611), Z-order naming: X[q][s] is level-1
# quadrant q (0=11, 1=12, 2=21, 3=22), level-2 sub-quadrant s.  Each row is
# (A terms, B terms, destinations) with terms/destinations as (quadrant, sign).
# ---------------------------------------------------------------------------------------
STRASSEN_TABLE = (
    # M1 = (A11 + A22)(B11 + B22) -> +C11, +C22
    (((0, 1), (3, 1)), ((0, 1), (3, 1)), ((0, 1), (3, 1))),
    # M2 = (A21 + A22) B11        -> +C21, -C22
    (((2, 1), (3, 1)), ((0, 1),), ((2, 1), (3, -1))),
    # M3 = A11 (B12 - B22)        -> +C12, +C22
    (((0, 1),), ((1, 1), (3, -1)), ((1, 1), (3, 1))),
    # M4 = A22 (B21 - B11)        -> +C11, +C21
    (((3, 1),), ((2, 1), (0, -1)), ((0, 1), (2, 1))),
    # M5 = (A11 + A12) B22        -> -C11, +C12
    (((0, 1), (1, 1)), ((3, 1),), ((0, -1), (1, 1))),
    # M6 = (A21 - A11)(B11 + B12) -> +C22
    (((2, 1), (0, -1)), ((0, 1), (1, 1)), ((3, 1),)),
    # M7 = (A12 - A22)(B21 + B22) -> +C11
    (((1, 1), (3, -1)), ((2, 1), (3, 1)), ((0, 1),)),
)


def strassen2_zorder_49(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """A @ B through the 49-product schedule of strassen.py:377-611.

    Group g forms a = sum(sign * A[q]) and b = sum(sign * B[q]) over level-1 quadrants
    (each a 4-vector of sub-quadrants), runs the inner seven products on the sub-quadrants
    and adds the inner result r[0..3] into C[q'][0..3] for each destination q'.  Sizes
    must be divisible by 4.  Computed in the dtype of the inputs (use fp64 to check the
    algebra, which is what this function exists for).
    """
    M, K = A.shape[-2:]
    N = B.shape[-1]
    assert M % 4 == 0 and N % 4 == 0 and K % 4 == 0
    Aq = [_quadrants(q, M // 4, K // 4) for q in _quadrants(A, M // 2, K // 2)]
    Bq = [_quadrants(q, K // 4, N // 4) for q in _quadrants(B, K // 2, N // 2)]
    Cq = [[torch.zeros(A.shape[:-2] + (M // 4, N // 4), dtype=A.dtype) for _ in range(4)]
          for _ in range(4)]
    for a_terms, b_terms, dests in STRASSEN_TABLE:
        a = [sum(s * Aq[q][t] for q, s in a_terms) for t in range(4)]
        b = [sum(s * Bq[q][t] for q, s in b_terms) for t in range(4)]
        r = [torch.zeros_like(Cq[0][0]) for _ in range(4)]
        for ia, ib, idst in STRASSEN_TABLE:
            m = torch.matmul(sum(s * a[q] for q, s in ia), sum(s * b[q] for q, s in ib))
            for q, s in idst:
                r[q] = r[q] + s * m
        for q, s in dests:
            for t in range(4):
                Cq[q][t] = Cq[q][t] + s * r[t]
    return _assemble(*[_assemble(*Cq[q]) for q in range(4)])


def winograd_base(A: torch.Tensor, B: torch.Tensor, base_dtype: torch.dtype | None = None,
                  fp32_agg: bool = True, mm=torch.matmul) -> torch.Tensor:
    """One level of Strassen-Winograd (7 products, 15 additions), rectangular allowed
    (even dimensions), batched allowed.

    S1=A21+A22 S2=S1-A11 S3=A11-A21 S4=A12-S2   T1=B12-B11 T2=B22-T1 T3=B22-B12 T4=T2-B21
    P1=A11 B11 P2=A12 B21 P3=S4 B22 P4=A22 T4 P5=S1 T1 P6=S2 T2 P7=S3 T3
    U2=P1+P6 U3=U2+P7 U4=U2+P5;  C11=P1+P2 C12=U4+P3 C21=U3-P4 C22=U3+P5

    With fp32_agg the cast schedule mirrors fixed_strassen_fp32_agg.py:26-50 (fp32 sums,
    one rounding to base_dtype per operand, fp32 recombination, one final rounding);
    otherwise everything stays in the input dtype as in fixed_strassen.py:39-51.
    """
    base_dtype = base_dtype or A.dtype
    M, K = A.shape[-2:]
    N = B.shape[-1]
    up = (lambda t: t.to(AGG_DTYPE)) if fp32_agg else (lambda t: t)
    A11, A12, A21, A22 = (up(q) for q in _quadrants(A, M // 2, K // 2))
    B11, B12, B21, B22 = (up(q) for q in _quadrants(B, K // 2, N // 2))
    S1 = A21 + A22
    S2 = S1 - A11
    S3 = A11 - A21
    S4 = A12 - S2
    T1 = B12 - B11
    T2 = B22 - T1
    T3 = B22 - B12
    T4 = T2 - B21

    def prod(x, y):
        return up(mm(x.to(base_dtype), y.to(base_dtype)))

    P1, P2, P3, P4 = prod(A11, B11), prod(A12, B21), prod(S4, B22), prod(A22, T4)
    P5, P6, P7 = prod(S1, T1), prod(S2, T2), prod(S3, T3)
    U2 = P1 + P6
    U3 = U2 + P7
    U4 = U2 + P5
    out = _assemble(P1 + P2, U4 + P3, U3 - P4, U3 + P5)
    return out.to(base_dtype)


# ---------------------------------------------------------------------------------------
# Extensions the reference does not have (rectangular, batched, odd sizes): defined by
# zero-padding every dimension up to a multiple of 2**levels, running the square-style
# formulas on half/quarter blocks, and slicing the result back.
# ---------------------------------------------------------------------------------------
def _pad_to(X: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    pr, pc = rows - X.shape[-2], cols - X.shape[-1]
    if pr == 0 and pc == 0:
        return X
    return torch.nn.functional.pad(X, (0, pc, 0, pr))


def _strassen_rect_level(A, B, levels, base_dtype, fp32_agg, mm=torch.matmul):
    """One-or-more levels on (possibly batched) rectangular operands with even dims."""
    if levels == 0:
        return mm(A.to(base_dtype), B.to(base_dtype))
    M, K = A.shape[-2:]
    N = B.shape[-1]
    up = (lambda t: t.to(AGG_DTYPE)) if fp32_agg else (lambda t: t)
    rd = lambda t: t.to(base_dtype)
    A11, A12, A21, A22 = (up(q) for q in _quadrants(A, M // 2, K // 2))
    B11, B12, B21, B22 = (up(q) for q in _quadrants(B, K // 2, N // 2))

    def f(x, y):
        return up(_strassen_rect_level(rd(x), rd(y), levels - 1, base_dtype, fp32_agg, mm))

    M1 = f(A11 + A22, B11 + B22)
    M2 = f(A21 + A22, B11)
    M3 = f(A11, B12 - B22)
    M4 = f(A22, B21 - B11)
    M5 = f(A11 + A12, B22)
    M6 = f(A21 - A11, B11 + B12)
    M7 = f(A12 - A22, B21 + B22)
    return _assemble(rd(M1 + M4 - M5 + M7), rd(M3 + M5), rd(M2 + M4), rd(M1 - M2 + M3 + M6))


def strassen_general(A: torch.Tensor, B: torch.Tensor, levels: int = 1,
                     base_dtype: torch.dtype | None = None, fp32_agg: bool = True,
                     winograd: bool = False, mm=torch.matmul) -> torch.Tensor:
    """(batch,) M x K times (batch,) K x N with `levels` Strassen levels, any sizes.

    Same formulas and cast schedule as strassen_base[_fp32_agg] / winograd_base, applied
    after zero-padding M, N, K to multiples of 2**levels (a padded Strassen product equals
    the unpadded product on the original index range).  No LEAF cut-off: `levels` is
    exact.  Every level's products run in base_dtype (the evident intent of
    fixed_strassen_fp32_agg.py).
    """
    base_dtype = base_dtype or A.dtype
    M, K = A.shape[-2:]
    N = B.shape[-1]
    q = 1 << levels
    Mp, Np, Kp = (-(-d // q) * q for d in (M, N, K))
    Ap, Bp = _pad_to(A, Mp, Kp), _pad_to(B, Kp, Np)
    if winograd:
        assert levels == 1
        C = winograd_base(Ap, Bp, base_dtype, fp32_agg, mm)
    else:
        C = _strassen_rect_level(Ap, Bp, levels, base_dtype, fp32_agg, mm)
    return C[..., :M, :N].contiguous()


def tile_kernel_semantics(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor,
                          operand_dtype: torch.dtype | None = torch.float16) -> torch.Tensor:
    """What run_strassen / run_strassen2 / run_matmul_fp32_accum /
    run_strassen_2_layer_fp32_accum leave in C: C_in + A @ B.

    strassen.py:150-163 casts every loaded operand tile to fp16 (operand_dtype), the
    products accumulate in fp32 (:130-133,:165-176) and the epilogue adds the old C and
    stores in C's dtype (:184-192).  strassen.py:31-64 and strassen_2_layer.py:103-162 use
    the operands as loaded (operand_dtype=None).  The per-tile Strassen regrouping changes
    only the rounding of the fp32 accumulation, so the oracle is the classical product of
    the cast operands accumulated in fp64 and rounded once (tolerance based comparison).
    """
    a = A if operand_dtype is None else A.to(operand_dtype)
    b = B if operand_dtype is None else B.to(operand_dtype)
    prod = torch.matmul(a.double(), b.double())
    return (C.double() + prod).to(C.dtype)


def linear_strassen_forward(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None,
                            depth: int = 1, mm=torch.mm) -> torch.Tensor:
    """model/layers.py:246-274: view to (M, D), M > D -> ValueError (:255-259), zero-pad
    rows to D (:261-262), Strassen product with weight.T (:264), slice, view, + bias."""
    *batch_dims, D_in = x.shape
    D = weight.shape[1]
    assert D_in == D, "Input dim mismatch"
    Mrows = x.numel() // D
    if Mrows > D:
        raise ValueError(
            f"Input M ({Mrows}) > D ({D}). Cannot pad input to DxD. "
            f"You MUST use the method that pads BOTH input and weights to PxP.")
    Xp = torch.nn.functional.pad(x.reshape(Mrows, D), (0, 0, 0, D - Mrows))
    if depth == 2:
        out = strassen_matmul_two_layers(Xp, weight.T, mm)
    else:
        out = strassen_base(Xp, weight.T, mm)
    out = out[:Mrows, :D].reshape(*batch_dims, D)
    return out + bias if bias is not None else out


def rel_fro(X: torch.Tensor, Y: torch.Tensor) -> float:
    """||X - Y||_F / ||Y||_F in fp64."""
    X, Y = X.double(), Y.double()
    return float(torch.linalg.norm(X - Y) / torch.linalg.norm(Y).clamp_min(1e-300))
