"""Pins the CPU oracle (oracle/strassen_oracle.py) with checks that do not retype it:
exact-arithmetic identities on small integers, a triple loop on tiny sizes, structured
inputs (identity, one-hot, block-diagonal) and algebraic invariants.  A dropped term, a
wrong sign, a swapped quadrant or a transposed operand fails at least one of them."""
import itertools

import pytest
import torch

from oracle import strassen_oracle as O


def _ints(shape, seed, lo=-2, hi=2, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).to(dtype)


def _triple_loop(A, B):
    M, K = A.shape
    N = B.shape[1]
    C = [[0.0] * N for _ in range(M)]
    a, b = A.tolist(), B.tolist()
    for i in range(M):
        for j in range(N):
            s = 0.0
            for k in range(K):
                s += a[i][k] * b[k][j]
            C[i][j] = s
    return torch.tensor(C, dtype=torch.float64)


ALGOS = {
    "base": lambda A, B: O.strassen_base(A, B),
    "base_agg": lambda A, B: O.strassen_base_fp32_agg(A, B, A.dtype),
    "n2": lambda A, B: O.strassen_matmul_n_layers(A, B, 2),
    "n3": lambda A, B: O.strassen_matmul_n_layers(A, B, 3),
    "n2_agg": lambda A, B: O.strassen_matmul_n_layers(A, B, 2, A.dtype, fp32_agg=True),
    "n3_agg_keep": lambda A, B: O.strassen_matmul_n_layers(
        A, B, 3, A.dtype, fp32_agg=True, inner_keeps_base_dtype=True),
    "two_layers": lambda A, B: O.strassen_matmul_two_layers(A, B),
    "zorder49": lambda A, B: O.strassen2_zorder_49(A, B),
    "winograd": lambda A, B: O.winograd_base(A, B, A.dtype, fp32_agg=False),
    "general_l1": lambda A, B: O.strassen_general(A, B, 1, fp32_agg=False),
    "general_l2": lambda A, B: O.strassen_general(A, B, 2, fp32_agg=False),
    "general_wino": lambda A, B: O.strassen_general(A, B, 1, fp32_agg=False, winograd=True),
}


@pytest.mark.parametrize("name", sorted(ALGOS))
@pytest.mark.parametrize("n", [32, 64, 128])
def test_integer_known_answer_exact_fp64(name, n):
    """Small integers: every partial sum is exact, so the result must equal A @ B bit for bit."""
    A, B = _ints((n, n), 1), _ints((n, n), 2)
    C = ALGOS[name](A, B)
    assert C.shape == (n, n)
    assert torch.equal(C, A @ B)


@pytest.mark.parametrize("name", sorted(ALGOS))
def test_integer_known_answer_exact_low_precision(name):
    """Same in fp32: entries in [-2, 2], n = 64 -- every pre-sum, product and partial sum is an
    integer far below 2**24, hence exact in fp32."""
    n = 64
    A, B = _ints((n, n), 3, dtype=torch.float32), _ints((n, n), 4, dtype=torch.float32)
    assert torch.equal(ALGOS[name](A, B).double(), A.double() @ B.double())


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_fp32_agg_schedule_exact_on_small_ints(dt):
    """fp32-aggregated variant on +-1/0 entries, n = 32: all values are integers of magnitude
    <= 64 < 256, exactly representable in bf16 and fp16 at every rounding point."""
    n = 32
    A, B = _ints((n, n), 5, -1, 1, dt), _ints((n, n), 6, -1, 1, dt)
    want = (A.double() @ B.double())
    assert want.abs().max() <= 256
    for C in (O.strassen_base_fp32_agg(A, B, dt),
              O.strassen_matmul_n_layers(A, B, 2, dt, fp32_agg=True),
              O.strassen_matmul_n_layers(A, B, 2, dt, fp32_agg=True, inner_keeps_base_dtype=True),
              O.strassen_general(A, B, 1, dt, True),
              O.strassen_general(A, B, 2, dt, True),
              O.strassen_general(A, B, 1, dt, True, winograd=True),
              O.strassen_base(A, B)):
        assert C.dtype == dt
        assert torch.equal(C.double(), want)


@pytest.mark.parametrize("name", ["zorder49", "winograd", "general_l1", "general_l2", "general_wino"])
@pytest.mark.parametrize("n", [4, 8])
def test_brute_force_tiny(name, n):
    """Sizes below the reference's n <= 16 cut-off exist only for the variants without it."""
    g = torch.Generator().manual_seed(n)
    A = torch.randn(n, n, generator=g, dtype=torch.float64)
    B = torch.randn(n, n, generator=g, dtype=torch.float64)
    torch.testing.assert_close(ALGOS[name](A, B), _triple_loop(A, B), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("name", sorted(ALGOS))
def test_brute_force_32(name):
    g = torch.Generator().manual_seed(7)
    A = torch.randn(32, 32, generator=g, dtype=torch.float64)
    B = torch.randn(32, 32, generator=g, dtype=torch.float64)
    # the fp32-aggregated variants round their sums and recombination to fp32 by construction
    tol = 1e-4 if "agg" in name else 1e-11
    torch.testing.assert_close(ALGOS[name](A, B), _triple_loop(A, B), rtol=tol, atol=tol)


@pytest.mark.parametrize("name", sorted(ALGOS))
def test_structured_inputs(name):
    n = 64
    f = ALGOS[name]
    I = torch.eye(n, dtype=torch.float64)
    X = _ints((n, n), 11)
    assert torch.equal(f(X, I), X)          # B = I
    assert torch.equal(f(I, X), X)          # A = I
    assert torch.equal(f(X, torch.zeros_like(X)), torch.zeros_like(X))
    E = torch.zeros(n, n, dtype=torch.float64)
    E[5, 41] = 1.0                          # one-hot A: row 5 of the result is row 41 of B
    R = f(E, X)
    assert torch.equal(R[5], X[41]) and R.abs().sum() == X[41].abs().sum()
    E2 = torch.zeros(n, n, dtype=torch.float64)
    E2[50, 9] = 1.0                         # one-hot B: column 9 of the result is column 50 of A
    R2 = f(X, E2)
    assert torch.equal(R2[:, 9], X[:, 50]) and R2.abs().sum() == X[:, 50].abs().sum()
    ones = torch.ones(n, n, dtype=torch.float64)
    assert torch.equal(f(ones, ones), ones * n)
    D = torch.zeros(n, n, dtype=torch.float64)  # block diagonal: no cross terms may leak
    D[:32, :32] = _ints((32, 32), 12)
    D[32:, 32:] = _ints((32, 32), 13)
    R3 = f(D, D)
    assert torch.equal(R3[:32, 32:], torch.zeros(32, 32, dtype=torch.float64))
    assert torch.equal(R3[:32, :32], D[:32, :32] @ D[:32, :32])


@pytest.mark.parametrize("name", sorted(ALGOS))
def test_invariants(name):
    n = 64
    f = ALGOS[name]
    A, B = _ints((n, n), 21), _ints((n, n), 22)
    # (A B)^T = B^T A^T catches a transposed or swapped operand
    assert torch.equal(f(A, B).T, f(B.T.contiguous(), A.T.contiguous()))
    # linearity with a power of two is exact
    assert torch.equal(f(4 * A, B), 4 * f(A, B))
    # non-commutativity witness: a swapped operand order would pass the symmetric checks above
    assert not torch.equal(f(A, B), f(B, A))


@pytest.mark.parametrize("shape", [(48, 80, 36), (33, 17, 65), (2, 2, 2), (1, 7, 3), (130, 66, 18)])
@pytest.mark.parametrize("levels,wino", [(1, False), (2, False), (1, True)])
def test_general_rectangular_and_odd(shape, levels, wino):
    M, N, K = shape
    A, B = _ints((M, K), 31), _ints((K, N), 32)
    C = O.strassen_general(A, B, levels, fp32_agg=False, winograd=wino)
    assert C.shape == (M, N) and torch.equal(C, A @ B)
    Ab, Bb = _ints((3, M, K), 33), _ints((3, K, N), 34)
    Cb = O.strassen_general(Ab, Bb, levels, fp32_agg=False, winograd=wino)
    assert torch.equal(Cb, Ab @ Bb)


def test_two_layers_validation_messages():
    with pytest.raises(ValueError, match="square"):
        O.strassen_matmul_two_layers(torch.zeros(8, 4), torch.zeros(4, 8))
    with pytest.raises(ValueError, match="divisible by 4"):
        O.strassen_matmul_two_layers(torch.zeros(6, 6), torch.zeros(6, 6))


def test_tolerance_schedule_bf16_fp16_fp32():
    """The documented tolerances hold between the oracle variants and an fp64 classical product."""
    n = 256
    g = torch.Generator().manual_seed(1234)
    A32 = torch.randn(n, n, generator=g) / n ** 0.5
    B32 = torch.randn(n, n, generator=g) / n ** 0.5
    want = A32.double() @ B32.double()
    assert O.rel_fro(O.strassen_base(A32, B32), want) < 1e-5
    assert O.rel_fro(O.strassen_matmul_n_layers(A32, B32, 2), want) < 1e-5
    for dt in (torch.bfloat16, torch.float16):
        A, B = A32.to(dt), B32.to(dt)
        want_dt = A.double() @ B.double()
        for C in (O.strassen_base_fp32_agg(A, B, dt),
                  O.strassen_matmul_n_layers(A, B, 2, dt, fp32_agg=True),
                  O.strassen_general(A, B, 2, dt, True),
                  O.strassen_general(A, B, 1, dt, True, winograd=True)):
            assert O.rel_fro(C, want_dt) < 2e-2


def test_tile_kernel_semantics_and_linear():
    A, B = _ints((32, 48), 41, dtype=torch.float32), _ints((48, 16), 42, dtype=torch.float32)
    C0 = _ints((32, 16), 43, dtype=torch.float32)
    out = O.tile_kernel_semantics(A, B, C0)
    assert torch.equal(out, C0 + A @ B)
    D = 64
    W, b = _ints((D, D), 44, dtype=torch.float32), _ints((D,), 45, dtype=torch.float32)
    x = _ints((3, 5, D), 46, dtype=torch.float32)
    for depth in (1, 2):
        y = O.linear_strassen_forward(x, W, b, depth)
        assert torch.equal(y, x @ W.T + b)
    with pytest.raises(ValueError, match="Cannot pad input"):
        O.linear_strassen_forward(torch.zeros(65, D), W, None)
