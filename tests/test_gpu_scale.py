"""GPU parity at the sizes the configurations name, through the reference-shaped surface:
multi-level recursion against the oracle's strassen_matmul_n_layers, the two-layer function
and the Linear adaptors on Gaussian inputs at thousands of rows, the GPT-2 Linear shapes
through the autograd layer, the benchmark harnesses as checked artefacts, and one 16384^3 run
checked through size-independent properties."""
import pytest
import torch

from oracle import strassen_oracle as O

pytestmark = pytest.mark.gpu

TOL16 = 2e-2   # rel. Frobenius bound for bf16 / fp16 inputs with fp32 aggregation


def _gauss(shape, seed, scale, dtype):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,depth", [(2048, 2), (4096, 2)])
def test_two_levels_against_the_oracle_recursion(dtype, n, depth):
    """strassen_matmul_n_layers, depth 2, Gaussian inputs, against the oracle's restatement of
    fixed_strassen_fp32_agg.py:58-125 (first-level sums rounded once, inner level in fp32) at the
    undoubled bound.  The inner level here runs on the 16-bit matrix cores, which is where the
    difference comes from."""
    import fixed_strassen_fp32_agg as agg
    A, B = _gauss((n, n), 101, n ** -0.5, dtype), _gauss((n, n), 102, n ** -0.5, dtype)
    C = agg.strassen_matmul_n_layers(A.cuda(), B.cuda(), depth, dtype).cpu()
    want = O.strassen_matmul_n_layers(A, B, depth, dtype, fp32_agg=True, mm=O.mm_fp32_upcast)
    err, err64 = O.rel_fro(C, want), O.rel_fro(C, A.double() @ B.double())
    print(f"depth {depth} {n}^3 {dtype}: vs oracle {err:.3e}, vs fp64 {err64:.3e}")
    assert err <= TOL16 and err64 <= TOL16


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_three_levels_against_the_oracle_recursion(dtype):
    """Depth 3 at 2048^3 against the oracle.  The reference runs everything below the first level
    in fp32 (fixed_strassen_fp32_agg.py:99-113 drop base_dtype); so does the library from three
    levels on: first-level sums rounded to the operand type, the seven half-size products as
    two-level fp32 products.  What is left is fp32 summation order seen through the final
    rounding (4.6e-5 on the CPU build of the library at 256^3), asserted at 1e-3, a twentieth of
    the configurations' bound."""
    import fixed_strassen_fp32_agg as agg
    n = 2048
    A, B = _gauss((n, n), 103, n ** -0.5, dtype), _gauss((n, n), 104, n ** -0.5, dtype)
    C = agg.strassen_matmul_n_layers(A.cuda(), B.cuda(), 3, dtype).cpu()
    want = O.strassen_matmul_n_layers(A, B, 3, dtype, fp32_agg=True, mm=O.mm_fp32_upcast)
    err, err64 = O.rel_fro(C, want), O.rel_fro(C, A.double() @ B.double())
    print(f"depth 3 {n}^3 {dtype}: vs oracle {err:.3e}, vs fp64 {err64:.3e}")
    assert err <= 1e-3 and err64 <= TOL16


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_three_levels_rounding_every_level(dtype):
    """schedule="fast" (STHIP_SCHEDULE_FAST): every level multiplies on the 16-bit matrix cores and
    rounds its operand sums and products once each, which about doubles the error per level:
    measured 2.3e-2 (bf16) against the oracle at 2048^3, outside the 2e-2 of the configurations --
    the reason three levels do not take this schedule unasked.  Bound 3e-2; fp16, with three more
    bits, must meet 2e-2 / 4."""
    import strassen_hip
    n = 2048
    A, B = _gauss((n, n), 103, n ** -0.5, dtype), _gauss((n, n), 104, n ** -0.5, dtype)
    C = strassen_hip.gemm(A.cuda(), B.cuda(), levels=3, schedule="fast").cpu()
    want = O.strassen_matmul_n_layers(A, B, 3, dtype, fp32_agg=True, mm=O.mm_fp32_upcast)
    err, err64 = O.rel_fro(C, want), O.rel_fro(C, A.double() @ B.double())
    print(f"depth 3 {n}^3 {dtype} rounding every level: vs oracle {err:.3e}, vs fp64 {err64:.3e}")
    assert err <= (3e-2 if dtype == torch.bfloat16 else TOL16 / 4)


def test_two_layers_function_gaussian_2048():
    """strassen.strassen_matmul_two_layers (reference strassen.py:742-812) at 2048^3 bf16 on
    Gaussian inputs against the oracle's restatement (all arithmetic in the input dtype there)."""
    import strassen
    n = 2048
    A, B = _gauss((n, n), 105, n ** -0.5, torch.bfloat16), _gauss((n, n), 106, n ** -0.5, torch.bfloat16)
    C = strassen.strassen_matmul_two_layers(A.cuda(), B.cuda()).cpu()
    want = O.strassen_matmul_two_layers(A, B, mm=O.mm_fp32_upcast)
    exact = A.double() @ B.double()
    err, err64, ora64 = O.rel_fro(C, want), O.rel_fro(C, exact), O.rel_fro(want, exact)
    print(f"two_layers 2048 bf16: vs oracle {err:.3e}, vs fp64 {err64:.3e} (oracle vs fp64 {ora64:.3e})")
    # the oracle adds in bf16 at both levels and is itself 1.6e-2 from fp64; the kernel adds in fp32
    assert err <= 2 * TOL16 and err64 <= TOL16 and err64 <= ora64


@pytest.mark.parametrize("depth,rows", [(1, 4096), (1, 1000), (2, 4096), (2, 1000)])
def test_linear_strassen_4096_against_the_oracle(depth, rows):
    """model.layers.LinearStrassen(4096) with rows == D and rows < D against the oracle's
    restatement of model/layers.py:246-274 (pad to D x D, _strassen_base or the two-layer
    function of strassen.py, slice, + bias), leaf products through mm_fp32_upcast."""
    from model.layers import LinearStrassen
    D, dtype = 4096, torch.bfloat16
    lin = LinearStrassen(D, D, bias=True, dtype=dtype, depth=depth, device="cuda")
    w, b = _gauss((D, D), 107, D ** -0.5, dtype), _gauss((D,), 108, 1.0, dtype)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    x = _gauss((rows, D), 109, 1.0, dtype)
    with torch.no_grad():
        y = lin(x.cuda()).cpu()
    want = O.linear_strassen_forward(x, w, b, depth, mm=O.mm_fp32_upcast)
    exact = x.double() @ w.double().t() + b.double()
    err, err64, ora64 = O.rel_fro(y, want), O.rel_fro(y, exact), O.rel_fro(want, exact)
    print(f"LinearStrassen 4096 depth {depth} rows {rows}: vs oracle {err:.3e}, vs fp64 {err64:.3e} (oracle vs fp64 {ora64:.3e})")
    assert y.shape == (rows, D) and y.dtype == dtype
    assert err64 <= TOL16 and err <= TOL16 * (1 if depth == 1 else 2) and err64 <= ora64 * 1.05


@pytest.mark.parametrize("cutoff", [False, True])
@pytest.mark.parametrize("d_in,d_out", [(768, 2304), (768, 768), (768, 3072), (3072, 768)])
def test_gpt2_linear_shapes_through_the_autograd_layer(d_in, d_out, cutoff):
    """The GPT-2-small Linear shapes with 8192 token rows through LinearStrassenRect: forward,
    input gradient and weight gradient against the oracle's one-level product on the same
    operands (strassen_general: fp32 aggregation, products in bf16).  cutoff=False runs one
    Strassen level in all three products; with the measured cutoff (the default) forward and
    input gradient run the classical kernel on these shapes and the weight gradients of the
    layers with at most 128 output tiles keep their level."""
    import strassen_hip
    from model.layers import LinearStrassenRect
    rows, dtype = 8192, torch.bfloat16
    if cutoff:
        assert strassen_hip.auto_levels(rows, d_out, d_in, dtype, 1) == 0
        assert strassen_hip.auto_levels(d_out, d_in, rows, dtype, 1) == (1 if d_in * d_out <= 128 * 128 * 128 else 0)
    lin = LinearStrassenRect(d_in, d_out, bias=True, dtype=dtype, device="cuda", cutoff=cutoff)
    w, b = _gauss((d_out, d_in), 111, 0.02, dtype), _gauss((d_out,), 112, 0.02, dtype)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    x, dy = _gauss((rows, d_in), 113, 0.02, dtype), _gauss((rows, d_out), 114, 0.02, dtype)
    xg = x.cuda().requires_grad_()
    y = lin(xg)
    y.backward(dy.cuda())
    mm = O.mm_fp32_upcast
    want_y = (O.strassen_general(x, w.t(), 1, dtype, mm=mm).float() + b.float()).to(dtype)
    want_dx = O.strassen_general(dy, w, 1, dtype, mm=mm)
    want_dw = O.strassen_general(dy.t(), x, 1, dtype, mm=mm)
    errs = {"fwd": O.rel_fro(y.detach().cpu(), want_y), "dgrad": O.rel_fro(xg.grad.cpu(), want_dx),
            "wgrad": O.rel_fro(lin.weight.grad.cpu(), want_dw)}
    print(f"GPT-2 {d_in}->{d_out}: " + ", ".join(f"{k} {v:.2e}" for k, v in errs.items()))
    assert all(v <= TOL16 for v in errs.values()), errs
    assert O.rel_fro(lin.bias.grad.cpu(), dy.double().sum(0)) <= TOL16


def test_benchmark_table_rows():
    """The main_profiling.py table (reference :236-302) as a checked artefact: the row of every
    (N, depth) has the reference's columns and a difference to nn.Linear inside the bf16 bound."""
    import main_profiling as mp
    flush = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    for n, depth in ((1024, 1), (2048, 2)):
        r = mp.benchmark_linear_layers(n, depth, num_warmup=2, num_runs=5, flush=flush)
        for key in ("N_dim", "strassen_depth", "std_mean_ms", "strassen_mean_ms", "speedup_mean", "std_tflops",
                    "strassen_tflops", "max_abs_diff", "allclose"):
            assert key in r, key
        assert r["N_dim"] == n and r["strassen_depth"] == depth
        assert r["std_mean_ms"] > 0 and r["strassen_mean_ms"] > 0 and r["strassen_tflops"] > 0
        # outputs are O(1) (N(0,1) inputs, |w| < 1/sqrt(N)): a few bf16 ulps of the largest entries
        assert r["max_abs_diff"] <= 0.125, r
        assert "|" in mp.format_row(r) and mp.HEADER.split("|")[0].strip() == "N_dim"


def test_block_demo_forward_and_backward():
    """The decoder-block demo (reference train.py:322-350 on model/model.py:4-32): all four Linear
    layers are replaced and the block's output and weight gradients stay inside the bf16 bound."""
    import gpt_block_demo as demo
    r = demo.compare_block(1024, 8, 2048, torch.bfloat16, backward=True, warmup=1, runs=2, verbose=False)
    assert r["replaced"] == ["LinearStrassenRect"] * 4
    assert r["rel_diff"] <= TOL16 and r["rel_diff_weight_grad"] <= TOL16, r
    assert r["std_ms"] > 0 and r["strassen_ms"] > 0


def test_one_level_16384_properties():
    """One level at 16384^3 bf16, too large for the CPU oracle: checked through properties that do
    not depend on size.  Scaling an operand by a power of two scales every sum, product and
    rounding exactly; (A B)^T = B^T A^T through transposed views exercises the other operand
    layouts and must agree to within rounding; a slab of 64 rows is compared with fp64."""
    import strassen_hip
    n, dtype = 16384, torch.bfloat16
    A, B = _gauss((n, n), 121, n ** -0.5, dtype).cuda(), _gauss((n, n), 122, n ** -0.5, dtype).cuda()
    C = strassen_hip.gemm(A, B, algo="strassen", levels=1)
    C4 = strassen_hip.gemm(A * 4, B, algo="strassen", levels=1)
    assert torch.equal(C4, C * 4)
    del C4
    Ct = strassen_hip.gemm(B.t(), A.t(), algo="strassen", levels=1)
    diff = float(torch.linalg.norm((Ct.t() - C).float()) / torch.linalg.norm(C.float()))
    assert diff <= TOL16 / 2, diff
    del Ct
    rows = slice(5000, 5064)
    exact = A[rows].double() @ B.double()
    err = float(torch.linalg.norm(C[rows].double() - exact) / torch.linalg.norm(exact))
    print(f"16384^3 bf16 one level: slab vs fp64 {err:.3e}, transpose identity {diff:.3e}")
    assert err <= TOL16


def test_result_does_not_depend_on_extra_workspace():
    """The kernels a multi-level call picks depend on the shape only: a workspace larger than the
    query asks for gives the same bits as one of exactly that size (host recursion, two and three
    levels -- the third on either rounding schedule -- and a shape the 49-product form does not take)."""
    import strassen_hip
    for levels, shape, schedule in ((2, (1024, 768, 1536), "auto"), (3, (1024, 1024, 2048), "auto"), (3, (1024, 1024, 2048), "fast")):
        M, N, K = shape
        A, B = _gauss((M, K), 131, K ** -0.5, torch.bfloat16).cuda(), _gauss((K, N), 132, 1.0, torch.bfloat16).cuda()
        need = strassen_hip.workspace_bytes(A, B, levels=levels, schedule=schedule)
        exact_ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        big_ws = torch.empty(3 * need + 4096, dtype=torch.uint8, device="cuda")
        c1 = strassen_hip.gemm(A, B, levels=levels, workspace=exact_ws, schedule=schedule)
        algo_code = strassen_hip.ALGO_STRASSEN | {"auto": 0, "fast": strassen_hip.SCHEDULE_FAST}[schedule]
        lib = strassen_hip._capi.load()
        c2 = torch.empty_like(c1)
        from strassen_hip.ops import _strides3
        strassen_hip._capi.check(lib.sthip_gemm(A.data_ptr(), B.data_ptr(), c2.data_ptr(), 1, M, N, K, _strides3(A), _strides3(B),
                                                _strides3(c2), 2, 2, algo_code, levels, 0, big_ws.data_ptr(), big_ws.numel(),
                                                torch.cuda.current_stream().cuda_stream))
        assert torch.equal(c1, c2), (levels, shape, schedule)


def test_kept_weight_sums_under_inference_mode():
    """Parameters created under torch.inference_mode track no version counter; the caching layer
    must still run (it forms the sums for the call instead of keeping them)."""
    from model.layers import LinearStrassen
    with torch.inference_mode():
        lin = LinearStrassen(1024, 1024, bias=False, dtype=torch.bfloat16, device="cuda", cache_weight_sums=True)
        plain = LinearStrassen(1024, 1024, bias=False, dtype=torch.bfloat16, device="cuda")
        plain.weight.copy_(lin.weight)
        x = _gauss((1024, 1024), 141, 1.0, torch.bfloat16).cuda()
        assert torch.equal(lin(x), plain(x))


def test_cutoff_table_rows():
    """The cutoff table of main_profiling.py (classical kernel against Strassen levels, beside the rule of sthip_auto_levels) on
    two small shapes: every column is there and timed, and the rule's column is what the library itself answers."""
    import main_profiling as mp
    import strassen_hip
    rows = mp.profile_cutoff(torch.bfloat16, [(1024, 1024, 1024), (2048, 1024, 512)], max_levels=2, b_transposed=True, runs=4)
    assert [(r["M"], r["N"], r["K"]) for r in rows] == [(1024, 1024, 1024), (2048, 1024, 512)]
    for r in rows:
        assert len(r["level_ms"]) == 3 and all(t > 0 for t in r["level_ms"]) and r["std_ms"] > 0
        assert r["best_levels"] in (0, 1, 2)
        assert r["rule_levels"] == strassen_hip.auto_levels(r["M"], r["N"], r["K"], torch.bfloat16, 2)
