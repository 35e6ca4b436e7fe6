"""GPU tests of the reference-shaped call surface: same names, arguments, return values
and exceptions as strassen.py / fixed_strassen*.py / strassen_2_layer.py / model/layers.py."""
import pytest
import torch

from oracle import strassen_oracle as O

pytestmark = pytest.mark.gpu


def _ints(shape, seed, lo=-1, hi=1, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).to(dtype)


def test_run_launchers_accumulate_in_place():
    """run_*: C += A @ B, return None (reference strassen.py:184-192; smoke of :815-825 uses
    512 x 512 fp32 with C = zeros)."""
    import strassen
    import strassen_2_layer
    torch.manual_seed(1234)
    a, b = torch.randn(512, 512), torch.randn(512, 512)
    for fn, cast in ((strassen.run_strassen, torch.float16), (strassen.run_strassen2, torch.float16),
                     (strassen.run_matmul_fp32_accum, None), (strassen_2_layer.run_strassen_2_layer_fp32_accum, None)):
        c0 = torch.randn(512, 512)
        c = c0.clone().cuda()
        assert fn(a.cuda(), b.cuda(), c) is None
        want = O.tile_kernel_semantics(a, b, c0, cast)
        tol = 2e-2 if cast is not None else 1e-5
        assert O.rel_fro(c.cpu(), want) <= tol, fn.__name__
    # batched, fp16 C, exact integers
    A, B = _ints((2, 128, 64), 1, dtype=torch.float16), _ints((2, 64, 256), 2, dtype=torch.float16)
    C0 = _ints((2, 128, 256), 3, -3, 3, torch.float16)
    C = C0.clone().cuda()
    strassen.run_strassen(A.cuda(), B.cuda(), C)
    assert torch.equal(C.cpu().double(), C0.double() + A.double() @ B.double())
    with pytest.raises(AssertionError):
        strassen.run_strassen(torch.zeros(4, 5).cuda(), torch.zeros(6, 4).cuda(), torch.zeros(4, 4).cuda())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,depth", [(16, 1), (64, 1), (256, 2), (256, 3), (512, 2), (64, 7)])
def test_matrix_level_functions(dtype, n, depth):
    import fixed_strassen as fs
    import fixed_strassen_fp32_agg as agg
    import strassen
    assert agg.agg_dtype == torch.float32
    A, B = _ints((n, n), 5, dtype=dtype), _ints((n, n), 6, dtype=dtype)
    want = A.double() @ B.double()
    outs = [fs.strassen_matmul_n_layers(A.cuda(), B.cuda(), depth),
            agg.strassen_matmul_n_layers(A.cuda(), B.cuda(), depth, dtype)]
    if depth == 1:
        outs += [fs._strassen_base(A.cuda(), B.cuda()), agg._strassen_base(A.cuda(), B.cuda(), dtype),
                 strassen._strassen_base(A.cuda(), B.cuda())]
    if depth == 2:
        outs.append(strassen.strassen_matmul_two_layers(A.cuda(), B.cuda()))
    for C in outs:
        assert C.dtype == dtype and C.shape == (n, n)
        if want.abs().max() <= 128:
            assert torch.equal(C.cpu().double(), want)
        else:
            assert O.rel_fro(C.cpu(), want) <= 2e-2


def test_two_layers_validation():
    import strassen
    with pytest.raises(ValueError, match="square"):
        strassen.strassen_matmul_two_layers(torch.zeros(8, 4).cuda(), torch.zeros(4, 8).cuda())
    with pytest.raises(ValueError, match="divisible by 4"):
        strassen.strassen_matmul_two_layers(torch.zeros(6, 6).cuda(), torch.zeros(6, 6).cuda())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("depth", [1, 2])
def test_linear_strassen_forward_backward(dtype, depth):
    from model.layers import LinearStrassen
    D = 256
    lin = LinearStrassen(D, D, bias=True, dtype=dtype, depth=depth, device="cuda")
    with torch.no_grad():
        lin.weight.copy_(_ints((D, D), 7).to(dtype))
        lin.bias.copy_(_ints((D,), 8).to(dtype))
    x = _ints((3, 40, D), 9).to(dtype)
    y = lin(x.cuda())
    want = O.linear_strassen_forward(x.float(), lin.weight.detach().cpu().float(), lin.bias.detach().cpu().float(), depth)
    assert y.shape == (3, 40, D) and y.dtype == dtype
    if want.abs().max() <= 128:
        assert torch.equal(y.detach().cpu().float(), want)
    else:
        assert O.rel_fro(y.detach().cpu(), want) <= 2e-2
    # gradients against plain autograd on the same integers
    xg = x.cuda().requires_grad_()
    g = _ints((3, 40, D), 10).to(dtype).cuda()
    lin.zero_grad()
    lin(xg).backward(g)
    xr = x.float().requires_grad_()
    Wr = lin.weight.detach().cpu().float().requires_grad_()
    br = lin.bias.detach().cpu().float().requires_grad_()
    (xr @ Wr.T + br).backward(g.cpu().float())
    for got, ref in ((xg.grad, xr.grad), (lin.weight.grad, Wr.grad), (lin.bias.grad, br.grad)):
        assert O.rel_fro(got.cpu(), ref) <= (1e-5 if dtype == torch.float32 else 2e-2)
    with pytest.raises(ValueError, match="Cannot pad input"):
        lin(torch.zeros(D + 1, D, dtype=dtype, device="cuda"))
    with pytest.raises(AssertionError, match="square and a power of 2"):
        LinearStrassen(96, 96, device="cuda")


def test_replace_linear_with_strassen(capsys):
    import torch.nn as nn
    from model.layers import LinearStrassen, replace_linear_with_strassen
    net = nn.Sequential(nn.Linear(256, 256), nn.ReLU(), nn.Sequential(nn.Linear(256, 64), nn.Linear(64, 64))).cuda()
    x = torch.randn(32, 256, device="cuda")
    before = net(x)
    replace_linear_with_strassen(net, min_size=128, depth=1)
    out = capsys.readouterr().out
    assert "Replacing '0' with LinearStrassen." in out and "Skipping" in out
    assert isinstance(net[0], LinearStrassen) and not isinstance(net[2][0], LinearStrassen)
    assert O.rel_fro(net(x).cpu(), before.cpu()) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(300, 768, 2304), (1000, 3072, 768), (77, 130, 129)])
def test_linear_strassen_rect_forward_backward(dtype, shape):
    """Non-square layer without padding: forward, dgrad and wgrad each against the same product
    in fp64 (rel. Frobenius <= 1e-5 fp32 / 2e-2 bf16), and bit for bit on small integers."""
    from model.layers import LinearStrassenRect
    rows, d_in, d_out = shape
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    g = torch.Generator().manual_seed(7)
    lin = LinearStrassenRect(d_in, d_out, bias=True, dtype=dtype, device="cuda", cutoff=False)
    x = (torch.randn(rows, d_in, generator=g) * 0.5).to(dtype).cuda().requires_grad_()
    dy = (torch.randn(rows, d_out, generator=g) * 0.5).to(dtype).cuda()
    y = lin(x)
    y.backward(dy)
    W, b = lin.weight.detach().double(), lin.bias.detach().double()
    rel = lambda got, ref: float(torch.linalg.norm(got.double() - ref) / torch.linalg.norm(ref))
    assert y.shape == (rows, d_out)
    assert rel(y.detach(), x.detach().double() @ W.T + b) <= tol
    assert rel(x.grad, dy.double() @ W) <= tol
    assert rel(lin.weight.grad, dy.double().T @ x.detach().double()) <= tol
    assert rel(lin.bias.grad, dy.double().sum(0)) <= tol
    # integers: every sum and product is exact, so the three GEMMs must be too
    xi = torch.randint(-2, 3, (rows, d_in), generator=g).to(dtype).cuda().requires_grad_()
    with torch.no_grad():
        lin.weight.copy_(torch.randint(-1, 2, (d_out, d_in), generator=g).to(dtype))
        lin.bias.zero_()
    lin.weight.grad = None
    di = torch.randint(-1, 2, (rows, d_out), generator=g).to(dtype).cuda()
    yi = lin(xi.view(1, rows, d_in))
    assert yi.shape == (1, rows, d_out)
    yi.backward(di.view(1, rows, d_out))
    Wi = lin.weight.detach().double()
    exact = lambda got, ref: torch.equal(got.double(), ref.to(dtype).double())
    assert exact(yi.detach()[0], xi.detach().double() @ Wi.T)
    assert exact(xi.grad, di.double() @ Wi)
    assert exact(lin.weight.grad, di.double().T @ xi.detach().double())


def test_replace_linear_with_strassen_rect(capsys):
    import torch.nn as nn
    from model.layers import LinearStrassen, LinearStrassenRect, replace_linear_with_strassen
    net = nn.Sequential(nn.Linear(256, 768), nn.GELU(), nn.Linear(768, 256), nn.Linear(256, 256),
                        nn.Linear(256, 32)).cuda()
    x = torch.randn(40, 256, device="cuda")
    before = net(x)
    replace_linear_with_strassen(net, min_size=128, depth=1, square_only=False)
    out = capsys.readouterr().out
    assert "Replacing '0' with LinearStrassenRect." in out and "Replacing '3' with LinearStrassenRect." in out
    assert all(isinstance(net[i], LinearStrassenRect) for i in (0, 2, 3)) and type(net[4]) is nn.Linear
    assert not isinstance(net[3], LinearStrassen)
    assert net(torch.randn(300, 256, device="cuda")).shape == (300, 32)   # more rows than features
    assert O.rel_fro(net(x).cpu(), before.cpu()) <= 1e-5


@pytest.mark.parametrize("levels,n", [(1, 1024), (2, 1024), (1, 384)])
def test_calls_can_be_captured_in_a_hip_graph(levels, n):
    """The C ABI only enqueues kernels on the stream it is given (no allocation, no memset, no
    synchronisation), so a call with caller-owned output and workspace can be captured into a HIP
    graph.  Every replay, with new operand values written in place and eager work in between, must
    reproduce the eager result bit for bit."""
    import strassen_hip
    g = torch.Generator().manual_seed(11)
    A = torch.randn(n, n, generator=g).to(torch.bfloat16).cuda()
    B = torch.randn(n, n, generator=g).to(torch.bfloat16).cuda()
    out = torch.empty(n, n, dtype=torch.bfloat16, device="cuda")
    ws = torch.empty(max(1, strassen_hip.workspace_bytes(A, B, levels=levels)), dtype=torch.uint8, device="cuda")
    strassen_hip.gemm(A, B, out, levels=levels, workspace=ws)          # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        strassen_hip.gemm(A, B, out, levels=levels, workspace=ws)
    for rep in range(3):
        A.copy_(torch.randn(n, n, generator=g).to(torch.bfloat16))
        B.copy_(torch.randn(n, n, generator=g).to(torch.bfloat16))
        eager = strassen_hip.gemm(A, B, levels=levels)
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep


def test_cpu_tensors_are_refused():
    import fixed_strassen
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        fixed_strassen._strassen_base(torch.zeros(32, 32), torch.zeros(32, 32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("depth", [1, 2])
def test_linear_strassen_bias_in_the_recombination_pass(dtype, depth):
    """On tile-aligned 16-bit problems the bias is added by the recombination pass instead of a
    pass of its own; the result is rounded before and after the addition, exactly as
    `strassen(x, W.T) + bias` rounds (reference model/layers.py:264-272), so it must equal the
    product computed without bias plus the bias added by torch, bit for bit."""
    import strassen_hip
    from model.layers import LinearStrassen
    D = 1024
    g = torch.Generator().manual_seed(31)
    lin = LinearStrassen(D, D, bias=True, dtype=dtype, depth=depth, device="cuda")
    with torch.no_grad():
        lin.weight.copy_((torch.randn(D, D, generator=g) * D ** -0.5).to(dtype))
        lin.bias.copy_(torch.randn(D, generator=g).to(dtype))
    x = torch.randn(D, D, generator=g).to(dtype).cuda()
    with torch.no_grad():
        y = lin(x)
        plain = strassen_hip.gemm(x, lin.weight.t(), levels=depth)
        want = plain + lin.bias            # torch: fp32 add of two 16-bit values, rounded once
    assert torch.equal(y, want)
    # fewer rows than features: not the grouped path, the bias is added by the separate pass
    with torch.no_grad():
        y2 = lin(x[:300])
    ref = x[:300].double() @ lin.weight.double().t() + lin.bias.double()
    assert float(torch.linalg.norm(y2.double() - ref) / torch.linalg.norm(ref)) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_linear_strassen_rect_bias_in_the_recombination_pass(dtype):
    """The non-square layer hands its bias to the forward product as well: same bits as the
    product without bias plus torch's add, and the bias gradient is the column sum of dY."""
    import strassen_hip
    from model.layers import LinearStrassenRect
    rows, d_in, d_out = 2048, 1024, 3072
    g = torch.Generator().manual_seed(33)
    lin = LinearStrassenRect(d_in, d_out, bias=True, dtype=dtype, device="cuda", cutoff=False)
    with torch.no_grad():
        lin.weight.copy_((torch.randn(d_out, d_in, generator=g) * d_in ** -0.5).to(dtype))
        lin.bias.copy_(torch.randn(d_out, generator=g).to(dtype))
    x = torch.randn(rows, d_in, generator=g).to(dtype).cuda().requires_grad_()
    y = lin(x)
    with torch.no_grad():
        want = strassen_hip.gemm(x.detach(), lin.weight.t(), levels=1) + lin.bias
    assert torch.equal(y.detach(), want)
    dy = torch.randn(rows, d_out, generator=g).to(dtype).cuda()
    y.backward(dy)
    ref = dy.double().sum(0)
    assert float(torch.linalg.norm(lin.bias.grad.double() - ref) / torch.linalg.norm(ref)) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("levels,rows,d_in,d_out,bias", [
    (1, 1024, 1024, 1024, False), (1, 2048, 1536, 1024, True), (1, 4096, 4096, 4096, True),
    (2, 1024, 1024, 1024, False), (2, 2048, 1536, 1024, True), (2, 4096, 4096, 4096, True),
    (3, 2048, 2048, 2048, True), (3, 4096, 2048, 3072, False), (4, 4096, 4096, 4096, True)])
def test_prepared_weight_sums_same_bits(dtype, levels, rows, d_in, d_out, bias):
    """The forward that reads weight-side sums formed ahead of the call gives the bits of the
    forward that forms them itself -- and does read them: handed the sums of another weight it
    gives another result."""
    import strassen_hip
    g = torch.Generator().manual_seed(rows + d_in + levels)
    x = torch.randn(rows, d_in, generator=g).to(dtype).cuda()
    w = (torch.randn(d_out, d_in, generator=g) * d_in ** -0.5).to(dtype).cuda()
    b = torch.randn(d_out, generator=g).to(dtype).cuda() if bias else None
    want = strassen_hip.linear_forward_any(x, w, b, levels)
    sums = strassen_hip.prepare_weight(w, levels)
    assert sums is not None
    got = strassen_hip.linear_forward_any(x, w, b, levels, sums)
    assert torch.equal(got, want)
    again = strassen_hip.linear_forward_any(x, w, b, levels, sums)   # the sums are read, never written
    assert torch.equal(again, want)
    other = strassen_hip.prepare_weight(w.flip(0).contiguous(), levels)
    assert not torch.equal(strassen_hip.linear_forward_any(x, w, b, levels, other), want)
    # every level rounds its sums to the operand type, so the error about doubles per level
    ref = x.double() @ w.double().t() + (b.double() if bias else 0)
    assert float(torch.linalg.norm(got.double() - ref) / torch.linalg.norm(ref)) <= 2e-2 * 2 ** max(0, levels - 2)


def test_prepared_weight_sums_where_none_are_kept():
    import strassen_hip
    assert strassen_hip.prepare_weight(torch.zeros(1024, 1024, device="cuda"), 1) is None                          # fp32
    assert strassen_hip.prepare_weight(torch.zeros(1024, 1024, device="cuda", dtype=torch.bfloat16), 5) is None    # depth
    assert strassen_hip.prepare_weight(torch.zeros(1000, 1000, device="cuda", dtype=torch.bfloat16), 1) is None    # shape
    # too few rows for the grouped form: the sums are ignored, the result is the plain forward's
    g = torch.Generator().manual_seed(5)
    x = torch.randn(24, 1024, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(1024, 1024, generator=g) / 32).to(torch.bfloat16).cuda()
    sums = strassen_hip.prepare_weight(w, 1)
    assert torch.equal(strassen_hip.linear_forward_any(x, w, None, 1, sums), strassen_hip.linear_forward_any(x, w, None, 1))


@pytest.mark.parametrize("depth", [1, 2, 3])
def test_layers_keep_weight_sums_between_calls(depth):
    """LinearStrassen and LinearStrassenRect with cache_weight_sums: same bits as without, the
    sums are formed once per weight version and again after the weight is written."""
    import strassen_hip
    from model.layers import LinearStrassen, LinearStrassenRect
    g = torch.Generator().manual_seed(8 + depth)
    for make, rows, d_in, d_out in ((LinearStrassen, 2048, 2048, 2048), (LinearStrassenRect, 1024, 1024, 3072)):
        kw = {"cutoff": False} if make is LinearStrassenRect else {}
        plain = make(d_in, d_out, bias=True, dtype=torch.bfloat16, depth=depth, device="cuda", **kw)
        keep = make(d_in, d_out, bias=True, dtype=torch.bfloat16, depth=depth, device="cuda", cache_weight_sums=True, **kw)
        with torch.no_grad():
            plain.weight.copy_((torch.randn(d_out, d_in, generator=g) * d_in ** -0.5).to(torch.bfloat16))
            plain.bias.copy_(torch.randn(d_out, generator=g).to(torch.bfloat16))
            keep.weight.copy_(plain.weight)
            keep.bias.copy_(plain.bias)
        x = torch.randn(rows, d_in, generator=g).to(torch.bfloat16).cuda()
        with torch.no_grad():
            assert torch.equal(keep(x), plain(x))
            first = keep.weight_sums._sums
            assert first is not None
            assert torch.equal(keep(x), plain(x))
            assert keep.weight_sums._sums is first          # not formed again
            plain.weight.mul_(0.5)
            keep.weight.mul_(0.5)
            assert torch.equal(keep(x), plain(x))
            assert keep.weight_sums._sums is not first      # the write moved the version counter
            import copy
            twin = copy.deepcopy(keep)
            assert twin.weight_sums._sums is None and torch.equal(twin(x), plain(x))
            second = keep.weight_sums._sums
            keep.weight = torch.nn.Parameter(plain.weight.detach().clone())   # another tensor object, same values
            assert torch.equal(keep(x), plain(x)) and keep.weight_sums._sums is not second
        # training step through the caching layer: gradients as without the cache
        xg = x.clone().requires_grad_()
        xk = x.clone().requires_grad_()
        dy = torch.randn(rows, d_out, generator=g).to(torch.bfloat16).cuda()
        plain(xg).backward(dy)
        keep(xk).backward(dy)
        assert torch.equal(xg.grad, xk.grad) and torch.equal(plain.weight.grad, keep.weight.grad)
        assert torch.equal(plain.bias.grad, keep.bias.grad)
