"""sthip_gemm_static: the entry point that allocates nothing.  Its workspace is a buffer inside
the library's device image, so a caller under graph capture or in a serving loop needs no
hipMalloc.  Checked through the C ABI against sthip_gemm (caller-provided workspace) on two calls
in a row, the second with a smaller input: same kernels, so the results must be bit-identical.
The file name makes pytest collect it last: a failure here must not hide the other GPU tests."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_BYTES = 144 << 20
_DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _s3(t):
    return (ctypes.c_int64 * 3)(0, t.stride(0), t.stride(1))


def _inputs(M, N, K, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    scale = 1.0 if dtype == torch.float32 else K ** -0.5
    A = (torch.randn(M, K, generator=g) * scale).to(dtype).cuda()
    B = (torch.randn(K, N, generator=g) * scale).to(dtype).cuda()
    return A, B


def _both(lib, A, B, algo, levels):
    """(result of sthip_gemm_static, result of sthip_gemm with a workspace of the queried size, that size)"""
    from strassen_hip import _capi
    M, K = A.shape
    N = B.shape[1]
    dt = _DT[A.dtype]
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.sthip_workspace_bytes(1, M, N, K, dt, dt, algo, levels)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    want = torch.full((M, N), float("nan"), dtype=A.dtype, device="cuda")
    _capi.check(lib.sthip_gemm(A.data_ptr(), B.data_ptr(), want.data_ptr(), 1, M, N, K, _s3(A), _s3(B), _s3(want),
                               dt, dt, algo, levels, 0, ws.data_ptr(), need, stream))
    got = torch.full((M, N), float("nan"), dtype=A.dtype, device="cuda")
    _capi.check(lib.sthip_gemm_static(A.data_ptr(), B.data_ptr(), got.data_ptr(), 1, M, N, K, _s3(A), _s3(B), _s3(got),
                                      dt, dt, algo, levels, 0, stream))
    torch.cuda.synchronize()
    return got, want, need


def test_static_scratch_matches_workspace_entry_on_two_calls_in_a_row():
    from strassen_hip import _capi
    lib = _capi.load()
    # first call: one level at 2048^3 bf16 (sums + grouped products + recombination, 34 MiB of scratch)
    A, B = _inputs(2048, 2048, 2048, torch.bfloat16, 11)
    got, want, need = _both(lib, A, B, 1, 1)
    assert 0 < need <= STATIC_BYTES
    assert torch.equal(got, want)
    exact = A.double() @ B.double()
    assert float(torch.linalg.norm(got.double() - exact) / torch.linalg.norm(exact)) <= 2e-2
    # second call, smaller input, two levels: the buffer still holds the first call's sums and products
    A2, B2 = _inputs(1024, 768, 512, torch.bfloat16, 12)
    got2, want2, need2 = _both(lib, A2, B2, 1, 2)
    assert 0 < need2 < need
    assert torch.equal(got2, want2)
    exact2 = A2.double() @ B2.double()
    assert float(torch.linalg.norm(got2.double() - exact2) / torch.linalg.norm(exact2)) <= 2e-2
    # and the first problem again: nothing the second call left behind leaks into it
    got3, _, _ = _both(lib, A, B, 1, 1)
    assert torch.equal(got3, want)


def test_static_scratch_fp32_and_winograd():
    from strassen_hip import _capi
    lib = _capi.load()
    A, B = _inputs(1024, 1024, 1024, torch.float32, 13)
    got, want, need = _both(lib, A, B, 1, 1)
    assert need > 0 and torch.equal(got, want)
    A, B = _inputs(1024, 1024, 2048, torch.float16, 14)
    got, want, need = _both(lib, A, B, 2, 1)
    assert need > 0 and torch.equal(got, want)
    # a shape that needs no workspace (odd sizes take the fused kernel) never touches the buffer
    A, B = _inputs(250, 130, 70, torch.bfloat16, 15)
    got, want, need = _both(lib, A, B, 1, 1)
    assert need == 0 and torch.equal(got, want)


def test_static_scratch_allocates_nothing_and_refuses_what_does_not_fit():
    from strassen_hip import _capi
    lib = _capi.load()
    A, B = _inputs(2048, 2048, 2048, torch.bfloat16, 16)
    out = torch.empty(2048, 2048, dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    call = lambda: lib.sthip_gemm_static(A.data_ptr(), B.data_ptr(), out.data_ptr(), 1, 2048, 2048, 2048, _s3(A), _s3(B),
                                         _s3(out), 2, 2, 1, 1, 0, stream)
    assert call() == 0          # set-up (address look-up, kernel attributes) happens on the first call at the latest
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        assert call() == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"device memory in use changed by {free0 - free1} bytes across calls"
    # 8192^3 needs 544 MiB of workspace: refused with a message, nothing launched, `out` untouched
    big = (ctypes.c_int64 * 3)(0, 8192, 1)
    before = out.clone()
    one = ctypes.c_void_p(out.data_ptr())
    rc = lib.sthip_gemm_static(one, one, one, 1, 8192, 8192, 8192, big, big, big, 2, 2, 1, 1, 0, stream)
    assert rc == -4
    msg = lib.sthip_last_error().decode()
    assert "static scratch" in msg and str(lib.sthip_workspace_bytes(1, 8192, 8192, 8192, 2, 2, 1, 1)) in msg
    torch.cuda.synchronize()
    assert torch.equal(out, before)
