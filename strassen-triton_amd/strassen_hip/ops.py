"""torch.Tensor front end of the C ABI.

PyTorch is used for device memory and streams only; all arithmetic happens in the HIP
kernels behind libstrassen_hip.so.  Tensors must live on the GPU: there is no CPU path.
"""
from __future__ import annotations

import ctypes
import weakref

import torch

from . import _capi

ALGO_CLASSIC, ALGO_STRASSEN, ALGO_WINOGRAD = 0, 1, 2
_ALGOS = {"classic": ALGO_CLASSIC, "strassen": ALGO_STRASSEN, "winograd": ALGO_WINOGRAD}
# OR-ed into the algo code (enum sthip_schedule): where 16-bit problems of two or more levels round below
# the first level.  "reference": only the first level's sums, everything deeper in fp32 as the reference's
# fp32-aggregating recursion does; "fast": every level, all products on the 16-bit matrix cores;
# "auto": fast at two levels, reference from three.
SCHEDULE_REFERENCE, SCHEDULE_FAST = 1 << 4, 2 << 4
_SCHEDULES = {"auto": 0, "reference": SCHEDULE_REFERENCE, "fast": SCHEDULE_FAST}


def _algo_code(algo, schedule: str = "auto") -> int:
    code = _ALGOS[algo] if isinstance(algo, str) else int(algo)
    try:
        return code | _SCHEDULES[schedule]
    except KeyError:
        raise ValueError(f"schedule must be one of {sorted(_SCHEDULES)}, got {schedule!r}") from None
_DTYPES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                "strassen_hip runs on MI355X tensors only (got a tensor on "
                f"{t.device}); there is no CPU implementation in this library")


def _dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}; use float32, float16 or bfloat16") from None


def _unit_stride(t: torch.Tensor) -> torch.Tensor:
    """The kernels read any matrix with a unit stride along rows or columns."""
    if t.stride(-1) == 1 or t.stride(-2) == 1:
        return t
    return t.contiguous()


def _strides3(t: torch.Tensor):
    if t.dim() == 2:
        s = (0, t.stride(0), t.stride(1))
    else:
        s = (t.stride(0) if t.shape[0] > 1 else 0, t.stride(1), t.stride(2))
    return (ctypes.c_int64 * 3)(*s)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _workspace(nbytes: int, device) -> tuple[torch.Tensor | None, int]:
    if nbytes == 0:
        return None, 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return ws, ws.data_ptr()


def workspace_bytes(A: torch.Tensor, B: torch.Tensor, *, algo="strassen", levels: int = 1,
                    out_dtype: torch.dtype | None = None, schedule: str = "auto") -> int:
    """Bytes of scratch gemm(A, B, ...) would allocate; pass a uint8 tensor of at least that size
    as `workspace=` to re-use one allocation across calls."""
    algo = _algo_code(algo, schedule)
    batch = A.shape[0] if A.dim() == 3 else 1
    dt = _dtype_code(A.dtype)
    return _capi.load().sthip_workspace_bytes(batch, A.shape[-2], B.shape[-1], A.shape[-1], dt,
                                              _dtype_code(out_dtype or A.dtype), algo, levels)


def auto_levels(M: int, N: int, K: int, dtype: torch.dtype, max_levels: int = 1) -> int:
    """Levels (0 = classical, at most max_levels) the library's measured cutoff picks for an
    M x K by K x N product (sthip_auto_levels)."""
    return _capi.load().sthip_auto_levels(M, N, K, _dtype_code(dtype), max_levels)


def gemm(A: torch.Tensor, B: torch.Tensor, out: torch.Tensor | None = None, *, algo="strassen",
         levels: int = 1, accumulate: bool = False, out_dtype: torch.dtype | None = None,
         workspace: torch.Tensor | None = None, schedule: str = "auto") -> torch.Tensor:
    """out (+)= A @ B through sthip_gemm.  A: (b,) M x K, B: (b,) K x N, same dtype.
    levels < 0: at most -levels levels, as many as the measured cutoff picks for the shape.
    schedule: "auto", "reference" or "fast" (see SCHEDULE_REFERENCE above)."""
    _require_gpu(A, B)
    lib = _capi.load()
    algo = _algo_code(algo, schedule)
    if levels < 0:
        levels = auto_levels(A.shape[-2], B.shape[-1], A.shape[-1], A.dtype, -levels)
        if levels == 0:
            algo = ALGO_CLASSIC
    if A.dim() != B.dim() or A.dim() not in (2, 3):
        raise ValueError(f"expected two 2-D or two 3-D tensors, got {tuple(A.shape)} and {tuple(B.shape)}")
    if A.dtype != B.dtype:
        raise TypeError(f"operand dtypes differ: {A.dtype} vs {B.dtype}")
    if A.shape[-1] != B.shape[-2] or (A.dim() == 3 and A.shape[0] != B.shape[0]):
        raise ValueError(f"shape mismatch: {tuple(A.shape)} @ {tuple(B.shape)}")
    batch = A.shape[0] if A.dim() == 3 else 1
    M, K, N = A.shape[-2], A.shape[-1], B.shape[-1]
    in_dt = _dtype_code(A.dtype)
    if out is None:
        if accumulate:
            raise ValueError("accumulate=True needs an `out` tensor")
        out = torch.empty(A.shape[:-1] + (N,), dtype=out_dtype or A.dtype, device=A.device)
    else:
        _require_gpu(out)
        if tuple(out.shape) != tuple(A.shape[:-1]) + (N,):
            raise ValueError(f"out has shape {tuple(out.shape)}, expected {tuple(A.shape[:-1]) + (N,)}")
    out_dt = _dtype_code(out.dtype)
    A, B = _unit_stride(A), _unit_stride(B)
    nbytes = lib.sthip_workspace_bytes(batch, M, N, K, in_dt, out_dt, algo, levels)
    if workspace is not None and nbytes > 0:
        if not workspace.is_cuda or workspace.dtype != torch.uint8 or workspace.numel() < nbytes:
            raise ValueError(f"workspace must be a uint8 GPU tensor of at least {nbytes} bytes")
        ws, ws_ptr = workspace, workspace.data_ptr()
    else:
        ws, ws_ptr = _workspace(nbytes, A.device)
    with torch.cuda.device(A.device):
        _capi.check(lib.sthip_gemm(A.data_ptr(), B.data_ptr(), out.data_ptr(), batch, M, N, K,
                                   _strides3(A), _strides3(B), _strides3(out), in_dt, out_dt, algo, levels,
                                   1 if accumulate else 0, ws_ptr, nbytes, _stream()))
    return out


class StrassenMatmul(torch.autograd.Function):
    """A @ B with gradients that are Strassen products themselves:
    dA = dC @ B^T and dB = A^T @ dC read the saved operands through transposed views."""

    @staticmethod
    def forward(ctx, A, B, algo, levels, schedule="auto"):
        ctx.save_for_backward(A, B)
        ctx.algo, ctx.levels, ctx.schedule = algo, levels, schedule
        return gemm(A, B, algo=algo, levels=levels, schedule=schedule)

    @staticmethod
    def backward(ctx, dC):
        A, B = ctx.saved_tensors
        dC = dC.contiguous()
        kw = dict(algo=ctx.algo, levels=ctx.levels, schedule=ctx.schedule)
        dA = gemm(dC, B.transpose(-1, -2), **kw) if ctx.needs_input_grad[0] else None
        dB = gemm(A.transpose(-1, -2), dC, **kw) if ctx.needs_input_grad[1] else None
        return dA, dB, None, None, None


def matmul(A: torch.Tensor, B: torch.Tensor, algo="strassen", levels: int = 1, schedule: str = "auto") -> torch.Tensor:
    """Differentiable A @ B."""
    if torch.is_grad_enabled() and (A.requires_grad or B.requires_grad):
        return StrassenMatmul.apply(A, B, algo, levels, schedule)
    return gemm(A, B, algo=algo, levels=levels, schedule=schedule)


def run_accumulate(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, *, algo="strassen", levels: int = 1,
                   operand_dtype: torch.dtype | None = torch.float16) -> None:
    """C += A @ B in place (sthip_run_accumulate).  Operands are cast to operand_dtype first
    when given, as the reference's Triton kernels cast every tile they load."""
    _require_gpu(A, B, C)
    lib = _capi.load()
    algo = _ALGOS[algo] if isinstance(algo, str) else int(algo)
    if operand_dtype is not None:
        A, B = A.to(operand_dtype), B.to(operand_dtype)
    A, B = A.contiguous(), B.contiguous()
    batch = A.shape[0] if A.dim() == 3 else 1
    M, K, N = A.shape[-2], A.shape[-1], B.shape[-1]
    op_dt = _dtype_code(A.dtype)
    target = C
    if not C.is_contiguous() or (C.dtype != A.dtype and C.dtype != torch.float32):
        target = C.to(torch.float32).contiguous()
    c_dt = _dtype_code(target.dtype)
    nbytes = lib.sthip_workspace_bytes(batch, M, N, K, op_dt, c_dt, algo, levels)
    ws, ws_ptr = _workspace(nbytes, A.device)
    with torch.cuda.device(A.device):
        _capi.check(lib.sthip_run_accumulate(A.data_ptr(), B.data_ptr(), target.data_ptr(), batch, M, N, K,
                                             op_dt, c_dt, algo, levels, ws_ptr, nbytes, _stream()))
    if target is not C:
        C.copy_(target)


def linear_forward(x2d: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, levels: int) -> torch.Tensor:
    """y = x2d @ weight.T (+ bias) for a square weight (sthip_linear_strassen_forward)."""
    _require_gpu(x2d, weight)
    lib = _capi.load()
    rows, D = x2d.shape
    x2d, weight = x2d.contiguous(), weight.contiguous()
    dt = _dtype_code(x2d.dtype)
    y = torch.empty((rows, D), dtype=x2d.dtype, device=x2d.device)
    nbytes = lib.sthip_workspace_bytes(1, D, D, D, dt, dt, ALGO_STRASSEN | SCHEDULE_FAST, levels)
    ws, ws_ptr = _workspace(nbytes, x2d.device)
    b_ptr = bias.contiguous().data_ptr() if bias is not None else 0
    with torch.cuda.device(x2d.device):
        _capi.check(lib.sthip_linear_strassen_forward(x2d.data_ptr(), weight.data_ptr(), b_ptr, y.data_ptr(),
                                                      rows, D, dt, levels, ws_ptr, nbytes, _stream()))
    return y


def linear_forward_any(x2d: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, levels: int,
                       weight_sums: torch.Tensor | None = None) -> torch.Tensor:
    """y = x2d @ weight.T (+ bias) for a weight of any shape (sthip_linear_forward): no padding,
    the bias is added inside the recombination pass where the call takes the grouped path.
    weight_sums: the buffer prepare_weight made for this weight and these levels; the call then
    forms the input-side sums only (sthip_linear_forward_prepared), with the same bits."""
    _require_gpu(x2d, weight)
    lib = _capi.load()
    rows, d_in = x2d.shape
    d_out = weight.shape[0]
    if weight.shape[1] != d_in:
        raise ValueError(f"shape mismatch: {tuple(x2d.shape)} @ {tuple(weight.shape)}^T")
    x2d, weight = x2d.contiguous(), weight.contiguous()
    dt = _dtype_code(x2d.dtype)
    if levels < 0:
        levels = lib.sthip_auto_levels(rows, d_out, d_in, dt, -levels)
    y = torch.empty((rows, d_out), dtype=x2d.dtype, device=x2d.device)
    nbytes = lib.sthip_workspace_bytes(1, rows, d_out, d_in, dt, dt, ALGO_STRASSEN | SCHEDULE_FAST, levels)
    ws, ws_ptr = _workspace(nbytes, x2d.device)
    b_ptr = bias.contiguous().data_ptr() if bias is not None else 0
    with torch.cuda.device(x2d.device):
        if weight_sums is not None and levels > 0:
            _capi.check(lib.sthip_linear_forward_prepared(x2d.data_ptr(), weight.data_ptr(), weight_sums.data_ptr(),
                                                          weight_sums.numel(), b_ptr, y.data_ptr(),
                                                          rows, d_in, d_out, dt, levels, ws_ptr, nbytes, _stream()))
        else:
            _capi.check(lib.sthip_linear_forward(x2d.data_ptr(), weight.data_ptr(), b_ptr, y.data_ptr(),
                                                 rows, d_in, d_out, dt, levels, ws_ptr, nbytes, _stream()))
    return y


def prepare_weight(weight: torch.Tensor, levels: int) -> torch.Tensor | None:
    """The quadrant sums of weight^T for `levels` Strassen levels as an opaque device buffer
    (sthip_linear_prepare_weight), or None where the library keeps none for this shape and type.
    Valid until the weight's contents change."""
    _require_gpu(weight)
    lib = _capi.load()
    if weight.dim() != 2 or not weight.is_contiguous():
        return None
    d_out, d_in = weight.shape
    if weight.dtype not in (torch.bfloat16, torch.float16):
        return None
    dt = _dtype_code(weight.dtype)
    nbytes = lib.sthip_linear_weight_sums_bytes(d_in, d_out, dt, levels)
    if nbytes == 0:
        return None
    sums = torch.empty(nbytes, dtype=torch.uint8, device=weight.device)
    with torch.cuda.device(weight.device):
        _capi.check(lib.sthip_linear_prepare_weight(weight.data_ptr(), d_in, d_out, dt, levels,
                                                    sums.data_ptr(), nbytes, _stream()))
    return sums


class WeightSums:
    """Keeps the prepared sums of one weight tensor and forms them again when the tensor is
    written (its version counter moves), replaced, or asked for at another depth.  A write through
    `.data` does not move the counter: call clear() (or refresh()) after one."""

    def __init__(self) -> None:
        self.clear()

    def get(self, weight: torch.Tensor, levels: int) -> torch.Tensor | None:
        try:
            version = weight._version
        except RuntimeError:
            # inference tensors (created under torch.inference_mode) track no version: nothing to key
            # the kept sums on, so form them for this call only
            self.clear()
            return prepare_weight(weight, levels)
        key = (weight.data_ptr(), version, tuple(weight.shape), weight.dtype, levels)
        same_tensor = self._owner is not None and self._owner() is weight
        if not same_tensor or key != self._key:
            self._sums = prepare_weight(weight, levels)
            self._key, self._owner = key, weakref.ref(weight)
        return self._sums

    def clear(self) -> None:
        self._key, self._sums, self._owner = None, None, None

    refresh = clear

    # a copied or unpickled layer starts without sums and forms its own on first use
    def __getstate__(self):
        return {}

    def __setstate__(self, state) -> None:
        self.clear()

    def __deepcopy__(self, memo):
        return WeightSums()
