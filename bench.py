"""Benchmark of the Strassen hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one C = A @ B through the fused one-level Strassen kernel (the C-ABI call, inputs
resident in HBM).  The default workload is the one BASELINE.json's metric is quoted on:
M = N = K = 8192, bf16 in / bf16 out, fp32 accumulation and aggregation.  Prints ONE JSON
line: effective TFLOP/s (2MNK / t, the classical flop count, as the reference's
main_profiling.py:190,216-217 does), the ratio to a hipBLASLt classical GEMM of the same
shape timed the same way, the MFMA roofline fraction of the Strassen kernel, and the CPU
oracle timed on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

os.environ.setdefault("TORCH_BLAS_PREFER_HIPBLASLT", "1")   # as the reference does on AMD (main_profiling.py:25-28)

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "strassen-triton_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}   # MI355X dense MFMA, vendor figures

WORKLOADS = {
    # name: (batch, M, N, K, dtype, algo, levels, input scale rule)
    "strassen1_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "strassen", 1),
    "strassen2_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "strassen", 2),
    "classic_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "classic", 0),
    "winograd1_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "winograd", 1),
    "strassen1_4096_f16": (1, 4096, 4096, 4096, torch.float16, "strassen", 1),
    "strassen1_1024_f32": (1, 1024, 1024, 1024, torch.float32, "strassen", 1),
    "winograd_b8_4096x8192x4096_bf16": (8, 4096, 4096, 8192, torch.bfloat16, "winograd", 1),
    "strassen1_16384_bf16": (1, 16384, 16384, 16384, torch.bfloat16, "strassen", 1),
}
DT_NAME = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}


def make_inputs(batch, M, N, K, dtype):
    """Seeded inputs, generated on the CPU so the oracle and the GPU see the same bits."""
    gA, gB = torch.Generator().manual_seed(1234), torch.Generator().manual_seed(1235)
    shape_a = (M, K) if batch == 1 else (batch, M, K)
    shape_b = (K, N) if batch == 1 else (batch, K, N)
    scale = 1.0 if dtype == torch.float32 else K ** -0.5
    A = (torch.randn(shape_a, generator=gA) * scale).to(dtype)
    B = (torch.randn(shape_b, generator=gB) * scale).to(dtype)
    return A, B


def time_gpu(fn, steps, warmup):
    """W untimed calls, then exactly K calls between two synchronisations; also HIP events on
    the stream the kernels run on, for the per-launch duration."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, start.elapsed_time(stop) * 1e-3


def cpu_baseline(A, B, levels, dtype, algo):
    """The oracle (a restatement of the reference's torch recursion) on the host cores."""
    from oracle import strassen_oracle as O
    cores = os.cpu_count() or 1
    cores = min(cores, 16) if os.environ.get("GRAFT_REPO_ROOT") else cores
    torch.set_num_threads(cores)
    if A.dim() == 3:
        A, B = A[0], B[0]
    M, K = A.shape
    N = B.shape[1]
    # torch's CPU GEMM for bf16/fp16 is fast only with AMX / AVX512-FP16; probe it and fall back
    # to the same recursion with fp32-upcast leaf products (sgemm) where it is not
    leaf, leaf_name = torch.mm, "native " + DT_NAME[dtype] + " leaf products"
    if dtype != torch.float32:
        P = torch.ones(1024, 1024, dtype=dtype)
        t0 = time.perf_counter()
        torch.mm(P, P)
        if time.perf_counter() - t0 > 0.25:     # < ~8 GFLOP/s
            leaf, leaf_name = O.mm_fp32_upcast, "fp32-upcast leaf products (native 16-bit CPU GEMM too slow here)"
    if algo == "winograd":
        f = lambda: O.winograd_base(A, B, dtype, fp32_agg=True, mm=leaf)
    elif algo == "classic":
        f = lambda: leaf(A, B)
    else:
        f = lambda: O.strassen_matmul_n_layers(A, B, levels, dtype, fp32_agg=True, mm=leaf)
    f()
    best = float("inf")
    spent = 0.0
    for _ in range(3):
        t0 = time.perf_counter()
        f()
        dt = time.perf_counter() - t0
        best, spent = min(best, dt), spent + dt
        if spent > 25.0:
            break
    return {"value": round(2.0 * M * N * K / best / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"one {M}x{N}x{K} {DT_NAME[dtype]} product through the CPU oracle "
                      f"({algo}, {levels} level(s), fp32 aggregation, {leaf_name}), best of 3 after 1 warm-up; "
                      f"best {best * 1e3:.1f} ms"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="strassen1_8192_bf16", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library runs on one GPU (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import strassen_hip
    from strassen_hip import _capi
    _capi.load()

    batch, M, N, K, dtype, algo, levels = WORKLOADS[args.workload]
    A, B = make_inputs(batch, M, N, K, dtype)
    Ag, Bg = A.cuda(), B.cuda()
    out = torch.empty(Ag.shape[:-1] + (N,), dtype=dtype, device="cuda")
    flops = 2.0 * batch * M * N * K

    fn = lambda: strassen_hip.gemm(Ag, Bg, out=out, algo=algo, levels=levels)
    wall, ev = time_gpu(fn, args.steps, args.warmup)
    tflops = flops * args.steps / wall / 1e12
    per_launch = ev / args.steps

    ref_out = torch.empty_like(out)
    wall_b, ev_b = time_gpu(lambda: torch.matmul(Ag, Bg, out=ref_out), args.steps, args.warmup)
    blas_tflops = flops * args.steps / wall_b / 1e12

    # numerical error of the timed result against fp64 and against hipBLASLt's result
    exact = torch.matmul(Ag[0].double() if batch > 1 else Ag.double(), Bg[0].double() if batch > 1 else Bg.double())
    mine = (out[0] if batch > 1 else out).double()
    err64 = float(torch.linalg.norm(mine - exact) / torch.linalg.norm(exact))
    err_blas = float(torch.linalg.norm((ref_out[0] if batch > 1 else ref_out).double() - exact) / torch.linalg.norm(exact))
    del exact, mine

    peak = PEAK_TFLOPS[DT_NAME[dtype]]
    achieved = flops / per_launch / 1e12
    result = {
        "metric": "effective TFLOP/s (2MNK/t) at 8192^2 bf16; ratio vs hipBLASLt GEMM",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": DT_NAME[dtype], "data": "synthetic",
        "config": {"workload": args.workload, "batch": batch, "M": M, "N": N, "K": K, "algo": algo, "levels": levels,
                   "accumulate": "fp32", "aggregate": "fp32", "out_dtype": DT_NAME[dtype]},
        "hipblaslt_tflops": round(blas_tflops, 2), "ratio_vs_hipblaslt": round(tflops / blas_tflops, 4),
        "hipblaslt_ms": round(wall_b / args.steps * 1e3, 4),
        "rel_fro_err_vs_fp64": err64, "hipblaslt_rel_fro_err_vs_fp64": err_blas,
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4), "traffic": None,
                     "kernel_ms": round(per_launch * 1e3, 4),
                     "executed_mfma_tflops": round(achieved * (7.0 / 8.0) ** (levels if algo != "classic" else 0), 2)},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(A, B, max(levels, 1), dtype, algo)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
