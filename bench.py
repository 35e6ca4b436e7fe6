"""Benchmark of the Strassen hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

A step is one C = A @ B through the library's C ABI with the inputs resident in HBM.  The
default workload is the one BASELINE.json's metric is quoted on: one-level Strassen,
M = N = K = 8192, bf16 in / bf16 out, fp32 accumulation and aggregation.  Prints ONE JSON
line:

  value / ms_per_step   effective TFLOP/s = 2MNK / t (the classical flop count, as the
                        reference's main_profiling.py:190,216-217 counts it) over exactly K
                        back-to-back steps between two synchronisations
  step_ms               min / median / mean over K further steps timed one by one with HIP events
  flushed_ms            median over steps that each follow a write of a 512 MiB buffer (larger than
                        the 256 MiB memory-side cache), the protocol of the reference's do_bench
                        (main_profiling.py:197); flushed_ratio_vs_hipblaslt is the same for both sides
  hipblaslt_*           torch.matmul (hipBLASLt) on the same tensors, same protocols, and the ratios
  roofline              the dominant kernel (the grouped-GEMM launch) timed alone with HIP events
                        on the stream it runs on, against the MI355X dense MFMA peak.  frac divides
                        the classical flop count of the call by that kernel's time (the convention
                        of the metric); frac_executed counts only the matrix work the kernel
                        executes (7/8 per level); frac_whole_call divides by the whole call's time.
                        traffic is not measured in this run: traffic_source names the committed
                        rocprofv3 counter summary it is read from.
  cpu_baseline          the CPU oracle (a restatement of the reference's torch recursion) on the
                        host cores, best of 3

The clocks of the card ramp for the first 20-30 ms of matrix work in a fresh process (both this
library and hipBLASLt run 10-15 % slower there), so the default warm-up is 50 steps.

`--workload copy_1gib` runs a plain 1 GiB device copy instead; it exists to calibrate the
FETCH_SIZE / WRITE_SIZE counters when the HBM traffic of the kernels is measured with rocprofv3.
"""
from __future__ import annotations

import argparse
import json
import os
import re
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
    # name: (batch, M, N, K, dtype, algo, levels)
    "strassen1_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "strassen", 1),
    "strassen2_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "strassen", 2),
    "classic_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "classic", 0),
    "winograd1_8192_bf16": (1, 8192, 8192, 8192, torch.bfloat16, "winograd", 1),
    "strassen1_4096_f16": (1, 4096, 4096, 4096, torch.float16, "strassen", 1),
    "strassen1_1024_f32": (1, 1024, 1024, 1024, torch.float32, "strassen", 1),
    "winograd_b8_4096x8192x4096_bf16": (8, 4096, 4096, 8192, torch.bfloat16, "winograd", 1),
    "strassen1_16384_bf16": (1, 16384, 16384, 16384, torch.bfloat16, "strassen", 1),
    "strassen1_8192_f32": (1, 8192, 8192, 8192, torch.float32, "strassen", 1),
    "strassen2_16384_f32": (1, 16384, 16384, 16384, torch.float32, "strassen", 2),
    "classic_8192_f32": (1, 8192, 8192, 8192, torch.float32, "classic", 0),
    "copy_1gib": None,
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
    """W untimed calls, then exactly K calls between two synchronisations.  Returns the wall
    time and the HIP-event time of the K calls (events recorded on the stream fn launches on)."""
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


def time_steps(fn, steps, flush=None):
    """Every step timed on its own with a pair of HIP events; with `flush`, a write of that buffer
    (larger than the memory-side cache) goes before every step, outside its timed region."""
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in events:
        if flush is not None:
            flush.zero_()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in events)
    return {"min": round(t[0], 4), "median": round(t[len(t) // 2], 4), "mean": round(sum(t) / len(t), 4)}


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


def measured_traffic(workload):
    """HBM bytes per launch of the dominant kernel, as measured with rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE and recorded in profiles/ (None if no such summary is committed)."""
    rel = os.path.join("profiles", f"gemm4p_kernel_{workload}_hbm_traffic.txt")
    try:
        m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", open(os.path.join(ROOT, rel)).read(), re.M)
        return (float(m.group(1)), rel) if m else (None, None)
    except OSError:
        return None, None


def copy_calibration(steps):
    """A plain device copy of known size: 1 GiB read + 1 GiB written per step."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    wall, ev = time_gpu(lambda: dst.copy_(src), steps, 2)
    print(json.dumps({"workload": "copy_1gib", "bytes_read_per_step": n, "bytes_written_per_step": n,
                      "steps": steps, "ms_per_step": round(ev / steps * 1e3, 4),
                      "GBps": round(2 * n * steps / ev / 1e9, 1)}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="strassen1_8192_bf16", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--force-tile", default=None, choices=["128x128", "128x128g", "256x128", "256x256", "64x64"],
                    help="override the library's tile table (STHIP_FORCE_TILE): 256x128 and 128x128 are the "
                         "kernels that recombine in registers, 128x128g / 256x256 the grouped paths")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library runs on one GPU (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.force_tile:
        os.environ["STHIP_FORCE_TILE"] = args.force_tile
    if args.workload == "copy_1gib":
        copy_calibration(args.steps)
        return
    import strassen_hip
    from strassen_hip import _capi
    lib = _capi.load()

    batch, M, N, K, dtype, algo, levels = WORKLOADS[args.workload]
    A, B = make_inputs(batch, M, N, K, dtype)
    Ag, Bg = A.cuda(), B.cuda()
    out = torch.empty(Ag.shape[:-1] + (N,), dtype=dtype, device="cuda")
    flops = 2.0 * batch * M * N * K
    nbytes = strassen_hip.workspace_bytes(Ag, Bg, algo=algo, levels=levels)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device="cuda")

    fn = lambda: strassen_hip.gemm(Ag, Bg, out=out, algo=algo, levels=levels, workspace=ws)
    wall, ev = time_gpu(fn, args.steps, args.warmup)
    tflops = flops * args.steps / wall / 1e12

    # the dominant kernel alone: with the pre-pass switched off the grouped GEMM re-uses the
    # quadrant sums the calls above left in the workspace
    kernel_s, prepass_s, recombine_s = ev / args.steps, 0.0, 0.0
    staged = levels in (1, 2) and algo != "classic" and nbytes > 0 and (levels == 1 or dtype != torch.float32)
    if staged:
        all_stages = lib.sthip_debug_set_stages(0)
        lib.sthip_debug_set_stages((all_stages & ~7) | 2)   # one stage at a time, the other switches as they were
        _, ev_k = time_gpu(fn, args.steps, 3)
        lib.sthip_debug_set_stages((all_stages & ~7) | 1)
        _, ev_p = time_gpu(fn, args.steps, 3)
        lib.sthip_debug_set_stages((all_stages & ~7) | 4)
        _, ev_r = time_gpu(fn, args.steps, 3)
        lib.sthip_debug_set_stages(all_stages)
        kernel_s, prepass_s, recombine_s = ev_k / args.steps, ev_p / args.steps, ev_r / args.steps
        fn()   # leave `out` holding a complete result for the error figures below

    ref_out = torch.empty_like(out)
    blas = lambda: torch.matmul(Ag, Bg, out=ref_out)
    wall_b, ev_b = time_gpu(blas, args.steps, args.warmup)
    blas_tflops = flops * args.steps / wall_b / 1e12

    # step by step, back to back and with the caches flushed before every step
    stat_steps = min(args.steps, 100)
    step_ms, blas_step_ms = time_steps(fn, stat_steps), time_steps(blas, stat_steps)
    flush = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    flushed, blas_flushed = time_steps(fn, stat_steps, flush), time_steps(blas, stat_steps, flush)
    del flush

    # numerical error of the timed result against fp64 and against hipBLASLt's result
    exact = torch.matmul(Ag[0].double() if batch > 1 else Ag.double(), Bg[0].double() if batch > 1 else Bg.double())
    mine = (out[0] if batch > 1 else out).double()
    err64 = float(torch.linalg.norm(mine - exact) / torch.linalg.norm(exact))
    err_blas = float(torch.linalg.norm((ref_out[0] if batch > 1 else ref_out).double() - exact) / torch.linalg.norm(exact))
    del exact, mine

    peak = PEAK_TFLOPS[DT_NAME[dtype]]
    achieved = flops / kernel_s / 1e12
    executed = (7.0 / 8.0) ** (levels if algo != "classic" else 0)
    traffic, traffic_source = measured_traffic(args.workload)
    metric = "effective TFLOP/s (2MNK/t) at 8192\u00b2 bf16; ratio vs hipBLASLt GEMM"
    if args.workload != "strassen1_8192_bf16":
        metric = f"effective TFLOP/s (2MNK/t) on {args.workload}; ratio vs hipBLASLt GEMM"
    result = {
        "metric": metric,
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": DT_NAME[dtype], "data": "synthetic",
        "config": {"workload": args.workload, "batch": batch, "M": M, "N": N, "K": K, "algo": algo, "levels": levels,
                   "accumulate": "fp32", "aggregate": "fp32", "out_dtype": DT_NAME[dtype],
                   "workspace_bytes": nbytes, "force_tile": args.force_tile},
        "hipblaslt_tflops": round(blas_tflops, 2), "ratio_vs_hipblaslt": round(tflops / blas_tflops, 4),
        "hipblaslt_ms": round(wall_b / args.steps * 1e3, 4),
        "step_ms": step_ms, "hipblaslt_step_ms": blas_step_ms,
        "flushed_ms": flushed["median"], "hipblaslt_flushed_ms": blas_flushed["median"],
        "flushed_ratio_vs_hipblaslt": round(blas_flushed["median"] / flushed["median"], 4),
        "mfma_peak_frac": round(tflops / peak, 4),
        "rel_fro_err_vs_fp64": err64, "hipblaslt_rel_fro_err_vs_fp64": err_blas,
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4),
                     "frac_executed": round(achieved * executed / peak, 4),
                     "frac_whole_call": round(tflops / peak, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "grouped GEMM launch of the call (stage mask 2)" if staged else "whole call",
                     "kernel_ms": round(kernel_s * 1e3, 4), "prepass_ms": round(prepass_s * 1e3, 4),
                     "recombine_ms": round(recombine_s * 1e3, 4),
                     "flops_per_launch": flops, "executed_mfma_tflops": round(achieved * executed, 2)},
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(A, B, max(levels, 1), dtype, algo)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
