"""LinearStrassen against nn.Linear on square N x N problems: the benchmark table of the
reference's main_profiling.py (:94-308), measured on MI355X.

Protocol kept from the reference: an N x N input through a bias-free N -> N layer, both
layers sharing weights; every timed call ends in .clone() (:201, :216); the cache is
flushed between calls; TFLOP/s = 2 N^3 / fastest time for both layers ("useful work",
:220); speed-up = ratio of mean times (:233).  Differences: nn.Linear runs eagerly (it is
a hipBLASLt call either way), timing uses HIP events around each call on the current
stream, and the grid is limited by --max-n.

    python main_profiling.py [--dtype bf16|fp16|fp32] [--max-n 16384] [--min-n 1024]
    python main_profiling.py --gpt2      # the Linear shapes of GPT-2 small, forward and backward
    python main_profiling.py --cutoff    # classical kernel against 1 - 3 Strassen levels: the measurement behind sthip_auto_levels
    python main_profiling.py --json out.json   # also write the rows as JSON
    python main_profiling.py --cache-weight-sums   # LinearStrassen keeps the weight's quadrant sums between calls
"""
from __future__ import annotations

import argparse
import json

import torch
import torch.nn as nn

from fixed_strassen import LinearStrassen

_DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}

# (N, depth) grid of reference main_profiling.py:250-261.
_GRID = [(1024, 1), (1024, 2), (2048, 1), (2048, 2), (4096, 1), (4096, 2),
         (8192, 1), (8192, 2), (8192, 3), (16384, 1), (16384, 2), (16384, 3),
         (32768, 1), (32768, 2), (32768, 3), (32768, 4),
         # beyond the reference's grid: where more levels start to pay on this machine
         (65536, 1), (65536, 2), (65536, 3)]


def _runs_for(n: int) -> tuple[int, int]:
    """(warm-up, timed calls) per problem size (reference main_profiling.py:279-289; fewer for
    the sizes where one call takes tens of milliseconds or more)."""
    if n >= 32768:
        return 3, 10
    if n >= 4096:
        return 10, 50
    if n >= 1024:
        return 10, 350
    return 25, 100


def _bench(fn, warmup: int, runs: int, flush: torch.Tensor) -> list[float]:
    """Milliseconds of each of `runs` calls, each preceded by a write over `flush` so no
    call finds its operands in the last-level cache."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(runs):
        flush.zero_()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        stop.synchronize()
        times.append(start.elapsed_time(stop))
    return times


@torch.no_grad()
def benchmark_linear_layers(N_dim: int, strassen_depth: int, use_bias: bool = False,
                            dtype=torch.bfloat16, device: str = "cuda",
                            num_warmup: int = 10, num_runs: int = 50, flush=None,
                            cache_weight_sums: bool = False) -> dict:
    assert N_dim > 0 and (N_dim & (N_dim - 1)) == 0, "N_dim (features) must be a power of 2."
    res = {"N_dim": N_dim, "strassen_depth": strassen_depth, "bias": use_bias}
    x = torch.randn(N_dim, N_dim, device=device, dtype=dtype)
    std = nn.Linear(N_dim, N_dim, bias=use_bias, device=device, dtype=dtype).eval()
    ours = LinearStrassen(N_dim, N_dim, bias=use_bias, dtype=dtype, depth=strassen_depth, device=device,
                          cache_weight_sums=cache_weight_sums).eval()
    ours.weight.data.copy_(std.weight.data)   # before the first forward: writes through .data do not refresh kept sums
    if use_bias:
        ours.bias.data.copy_(std.bias.data)

    out_std, out_ours = std(x).clone(), ours(x).clone()
    res["max_abs_diff"] = (out_std.float() - out_ours.float()).abs().max().item()
    res["allclose"] = bool(torch.allclose(out_std, out_ours))
    del out_std, out_ours

    if flush is None:
        flush = torch.empty(512 << 20, dtype=torch.uint8, device=device)
    flops = 2 * N_dim ** 3 + (N_dim * N_dim if use_bias else 0)
    for key, layer in (("std", std), ("strassen", ours)):
        t = _bench(lambda: layer(x).clone(), num_warmup, num_runs, flush)
        res[f"{key}_mean_ms"] = sum(t) / len(t)
        res[f"{key}_min_ms"] = min(t)
        res[f"{key}_tflops"] = flops / (min(t) * 1e-3) / 1e12
    res["speedup_mean"] = res["std_mean_ms"] / res["strassen_mean_ms"]
    return res


HEADER = (f"{'N_dim':>7s} | {'Depth':>5s} | {'Std Mean(ms)':>14s} | {'Strassen Mean(ms)':>18s} | "
          f"{'Speedup':>9s} | {'Std TFLOPs':>12s} | {'Strassen TFLOPs':>17s} | "
          f"{'MaxAbsDiff':>12s} | {'Allclose':>8s}")


def format_row(r: dict) -> str:
    return (f"{r['N_dim']:>7} | {r['strassen_depth']:>5} | {r['std_mean_ms']:>14.4f} | "
            f"{r['strassen_mean_ms']:>18.4f} | {r['speedup_mean']:>8.2f}x | {r['std_tflops']:>12.2f} | "
            f"{r['strassen_tflops']:>17.2f} | {r['max_abs_diff']:>12.3e} | {str(r['allclose']):>8s}")


def profile_linear_layers(dtype=torch.bfloat16, min_n: int = 1024, max_n: int = 16384,
                          cache_weight_sums: bool = False) -> list[dict]:
    flush = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    rows = []
    print(HEADER)
    print("-" * len(HEADER))
    for n, depth in _GRID:
        if n < min_n or n > max_n:
            continue
        warmup, runs = _runs_for(n)
        r = benchmark_linear_layers(n, depth, dtype=dtype, num_warmup=warmup, num_runs=runs, flush=flush,
                                    cache_weight_sums=cache_weight_sums)
        rows.append(r)
        print(format_row(r), flush=True)
        torch.cuda.empty_cache()
    return rows


# (name, in_features, out_features) of the Linear layers of GPT-2 small.
_GPT2_LINEARS = [("qkv", 768, 2304), ("attn_proj", 768, 768), ("mlp_up", 768, 3072), ("mlp_down", 3072, 768)]


@torch.no_grad()
def profile_gpt2_linears(tokens: int = 8192, dtype=torch.bfloat16) -> list[dict]:
    """Forward x W^T, dgrad dY W and wgrad dY^T X of each GPT-2-small Linear for `tokens`
    rows on strided views: torch.matmul, one Strassen level, the library's classical kernel, and
    what the measured cutoff picks between the latter two (levels = -1, the default of
    LinearStrassenRect)."""
    import strassen_hip
    flush = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    rows = []
    print(f"{'layer':>10s} | {'pass':>5s} | {'M x N x K':>18s} | {'matmul ms':>10s} | {'strassen ms':>11s} | "
          f"{'classic ms':>10s} | {'cutoff ms':>9s} | {'levels':>6s} | {'matmul TF':>9s} | {'strassen TF':>11s} | {'rel err':>9s}")
    for name, d_in, d_out in _GPT2_LINEARS:
        x = torch.randn(tokens, d_in, device="cuda", dtype=dtype) * 0.02
        w = torch.randn(d_out, d_in, device="cuda", dtype=dtype) * 0.02
        dy = torch.randn(tokens, d_out, device="cuda", dtype=dtype) * 0.02
        for which, a, b in (("fwd", x, w.t()), ("dgrad", dy, w), ("wgrad", dy.t(), x)):
            M, K, N = a.shape[0], a.shape[1], b.shape[1]
            ws = torch.empty(max(1, strassen_hip.workspace_bytes(a, b)), dtype=torch.uint8, device="cuda")
            out = torch.empty(M, N, device="cuda", dtype=dtype)
            t_std = _bench(lambda: torch.matmul(a, b, out=out), 10, 50, flush)
            ref = out.double()
            t_str = _bench(lambda: strassen_hip.gemm(a, b, out, workspace=ws), 10, 50, flush)
            err = float(torch.linalg.norm(out.double() - ref) / torch.linalg.norm(ref))
            t_cls = _bench(lambda: strassen_hip.gemm(a, b, out, algo="classic", levels=0), 10, 50, flush)
            t_auto = _bench(lambda: strassen_hip.gemm(a, b, out, levels=-1, workspace=ws), 10, 50, flush)
            picked = strassen_hip.auto_levels(M, N, K, dtype, 1)
            tf = lambda t: 2.0 * M * N * K / (min(t) * 1e-3) / 1e12
            r = dict(layer=name, which=which, M=M, N=N, K=K, std_ms=min(t_std), strassen_ms=min(t_str),
                     classic_ms=min(t_cls), cutoff_ms=min(t_auto), cutoff_levels=picked,
                     std_tflops=tf(t_std), strassen_tflops=tf(t_str), rel_err=err)
            rows.append(r)
            print(f"{name:>10s} | {which:>5s} | {f'{M}x{N}x{K}':>18s} | {r['std_ms']:>10.4f} | {r['strassen_ms']:>11.4f} | "
                  f"{r['classic_ms']:>10.4f} | {r['cutoff_ms']:>9.4f} | {picked:>6d} | {r['std_tflops']:>9.1f} | "
                  f"{r['strassen_tflops']:>11.1f} | {err:>9.2e}", flush=True)
    return rows


# M x N x K of the cutoff table: the square sizes around which a level starts to pay, and some that are not square.
_CUTOFF_SHAPES = [(4096, 4096, 4096), (8192, 8192, 8192), (12288, 12288, 12288), (16384, 16384, 16384), (8192, 16384, 16384),
                  (16384, 8192, 16384), (20480, 20480, 20480), (24576, 24576, 24576), (32768, 32768, 32768)]


def _steady(fn, runs: int) -> float:
    """Milliseconds per call of `runs` calls back to back (the state of a training or serving loop: operands of the next call
    partly in the last-level cache, clocks settled), after a quarter as many warm-up calls."""
    for _ in range(max(3, runs // 4)):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(runs):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / runs


@torch.no_grad()
def profile_cutoff(dtype=torch.bfloat16, shapes=None, max_levels: int = 2, b_transposed: bool = False, runs=None) -> list[dict]:
    """The library's classical kernel against 1 .. max_levels Strassen levels on C = A B, beside torch.matmul and what
    strassen_hip.auto_levels picks for the shape: the table from which the rule of sthip_auto_levels is read (a level pays
    where its column is below the classical one).  The reference has no such cutoff; its replace_linear_with_strassen takes
    every layer of at least min_size features (model/layers.py:279-300)."""
    import strassen_hip
    rows = []
    print(f"{'M x N x K':>20s} | {'matmul ms':>9s} | {'classic ms':>10s} | " +
          " | ".join(f"{f'{l} level ms':>10s}" for l in range(1, max_levels + 1)) + f" | {'best':>4s} | {'rule':>4s}")
    for M, N, K in shapes or _CUTOFF_SHAPES:
        a = torch.randn(M, K, device="cuda", dtype=dtype) * K ** -0.5
        b = torch.randn(N, K, device="cuda", dtype=dtype).t() if b_transposed else torch.randn(K, N, device="cuda", dtype=dtype)
        out = torch.empty(M, N, device="cuda", dtype=dtype)
        n = runs or (30 if 2.0 * M * N * K <= 1e13 else 8)
        r = dict(M=M, N=N, K=K, b_transposed=b_transposed, std_ms=_steady(lambda: torch.matmul(a, b, out=out), n))
        r["level_ms"] = [_steady(lambda: strassen_hip.gemm(a, b, out, algo="classic", levels=0), n)]
        for levels in range(1, max_levels + 1):
            # "fast": every level on the 16-bit matrix cores (the default from three levels on runs its inner products in fp32)
            ws = torch.empty(max(1, strassen_hip.workspace_bytes(a, b, levels=levels, schedule="fast")), dtype=torch.uint8, device="cuda")
            r["level_ms"].append(_steady(lambda: strassen_hip.gemm(a, b, out, levels=levels, workspace=ws, schedule="fast"), n))
            del ws
        r["best_levels"] = min(range(max_levels + 1), key=lambda l: r["level_ms"][l])
        r["rule_levels"] = strassen_hip.auto_levels(M, N, K, dtype, max_levels)
        rows.append(r)
        print(f"{f'{M}x{N}x{K}':>20s} | {r['std_ms']:>9.4f} | " + " | ".join(f"{t:>10.4f}" for t in r["level_ms"]) +
              f" | {r['best_levels']:>4d} | {r['rule_levels']:>4d}", flush=True)
        del a, b, out
        torch.cuda.empty_cache()
    return rows


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--dtype", choices=sorted(_DTYPES), default="bf16")
    ap.add_argument("--min-n", type=int, default=1024)
    ap.add_argument("--max-n", type=int, default=16384)
    ap.add_argument("--gpt2", action="store_true", help="GPT-2-small Linear shapes instead of the square grid")
    ap.add_argument("--cutoff", action="store_true", help="classical kernel against Strassen levels on a grid of shapes up to --max-n")
    ap.add_argument("--b-transposed", action="store_true", help="--cutoff: B as the transposed view of an N x K matrix (the layout of x W^T)")
    ap.add_argument("--cache-weight-sums", action="store_true",
                    help="keep the quadrant sums of the weight between calls (16-bit weights)")
    ap.add_argument("--json", default=None, help="write the measured rows to this file as JSON")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("no GPU visible: this benchmark needs an MI355X")
    print(f"device: {torch.cuda.get_device_name(0)}  dtype: {args.dtype}")
    if args.gpt2:
        rows = profile_gpt2_linears(dtype=_DTYPES[args.dtype])
    elif args.cutoff:
        rows = profile_cutoff(_DTYPES[args.dtype], [s for s in _CUTOFF_SHAPES if args.min_n <= max(s) <= args.max_n],
                              max_levels=3 if args.max_n > 16384 else 2, b_transposed=args.b_transposed)
    else:
        rows = profile_linear_layers(_DTYPES[args.dtype], args.min_n, args.max_n, args.cache_weight_sums)
    if args.json:
        with open(args.json, "w") as f:
            json.dump({"device": torch.cuda.get_device_name(0), "dtype": args.dtype, "rows": rows}, f, indent=1)
