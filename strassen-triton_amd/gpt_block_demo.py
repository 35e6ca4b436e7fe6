"""Before / after timing of one pre-norm decoder block with its Linear layers swapped for
Strassen layers, the experiment of the reference's train.py (:322-350) on one block of the
shape of its model/model.py Decoder (:4-32): LayerNorm, causal attention (qkv and output
projections), LayerNorm, feed-forward with 4 x expansion and SiLU, residuals.

    python gpt_block_demo.py [--dim 4096] [--heads 32] [--tokens 8192] [--dtype bf16] [--backward]

The block runs eagerly; attention itself is torch's scaled_dot_product_attention in both runs,
only the four Linear layers change (replace_linear_with_strassen(..., square_only=False): all four
become LinearStrassenRect, which takes any number of token rows).
"""
from __future__ import annotations

import argparse
import copy

import torch
import torch.nn as nn
import torch.nn.functional as F

from model.layers import replace_linear_with_strassen

_DTYPES = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


class Block(nn.Module):
    def __init__(self, dim: int, heads: int, expansion: int = 4, bias: bool = True, device="cuda", dtype=None):
        super().__init__()
        kw = dict(device=device, dtype=dtype)
        self.heads = heads
        self.l1, self.l2 = nn.LayerNorm(dim, **kw), nn.LayerNorm(dim, **kw)
        self.qkv = nn.Linear(dim, 3 * dim, bias=bias, **kw)
        self.proj = nn.Linear(dim, dim, bias=bias, **kw)
        self.up = nn.Linear(dim, expansion * dim, bias=bias, **kw)
        self.down = nn.Linear(expansion * dim, dim, bias=bias, **kw)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        b, t, d = x.shape
        q, k, v = self.qkv(self.l1(x)).view(b, t, 3, self.heads, d // self.heads).permute(2, 0, 3, 1, 4)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(b, t, d)
        x = x + self.proj(a)
        return x + self.down(F.silu(self.up(self.l2(x))))


def _time(fn, warmup: int = 3, runs: int = 10) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(runs):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / runs


def compare_block(dim: int, heads: int, tokens: int, dtype=torch.bfloat16, backward: bool = False,
                  cache_weight_sums: bool = False, warmup: int = 3, runs: int = 10, verbose: bool = True) -> dict:
    """Builds one block, swaps the Linear layers of a copy, and returns the times of both and the
    relative difference of their outputs (and, with backward, of the input gradients)."""
    torch.manual_seed(0)
    std = Block(dim, heads, dtype=dtype)
    ours = copy.deepcopy(std)
    if verbose:
        replace_linear_with_strassen(ours, min_size=128, depth=1, square_only=False, cache_weight_sums=cache_weight_sums)
    else:
        import contextlib, io
        with contextlib.redirect_stdout(io.StringIO()):
            replace_linear_with_strassen(ours, min_size=128, depth=1, square_only=False, cache_weight_sums=cache_weight_sums)
    seq = min(1024, tokens)
    x = torch.randn(tokens // seq, seq, dim, device="cuda", dtype=dtype)

    def step(block):
        if not backward:
            with torch.no_grad():
                return block(x)
        block.zero_grad(set_to_none=True)
        y = block(x)
        y.float().square().mean().backward()
        return y

    rel = lambda got, ref: float(torch.linalg.norm(got.float() - ref.float()) / torch.linalg.norm(ref.float()))
    with torch.no_grad():
        res = {"dim": dim, "heads": heads, "tokens": tokens, "backward": backward, "rel_diff": rel(ours(x), std(x))}
    if backward:
        step(std), step(ours)
        res["rel_diff_weight_grad"] = max(rel(po.grad, ps.grad) for (_, po), (_, ps) in
                                          zip(ours.named_parameters(), std.named_parameters()) if ps.dim() == 2)
    res["std_ms"], res["strassen_ms"] = _time(lambda: step(std), warmup, runs), _time(lambda: step(ours), warmup, runs)
    res["replaced"] = sorted(type(m).__name__ for m in ours.modules() if type(m).__name__.startswith("LinearStrassen"))
    return res


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--dim", type=int, default=4096)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--tokens", type=int, default=8192, help="batch x sequence; sequences of 1024")
    ap.add_argument("--dtype", choices=sorted(_DTYPES), default="bf16")
    ap.add_argument("--backward", action="store_true", help="time forward + backward instead of forward only")
    ap.add_argument("--cache-weight-sums", action="store_true",
                    help="the replaced layers keep their weights' quadrant sums between calls (inference)")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("no GPU visible: this demo needs an MI355X")
    r = compare_block(args.dim, args.heads, args.tokens, _DTYPES[args.dtype], args.backward, args.cache_weight_sums)
    what = "forward + backward" if args.backward else "forward"
    print(f"block dim {args.dim}, {args.tokens} tokens, {args.dtype}, {what}:")
    print(f"  nn.Linear       {r['std_ms']:9.3f} ms")
    print(f"  Strassen layers {r['strassen_ms']:9.3f} ms   ({r['std_ms'] / r['strassen_ms']:.2f}x)   "
          f"output rel. difference {r['rel_diff']:.2e}")


if __name__ == "__main__":
    main()
