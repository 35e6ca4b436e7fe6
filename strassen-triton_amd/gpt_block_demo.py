"""Before / after timing of one pre-norm decoder block with its Linear layers swapped for
Strassen layers, the experiment of the reference's train.py (:322-350) on one block of the
shape of its model/model.py Decoder (:4-32): LayerNorm, causal attention (qkv and output
projections), LayerNorm, feed-forward with 4 x expansion and SiLU, residuals.

    python gpt_block_demo.py [--dim 4096] [--heads 32] [--tokens 8192] [--dtype bf16] [--backward]

The block runs eagerly; attention itself is torch's scaled_dot_product_attention in both runs,
only the four Linear layers change (replace_linear_with_strassen(..., square_only=False): the
square projection becomes LinearStrassen, the non-square ones LinearStrassenRect).
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
    dtype = _DTYPES[args.dtype]
    torch.manual_seed(0)
    std = Block(args.dim, args.heads, dtype=dtype)
    ours = copy.deepcopy(std)
    replace_linear_with_strassen(ours, min_size=128, depth=1, square_only=False,
                                 cache_weight_sums=args.cache_weight_sums)
    seq = min(1024, args.tokens)
    x = torch.randn(args.tokens // seq, seq, args.dim, device="cuda", dtype=dtype)

    def step(block):
        if not args.backward:
            with torch.no_grad():
                return block(x)
        block.zero_grad(set_to_none=True)
        y = block(x)
        y.float().square().mean().backward()
        return y

    with torch.no_grad():
        ref, got = std(x).float(), ours(x).float()
    rel = float(torch.linalg.norm(got - ref) / torch.linalg.norm(ref))
    t_std, t_ours = _time(lambda: step(std)), _time(lambda: step(ours))
    what = "forward + backward" if args.backward else "forward"
    print(f"block dim {args.dim}, {args.tokens} tokens, {args.dtype}, {what}:")
    print(f"  nn.Linear       {t_std:9.3f} ms")
    print(f"  Strassen layers {t_ours:9.3f} ms   ({t_std / t_ours:.2f}x)   output rel. difference {rel:.2e}")


if __name__ == "__main__":
    main()
