"""The Linear adaptor of the reference's model/layers.py (:225-300) on MI355X.

Only the Strassen Linear path lives here; attention, RoPE and the feed-forward block of
the reference's model code are consumers of this layer, not part of it.
"""
from __future__ import annotations

import torch
import torch.nn as nn

import strassen_hip
from fixed_strassen import LinearStrassen as _LinearStrassen
from strassen import _strassen_base, strassen_matmul_two_layers


class LinearStrassen(_LinearStrassen):
    """Same module as fixed_strassen.LinearStrassen with the constructor and the depth rule of
    reference model/layers.py:232-244: dtype defaults to None; depth 2 selects the two-layer
    product, every other depth the one-level routine (there depth 3 is one level, not three).
    strassen_func names the function of the reference-shaped surface that computes the same
    product; forward itself goes through the fused Linear entry of the C ABI (no padding copy)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, dtype=None,
                 depth: int = 1, device: str = "cuda", cache_weight_sums: bool = False) -> None:
        super().__init__(in_features, out_features, bias, dtype, depth, device, cache_weight_sums)
        self.strassen_func = strassen_matmul_two_layers if depth == 2 else _strassen_base

    def _levels_for(self, D: int) -> int:
        from _levels import practical_levels
        return max(1, practical_levels(D, 2 if self.depth == 2 else 1))


class _RectLinearFn(torch.autograd.Function):
    """y = x W^T + b for any (rows, in) x (out, in): forward, dgrad dX = dY W and wgrad
    dW = dY^T X are each one Strassen product over strided views, no padding, no copies; the
    bias is added by the forward product's recombination pass where it has one."""

    @staticmethod
    def forward(ctx, x2d, weight, bias, levels, weight_sums=None):
        ctx.save_for_backward(x2d, weight)
        ctx.levels, ctx.has_bias = levels, bias is not None
        return strassen_hip.linear_forward_any(x2d, weight, bias, levels, weight_sums)

    @staticmethod
    def backward(ctx, dy):
        x2d, weight = ctx.saved_tensors
        dy = dy.contiguous()
        # a negative ctx.levels carries the measured cutoff to each of the two gradient products
        dx = strassen_hip.gemm(dy, weight, levels=ctx.levels) if ctx.needs_input_grad[0] else None
        dw = strassen_hip.gemm(dy.t(), x2d, levels=ctx.levels) if ctx.needs_input_grad[1] else None
        db = dy.sum(0) if ctx.has_bias and ctx.needs_input_grad[2] else None
        return dx, dw, db, None, None


class LinearStrassenRect(nn.Linear):
    """nn.Linear of any shape whose three GEMMs are Strassen products.  Lifts the constraints
    of the reference's layer (model/layers.py:240, :255-262: square, power of two, at most D
    input rows, input padded to D x D): sizes that are odd or not tile multiples are handled
    by the kernels' zero-padding edge tiles, so nothing is padded or sliced in memory.
    cache_weight_sums: as for LinearStrassen; shapes for which no sums are kept run as before.
    cutoff (default on): each of the three products runs at most `depth` levels, and fewer -- down
    to the library's classical kernel -- where the measured cutoff (sthip_auto_levels) says that is
    faster on its shape; cutoff=False always runs `depth` levels, as the reference's layer does."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, dtype=None,
                 depth: int = 1, device: str = "cuda", cache_weight_sums: bool = False, cutoff: bool = True) -> None:
        super().__init__(in_features, out_features, bias, device, dtype)
        self.depth = depth
        self.cutoff = cutoff
        self.cache_weight_sums = cache_weight_sums
        self.weight_sums = strassen_hip.WeightSums()

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        *batch_dims, d_in = input.shape
        assert d_in == self.in_features, "Input dim mismatch"
        x2d = input.reshape(-1, d_in)
        levels = max(1, int(self.depth))
        if self.cutoff:
            fwd = strassen_hip.auto_levels(x2d.shape[0], self.out_features, d_in, x2d.dtype, levels)
            sums = self.weight_sums.get(self.weight, fwd) if self.cache_weight_sums and fwd > 0 else None
            y = _RectLinearFn.apply(x2d, self.weight, self.bias, -levels, sums)
        else:
            sums = self.weight_sums.get(self.weight, levels) if self.cache_weight_sums else None
            y = _RectLinearFn.apply(x2d, self.weight, self.bias, levels, sums)
        return y.view(*batch_dims, self.out_features)


def replace_linear_with_strassen(module: nn.Module, min_size: int = 128, depth: int = 1,
                                 square_only: bool = True, cache_weight_sums: bool = False, cutoff: bool = True):
    """Swap every square nn.Linear of at least min_size features for LinearStrassen, in
    place, keeping weights and bias (reference model/layers.py:279-300).  With
    square_only=False every layer whose smaller side is at least min_size becomes a
    LinearStrassenRect instead (any shape, any number of input rows -- the reference's layer
    refuses more than D rows); below min_size a layer stays an nn.Linear, i.e. a classical GEMM.
    cache_weight_sums and cutoff are handed to the new layers (cutoff: see LinearStrassenRect)."""
    for name, child in module.named_children():
        if isinstance(child, nn.Linear) and not isinstance(child, (_LinearStrassen, LinearStrassenRect)):
            if not square_only and min(child.in_features, child.out_features) >= min_size:
                print(f"Replacing '{name}' with LinearStrassenRect.")
                new_layer = LinearStrassenRect(child.in_features, child.out_features,
                                               bias=child.bias is not None, device=child.weight.device,
                                               dtype=child.weight.dtype, depth=depth,
                                               cache_weight_sums=cache_weight_sums, cutoff=cutoff)
                new_layer.weight.data.copy_(child.weight.data)
                new_layer.weight_sums.clear()   # a write through .data does not move the version counter
                if child.bias is not None:
                    new_layer.bias.data.copy_(child.bias.data)
                setattr(module, name, new_layer)
            elif child.in_features == child.out_features and child.in_features >= min_size:
                print(f"Replacing '{name}' with LinearStrassen.")
                new_layer = LinearStrassen(child.in_features, child.out_features,
                                           bias=child.bias is not None, device=child.weight.device,
                                           dtype=child.weight.dtype, depth=depth,
                                           cache_weight_sums=cache_weight_sums)
                new_layer.weight.data.copy_(child.weight.data)
                new_layer.weight_sums.clear()   # a write through .data does not move the version counter
                if child.bias is not None:
                    new_layer.bias.data.copy_(child.bias.data)
                setattr(module, name, new_layer)
            else:
                print(f"Skipping '{name}': Not square or too small.")
        elif len(list(child.children())) > 0:
            replace_linear_with_strassen(child, min_size, depth, square_only, cache_weight_sums, cutoff)
