"""Drop-in for the reference's fixed_strassen.py on MI355X.

Same names and call signatures (`_strassen_base`, `strassen_matmul_n_layers`,
`LinearStrassen`), but the quadrant sums, the seven products and the recombination run in
one hand-written HIP kernel per level instead of torch ops under torch.compile.  Tensors
must be on the GPU.
"""
from __future__ import annotations

from math import log2

import torch
import torch.nn as nn
from torch import Tensor

import strassen_hip
from _levels import LEAF, practical_levels, reference_levels


def _check_square(A: Tensor, B: Tensor) -> int:
    if A.dim() != 2 or B.dim() != 2 or A.shape[0] != A.shape[1] or tuple(A.shape) != tuple(B.shape):
        raise ValueError("Input matrices must be square and have the same dimensions.")
    return A.shape[0]


def _strassen_base(A: Tensor, B: Tensor, base_dtype=torch.float32) -> Tensor:
    """One Strassen level (reference fixed_strassen.py:11-57); base_dtype is ignored here as
    it is there.  Inputs of 16 rows or fewer are multiplied classically (:20-21)."""
    n = _check_square(A, B)
    if n <= LEAF:
        return strassen_hip.matmul(A, B, algo="classic", levels=0)
    return strassen_hip.matmul(A, B, algo="strassen", levels=1)


def strassen_matmul_n_layers(A: Tensor, B: Tensor, n_depth: int = 2, base_dtype=torch.float32) -> Tensor:
    """n_depth-level Strassen product (reference fixed_strassen.py:59-126).  The reference does all
    of its arithmetic in the input dtype at every level, so 16-bit inputs take the schedule that
    rounds every level's operand sums and products to that dtype (sums and recombination are
    still formed in fp32 and rounded once, which is closer to the exact product than the
    reference's own additions in 16 bits)."""
    n = _check_square(A, B)
    levels = practical_levels(n, reference_levels(n, n_depth))
    if levels == 0:
        return strassen_hip.matmul(A, B, algo="classic", levels=0)
    return strassen_hip.matmul(A, B, algo="strassen", levels=levels, schedule="fast")


class _LinearFn(torch.autograd.Function):
    """y = x W^T + b with the forward in one C-ABI call; dgrad dX = dY W and wgrad
    dW = dY^T X are Strassen products over views of the saved tensors."""

    @staticmethod
    def forward(ctx, x2d, weight, bias, levels, weight_sums=None):
        ctx.save_for_backward(x2d, weight)
        ctx.levels, ctx.has_bias = levels, bias is not None
        if weight_sums is not None:
            return strassen_hip.linear_forward_any(x2d, weight, bias, levels, weight_sums)
        return strassen_hip.linear_forward(x2d, weight, bias, levels)

    @staticmethod
    def backward(ctx, dy):
        x2d, weight = ctx.saved_tensors
        dy = dy.contiguous()
        dx = strassen_hip.gemm(dy, weight, levels=1) if ctx.needs_input_grad[0] else None
        dw = strassen_hip.gemm(dy.t(), x2d, levels=1) if ctx.needs_input_grad[1] else None
        db = dy.sum(0) if ctx.has_bias and ctx.needs_input_grad[2] else None
        return dx, dw, db, None, None


class LinearStrassen(nn.Linear):
    """nn.Linear whose matmul is the Strassen kernel (reference fixed_strassen.py:128-169,
    model/layers.py:232-274): square power-of-two features, at most D input rows.

    cache_weight_sums (not in the reference, off by default): keep the quadrant sums of the
    weight in device memory between calls (1.25 x the weight's bytes at depth 1, 3.4 x at
    depth 2, 7.3 x at depth 3) instead of forming them in every forward; for 16-bit weights,
    D x D inputs and up to four levels, same bits.  The sums follow the weight's version counter: after a write that
    bypasses it (through .data) call weight_sums.clear()."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, dtype=torch.float32,
                 depth: int = 1, device: str = "cuda", cache_weight_sums: bool = False) -> None:
        assert in_features == out_features and (log2(in_features)).is_integer(), \
            "Transform must be square and a power of 2"
        super().__init__(in_features, out_features, bias, device, dtype)
        self.depth = depth
        self.cache_weight_sums = cache_weight_sums
        self.weight_sums = strassen_hip.WeightSums()

    def _levels_for(self, D: int) -> int:
        """Levels strassen_matmul_n_layers(X, W.T, n_depth=self.depth) takes (fixed_strassen.py:157)."""
        return max(1, practical_levels(D, reference_levels(D, self.depth)))

    def forward(self, input: Tensor):
        *batch_dims, D_in = input.shape
        assert D_in == self.in_features, "Input dim mismatch"
        D = self.in_features
        M = input.numel() // D
        if M > D:
            raise ValueError(
                f"Input M ({M}) > D ({D}). Cannot pad input to DxD. "
                f"You MUST use the method that pads BOTH input and weights to PxP.")
        levels = self._levels_for(D)
        sums = self.weight_sums.get(self.weight, levels) if self.cache_weight_sums and M == D else None
        out = _LinearFn.apply(input.reshape(M, D), self.weight, self.bias, levels, sums)
        return out.view(*batch_dims, D)
