"""Drop-in for the reference's fixed_strassen_fp32_agg.py on MI355X.

The reference forms the quadrant sums and the recombination in `agg_dtype` (fp32) and the
products in `base_dtype` (fixed_strassen_fp32_agg.py:26-50).  The HIP kernel does exactly
that in registers: operand sums in fp32 rounded once to base_dtype, MFMA products with fp32
accumulation, fp32 recombination, one final rounding.
"""
from __future__ import annotations

import torch
from torch import Tensor

import strassen_hip
from _levels import LEAF, practical_levels, reference_levels
from fixed_strassen import LinearStrassen, _check_square  # noqa: F401  (same class, same kernel)

agg_dtype = torch.float32   # reference fixed_strassen_fp32_agg.py:10


def _strassen_base(A: Tensor, B: Tensor, base_dtype=torch.float32) -> Tensor:
    """One level with fp32 aggregation (reference fixed_strassen_fp32_agg.py:12-56); the
    result has dtype base_dtype."""
    n = _check_square(A, B)
    A, B = A.to(base_dtype), B.to(base_dtype)
    if n <= LEAF:
        return strassen_hip.matmul(A, B, algo="classic", levels=0)
    return strassen_hip.matmul(A, B, algo="strassen", levels=1)


def strassen_matmul_n_layers(A: Tensor, B: Tensor, n_depth: int = 2, base_dtype=torch.float32) -> Tensor:
    """n_depth levels with fp32 aggregation (reference fixed_strassen_fp32_agg.py:58-125).
    The reference's inner calls do not forward base_dtype (:99-113), so below the first level
    it multiplies in fp32.  From three levels on this does the same (first-level sums rounded
    to base_dtype, the seven half-size products on the fp32 kernels); at two levels all 49
    quarter-size products run in base_dtype on the 16-bit matrix cores, 1.2e-2 from the
    reference in bf16.  strassen_hip.gemm(..., schedule="reference") gives the reference's
    schedule at two levels as well, schedule="fast" 16-bit products at every depth."""
    n = _check_square(A, B)
    A, B = A.to(base_dtype), B.to(base_dtype)
    levels = practical_levels(n, reference_levels(n, n_depth))
    if levels == 0:
        return strassen_hip.matmul(A, B, algo="classic", levels=0)
    return strassen_hip.matmul(A, B, algo="strassen", levels=levels)
