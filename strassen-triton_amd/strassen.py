"""Drop-in for the reference's strassen.py on MI355X: the in-place launchers
(`run_matmul_fp32_accum`, `run_strassen`, `run_strassen2`, all C += A @ B, returning None)
and the torch-level two-layer recursion (`_strassen_base`, `strassen_matmul_two_layers`),
backed by the HIP kernels instead of Triton.  BLOCK_SIZE arguments are accepted and ignored
(the reference's autotuner overrides them too); tiles come from a fixed gfx950 table.
"""
from __future__ import annotations

import torch

import strassen_hip
from _levels import LEAF, practical_levels


def _shapes(A, B, C):
    if A.dim() == 3:
        return
    M, K = A.shape
    _, N = B.shape
    assert K == B.shape[0] and A.shape[0] == M and B.shape[1] == N
    assert tuple(C.shape) == (M, N)


def run_matmul_fp32_accum(A, B, C, BLOCK_SIZE=32):
    """C += A @ B, classical tiling, operands as given (reference strassen.py:66-88)."""
    _shapes(A, B, C)
    strassen_hip.run_accumulate(A, B, C, algo="classic", levels=0, operand_dtype=None)


def run_strassen(A, B, C, BLOCK_SIZE=32):
    """C += A @ B with one Strassen level, operands cast to fp16, fp32 accumulation
    (reference strassen.py:195-213 and the casts at :150-163)."""
    _shapes(A, B, C)
    strassen_hip.run_accumulate(A, B, C, algo="strassen", levels=1, operand_dtype=torch.float16)


def run_strassen2(A, B, C, BLOCK_SIZE=64):
    """C += A @ B with two Strassen levels (the 49-product schedule of reference
    strassen.py:373-611), operands cast to fp16 (:311-370)."""
    _shapes(A, B, C)
    n = min(A.shape[-2], A.shape[-1], B.shape[-1])
    strassen_hip.run_accumulate(A, B, C, algo="strassen", levels=max(1, practical_levels(n, 2)),
                                operand_dtype=torch.float16)


def _strassen_base(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """One Strassen level (reference strassen.py:697-740)."""
    if A.shape[0] <= LEAF:
        return strassen_hip.matmul(A, B, algo="classic", levels=0)
    return strassen_hip.matmul(A, B, algo="strassen", levels=1)


def strassen_matmul_two_layers(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """Two Strassen levels with the reference's validation (strassen.py:742-812)."""
    n = A.shape[0]
    if n != B.shape[0] or A.shape[1] != B.shape[0] or A.shape[0] != A.shape[1]:
        raise ValueError("Input matrices must be square and have the same dimensions.")
    if n % 4 != 0:
        raise ValueError("Matrix size must be divisible by 4 for two Strassen layers.")
    if not n > 0:
        raise ValueError("Matrix size must be positive.")
    levels = practical_levels(n, 2 if n // 2 > LEAF else 1)
    if levels == 0:
        return strassen_hip.matmul(A, B, algo="classic", levels=0)
    return strassen_hip.matmul(A, B, algo="strassen", levels=levels)
