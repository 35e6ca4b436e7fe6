"""Drop-in for the reference's strassen_2_layer.py on MI355X."""
from __future__ import annotations

import strassen_hip
from _levels import practical_levels


def run_strassen_2_layer_fp32_accum(A, B, C, BLOCK_SIZE=64):
    """C += A @ B with two levels on the operands as given (reference
    strassen_2_layer.py:7-15; its kernel keeps fp32 operands, :103-162).  The whole of C is
    updated; the reference's grid drops rows and columns beyond a multiple of BLOCK_SIZE (:12)."""
    M, N = C.shape
    K = A.shape[1]
    assert K == B.shape[0] and A.shape[0] == M and B.shape[1] == N
    levels = max(1, practical_levels(min(M, N, K), 2))
    strassen_hip.run_accumulate(A, B, C, algo="strassen", levels=levels, operand_dtype=None)
