"""How many Strassen levels a call of the reference's recursion actually takes."""
from __future__ import annotations

# The reference multiplies blocks of 16 rows or fewer classically (fixed_strassen.py:20-21).
LEAF = 16
# Splitting further than this only adds launches: blocks below 32 rows are multiplied classically.
MIN_HALF = 32


def reference_levels(n: int, n_depth: int) -> int:
    """Levels taken by strassen_matmul_n_layers(A, B, n_depth) on n x n inputs
    (fixed_strassen.py:71-114): one split per recursion step until n_depth reaches 2 or the
    half size reaches 2, then the one-level routine, which splits once more if its input has
    more than LEAF rows."""
    levels = 0
    while True:
        if n_depth == 1:
            return levels + (1 if n > LEAF else 0)
        mid = n // 2
        levels += 1
        if mid == 2 or n_depth == 2:
            return levels + (1 if mid > LEAF else 0)
        n, n_depth = mid, n_depth - 1


def practical_levels(n: int, levels: int) -> int:
    """Clamp so that the innermost half block keeps at least MIN_HALF rows."""
    while levels > 0 and (n >> levels) < MIN_HALF:
        levels -= 1
    return levels
