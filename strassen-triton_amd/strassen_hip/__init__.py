"""Host side of the MI355X Strassen library: tensors in, C-ABI calls out."""
from . import _capi
from .ops import (ALGO_CLASSIC, ALGO_STRASSEN, ALGO_WINOGRAD, SCHEDULE_FAST, SCHEDULE_REFERENCE, StrassenMatmul, WeightSums, auto_levels, gemm, linear_forward,
                  linear_forward_any, matmul, prepare_weight, run_accumulate, workspace_bytes)

__all__ = ["gemm", "matmul", "run_accumulate", "linear_forward", "linear_forward_any", "StrassenMatmul", "workspace_bytes",
           "prepare_weight", "WeightSums", "auto_levels",
           "ALGO_CLASSIC", "ALGO_STRASSEN", "ALGO_WINOGRAD", "SCHEDULE_REFERENCE", "SCHEDULE_FAST"]
