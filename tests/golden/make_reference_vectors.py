"""Writes tests/golden/reference_cast_schedule.npz: outputs of the reference's own
matrix-level Strassen functions (fixed_strassen.py, fixed_strassen_fp32_agg.py) on small
seeded CPU inputs, run eagerly (torch.compile disabled).

Why this exists: mathematics pins the oracle's formulas (C = A @ B in exact arithmetic), but
not where the reference rounds to bf16 / fp16 / fp32.  These vectors pin that cast schedule
bit for bit.  Only the vectors are committed; the reference itself is read from
/root/reference, which exists in the build container only.

    TORCHDYNAMO_DISABLE=1 python tests/golden/make_reference_vectors.py
"""
import os
import sys

os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
import numpy as np
import torch

REF = os.environ.get("STRASSEN_REFERENCE", "/root/reference")
sys.path.insert(0, REF)
import fixed_strassen as ref_plain          # noqa: E402
import fixed_strassen_fp32_agg as ref_agg   # noqa: E402

DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def bits(t: torch.Tensor) -> np.ndarray:
    """Raw storage as integers, so bf16 survives the trip through numpy."""
    if t.dtype == torch.float32:
        return t.contiguous().view(torch.int32).numpy().copy()
    return t.contiguous().view(torch.int16).numpy().copy()


def main():
    out = {}
    for n in (32, 64, 128):
        g = torch.Generator().manual_seed(1234 + n)
        A32 = torch.randn(n, n, generator=g) / n ** 0.5
        B32 = torch.randn(n, n, generator=g) / n ** 0.5
        for name, dt in DT.items():
            if n == 128 and name != "bf16":   # keep the fixture small
                continue
            A, B = A32.to(dt), B32.to(dt)
            out[f"A_{n}_{name}"] = bits(A)
            out[f"B_{n}_{name}"] = bits(B)
            out[f"plain_base_{n}_{name}"] = bits(ref_plain._strassen_base(A, B))
            out[f"agg_base_{n}_{name}"] = bits(ref_agg._strassen_base(A, B, dt))
            for depth in (2, 3):
                out[f"plain_d{depth}_{n}_{name}"] = bits(ref_plain.strassen_matmul_n_layers(A, B, depth))
                try:
                    r = ref_agg.strassen_matmul_n_layers(A, B, depth, dt)
                except RuntimeError as e:
                    # the reference itself fails here: a 16-row leaf gets one bf16/fp16 and one
                    # fp32 operand (fixed_strassen_fp32_agg.py:20 reached from :99-113)
                    out[f"agg_d{depth}_{n}_{name}_error"] = np.array(str(e)[:120])
                    continue
                out[f"agg_d{depth}_{n}_{name}"] = bits(r)
                out[f"agg_d{depth}_{n}_{name}_dtype"] = np.array(str(r.dtype))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_cast_schedule.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
