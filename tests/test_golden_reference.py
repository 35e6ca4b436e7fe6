"""The oracle against vectors produced by the reference's own functions.

tests/golden/reference_cast_schedule.npz holds outputs of the reference's
fixed_strassen.py / fixed_strassen_fp32_agg.py (run eagerly on CPU by
tests/golden/make_reference_vectors.py).  Mathematics pins the oracle's formulas; these
vectors pin the one thing it cannot: where the reference rounds to bf16 / fp16 / fp32.
Outputs are compared bit for bit."""
import os

import numpy as np
import pytest
import torch

from oracle import strassen_oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_cast_schedule.npz")
DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
CASES = [(n, name) for n in (32, 64, 128) for name in DT if not (n == 128 and name != "bf16")]


@pytest.fixture(scope="module")
def vec():
    return np.load(PATH)


def _tensor(arr, dt):
    t = torch.from_numpy(np.ascontiguousarray(arr))
    return t.view(dt)


@pytest.mark.parametrize("n,name", CASES)
def test_oracle_reproduces_reference_bits(vec, n, name):
    dt = DT[name]
    A, B = _tensor(vec[f"A_{n}_{name}"], dt), _tensor(vec[f"B_{n}_{name}"], dt)
    checks = {
        f"plain_base_{n}_{name}": lambda: O.strassen_base(A, B),
        f"agg_base_{n}_{name}": lambda: O.strassen_base_fp32_agg(A, B, dt),
    }
    for d in (2, 3):
        checks[f"plain_d{d}_{n}_{name}"] = lambda d=d: O.strassen_matmul_n_layers(A, B, d)
        checks[f"agg_d{d}_{n}_{name}"] = lambda d=d: O.strassen_matmul_n_layers(A, B, d, dt, fp32_agg=True)
    seen = 0
    for key, fn in checks.items():
        if key + "_error" in vec.files:
            continue   # the reference itself raises on this input (mixed-dtype leaf product)
        got = fn()
        want_dtype = dt
        if key + "_dtype" in vec.files:
            want_dtype = getattr(torch, str(vec[key + "_dtype"]).split(".")[1])
        assert got.dtype == want_dtype, key
        want = _tensor(vec[key], want_dtype)
        assert torch.equal(got, want), f"{key}: max abs diff {(got.double() - want.double()).abs().max():.3e}"
        seen += 1
    assert seen >= 4


def test_reference_failure_cases_are_recorded(vec):
    """The fp32-aggregated reference cannot run two levels on 32 x 32 bf16/fp16 inputs: its
    16-row leaf product gets one rounded and one fp32 operand (fixed_strassen_fp32_agg.py:20)."""
    errs = sorted(k for k in vec.files if k.endswith("_error"))
    assert errs == ["agg_d2_32_bf16_error", "agg_d2_32_f16_error"]
    assert "same dtype" in str(vec[errs[0]])
