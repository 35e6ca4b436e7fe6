"""The five benchmark configurations at their REAL shapes on the CPU build of the library (tests/host_model/: the
library's own sources compiled for the host, one host thread per lane), against the oracle at the configurations' bounds.
What tests/test_gpu_parity.py checks on the card, checked where no card is at hand: the same seeded inputs, the same calls
through the C ABI, the same kernels and path selection -- everything but the hardware's own execution.

Minutes to hours each, so none of it runs unasked:

    STHIP_HOST_CONFIGS=C1,C2 python -m pytest tests/test_host_configs.py -s     # or C3a (one level), C3b (two), C3c (two at 4096^3), C4, C5, L4 (LinearStrassen 4096), all

Measured (8 host cores; relative Frobenius distance from the oracle / from the fp64 product): C1 7.2e-7 / 4.3e-7 in 4
minutes; C2 3.0e-5 / 7.2e-4 in 25 minutes (a GPU gave 3.1e-5 / 7.2e-4 on the same inputs); C4, entry 0, 9.2e-5 / 7.7e-3 in an
hour; C5 between 3.3e-5 and 8.1e-5 from the oracle on the paths that round their products as the reference does and 4.0e-3
on the kernels that keep them in fp32 (4.7e-3 from fp64 instead of 5.8e-3), two hours for the fifteen products; C3, one level,
6.9e-5 / 5.8e-3 in three hours (a GPU: 8.5e-5 / 5.8e-3); two levels at 4096^3 1.13e-2 / 1.20e-2 in twenty minutes (a GPU at
8192^3: 1.18e-2 / 1.24e-2); LinearStrassen(4096) on 1000 rows 3.1e-3 / 2.9e-3 at depth 1 and 4.7e-3 / 4.3e-3 at depth 2, whose
oracle adds in bf16 and is itself 3.6e-3 and 5.8e-3 from fp64 (seventy minutes for the two).
"""
import os

import pytest
import torch

from oracle import strassen_oracle as O
import test_host_parity
from test_host_parity import BF, DT, HF, SCHEDULE, SG, Script, host_gemm, cli  # noqa: F401  (cli is the fixture that builds the driver)
from test_kernel_host_model import _clang

if os.environ.get("STHIP_HOST_CONFIGS"):
    test_host_parity.Script.timeout = 8 * 3600

ASKED = {c.strip() for c in os.environ.get("STHIP_HOST_CONFIGS", "").split(",") if c.strip()}
pytestmark = pytest.mark.skipif(_clang() is None, reason="no clang++ for the host build")
TOL = {SG: 1e-5, HF: 2e-2, BF: 2e-2}


def _wanted(name):
    return pytest.mark.skipif(not ({name, name[:2], "all"} & ASKED), reason="set STHIP_HOST_CONFIGS=%s (or all): minutes to hours on the host" % name)


def _gauss(shape, seed, scale, dtype):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


def _report(name, C, want, A, B, tol):
    e_ref, e_exact = O.rel_fro(C.double(), want.double()), O.rel_fro(C.double(), A.double() @ B.double())
    print(f"{name}: {e_ref:.3e} from the oracle, {e_exact:.3e} from fp64", flush=True)
    assert e_ref <= tol and e_exact <= tol


@_wanted("C1")
def test_config1_fp32_one_level_1024(cli):  # noqa: F811
    """1024^3 fp32, N(0,1), one level (fixed_strassen.py:11-57); on the card this is the 64 x 64 kernel with the sums formed
    in the operand loads.  7.2e-7 from the oracle."""
    A, B = _gauss((1024, 1024), 1234, 1.0, SG), _gauss((1024, 1024), 1235, 1.0, SG)
    _report("config 1", host_gemm(cli, A, B, levels=1, cus=8), O.strassen_base(A, B), A, B, TOL[SG])


@_wanted("C2")
def test_config2_fp16_one_level_4096(cli):  # noqa: F811
    """4096^3 fp16, N(0,1)/sqrt(K), one level with fp32 aggregation (fixed_strassen_fp32_agg.py:12-56): sums pass, seven
    products on 256 x 256 tiles walked by the workgroups, recombination pass."""
    n = 4096
    A, B = _gauss((n, n), 1234, n ** -0.5, HF), _gauss((n, n), 1235, n ** -0.5, HF)
    want = O.strassen_base_fp32_agg(A, B, HF, mm=O.mm_fp32_upcast)
    _report("config 2", host_gemm(cli, A, B, levels=1, cus=16), want, A, B, TOL[HF])


@pytest.mark.parametrize("depth", [pytest.param(1, marks=_wanted("C3a")), pytest.param(2, marks=_wanted("C3b"))])
def test_config3_bf16_8192(cli, depth):  # noqa: F811
    """8192^3 bf16, N(0,1)/sqrt(K): one level (the headline path) and two levels (49 products in one launch)."""
    n = 8192
    A, B = _gauss((n, n), 1234, n ** -0.5, BF), _gauss((n, n), 1235, n ** -0.5, BF)
    want = O.strassen_matmul_n_layers(A, B, depth, BF, fp32_agg=True, mm=O.mm_fp32_upcast)
    _report("config 3, %d level(s)" % depth, host_gemm(cli, A, B, levels=depth, cus=16), want, A, B, TOL[BF])


@_wanted("C3c")
def test_two_levels_bf16_4096(cli):  # noqa: F811
    """The two-level form of configuration 3 at an eighth of its work (4096^3; the 8192^3 run takes some thirteen core-hours
    on the host): sums of both levels in one pass, the 49 quarter-size products as one launch, both recombinations in one pass."""
    n = 4096
    A, B = _gauss((n, n), 1234, n ** -0.5, BF), _gauss((n, n), 1235, n ** -0.5, BF)
    want = O.strassen_matmul_n_layers(A, B, 2, BF, fp32_agg=True, mm=O.mm_fp32_upcast)
    _report("two levels, 4096^3 bf16", host_gemm(cli, A, B, levels=2, cus=16), want, A, B, TOL[BF])


@_wanted("C4")
def test_config4_winograd_bf16(cli):  # noqa: F811
    """Strassen-Winograd, 4096 x 8192 x 4096 bf16, U[-1,1]/sqrt(K): entry 0 of the configuration's batch of eight as a call of
    its own (that batch entries do not influence each other is checked at small sizes, tests/test_host_parity.py)."""
    b, M, K, N = 8, 4096, 8192, 4096
    A = ((torch.rand((b, M, K), generator=torch.Generator().manual_seed(1234))[0] * 2 - 1) * K ** -0.5).to(BF)
    B = ((torch.rand((b, K, N), generator=torch.Generator().manual_seed(1235))[0] * 2 - 1) * K ** -0.5).to(BF)
    want = O.winograd_base(A, B, BF, fp32_agg=True, mm=O.mm_fp32_upcast)
    _report("config 4, entry 0", host_gemm(cli, A, B, algo="winograd", levels=1, cus=16), want, A, B, TOL[BF])


@_wanted("C5")
@pytest.mark.parametrize("d_in,d_out", [(768, 768), (768, 2304), (768, 3072), (3072, 768), (768, 769)])
def test_config5_gpt2_linears(cli, d_in, d_out):  # noqa: F811
    """GPT-2-small Linear shapes, 8192 token rows, bf16 ~ N(0, 0.02), one level: forward x W^T (NT), input gradient dY W (NN),
    weight gradient dY^T x (TN); 769 is the odd size that pads to even quadrants."""
    rows = 8192
    X, W, dY = _gauss((rows, d_in), 1234, 0.02, BF), _gauss((d_out, d_in), 1235, 0.02, BF), _gauss((rows, d_out), 1236, 0.02, BF)
    for name, A, B in (("fwd", X, W.t()), ("dgrad", dY, W), ("wgrad", dY.t(), X)):
        want = O.strassen_general(A, B, levels=1, base_dtype=BF, fp32_agg=True, mm=O.mm_fp32_upcast)
        _report("config 5, %d -> %d %s" % (d_in, d_out, name), host_gemm(cli, A, B, levels=1, cus=16), want, A, B, TOL[BF])


@pytest.mark.parametrize("depth", [pytest.param(1, marks=_wanted("L4")), pytest.param(2, marks=_wanted("L4"))])
def test_linear_strassen_4096(cli, depth):  # noqa: F811
    """LinearStrassen(4096) with 1000 input rows, bias, bf16, depth 1 and 2 (sthip_linear_strassen_forward) against the oracle's
    restatement of model/layers.py:246-274 -- pad to D x D, _strassen_base or the two-layer function of strassen.py (which adds in
    bf16 at both levels, hence twice the bound at depth 2, as in tests/test_gpu_scale.py), slice, + bias."""
    D, rows = 4096, 1000
    w, b, x = _gauss((D, D), 107, D ** -0.5, BF), _gauss((D,), 108, 1.0, BF), _gauss((rows, D), 109, 1.0, BF)
    y = torch.zeros(rows, D, dtype=BF)
    sc = Script(cli)
    sc.add("units", 16)
    sc.add("linear_strassen", sc.buf(x), sc.buf(w), sc.buf(b), sc.buf(y, back=True), rows, D, DT[BF], depth,
           sc.workspace(1, D, D, D, DT[BF], DT[BF], 1 | SCHEDULE["fast"], depth))
    sc.run()
    want = O.linear_strassen_forward(x, w, b, depth, mm=O.mm_fp32_upcast)
    exact = x.double() @ w.double().t() + b.double()
    err, err64, ora64 = O.rel_fro(y, want), O.rel_fro(y, exact), O.rel_fro(want, exact)
    print(f"LinearStrassen 4096, {rows} rows, depth {depth}: {err:.3e} from the oracle, {err64:.3e} from fp64 (the oracle: {ora64:.3e})", flush=True)
    assert err64 <= TOL[BF] and err <= TOL[BF] * depth and err64 <= ora64 * 1.05
