"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares,
argument errors are reported without touching a GPU, and the host logic that mirrors the
reference (recursion depth, validation, refusal of CPU tensors) behaves."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    names = set()
    for header in ("strassen_hip.h", "strassen_hip_debug.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(sthip_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    from strassen_hip import _capi
    lib = _capi.load()
    names = _header_symbols()
    assert len(names) >= 8
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ but not exported"
        assert n in _capi.SIGNATURES, f"{n} has no ctypes prototype"
    assert set(_capi.SIGNATURES) == set(names)
    assert lib.sthip_version() == 100


def test_argument_errors_need_no_gpu():
    from strassen_hip import _capi
    lib = _capi.load()
    s3 = (ctypes.c_int64 * 3)(0, 4, 1)
    one = ctypes.c_void_p(16)
    assert lib.sthip_gemm(one, one, one, 1, -1, 4, 4, s3, s3, s3, 0, 0, 1, 1, 0, None, 0, None) == -1
    assert b"negative" in lib.sthip_last_error()
    assert lib.sthip_gemm(one, one, one, 1, 4, 4, 4, s3, s3, s3, 7, 0, 1, 1, 0, None, 0, None) == -2
    assert lib.sthip_gemm(one, one, one, 1, 4, 4, 4, s3, s3, s3, 2, 1, 1, 1, 0, None, 0, None) == -2
    assert lib.sthip_gemm(one, one, one, 1, 4, 4, 4, s3, s3, s3, 0, 0, 9, 1, 0, None, 0, None) == -5
    assert lib.sthip_gemm(None, one, one, 1, 4, 4, 4, s3, s3, s3, 0, 0, 1, 1, 0, None, 0, None) == -5
    assert lib.sthip_gemm(one, one, one, 0, 4, 4, 4, s3, s3, s3, 0, 0, 1, 1, 0, None, 0, None) == 0   # empty batch
    assert lib.sthip_gemm(one, one, one, 1, 0, 4, 4, s3, s3, s3, 0, 0, 1, 1, 0, None, 0, None) == 0   # empty M
    assert lib.sthip_linear_strassen_forward(one, one, None, one, 9, 8, 0, 1, None, 0, None) == -1
    assert b"cannot be padded" in lib.sthip_last_error()
    # the entry point that brings its own scratch refuses a problem whose workspace exceeds that buffer
    wide = (ctypes.c_int64 * 3)(0, 8192, 1)
    assert lib.sthip_gemm_static(one, one, one, 1, 8192, 8192, 8192, wide, wide, wide, 2, 2, 1, 1, 0, None) == -4
    assert b"static scratch" in lib.sthip_last_error()
    assert lib.sthip_gemm_static(one, one, one, 1, -1, 4, 4, s3, s3, s3, 0, 0, 1, 1, 0, None) == -1
    assert lib.sthip_workspace_bytes(1, 4096, 4096, 4096, 2, 2, 1, 1) <= 144 << 20 < lib.sthip_workspace_bytes(1, 8192, 8192, 8192, 2, 2, 1, 1)
    # two or more levels need the workspace the query asks for: refused before anything is launched
    big = (ctypes.c_int64 * 3)(0, 1024, 1)
    for dt in (0, 2):
        assert lib.sthip_gemm(one, one, one, 1, 1024, 1024, 1024, big, big, big, dt, dt, 1, 2, 0, None, 0, None) == -4
        assert b"workspace too small" in lib.sthip_last_error()
        es = 4 if dt == 0 else 2
        mandatory = 2 * 5 * 512 * 512 * es + 7 * 512 * 512 * 4   # sums and fp32 products of the top level
        assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, dt, dt, 1, 2) >= mandatory
        assert lib.sthip_gemm(one, one, one, 1, 1024, 1024, 1024, big, big, big, dt, dt, 1, 2, 0,
                              ctypes.c_void_p(4096), mandatory - 1, None) == -4
    assert lib.sthip_gemm(one, one, one, 1, 1024, 1024, 1024, big, big, big, 2, 2, 1, 9, 0, None, 0, None) == -5   # levels > 8
    # an operand without a unit stride is a layout error
    bad = (ctypes.c_int64 * 3)(0, 2048, 2)
    assert lib.sthip_gemm(one, one, one, 1, 64, 64, 64, bad, big, big, 2, 2, 1, 1, 0, None, 0, None) == -3
    assert b"no unit stride" in lib.sthip_last_error()
    # workspace.  One level: room for the ten quadrant sums (5 per operand) and the parked accumulator when the shape is
    # tile aligned, per batch entry; nothing for fp32, odd or unaligned shapes, or classic.
    sums = lambda h: 2 * 5 * h * h * 2 + 7 * h * h * 2 + 256   # ten 16-bit sums + seven 16-bit products (or parked fp32 tiles) + counters
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 1, 1) == sums(512)
    assert lib.sthip_workspace_bytes(3, 1024, 1024, 1024, 1, 1, 2, 1) == 3 * sums(512)
    # 16-bit operands with an fp32 result: the seven products stay fp32
    assert lib.sthip_workspace_bytes(2, 1024, 1024, 1024, 2, 0, 1, 1) == 2 * (2 * 5 * 512 * 512 * 2 + 7 * 512 * 512 * 4) + 256
    # fp32, tile aligned: seven dense A operands, seven B operands, seven fp32 products
    f32 = lambda h: 7 * 3 * h * h * 4
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 0, 0, 1, 1) == f32(512)
    assert lib.sthip_workspace_bytes(1, 1000, 1000, 1000, 0, 0, 1, 1) == 0
    assert lib.sthip_workspace_bytes(4, 1024, 1024, 1024, 0, 0, 1, 1) == 0   # one problem per call on that path
    assert lib.sthip_workspace_bytes(1, 1000, 1024, 1024, 2, 2, 1, 1) == 0
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 0, 1) == 0
    # Two levels: five S_A, five S_B and seven fp32 M buffers of half size, plus the leaf's workspace
    # (host recursion; a leaf under an upper level hands its result over in fp32 and keeps its seven
    # products in fp32 too), or -- for tile-aligned 16-bit problems, which may run as one 49-product
    # launch -- ten half-size sums, 70 quarter-size sums and 49 quarter-size products; the query covers
    # whichever is larger.
    upper = lambda h: 2 * 5 * h * h * 2 + 7 * h * h * 4
    inner_sums = lambda h: 2 * 5 * h * h * 2 + 7 * h * h * 4 + 256
    flat = lambda h: 10 * h * h * 2 + (70 + 49) * (h // 2) ** 2 * 2
    two = lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 1, 2)
    assert two == max(upper(512) + inner_sums(256), flat(512))
    # three levels, every level in the operand type (STHIP_SCHEDULE_FAST = 2 << 4 OR-ed into algo)
    three = lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 1 | (2 << 4), 3)
    assert three == upper(512) + max(upper(256) + inner_sums(128), flat(256))
    # fp32 never takes the one-launch form
    f32_two = lambda h: 2 * 5 * h * h * 4 + 7 * h * h * 4 + f32(h // 2)
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 0, 0, 1, 2) == f32_two(512)
    # three levels by default, and two with STHIP_SCHEDULE_REFERENCE (1 << 4): one widened operand pair and seven fp32
    # products of half size, then the fp32 problem of one level less
    widened = lambda h: 2 * h * h * 4 + 7 * h * h * 4
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 1, 3) == widened(512) + f32_two(256)
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 1 | (1 << 4), 3) == widened(512) + f32_two(256)
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 1, 1, 1 | (1 << 4), 2) == widened(512) + f32(256)
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 1 | (2 << 4), 2) == two            # two levels are fast by default
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 0, 0, 1 | (1 << 4), 2) == f32_two(512)   # fp32 ignores the flags
    assert lib.sthip_workspace_bytes(1, 1024, 1024, 1024, 2, 2, 1 | (3 << 4), 2) == 0              # no such schedule
    assert lib.sthip_gemm(one, one, one, 1, 64, 64, 64, big, big, big, 2, 2, 1 | (3 << 4), 2, 0, None, 0, None) == -5


def test_weight_sums_size_and_argument_errors():
    """Sums of a constant weight: five half-size blocks for one level, 35 quarter-size ones more
    for two; three and four levels keep
    such a buffer per first-level product; none for fp32, other depths or blocks the grouped paths do not take.  Bad buffers are
    refused before anything is launched."""
    from strassen_hip import _capi
    lib = _capi.load()
    assert lib.sthip_linear_weight_sums_bytes(1024, 1024, 2, 1) == 5 * 512 * 512 * 2
    assert lib.sthip_linear_weight_sums_bytes(1024, 1024, 1, 2) == 5 * 512 * 512 * 2 + 35 * 256 * 256 * 2
    assert lib.sthip_linear_weight_sums_bytes(768, 3072, 2, 1) == 5 * 384 * 1536 * 2
    assert lib.sthip_linear_weight_sums_bytes(1024, 1024, 0, 1) == 0      # fp32
    two_of_half = 5 * 256 * 256 * 2 + 35 * 128 * 128 * 2
    assert lib.sthip_linear_weight_sums_bytes(1024, 1024, 2, 3) == 5 * 512 * 512 * 2 + 7 * two_of_half
    assert lib.sthip_linear_weight_sums_bytes(2048, 2048, 2, 4) == 5 * 1024 * 1024 * 2 + 7 * (5 * 512 * 512 * 2 + 7 * two_of_half)
    assert lib.sthip_linear_weight_sums_bytes(1024, 1024, 2, 4) == 0      # 64-wide blocks of out_features
    assert lib.sthip_linear_weight_sums_bytes(1 << 16, 1 << 16, 2, 5) == 0   # more than four levels
    assert lib.sthip_linear_weight_sums_bytes(1024, 1024, 2, 0) == 0
    assert lib.sthip_linear_weight_sums_bytes(1000, 1024, 2, 1) == 0      # 500 is no multiple of 64
    assert lib.sthip_linear_weight_sums_bytes(1024, 768, 2, 2) == 0       # 192 is no multiple of 128
    w, buf = ctypes.c_void_p(4096), ctypes.c_void_p(8192)
    assert lib.sthip_linear_prepare_weight(w, 1024, 1024, 0, 1, buf, 1 << 30, None) == -1
    assert b"no weight-side sums" in lib.sthip_last_error()
    assert lib.sthip_linear_prepare_weight(w, 1024, 1024, 2, 1, buf, 100, None) == -4
    assert b"too small" in lib.sthip_last_error()
    assert lib.sthip_linear_prepare_weight(w, 1024, 1024, 2, 1, ctypes.c_void_p(8200), 1 << 30, None) == -5
    assert lib.sthip_linear_prepare_weight(None, 1024, 1024, 2, 1, buf, 1 << 30, None) == -5
    assert lib.sthip_linear_forward_prepared(w, w, buf, 100, None, w, 1024, 1024, 1024, 2, 1, None, 0, None) == -4
    assert lib.sthip_linear_forward_prepared(w, w, None, 1 << 30, None, w, 1024, 1024, 1024, 2, 1, None, 0, None) == -5
    assert lib.sthip_linear_forward_prepared(w, w, buf, 1 << 30, None, w, 1024, 1024, 1024, 0, 1, None, 0, None) == -1


def test_weight_sums_holder_survives_copy_and_pickle():
    """A layer that keeps weight sums can be deep-copied and pickled: the copy starts empty."""
    import copy
    import pickle
    import strassen_hip
    held = strassen_hip.WeightSums()
    held._key, held._sums = ("stale",), object()
    for twin in (copy.deepcopy(held), pickle.loads(pickle.dumps(held))):
        assert twin._key is None and twin._sums is None and twin._owner is None


def test_reference_recursion_depth():
    from _levels import practical_levels, reference_levels
    # fixed_strassen.py:71-114 traced by hand
    assert reference_levels(8192, 1) == 1 and reference_levels(8192, 2) == 2 and reference_levels(8192, 3) == 3
    assert reference_levels(16, 1) == 0          # n <= 16 -> classical (:20-21)
    assert reference_levels(32, 2) == 1          # halves of 16 are multiplied classically
    assert reference_levels(64, 7) == 5          # the D=64, depth=7 demo (:173-184) stops at mid == 2
    assert practical_levels(64, 5) == 1 and practical_levels(8192, 3) == 3 and practical_levels(32, 1) == 0


def test_cpu_tensors_and_bad_shapes_are_refused():
    import fixed_strassen
    import fixed_strassen_fp32_agg
    import strassen
    import strassen_2_layer  # noqa: F401
    from model.layers import LinearStrassen, replace_linear_with_strassen  # noqa: F401
    assert fixed_strassen_fp32_agg.agg_dtype == torch.float32
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        fixed_strassen._strassen_base(torch.zeros(32, 32), torch.zeros(32, 32))
    with pytest.raises(ValueError, match="square"):
        strassen.strassen_matmul_two_layers(torch.zeros(8, 4), torch.zeros(4, 8))
    with pytest.raises(ValueError, match="divisible by 4"):
        strassen.strassen_matmul_two_layers(torch.zeros(6, 6), torch.zeros(6, 6))
    with pytest.raises(AssertionError, match="square and a power of 2"):
        LinearStrassen(96, 96, device="cpu")
    lin = LinearStrassen(64, 64, device="cpu")
    with pytest.raises(ValueError, match="Cannot pad input"):
        lin(torch.zeros(65, 64))


def test_product_code_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "strassen-triton_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)


def test_measured_cutoff_rule():
    """sthip_auto_levels: host-only arithmetic.  Classical for the forward shapes of a small
    transformer, one level for its weight gradients (few output tiles, long k) and for very large
    products, more levels only beyond that; never more than max_levels."""
    from strassen_hip import _capi
    lib = _capi.load()
    bf16, f32 = 2, 0
    assert lib.sthip_auto_levels(8192, 2304, 768, bf16, 1) == 0
    assert lib.sthip_auto_levels(8192, 8192, 8192, bf16, 2) == 0
    assert lib.sthip_auto_levels(768, 768, 8192, bf16, 1) == 1
    assert lib.sthip_auto_levels(2304, 768, 8192, bf16, 1) == 1
    assert lib.sthip_auto_levels(3072, 768, 8192, bf16, 1) == 0        # 144 output tiles: the classical kernel fills enough CUs
    assert lib.sthip_auto_levels(768, 768, 2048, bf16, 1) == 0         # k too short to pay for the passes
    assert lib.sthip_auto_levels(16384, 16384, 16384, bf16, 3) == 0    # within 2 % of the classical kernel either way
    assert lib.sthip_auto_levels(20480, 20480, 20480, bf16, 3) == 1
    assert lib.sthip_auto_levels(32768, 32768, 32768, bf16, 3) == 2
    assert lib.sthip_auto_levels(65536, 65536, 65536, bf16, 3) == 2    # a third 16-bit level would run in fp32 by default
    assert lib.sthip_auto_levels(32768, 32768, 32768, bf16, 1) == 1
    assert lib.sthip_auto_levels(8192, 8192, 8192, f32, 3) == 2 and lib.sthip_auto_levels(8192, 8192, 4096, f32, 3) == 1
    assert lib.sthip_auto_levels(2048, 4096, 2048, f32, 3) == 0      # the classical product on 64 x 64 tiles is faster
    assert lib.sthip_auto_levels(16384, 16384, 16384, f32, 3) == 2
    assert lib.sthip_auto_levels(4096, 4096, 4096, f32, 3) == 0
    assert lib.sthip_auto_levels(768, 768, 8192, f32, 1) == 0
    assert lib.sthip_auto_levels(8192, 8192, 8192, bf16, 0) == 0 and lib.sthip_auto_levels(0, 8, 8, bf16, 1) == 0


class _HostEvent:
    """Stand-in for torch.cuda.Event on a machine without a GPU: wall-clock stamps."""

    def __init__(self, enable_timing=False):
        self.t = 0.0

    def record(self):
        import time
        self.t = time.perf_counter()

    def synchronize(self):
        pass

    def elapsed_time(self, other):
        return (other.t - self.t) * 1e3 + 1e-3


def test_cutoff_table_host_logic(monkeypatch, capsys):
    """main_profiling.profile_cutoff with the GPU taken out: tensors on the CPU, host clock for events, and a stand-in for
    strassen_hip.gemm that checks how it is called (positional out, `levels` / `algo` / `workspace` / `schedule` keywords, a workspace of
    at least the size the library's own query returns).  What is left is the table's own logic: one classical column and
    one per level, `best` = the fastest column, `rule` = the library's sthip_auto_levels (the real one, host arithmetic)."""
    import main_profiling as mp
    import strassen_hip
    monkeypatch.setattr(torch.cuda, "Event", _HostEvent)
    monkeypatch.setattr(torch.cuda, "empty_cache", lambda: None)
    for name in ("randn", "empty"):
        real = getattr(torch, name)
        monkeypatch.setattr(torch, name, (lambda real: lambda *a, **k: real(*a, **{kk: v for kk, v in k.items() if kk != "device"}))(real))
    calls = []

    def gemm(a, b, out=None, *, algo="strassen", levels=1, workspace=None, schedule="auto"):
        assert out is not None and out.shape == (a.shape[0], b.shape[1]) and out.dtype == a.dtype
        lv = 0 if algo == "classic" else levels
        assert lv == 0 or schedule == "fast"   # the table times 16-bit products at every level
        need = strassen_hip.workspace_bytes(a, b, levels=lv, schedule=schedule) if lv else 0
        assert algo in ("classic", "strassen") and (lv == 0 or (workspace is not None and workspace.numel() >= need))
        calls.append((tuple(a.shape), tuple(b.shape), tuple(b.stride()), lv))
        out.copy_(torch.matmul(a.float(), b.float()))
        return out

    monkeypatch.setattr(strassen_hip, "gemm", gemm)
    rows = mp.profile_cutoff(torch.bfloat16, [(128, 128, 128), (256, 128, 64)], max_levels=2, b_transposed=True, runs=4)
    assert [(r["M"], r["N"], r["K"]) for r in rows] == [(128, 128, 128), (256, 128, 64)]
    for r in rows:
        assert len(r["level_ms"]) == 3 and all(t > 0 for t in r["level_ms"]) and r["std_ms"] > 0
        assert r["best_levels"] == min(range(3), key=lambda l: r["level_ms"][l])
        assert r["rule_levels"] == strassen_hip.auto_levels(r["M"], r["N"], r["K"], torch.bfloat16, 2) == 0
    assert {c[3] for c in calls} == {0, 1, 2}
    assert all(c[2] == (1, c[1][0]) for c in calls)   # B is the transposed view of an N x K matrix
    calls.clear()
    rows = mp.profile_cutoff(torch.float32, [(128, 64, 128)], max_levels=3, runs=2)
    assert len(rows[0]["level_ms"]) == 4 and {c[3] for c in calls} == {0, 1, 2, 3}
    assert all(c[2] == (64, 1) for c in calls)
    out = capsys.readouterr().out
    assert out.count("M x N x K") == 2 and "128x64x128" in out and "3 level ms" in out
    # the shapes --cutoff --max-n 32768 walks, and the level count it asks for
    assert max(max(s) for s in mp._CUTOFF_SHAPES) == 32768 and all(len(s) == 3 for s in mp._CUTOFF_SHAPES)
