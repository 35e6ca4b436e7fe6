"""The library against the oracle WITHOUT a GPU: libstrassen_hip's sources compiled for the host
(tests/host_model/, see tests/test_kernel_host_model.py) and sthip_gemm called through a small command-line
driver with the tensors' storage as "device" memory.  The cases mirror tests/test_gpu_parity.py at sizes a CPU
finishes in seconds: exact on small-integer inputs, within the same tolerances on seeded Gaussian inputs
(fp32 <= 1e-5, bf16 / fp16 <= 2e-2 relative Frobenius error against the oracle's fp32-aggregating recursion).
One host thread stands for one lane, so a 512^3 product takes seconds: the default run keeps about a minute's worth of
cases, STHIP_HOST_FULL=1 in the environment runs the whole grid (five to six minutes on 8 cores).
"""
import ctypes
import os
import struct
import subprocess

import pytest
import torch

from oracle import strassen_oracle as O
from test_kernel_host_model import _clang

pytestmark = pytest.mark.skipif(_clang() is None, reason="no clang++ for the host build")

DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
ALGO = {"classic": 0, "strassen": 1, "winograd": 2}
TILE = {None: 0, "128x128": 1, "256x128": 2, "128x128g": 3, "256x256": 4, "64x64": 5}
TOL = {torch.float32: 1e-5, torch.float16: 2e-2, torch.bfloat16: 2e-2}
FULL = bool(os.environ.get("STHIP_HOST_FULL"))
BF, HF, SG = torch.bfloat16, torch.float16, torch.float32
ALGOS = ["classic", "strassen", "winograd"]


def _grid(full, short):
    """The whole grid of cases, or the part of it that the default run keeps."""
    return full if FULL else short



@pytest.fixture(scope="module")
def cli(host_builds, tmp_path_factory):
    return host_builds("library")["library_cli.cpp"], str(tmp_path_factory.mktemp("jobs"))


def _storage_bytes(t):
    s = t.untyped_storage()
    return ctypes.string_at(s.data_ptr(), s.nbytes())


def _strides3(t):
    assert t.storage_offset() == 0
    if t.dim() == 2:
        return (0, t.stride(0), t.stride(1))
    return (t.stride(0), t.stride(1), t.stride(2))


def host_gemm(cli, A, B, algo="strassen", levels=1, out_dtype=None, out=None, accumulate=False, workspace=True, tile=None, cus=4):
    exe, tmp = cli
    batch = A.shape[0] if A.dim() == 3 else 1
    M, K = A.shape[-2:]
    N = B.shape[-1]
    out_dtype = out_dtype or (out.dtype if out is not None else A.dtype)
    C = out if out is not None else torch.full((batch, M, N) if A.dim() == 3 else (M, N), 99.0).to(out_dtype)
    a, b, c = _storage_bytes(A), _storage_bytes(B), _storage_bytes(C)
    hdr = struct.pack("<4q9q3q8i", batch, M, N, K, *_strides3(A), *_strides3(B), *_strides3(C), len(a), len(b), len(c),
                      DT[A.dtype], DT[out_dtype], ALGO[algo], levels, int(accumulate), int(workspace), TILE[tile], cus)
    job, res = os.path.join(tmp, "job.bin"), os.path.join(tmp, "out.bin")
    with open(job, "wb") as f:
        f.write(hdr + a + b + c)
    r = subprocess.run([exe, job, res], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    data = open(res, "rb").read()
    ctypes.memmove(C.untyped_storage().data_ptr(), data, len(data))
    return C


def _ints(shape, seed, lo=-2, hi=2, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, shape, generator=g).to(dtype)


def _gauss(shape, seed, scale, dtype):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _layout(X, transposed):
    return X.transpose(-1, -2).contiguous().transpose(-1, -2) if transposed else X.contiguous()


KAT_SHAPES = [(False, False, (256, 256, 256)), (False, True, (200, 136, 72)), (True, False, (33, 17, 65)), (True, True, (130, 258, 2)),
              (False, False, (1, 5, 3)), (True, True, (512, 256, 384))]
KAT = _grid([(d, a, *s) for d in (BF, HF, SG) for a in ALGOS for s in KAT_SHAPES],
            [(BF, a, *s) for a in ALGOS for s in KAT_SHAPES[:5]] + [(BF, "strassen", *KAT_SHAPES[5])] +
            [(d, a, *s) for d in (HF, SG) for a in ("strassen", "winograd") for s in KAT_SHAPES[:3]] + [(SG, "classic", *KAT_SHAPES[1])])


@pytest.mark.parametrize("dtype,algo,ta,tb,shape", KAT)
def test_integer_kat_exact(cli, dtype, algo, ta, tb, shape):
    """Entries in [-2, 2]: the fp32 result must equal the fp64 classical product bit for bit (test_gpu_parity.py:65)."""
    M, N, K = shape
    A, B = _ints((M, K), 1, dtype=dtype), _ints((K, N), 2, dtype=dtype)
    C = host_gemm(cli, _layout(A, ta), _layout(B, tb), algo=algo, levels=1, out_dtype=torch.float32)
    assert torch.equal(C.double(), A.double() @ B.double())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("algo", ["classic", "strassen", "winograd"])
@pytest.mark.parametrize("shape", [(256, 256, 128), (96, 40, 100)])
def test_integer_kat_exact_native_output(cli, dtype, algo, shape):
    M, N, K = shape
    A, B = _ints((M, K), 3, -1, 1, dtype), _ints((K, N), 4, -1, 1, dtype)
    C = host_gemm(cli, A, B, algo=algo, levels=1)
    assert C.dtype == dtype and torch.equal(C.double(), A.double() @ B.double())


DEEP = _grid([(d, l, s) for d in (BF, SG) for l, s in [(2, (512, 512, 512)), (2, (300, 260, 200)), (3, (512, 512, 512)), (2, (67, 35, 129))]],
             [(BF, 2, (512, 512, 512)), (BF, 2, (67, 35, 129)), (BF, 3, (256, 256, 256)), (HF, 2, (256, 320, 192)), (SG, 2, (67, 35, 129))])


@pytest.mark.parametrize("dtype,levels,shape", DEEP)
def test_integer_kat_multi_level(cli, dtype, levels, shape):
    M, N, K = shape
    A, B = _ints((M, K), 5, -1, 1, dtype), _ints((K, N), 6, -1, 1, dtype)
    C = host_gemm(cli, A, B, algo="strassen", levels=levels, out_dtype=torch.float32)
    assert torch.equal(C.double(), A.double() @ B.double())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_accumulate_and_batch(cli, dtype):
    b, M, N, K = 3, 256, 256, 128
    A, B = _ints((b, M, K), 21, -1, 1, dtype), _ints((b, K, N), 22, -1, 1, dtype)
    C0 = _ints((b, M, N), 23, -4, 4, torch.float32)
    C = host_gemm(cli, A, B, out=C0.clone(), algo="strassen", accumulate=True)
    assert torch.equal(C.double(), C0.double() + A.double() @ B.double())
    A3, B3 = _ints((b, 70, 50), 24, -1, 1, dtype), _ints((50, 30), 25, -1, 1, dtype)
    C3 = host_gemm(cli, A3, B3.unsqueeze(0).expand(b, -1, -1), algo="strassen", out_dtype=torch.float32)
    assert torch.equal(C3.double(), A3.double() @ B3.double())


TILES = ["128x128", "128x128g", "256x128", "256x256"]
TILE_CASES = _grid([(t, d, a) for t in TILES for d in (BF, HF) for a in ALGOS],
                   [(t, d, "strassen") for t in TILES for d in (BF, HF)] + [(t, BF, a) for t in TILES[2:] for a in ("classic", "winograd")] +
                   [("128x128g", HF, "winograd")])


@pytest.mark.parametrize("tile,dtype,algo", TILE_CASES)
def test_every_pipelined_tile_exact(cli, tile, dtype, algo):
    """Every tile of the pipelined paths, forced, on a problem it fits (test_gpu_parity.py:389)."""
    M, N, K = 512, 512, 256
    A, B = _ints((M, K), 31, -1, 1, dtype), _ints((K, N), 32, -1, 1, dtype)
    C = host_gemm(cli, A, _layout(B, tile != "256x128"), algo=algo, levels=1, out_dtype=torch.float32, tile=tile)
    assert torch.equal(C.double(), A.double() @ B.double())


GAUSS_SHAPES = [(1, (512, 512, 256), "256x256"), (1, (384, 256, 320), None), (2, (512, 512, 512), None)]
GAUSS = _grid([(d, *g) for d in (BF, HF, SG) for g in GAUSS_SHAPES], [(d, *g) for d in (BF, HF) for g in GAUSS_SHAPES] + [(SG, *GAUSS_SHAPES[1])])


@pytest.mark.parametrize("dtype,levels,shape,tile", GAUSS)
def test_gaussian_against_the_oracle(cli, dtype, levels, shape, tile):
    """N(0, 1/K) inputs against the oracle's recursion with fp32 aggregation, the tolerances of test_gpu_parity.py."""
    M, N, K = shape
    A, B = _gauss((M, K), 41, 1.0, dtype), _gauss((K, N), 42, K ** -0.5, dtype)
    C = host_gemm(cli, A, B, algo="strassen", levels=levels, tile=tile if dtype != torch.float32 else None)
    want = O.strassen_general(A, B, levels=levels, base_dtype=dtype, fp32_agg=True)
    assert O.rel_fro(C.double(), want.double()) <= TOL[dtype]
    assert O.rel_fro(C.double(), A.double() @ B.double()) <= TOL[dtype]
