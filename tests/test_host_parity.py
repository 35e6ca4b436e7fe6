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
import subprocess

import pytest
import torch

from oracle import strassen_oracle as O
from test_kernel_host_model import _clang

pytestmark = pytest.mark.skipif(_clang() is None, reason="no clang++ for the host build")

DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
ALGO = {"classic": 0, "strassen": 1, "winograd": 2}
TOL = {torch.float32: 1e-5, torch.float16: 2e-2, torch.bfloat16: 2e-2}
FULL = bool(os.environ.get("STHIP_HOST_FULL"))
BF, HF, SG = torch.bfloat16, torch.float16, torch.float32
ALGOS = ["classic", "strassen", "winograd"]


def _name(v):
    """Readable test ids: bf16, 512x256x384, NT ..."""
    if isinstance(v, torch.dtype):
        return {BF: "bf16", HF: "fp16", SG: "fp32"}[v]
    if isinstance(v, tuple):
        return "x".join(str(x) for x in v)
    return None


def _grid(full, short):
    """The whole grid of cases, or the part of it that the default run keeps."""
    return full if FULL else short



@pytest.fixture(scope="module")
def cli(host_builds, tmp_path_factory):
    return host_builds("library")["library_cli.cpp"], str(tmp_path_factory.mktemp("jobs"))


def _strides3(t):
    if t.dim() == 2:
        return (0, t.stride(0), t.stride(1))
    return (t.stride(0), t.stride(1), t.stride(2))


class Script:
    """Statements for tests/host_model/library_cli.cpp: tensors become buffers of "device" memory (their whole storage, so
    views keep their strides), calls name them, results are read back into the tensors after run()."""

    timeout = 900   # seconds for one run of the driver (tests/test_host_configs.py raises it)

    def __init__(self, cli):
        self.exe, self.tmp = cli
        self.lines, self.back, self.count = [], [], 0

    def buf(self, t, back=False):
        if t is None:
            return "-"
        name = "b%d" % self.count
        self.count += 1
        s = t.untyped_storage()
        path = os.path.join(self.tmp, name + ".bin")
        with open(path, "wb") as f:
            f.write(ctypes.string_at(s.data_ptr(), s.nbytes()))
        self.lines.append("buf %s %d %s" % (name, s.nbytes(), path))
        if back:
            self.back.append((name, t))
        off = t.storage_offset() * t.element_size()
        return name + "+%d" % off if off else name

    def add(self, *words):
        self.lines.append(" ".join(str(int(w)) if isinstance(w, bool) else str(w) for w in words))

    def workspace(self, batch, M, N, K, dt, odt, algo, levels):
        name = "w%d" % self.count
        self.count += 1
        self.add("wsbuf", name, batch, M, N, K, dt, odt, algo, levels)
        return name

    def run(self):
        for name, _ in self.back:
            self.add("save", name, os.path.join(self.tmp, name + ".out"))
        path = os.path.join(self.tmp, "script.txt")
        with open(path, "w") as f:
            f.write("\n".join(self.lines) + "\n")
        r = subprocess.run([self.exe, path], capture_output=True, text=True, timeout=self.timeout)
        assert r.returncode == 0, r.stderr[-2000:]
        for name, t in self.back:
            data = open(os.path.join(self.tmp, name + ".out"), "rb").read()
            ctypes.memmove(t.untyped_storage().data_ptr(), data, len(data))


SCHEDULE = {"auto": 0, "reference": 1 << 4, "fast": 2 << 4}   # enum sthip_schedule, OR-ed into the algo argument


def host_gemm(cli, A, B, algo="strassen", levels=1, out_dtype=None, out=None, accumulate=False, workspace=True, tile=None, cus=4,
              static=False, schedule="auto"):
    """strassen_hip.gemm on the host build: C = A B (or C += A B) through sthip_gemm, or sthip_gemm_static."""
    batch = A.shape[0] if A.dim() == 3 else 1
    M, K = A.shape[-2:]
    N = B.shape[-1]
    out_dtype = out_dtype or (out.dtype if out is not None else A.dtype)
    C = out if out is not None else torch.full((batch, M, N) if A.dim() == 3 else (M, N), 99.0).to(out_dtype)
    sc = Script(cli)
    sc.add("units", cus)
    sc.add("tile", tile or "-")
    code = ALGO[algo] | SCHEDULE[schedule]
    args = [sc.buf(A), sc.buf(B), sc.buf(C, back=True), batch, M, N, K, *_strides3(A), *_strides3(B), *_strides3(C),
            DT[A.dtype], DT[out_dtype], code, levels, accumulate]
    if static:
        sc.add("gemm_static", *args)
    else:
        sc.add("gemm", *args, sc.workspace(batch, M, N, K, DT[A.dtype], DT[out_dtype], code, levels) if workspace else "-")
    sc.run()
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
            [(d, a, *s) for d in (HF, SG) for a in ("strassen", "winograd") for s in KAT_SHAPES[:3]] + [(SG, "classic", *KAT_SHAPES[1]), (SG, "classic", *KAT_SHAPES[0])])


@pytest.mark.parametrize("dtype,algo,ta,tb,shape", KAT, ids=_name)
def test_integer_kat_exact(cli, dtype, algo, ta, tb, shape):
    """Entries in [-2, 2]: the fp32 result must equal the fp64 classical product bit for bit (test_gpu_parity.py:65)."""
    M, N, K = shape
    A, B = _ints((M, K), 1, dtype=dtype), _ints((K, N), 2, dtype=dtype)
    C = host_gemm(cli, _layout(A, ta), _layout(B, tb), algo=algo, levels=1, out_dtype=torch.float32)
    assert torch.equal(C.double(), A.double() @ B.double())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("algo", ["classic", "strassen", "winograd"])
@pytest.mark.parametrize("shape", [(256, 256, 128), (96, 40, 100)], ids=_name)
def test_integer_kat_exact_native_output(cli, dtype, algo, shape):
    M, N, K = shape
    A, B = _ints((M, K), 3, -1, 1, dtype), _ints((K, N), 4, -1, 1, dtype)
    C = host_gemm(cli, A, B, algo=algo, levels=1)
    assert C.dtype == dtype and torch.equal(C.double(), A.double() @ B.double())


DEEP = _grid([(d, l, s) for d in (BF, SG) for l, s in [(2, (512, 512, 512)), (2, (300, 260, 200)), (3, (512, 512, 512)), (2, (67, 35, 129))]],
             [(BF, 2, (512, 512, 512)), (BF, 2, (67, 35, 129)), (HF, 2, (128, 192, 64)), (SG, 2, (67, 35, 129))])


@pytest.mark.parametrize("dtype,levels,shape", DEEP, ids=_name)
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


@pytest.mark.parametrize("tile,dtype,algo", TILE_CASES, ids=_name)
def test_every_pipelined_tile_exact(cli, tile, dtype, algo):
    """Every tile of the pipelined paths, forced, on a problem it fits (test_gpu_parity.py:389)."""
    M, N, K = 512, 512, 256
    A, B = _ints((M, K), 31, -1, 1, dtype), _ints((K, N), 32, -1, 1, dtype)
    C = host_gemm(cli, A, _layout(B, tile != "256x128"), algo=algo, levels=1, out_dtype=torch.float32, tile=tile)
    assert torch.equal(C.double(), A.double() @ B.double())


GAUSS_SHAPES = [(1, (512, 512, 256), "256x256"), (1, (384, 256, 320), None), (2, (512, 512, 512), None)]
GAUSS = _grid([(d, *g) for d in (BF, HF, SG) for g in GAUSS_SHAPES], [(d, *g) for d in (BF, HF) for g in GAUSS_SHAPES] + [(SG, *GAUSS_SHAPES[1])])


@pytest.mark.parametrize("dtype,levels,shape,tile", GAUSS, ids=_name)
def test_gaussian_against_the_oracle(cli, dtype, levels, shape, tile):
    """N(0, 1/K) inputs against the oracle's recursion with fp32 aggregation, the tolerances of test_gpu_parity.py."""
    M, N, K = shape
    A, B = _gauss((M, K), 41, 1.0, dtype), _gauss((K, N), 42, K ** -0.5, dtype)
    C = host_gemm(cli, A, B, algo="strassen", levels=levels, tile=tile if dtype != torch.float32 else None)
    want = O.strassen_general(A, B, levels=levels, base_dtype=dtype, fp32_agg=True)
    assert O.rel_fro(C.double(), want.double()) <= TOL[dtype]
    assert O.rel_fro(C.double(), A.double() @ B.double()) <= TOL[dtype]



# measured on the host build: 4.6e-5 (bf16, three levels), 1.8e-5 (fp16), 4.5e-5 (bf16, two levels, reference), 2.0e-2 (bf16,
# three levels, fast), 9.2e-3 (bf16, two levels, fast)
SCHEDULES = [(BF, 128, 3, "auto", 2e-4), (BF, 128, 2, "reference", 2e-4)]


@pytest.mark.parametrize("dtype,n,depth,schedule,bound",
                         _grid(SCHEDULES + [(BF, 256, 3, "fast", 3e-2), (HF, 256, 3, "auto", 1e-4), (BF, 256, 2, "auto", 2e-2)], SCHEDULES), ids=_name)
def test_cast_schedule_below_the_first_level(cli, dtype, n, depth, schedule, bound):
    """The reference rounds the first level's sums to base_dtype and runs everything deeper in fp32
    (fixed_strassen_fp32_agg.py:87-113; the oracle reproduces its outputs bit for bit, tests/test_golden_reference.py).
    The library does the same from three levels on, and at two when asked (STHIP_SCHEDULE_REFERENCE): what is left is fp32
    summation order, seen through the final rounding -- a few entries one unit in the last place apart, far inside the
    2e-2 bound.  STHIP_SCHEDULE_FAST (the default at two levels) rounds every level: inside 2e-2 at two levels, not at
    three, which is why three levels do not take it unasked."""
    A, B = _gauss((n, n), 151, n ** -0.5, dtype), _gauss((n, n), 152, n ** -0.5, dtype)
    C = host_gemm(cli, A, B, levels=depth, schedule=schedule)
    want = O.strassen_matmul_n_layers(A, B, depth, dtype, fp32_agg=True)
    err = O.rel_fro(C.double(), want.double())
    print(f"{depth} levels {dtype} schedule {schedule}: {err:.3e} from the oracle, {(C != want).float().mean():.2e} of the entries differ")
    assert err <= bound
    if schedule != "fast" and (depth >= 3 or schedule == "reference"):
        assert (C != want).float().mean() <= 0.02


@pytest.mark.parametrize("dtype,shape,levels,out_dtype,tile", [
    (BF, (512, 512, 256), 1, BF, "256x256"),    # recombination pass adds into a 16-bit C
    (HF, (512, 512, 256), 1, SG, "256x256"),    # products kept in fp32, recombination adds into an fp32 C
    (BF, (256, 256, 128), 1, BF, "128x128g"),
    (HF, (512, 256, 128), 1, HF, "256x128"),    # recombined in registers around the parked tile, added into a 16-bit C
    (HF, (33, 17, 65), 1, HF, None),            # fused kernel, edge tiles, element-wise read-modify-write
    (BF, (132, 100, 72), 2, BF, None),          # two levels by host recursion, 16-bit C
    (SG, (256, 256, 128), 1, SG, "256x128"),    # fp32: sums written once, the seven products as one batched launch
    (SG, (128, 192, 64), 1, SG, "64x64")], ids=_name)
def test_accumulate_on_every_path(cli, dtype, shape, levels, out_dtype, tile):
    M, N, K = shape
    A, B = _ints((M, K), 101, -1, 1, dtype), _ints((K, N), 102, -1, 1, dtype)
    C0 = _ints((M, N), 103, -4, 4, out_dtype)
    C = host_gemm(cli, A, B, out=C0.clone(), algo="strassen", levels=levels, accumulate=True, tile=tile)
    assert torch.equal(C.double(), C0.double() + A.double() @ B.double())


@pytest.mark.parametrize("dtype,shape", [(BF, (256, 256, 256)), (SG, (128, 64, 96)), (HF, (100, 36, 52))], ids=_name)
def test_winograd_two_levels(cli, dtype, shape):
    M, N, K = shape
    A, B = _ints((M, K), 111, -1, 1, dtype), _ints((K, N), 112, -1, 1, dtype)
    C = host_gemm(cli, A, B, algo="winograd", levels=2, out_dtype=SG)
    assert torch.equal(C.double(), A.double() @ B.double())


LARGE = [("classic", 0, SG, (14, 1024, 1024, 32)),     # fp32 classical on the walking 256 x 256 kernel: 224 tiles
         ("strassen", 1, SG, (1, 4096, 2048, 64)),     # fp32 one level: sums, one grouped launch of 7 x 32 tiles, recombination
         ("winograd", 1, SG, (1, 4096, 2048, 64)),
         ("strassen", 2, SG, (1, 3072, 2048, 128)),    # fp32 two levels as three launches: 49 x 6 tiles
         ("strassen", 2, BF, (1, 1024, 1024, 4096)),   # 16-bit two levels with the 49 products on 256 x 256 tiles (quarter k >= 1024)
         ("strassen", 3, BF, (1, 1024, 1024, 512))]    # three levels: seven two-level calls with fp32 results inside


@pytest.mark.skipif(not FULL, reason="a minute or two each on the host: STHIP_HOST_FULL=1")
@pytest.mark.parametrize("algo,levels,dtype,shape", LARGE, ids=_name)
def test_paths_that_only_large_problems_take(cli, algo, levels, dtype, shape):
    batch, M, N, K = shape
    lead = (batch,) if batch > 1 else ()
    A, B = _ints(lead + (M, K), 121, -1, 1, dtype), _ints(lead + (K, N), 122, -1, 1, dtype)
    if dtype != SG and levels == 2:
        # the 49-product form needs a result in the operand type and rounds every product to it: one entry in eight kept, so
        # that sums over k = 4096 of products of up to four-term sums stay far below 256 and every rounding is exact
        g = torch.Generator().manual_seed(123)
        A, B = A * (torch.rand(A.shape, generator=g) < 0.125), B * (torch.rand(B.shape, generator=g) < 0.125)
        C = host_gemm(cli, A, B, algo=algo, levels=levels, cus=8)
    else:
        C = host_gemm(cli, A, B, algo=algo, levels=levels, out_dtype=SG, cus=8, schedule="fast")
    assert torch.equal(C.double(), A.double() @ B.double())


@pytest.mark.skipif(not FULL, reason="four minutes on the host: STHIP_HOST_FULL=1")
def test_configuration_1_at_full_size(cli):
    """One-level Strassen, 1024^3 fp32, N(0,1) from seeds 1234 / 1235 -- the first configuration at its real shape, on the kernel
    it takes on the card (64 x 64 tiles, the quadrant sums formed in the operand loads) -- against the oracle's restatement of
    fixed_strassen.py:11-57 at the configuration's bound.  Measured on the host build: 7.2e-7 (4.3e-7 from fp64)."""
    n = 1024
    A = torch.randn(n, n, generator=torch.Generator().manual_seed(1234))
    B = torch.randn(n, n, generator=torch.Generator().manual_seed(1235))
    C = host_gemm(cli, A, B, levels=1, cus=8)
    assert O.rel_fro(C.double(), O.strassen_base(A, B).double()) <= 1e-5
    assert O.rel_fro(C.double(), A.double() @ B.double()) <= 1e-5


@pytest.mark.parametrize("stages", _grid([47, 31], [47]))
def test_other_launch_forms_give_the_same_bits(cli, stages):
    """The 256 x 256 kernel with one workgroup per tile instead of workgroups that walk their tiles (stage bit 5), and the
    whole level as ONE launch whose workgroups are sums, product tiles and recombination ordered by counters (bit 4; the host
    runs the workgroups one after the other in launch order, which is the order the counters assume)."""
    A, B = _gauss((512, 256), 131, 1.0, BF), _gauss((256, 512), 132, 1 / 16, BF)
    outs = []
    for mask in (15, stages):
        C = torch.zeros(512, 512, dtype=BF)
        sc = Script(cli)
        sc.add("tile", "256x256")
        sc.add("stages", mask)
        ws = sc.workspace(1, 512, 512, 256, DT[BF], DT[BF], 1, 1)
        sc.add("gemm", sc.buf(A), sc.buf(B), sc.buf(C, back=True), 1, 512, 512, 256, *_strides3(A), *_strides3(B), *_strides3(C),
               DT[BF], DT[BF], 1, 1, 0, ws)
        if mask & 16:   # the debug query: no workgroup gave up waiting, each product counted its one tile
            sc.add("one_launch_counters", ws, 512, 512, 256, 1)
        sc.run()
        outs.append(C)
    assert torch.equal(outs[0], outs[1])
    assert O.rel_fro(outs[0].double(), A.double() @ B.double()) <= 2e-2


def test_two_levels_by_host_recursion(cli):
    """Stage bit 3 cleared: two levels never run as one 49-product launch but as seven one-level calls with fp32 results."""
    A, B = _ints((512, 512), 141, -1, 1, BF), _ints((512, 256), 142, -1, 1, BF)
    C = torch.zeros(512, 256, dtype=SG)
    sc = Script(cli)
    sc.add("stages", 7)
    sc.add("gemm", sc.buf(A), sc.buf(B), sc.buf(C, back=True), 1, 512, 256, 512, *_strides3(A), *_strides3(B), *_strides3(C),
           DT[BF], DT[SG], 1, 2, 0, sc.workspace(1, 512, 256, 512, DT[BF], DT[SG], 1, 2))
    sc.run()
    assert torch.equal(C.double(), A.double() @ B.double())


def _random_call(case, deep=False):
    """A seeded random sthip_gemm call: sizes aligned to tiles, to 8, or arbitrary; either layout of A and B; leading dimensions
    with padding; views that start 2 or 16 bytes into their storage; batch; fp32 or native result; accumulate; with and without
    workspace; a forced tile; 1 .. 16 compute units.  deep: 16-bit operands, two or three levels, either rounding schedule
    or the default."""
    import random
    rnd = random.Random((5000 if deep else 1000) + case)
    dt = rnd.choice([BF, HF] if deep else [BF, BF, HF, SG])
    algo = rnd.choice(["strassen", "strassen", "winograd"] if deep else ["classic", "strassen", "strassen", "winograd"])
    levels = rnd.choice([2, 3, 3]) if deep else 0 if algo == "classic" else rnd.choice([1, 1, 1, 2])
    kind = rnd.random()
    if kind < 0.35:
        M, N, K = (rnd.choice([64, 128]) * rnd.randint(1, 3) for _ in range(3))
    elif kind < 0.65:
        M, N, K = (8 * rnd.randint(1, 30) for _ in range(3))
    else:
        M, N, K = (rnd.randint(1, 200) for _ in range(3))
    if dt == SG:
        K = min(K, 96)
    batch = rnd.choice([0, 0, 0, 2])
    opts = dict(algo=algo, levels=levels, accumulate=rnd.random() < 0.3, workspace=rnd.random() < 0.8 or levels >= 2,
                tile=rnd.choice([None, None, None, "128x128", "128x128g", "256x128", "256x256", "64x64"]), cus=rnd.choice([1, 2, 4, 8, 16]))
    if deep:
        opts["schedule"] = rnd.choice(["auto", "reference", "fast"])
    g = torch.Generator().manual_seed(case)

    def make(rows, cols, transposed, dtype, lo, hi):
        pad, off = rnd.choice([0, 0, 8, 3]), rnd.choice([0, 0, 0, 8, 1])
        r, c = (cols, rows) if transposed else (rows, cols)
        flat = torch.randint(lo, hi + 1, (off + (batch or 1) * r * (c + pad),), generator=g).to(dtype)
        v = flat[off:].view(*((batch,) if batch else ()), r, c + pad)[..., :c]
        return v.transpose(-1, -2) if transposed else v

    A = make(M, K, rnd.random() < 0.4, dt, -1, 1)
    B = make(K, N, rnd.random() < 0.5, dt, -1, 1)
    C = make(M, N, False, rnd.choice([dt, SG]), -3, 3)
    return A, B, C, opts


@pytest.mark.parametrize("case", range(_grid(200, 16)))
def test_random_calls_exact(cli, case):
    A, B, C, opts = _random_call(case)
    C0, around = C.clone(), C._base.clone()
    host_gemm(cli, A, B, out=C, **opts)
    assert torch.equal(C.double(), A.double() @ B.double() + (C0.double() if opts["accumulate"] else 0)), opts
    after = C._base.clone()     # nothing outside the view of C (padding of its rows, the elements in front of it) was written
    for whole in (around, after):
        whole.as_strided(C.size(), C.stride(), C.storage_offset()).zero_()
    assert torch.equal(around, after), opts


@pytest.mark.parametrize("case", _grid(list(range(60)), [4]))   # twenty seconds and more each: the default run keeps one
def test_random_deep_calls_exact(cli, case):
    """The same for two and three levels of 16-bit operands on either rounding schedule (inner products in fp32, or every
    level in the operand type) and on the default: small integers come out exact on all of them."""
    A, B, C, opts = _random_call(case, deep=True)
    C0, around = C.clone(), C._base.clone()
    host_gemm(cli, A, B, out=C, **opts)
    assert torch.equal(C.double(), A.double() @ B.double() + (C0.double() if opts["accumulate"] else 0)), opts
    after = C._base.clone()
    for whole in (around, after):
        whole.as_strided(C.size(), C.stride(), C.storage_offset()).zero_()
    assert torch.equal(around, after), opts


# ---- the other entry points of include/strassen_hip.h (tests/test_gpu_api.py, tests/test_zz_no_alloc.py on the GPU) ----

def test_static_entry_point_on_two_calls_in_a_row(cli):
    """sthip_gemm_static against sthip_gemm, bit for bit: a first call, a smaller one with two levels, the first again."""
    A, B = _gauss((256, 256), 51, 1.0, BF), _gauss((256, 256), 52, 1 / 16, BF)
    A2, B2 = _gauss((256, 64), 53, 1.0, BF), _gauss((64, 128), 54, 1 / 8, BF)
    sc = Script(cli)
    outs = []
    for a, b, levels in ((A, B, 1), (A2, B2, 2), (A, B, 1)):
        M, K, N = *a.shape, b.shape[1]
        for static in (True, False):
            c = torch.full((M, N), 7.0).to(BF)
            outs.append(c)
            args = [sc.buf(a), sc.buf(b), sc.buf(c, back=True), 1, M, N, K, *_strides3(a), *_strides3(b), *_strides3(c), DT[BF], DT[BF], 1, levels, 0]
            sc.add("gemm_static" if static else "gemm", *args, *([] if static else [sc.workspace(1, M, N, K, DT[BF], DT[BF], 1, levels)]))
    sc.run()
    for i in (0, 2, 4):
        assert torch.equal(outs[i], outs[i + 1])
    assert torch.equal(outs[0], outs[4])
    assert O.rel_fro(outs[0].double(), A.double() @ B.double()) <= 2e-2
    assert O.rel_fro(outs[2].double(), A2.double() @ B2.double()) <= 2e-2


def test_static_entry_point_refuses_what_does_not_fit(cli):
    sc = Script(cli)      # two levels at 8192^3 bf16 need more than the 144 MiB buffer; nothing is launched, no operand is read
    tiny = torch.zeros(64, dtype=BF)
    sc.add("expect", -4)
    sc.add("gemm_static", sc.buf(tiny), sc.buf(tiny), sc.buf(tiny), 1, 8192, 8192, 8192, 0, 8192, 1, 0, 8192, 1, 0, 8192, 1, DT[BF], DT[BF], 1, 2, 0)
    sc.run()


@pytest.mark.parametrize("dtype,n,levels", _grid([(BF, 256, 1), (SG, 128, 2), (HF, 256, 2), (BF, 64, 3)], [(BF, 256, 1), (SG, 128, 2), (HF, 256, 2)]),
                         ids=_name)
def test_n_layers_entry_point(cli, dtype, n, levels):
    """sthip_strassen_matmul_n_layers: square operands, B a transposed view (test_gpu_api.py:43)."""
    A, Bt = _ints((n, n), 61, -1, 1, dtype), _ints((n, n), 62, -1, 1, dtype)
    C = torch.zeros(n, n, dtype=dtype)
    sc = Script(cli)
    sc.add("n_layers", sc.buf(A), sc.buf(Bt), sc.buf(C, back=True), n, n, 1, 1, n, DT[dtype], levels, sc.workspace(1, n, n, n, DT[dtype], DT[dtype], 1, levels))
    sc.run()
    assert torch.equal(C.double(), A.double() @ Bt.double().t())


@pytest.mark.parametrize("algo,levels", [("strassen", 1), ("strassen", 2), ("classic", 0)], ids=_name)
def test_run_accumulate_entry_point(cli, algo, levels):
    """sthip_run_accumulate: C += A B with fp16 operands and an fp32 C, batched (the contract of the reference's launchers)."""
    A, B = _ints((2, 128, 64), 71, -1, 1, HF), _ints((2, 64, 256), 72, -1, 1, HF)
    C0 = _ints((2, 128, 256), 73, -3, 3, SG)
    C = C0.clone()
    sc = Script(cli)
    sc.add("run_accumulate", sc.buf(A), sc.buf(B), sc.buf(C, back=True), 2, 128, 256, 64, DT[HF], DT[SG], ALGO[algo], levels,
           sc.workspace(2, 128, 256, 64, DT[HF], DT[SG], ALGO[algo], levels))
    sc.run()
    assert torch.equal(C.double(), C0.double() + A.double() @ B.double())


@pytest.mark.parametrize("dtype,rows,D,levels,bias,tile", [(BF, 256, 256, 1, True, None), (HF, 100, 256, 1, True, None), (BF, 512, 512, 2, False, None),
                                                          (SG, 77, 128, 1, True, None), (HF, 512, 512, 1, True, "256x256"), (BF, 256, 256, 1, True, "128x128g")], ids=_name)
def test_linear_strassen_forward_entry_point(cli, dtype, rows, D, levels, bias, tile):
    """sthip_linear_strassen_forward: y = x W^T + bias with rows <= D (reference model/layers.py:246-274 pads x instead)."""
    x, W = _ints((rows, D), 81, -1, 1, dtype), _ints((D, D), 82, -1, 1, dtype)
    b = _ints((D,), 83, -2, 2, dtype) if bias else None
    y = torch.zeros(rows, D, dtype=dtype)
    sc = Script(cli)
    sc.add("tile", tile or "-")
    sc.add("linear_strassen", sc.buf(x), sc.buf(W), sc.buf(b), sc.buf(y, back=True), rows, D, DT[dtype], levels,
           sc.workspace(1, rows, D, D, DT[dtype], DT[dtype], 1 | SCHEDULE["fast"], levels))
    sc.run()
    assert torch.equal(y.double(), x.double() @ W.double().t() + (b.double() if bias else 0))


PREPARED = [(BF, 1, 256, 256, 512, True), (HF, 2, 512, 512, 512, False), (BF, -2, 200, 136, 72, True)]


@pytest.mark.parametrize("dtype,levels,rows,d_in,d_out,bias", _grid(PREPARED + [(BF, 3, 512, 512, 1024, True)], PREPARED), ids=_name)
def test_linear_forward_and_prepared_sums_same_bits(cli, dtype, levels, rows, d_in, d_out, bias):
    """sthip_linear_forward on a layer of any shape; where sums of the weight can be kept, the forward that reads them gives the
    same bits, and does read them: with the sums of another weight it gives another result (test_gpu_api.py:264)."""
    x, W = _gauss((rows, d_in), 91, 1.0, dtype), _gauss((d_out, d_in), 92, d_in ** -0.5, dtype)
    b = _gauss((d_out,), 93, 1.0, dtype) if bias else None
    ys = [torch.zeros(rows, d_out, dtype=dtype) for _ in range(3)]
    sc = Script(cli)
    bx, bw, bb = sc.buf(x), sc.buf(W), sc.buf(b)
    ws = sc.workspace(1, rows, d_out, d_in, DT[dtype], DT[dtype], 1 | SCHEDULE["fast"], abs(levels))   # as the header says for this entry
    sc.add("linear", bx, bw, bb, sc.buf(ys[0], back=True), rows, d_in, d_out, DT[dtype], levels, ws)
    if levels > 0:
        other = sc.buf(W.flip(0).contiguous())
        for w_for_sums, y in ((bw, ys[1]), (other, ys[2])):
            sc.add("sumsbuf", "sums", d_in, d_out, DT[dtype], levels)
            sc.add("prepare", w_for_sums, d_in, d_out, DT[dtype], levels, "sums")
            sc.add("linear_prepared", bx, bw, "sums", bb, sc.buf(y, back=True), rows, d_in, d_out, DT[dtype], levels, ws)
    sc.run()
    want = x.double() @ W.double().t() + (b.double() if bias else 0)
    assert O.rel_fro(ys[0].double(), want) <= TOL[dtype]
    if levels > 0:
        assert torch.equal(ys[1], ys[0])
        assert not torch.equal(ys[2], ys[0])
