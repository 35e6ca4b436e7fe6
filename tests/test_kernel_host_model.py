"""The 256 x 256 kernels of strassen-triton_amd/csrc/sthip_kernel4.hpp, the 256 x 128 and 128 x 128 pipelined
kernels of sthip_kernel3.hpp / sthip_kernel2.hpp (classical, and Strassen / Winograd recombined in registers), the
fused kernel of sthip_kernel.hpp (whole problems C = A B with the quadrant sums formed in registers, odd sizes included) and the 64 x 64 fp32 kernel of sthip_kernel6.hpp
compiled for the host and run on the CPU, one thread per lane (tests/host_model/kernel4_host.cpp).

The kernel headers are the library's own; only their inline-assembly statements are taken out (scheduling
hints, waits that builtins repeat, and the instructions of sthip_prims.hpp, which the host build replaces by
functions that exchange operands among the threads of a wave and copy direct-to-LDS loads by hand, at once or
at the last moment the waits allow, checking every source against the operands and every destination
against the LDS allocation).  Products of small integers must come out exact for walking and one-tile-per-
workgroup launches, both B layouts, bf16 / fp16 / fp32, plain, fp32-result and accumulating stores, a batch;
every tile id of a launch must map to a different tile (plain and XCD-chunked numbering).  Two
deliberately broken copies of the large kernel must be caught: one without the wait for the loads before the
k-step's barrier, one that moves the loader's cursor before the last load of a step; and one of the small
kernel that waits one load short.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "strassen-triton_amd", "csrc")
MODEL = os.path.join(ROOT, "tests", "host_model")
HEADERS = ("sthip_kernel.hpp", "sthip_kernel2.hpp", "sthip_kernel3.hpp", "sthip_kernel4.hpp", "sthip_kernel6.hpp")


def _clang():
    for cand in (os.environ.get("STHIP_HOST_CXX"), "/opt/rocm/lib/llvm/bin/clang++", shutil.which("clang++")):
        if cand and os.path.exists(cand):
            return cand
    return None


def strip_asm(text: str) -> str:
    """Replaces every `asm volatile(...);` statement by an empty statement."""
    out, i = [], 0
    pat = re.compile(r"\basm\s+volatile\s*\(")
    while True:
        m = pat.search(text, i)
        if not m:
            out.append(text[i:])
            return "".join(out)
        out.append(text[i:m.start()])
        j, depth, in_str = m.end(), 1, False
        while depth:
            c = text[j]
            if in_str:
                if c == "\\":
                    j += 1
                elif c == '"':
                    in_str = False
            elif c == '"':
                in_str = True
            elif c == "(":
                depth += 1
            elif c == ")":
                depth -= 1
            j += 1
        k = j
        while text[k] in " \t":
            k += 1
        assert text[k] == ";", text[m.start():k + 20]
        out.append("((void)0);")
        i = k + 1


def _build(tmp, name, mutate=None, mutate_header="sthip_kernel4.hpp", extra=()):
    inc = os.path.join(tmp, name)
    os.makedirs(inc)
    for h in HEADERS:
        text = strip_asm(open(os.path.join(CSRC, h)).read()).replace("extern __shared__", "extern")
        if mutate and h == mutate_header:
            text = mutate(text)
        open(os.path.join(inc, h), "w").write(text)
    exe = os.path.join(inc, "kernel4_host")
    cmd = [_clang(), "-std=c++17", "-O1", "-Wno-everything", "-no-pie", "-pthread", *extra, "-I", inc, "-I", MODEL,
           "-I", os.path.join(ROOT, "include"), os.path.join(MODEL, "kernel4_host.cpp"), os.path.join(MODEL, "host_runtime.cpp"),
           "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return exe


def _build_library(tmp, name, extra=(), drivers=("library_host.cpp",)):
    """Every translation unit of the library (strassen-triton_amd/build.py lists them) compiled for the host against the
    stand-in HIP runtime of tests/host_model/hip/hip_runtime.h, linked with library_host.cpp and host_runtime.cpp."""
    import glob
    import importlib.util
    from concurrent.futures import ThreadPoolExecutor
    out = os.path.join(tmp, name)
    os.makedirs(out)
    for f in glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(CSRC, "*.hip")):
        if os.path.basename(f) == "sthip_prims.hpp":   # the host build has its own (tests/host_model/sthip_prims.hpp)
            continue
        open(os.path.join(out, os.path.basename(f)), "w").write(strip_asm(open(f).read()).replace("extern __shared__", "extern"))
    spec = importlib.util.spec_from_file_location("sthip_build", os.path.join(ROOT, "strassen-triton_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    common = ["-std=c++17", "-O1", "-Wno-everything", "-pthread", *extra, "-I", MODEL, "-I", out, "-I", os.path.join(ROOT, "include")]

    def compile_unit(unit):
        obj, src, defs = unit
        r = subprocess.run([_clang(), "-x", "c++", *common, *defs, "-c", os.path.join(out, src), "-o", os.path.join(out, obj)],
                           capture_output=True, text=True)
        assert r.returncode == 0, obj + "\n" + r.stderr[-3000:]
        return os.path.join(out, obj)

    with ThreadPoolExecutor(8) as pool:
        objs = list(pool.map(compile_unit, build._units()))
    runtime = os.path.join(out, "host_runtime.o")
    r = subprocess.run([_clang(), *common, "-c", os.path.join(MODEL, "host_runtime.cpp"), "-o", runtime], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    exes = {}
    for driver in drivers:
        exes[driver] = os.path.join(out, driver[:-4])
        r = subprocess.run([_clang(), *common, "-no-pie", os.path.join(MODEL, driver), runtime, *objs, "-o", exes[driver]],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-3000:]
    return exes


def run_shares(exe, shares=4, timeout=1800):
    """The driver's cases dealt to `shares` processes that run side by side (a launch spends much of its time in barriers);
    returns the worst exit code and everything printed."""
    procs = [subprocess.Popen([exe, "%d/%d" % (i, shares)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True) for i in range(shares)]
    outs = [p.communicate(timeout=timeout) for p in procs]
    return max(abs(p.returncode) for p in procs), "".join(o[0] for o in outs), "".join(o[1] for o in outs)


needs_clang = pytest.mark.skipif(_clang() is None, reason="no clang++ (the kernel headers use ext_vector_type)")


def test_strip_asm_takes_out_whole_statements():
    src = 'a(); asm volatile("s_nop 0\\n\\t(x)" :: "s"(f(1, 2)) : "memory");\nb = asm_volatile_count;'
    assert strip_asm(src) == "a(); ((void)0);\nb = asm_volatile_count;"


@needs_clang
def test_kernels_exact_on_the_host(host_builds):
    # under AddressSanitizer where the compiler has it (operands, results and the parked tile are heap buffers), with
    # misaligned vector accesses, indices out of a static array's bounds and out-of-range shifts ending the run as well
    exe = host_builds("asan") if host_builds.ok("asan") else host_builds("plain")
    rc, out, err = run_shares(exe)
    assert "AddressSanitizer" not in err and "runtime error" not in err, err[:4000]
    assert rc == 0, out[-2000:] + err[-2000:]
    lines = [l for l in out.splitlines() if "wrong of" in l]
    # 24 launches of the pipelined kernels x 2 load timings, 6 of the fused kernel, 9 tile numberings
    assert len(lines) == 63 and all(": 0 wrong of" in l for l in lines), out
    assert out.count("ALL EXACT") == 4


@needs_clang
def test_no_data_race_under_thread_sanitizer(host_builds):
    """Lanes are threads, barriers are barriers, a direct-to-LDS load is a write by the issuing thread: an LDS
    buffer that is overwritten while another wave may still read it, or read before its barrier, is a data
    race that ThreadSanitizer reports whatever the timing of this run was."""
    if not host_builds.ok("tsan"):   # no ThreadSanitizer runtime with this compiler
        pytest.skip(host_builds.why("tsan")[-300:])
    rc, out, err = run_shares(host_builds("tsan"))
    assert "ThreadSanitizer" not in err, err[:4000]
    assert rc == 0 and out.count("ALL EXACT") == 4, out[-2000:]


@needs_clang
def test_library_through_its_c_abi_on_the_host(host_builds):
    """sthip_gemm itself, host code and kernels, on the CPU: the headline path (sums, grouped 256 x 256 products walked by
    fewer workgroups than tiles, recombination) and the two-level path (49 products) bit for bit against the cast schedule
    written out in library_host.cpp, fp32 results, the classical product, the 64 x 64 fp32 path, the fused kernel on odd
    sizes, Winograd on grouped 128 x 128 tiles accumulating into fp32."""
    rc, out, err = run_shares(host_builds("library")["library_host.cpp"], shares=3)
    assert rc == 0, out[-3000:] + err[-3000:]
    lines = [l for l in out.splitlines() if "wrong of" in l]
    assert len(lines) == 7 and all(": 0 wrong of" in l for l in lines), out
    assert out.count("ALL EXACT") == 3


def _drop_barrier(text):
    old = "                    wait_vmcnt_imm<0>();\n                    __syncthreads();\n                }\n                const uint32_t wave_stage"
    assert old in text
    return text.replace(old, "                    wait_vmcnt_imm<0>();\n                }\n                const uint32_t wave_stage", 1)


@needs_clang
def test_thread_sanitizer_sees_a_missing_barrier(host_builds):
    if not host_builds.ok("tsan_broken"):
        pytest.skip(host_builds.why("tsan_broken")[-300:])
    r = subprocess.run([host_builds("tsan_broken"), "0"], capture_output=True, text=True, timeout=900)
    assert "ThreadSanitizer: data race" in r.stderr


def _drop_wait(text):
    old = "                    wait_vmcnt_imm<0>();\n                    __syncthreads();\n                }\n                const uint32_t wave_stage"
    assert old in text
    return text.replace(old, "                    __syncthreads();\n                }\n                const uint32_t wave_stage", 1)


def _advance_too_early(text):
    old = "                        ld.issue_one_masked(wave_stage, i, live);\n                        if (i == 7 && !ld.done()) ld.advance();"
    assert old in text
    return text.replace(old, "                        if (i == 7 && !ld.done()) ld.advance();\n                        ld.issue_one_masked(wave_stage, i, live);", 1)


def _short_wait6(text):   # 64 x 64 kernel: one load of the older register set may still be in flight when it is used
    old = "        wait_vmcnt_imm<kLoadsPerSet>();\n"
    assert old in text
    return text.replace(old, "        wait_vmcnt_imm<kLoadsPerSet + 1>();\n", 1)


BROKEN = {"no wait before the barrier": (_drop_wait, "sthip_kernel4.hpp", "0"),
          "cursor moved before the last load": (_advance_too_early, "sthip_kernel4.hpp", "0"),
          "64x64: wait one load short": (_short_wait6, "sthip_kernel6.hpp", "12")}


@needs_clang
@pytest.mark.parametrize("name", list(BROKEN))
def test_broken_copies_are_caught(host_builds, name):
    r = subprocess.run([host_builds(name), BROKEN[name][2]], capture_output=True, text=True, timeout=600)   # one launch is enough
    assert r.returncode != 0, r.stdout
    assert "MODEL VIOLATION" in r.stderr or "FAILED" in r.stdout


class HostBuilds:
    """Every host build these tests and tests/test_host_parity.py use, made side by side once per session."""

    def __init__(self, tmp):
        from concurrent.futures import ThreadPoolExecutor
        def checked():   # with the alignment, bounds and shift checks of UndefinedBehaviorSanitizer where its runtime is there
            try:
                return _build(tmp, "asan_ub", extra=("-g", "-fsanitize=address,alignment,bounds,shift", "-fno-sanitize-recover=all"))
            except AssertionError:
                return _build(tmp, "asan", extra=("-g", "-fsanitize=address"))
        jobs = {"asan": checked,
                "tsan": lambda: _build(tmp, "tsan", extra=("-g", "-fsanitize=thread")),
                "tsan_broken": lambda: _build(tmp, "tsan_broken", _drop_barrier, extra=("-g", "-fsanitize=thread")),
                "library": lambda: _build_library(tmp, "lib", drivers=("library_host.cpp", "library_cli.cpp"))}
        for name, (mutate, header, _) in BROKEN.items():
            jobs[name] = lambda mutate=mutate, header=header, name=name: _build(tmp, "broken%d" % list(BROKEN).index(name), mutate, header)
        self.tmp, self.done = tmp, {}
        with ThreadPoolExecutor(4) as pool:
            for name, fut in [(n, pool.submit(j)) for n, j in jobs.items()]:
                try:
                    self.done[name] = fut.result()
                except AssertionError as e:
                    self.done[name] = e

    def ok(self, name):
        return not isinstance(self.done[name], Exception)

    def why(self, name):
        return str(self.done[name])

    def __call__(self, name):
        if name == "plain" and name not in self.done:
            self.done[name] = _build(self.tmp, "plain")
        if not self.ok(name):
            raise self.done[name]
        return self.done[name]
