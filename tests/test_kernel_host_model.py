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
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "host_model"))
import hostbuild  # noqa: E402
from hostbuild import clang as _clang, strip_asm, run_shares, build_kernels as _build, build_library as _build_library  # noqa: E402,F401

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


@needs_clang
def test_preflight_gate_takes_the_kernel_directory_from_the_environment(tmp_path):
    """tests/host_model/preflight.py is the one command a kernel source passes before it goes to a GPU.  Here it runs on a
    directory that holds a copy of the committed 256 x 256 kernel header (kernel cases only: the library-level run is
    test_library_through_its_c_abi_on_the_host), named through STHIP_KERNEL_DIR as a working copy would be."""
    work = tmp_path / "variant"
    work.mkdir()
    (work / "sthip_kernel4.hpp").write_text(open(os.path.join(hostbuild.CSRC, "sthip_kernel4.hpp")).read())
    env = dict(os.environ, STHIP_KERNEL_DIR=str(work))
    r = subprocess.run([sys.executable, os.path.join(hostbuild.MODEL, "preflight.py"), "--no-library"], env=env,
                       capture_output=True, text=True, timeout=1500)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "kernel sources from " + str(work) in r.stdout and "preflight: PASSED" in r.stdout


@needs_clang
def test_preflight_gate_refuses_a_broken_working_copy(tmp_path):
    """The same command on a working copy with the mistake that once reached a GPU (the loader's cursor moved before the
    step's last load, so that the last k-step reads past the operand) must fail."""
    work = tmp_path / "variant"
    work.mkdir()
    (work / "sthip_kernel4.hpp").write_text(_advance_too_early(open(os.path.join(hostbuild.CSRC, "sthip_kernel4.hpp")).read()))
    r = subprocess.run([sys.executable, os.path.join(hostbuild.MODEL, "preflight.py"), "--no-library", "--kernel-dir", str(work)],
                       capture_output=True, text=True, timeout=1500)
    assert r.returncode == 1, r.stdout[-3000:]
    assert "preflight: FAILED" in r.stdout


class HostBuilds:
    """Every host build these tests and tests/test_host_parity.py use, made side by side once per session."""

    def __init__(self, tmp):
        from concurrent.futures import ThreadPoolExecutor
        # "asan": with the alignment, bounds and shift checks of UndefinedBehaviorSanitizer where its runtime is there
        jobs = {"asan": lambda: hostbuild.build_checked(tmp),
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
