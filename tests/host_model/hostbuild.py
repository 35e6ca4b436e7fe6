"""Builds of the library's kernels for the CPU executor in this directory, shared by the tests and by
preflight.py.

Every kernel header is taken from KERNEL_DIR: the library's own strassen-triton_amd/csrc, or the directory named
by STHIP_KERNEL_DIR in the environment.  A working copy of one header (an experiment on sthip_kernel4.hpp, say)
goes through exactly the same bounds-checked runs as the committed one by pointing that variable at a directory
that holds it; files the directory does not hold come from the library.
"""
import glob
import importlib.util
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
CSRC = os.path.join(ROOT, "strassen-triton_amd", "csrc")
MODEL = os.path.join(ROOT, "tests", "host_model")
HEADERS = ("sthip_kernel.hpp", "sthip_kernel2.hpp", "sthip_kernel3.hpp", "sthip_kernel4.hpp", "sthip_kernel6.hpp")


def kernel_dir():
    """Directory the kernel sources are read from (STHIP_KERNEL_DIR, else the library's csrc)."""
    d = os.environ.get("STHIP_KERNEL_DIR")
    if not d:
        return CSRC
    d = os.path.abspath(d)
    if not os.path.isdir(d):
        raise FileNotFoundError("STHIP_KERNEL_DIR=%s is not a directory" % d)
    return d


def source_path(name):
    """`name` in the kernel directory if it is there, else the library's own file."""
    p = os.path.join(kernel_dir(), name)
    return p if os.path.exists(p) else os.path.join(CSRC, name)


def clang():
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


def host_text(path):
    return strip_asm(open(path).read()).replace("extern __shared__", "extern")


def build_kernels(tmp, name, mutate=None, mutate_header="sthip_kernel4.hpp", extra=()):
    """kernel4_host.cpp against the kernel headers (asm statements taken out); `mutate` edits one header's text first."""
    inc = os.path.join(tmp, name)
    os.makedirs(inc)
    for h in HEADERS:
        text = host_text(source_path(h))
        if mutate and h == mutate_header:
            text = mutate(text)
        open(os.path.join(inc, h), "w").write(text)
    exe = os.path.join(inc, "kernel4_host")
    cmd = [clang(), "-std=c++17", "-O1", "-Wno-everything", "-no-pie", "-pthread", *extra, "-I", inc, "-I", MODEL,
           "-I", os.path.join(ROOT, "include"), os.path.join(MODEL, "kernel4_host.cpp"), os.path.join(MODEL, "host_runtime.cpp"),
           "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return exe


def build_library(tmp, name, extra=(), drivers=("library_host.cpp",)):
    """Every translation unit of the library (strassen-triton_amd/build.py lists them) compiled for the host against the
    stand-in HIP runtime of tests/host_model/hip/hip_runtime.h, linked with the drivers and host_runtime.cpp."""
    out = os.path.join(tmp, name)
    os.makedirs(out)
    names = {os.path.basename(f) for d in (CSRC, kernel_dir()) for f in glob.glob(os.path.join(d, "*.hpp")) + glob.glob(os.path.join(d, "*.hip"))}
    for f in sorted(names):
        if f == "sthip_prims.hpp":   # the host build has its own (tests/host_model/sthip_prims.hpp)
            continue
        open(os.path.join(out, f), "w").write(host_text(source_path(f)))
    spec = importlib.util.spec_from_file_location("sthip_build", os.path.join(ROOT, "strassen-triton_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    common = ["-std=c++17", "-O1", "-Wno-everything", "-pthread", *extra, "-I", MODEL, "-I", out, "-I", os.path.join(ROOT, "include")]

    def compile_unit(unit):
        obj, src, defs = unit
        r = subprocess.run([clang(), "-x", "c++", *common, *defs, "-c", os.path.join(out, src), "-o", os.path.join(out, obj)],
                           capture_output=True, text=True)
        assert r.returncode == 0, obj + "\n" + r.stderr[-3000:]
        return os.path.join(out, obj)

    with ThreadPoolExecutor(8) as pool:
        objs = list(pool.map(compile_unit, build._units()))
    runtime = os.path.join(out, "host_runtime.o")
    r = subprocess.run([clang(), *common, "-c", os.path.join(MODEL, "host_runtime.cpp"), "-o", runtime], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    exes = {}
    for driver in drivers:
        exes[driver] = os.path.join(out, driver[:-4])
        r = subprocess.run([clang(), *common, "-no-pie", os.path.join(MODEL, driver), runtime, *objs, "-o", exes[driver]],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-3000:]
    return exes


def run_shares(exe, shares=4, timeout=1800):
    """The driver's cases dealt to `shares` processes that run side by side (a launch spends much of its time in barriers);
    returns the worst exit code and everything printed."""
    procs = [subprocess.Popen([exe, "%d/%d" % (i, shares)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True) for i in range(shares)]
    outs = [p.communicate(timeout=timeout) for p in procs]
    return max(abs(p.returncode) for p in procs), "".join(o[0] for o in outs), "".join(o[1] for o in outs)


SANITIZE = ("-g", "-fsanitize=address,alignment,bounds,shift", "-fno-sanitize-recover=all")


def build_checked(tmp, name="asan"):
    """The kernel executor under AddressSanitizer with the alignment, bounds and shift checks of
    UndefinedBehaviorSanitizer; AddressSanitizer alone where that runtime is missing."""
    try:
        return build_kernels(tmp, name + "_ub", extra=SANITIZE)
    except AssertionError:
        return build_kernels(tmp, name, extra=("-g", "-fsanitize=address"))
