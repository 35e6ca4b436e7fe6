"""Builds libstrassen_hip.so (gfx950) from csrc/ with hipcc.

    python build.py            # rebuild what changed
    python build.py --force    # rebuild everything

The fused kernel is instantiated once per (element type, algorithm) pair; the nine units
plus the C-ABI front end compile in parallel and are linked into one shared library next to
this file.  Object files go to csrc/build/ (git-ignored).
"""
from __future__ import annotations

import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libstrassen_hip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# Packed fp32 VALU ops are disabled on purpose (hipcc's host pass prints a harmless note
# that it does not know the feature).
FLAGS = ["-O3", "-fPIC", "-std=c++17", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-I", CSRC]


def _units():
    units = [("sthip_api.o", "sthip_api.hip", [])]
    for t in range(3):
        for a in range(3):
            units.append((f"sthip_inst_{t}_{a}.o", "sthip_inst.hip",
                          [f"-DSTHIP_INST_TYPE={t}", f"-DSTHIP_INST_ALGO={a}"]))
    for t in (1, 2):
        for a in range(3):
            units.append((f"sthip_inst2_{t}_{a}.o", "sthip_inst2.hip",
                          [f"-DSTHIP_INST_TYPE={t}", f"-DSTHIP_INST_ALGO={a}"]))
    for t in (1, 2):
        for a in range(3):
            units.append((f"sthip_inst3_{t}_{a}.o", "sthip_inst3.hip",
                          [f"-DSTHIP_INST_TYPE={t}", f"-DSTHIP_INST_ALGO={a}"]))
        units.append((f"sthip_inst4_{t}.o", "sthip_inst4.hip", [f"-DSTHIP_INST_TYPE={t}"]))
        units.append((f"sthip_inst5_{t}.o", "sthip_inst5.hip", [f"-DSTHIP_INST_TYPE={t}"]))
    units.append(("sthip_inst4_0.o", "sthip_inst4.hip", ["-DSTHIP_INST_TYPE=0"]))
    units.append(("sthip_inst6.o", "sthip_inst6.hip", []))
    return units


def _digest(extra):
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        path = os.path.join(CSRC, name)
        if os.path.isfile(path):
            h.update(name.encode())
            h.update(open(path, "rb").read())
    for hdr in ("strassen_hip.h", "strassen_hip_debug.h"):
        h.update(open(os.path.join(HERE, "..", "include", hdr), "rb").read())
    h.update(" ".join(FLAGS + extra).encode())
    return h.hexdigest()


def _compile(unit, force):
    obj, src, defs = unit
    out = os.path.join(OBJ, obj)
    stamp = out + ".sha"
    dig = _digest(defs)
    if not force and os.path.exists(out) and os.path.exists(stamp) and open(stamp).read() == dig:
        return obj, "cached"
    cmd = [HIPCC, *FLAGS, *defs, "-c", os.path.join(CSRC, src), "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {obj}:\n{r.stderr[-4000:]}")
    open(stamp, "w").write(dig)
    return obj, "built"


def build(force: bool = False, jobs: int | None = None, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    units = _units()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda u: _compile(u, force), units))
    if verbose:
        print("objects:", ", ".join(f"{o}:{s}" for o, s in results))
    if force or not os.path.exists(LIB) or any(s == "built" for _, s in results):
        objs = [os.path.join(OBJ, u[0]) for u in units]
        cmd = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", LIB]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
        if verbose:
            print("linked", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
