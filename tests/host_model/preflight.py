#!/usr/bin/env python3
"""Pre-flight gate for kernel sources: run them on the CPU executor before they are ever launched on a GPU.

    python tests/host_model/preflight.py                      # the library's own csrc
    python tests/host_model/preflight.py --kernel-dir DIR     # a working copy (DIR holds the edited files only)
    STHIP_KERNEL_DIR=DIR python -m pytest tests/test_kernel_host_model.py tests/test_host_parity.py   # the same sources under the whole CPU suite

What runs (tests/host_model/hostbuild.py builds it):
  1. kernel4_host: every pipelined kernel as the library launches it, one host thread per lane, under
     AddressSanitizer with alignment / bounds / shift checks.  Every direct-to-LDS load is checked against the
     operand it reads and the LDS allocation it writes, and every case runs at both load timings (data lands at
     once / not before the lane's next wait).  The cases include the ones an addressing mistake shows in first: the last
     k-steps of a workgroup's last tile, fewer workgroups than tiles, odd and single k-steps, both layouts of B.
  2. library_host: sthip_gemm through the C ABI on the host build of all translation units (headline one-level path,
     two levels as 49 products, fp32 paths, odd sizes on the fused kernel), bit for bit.
  3. with --tsan: the kernel cases again under ThreadSanitizer (missing barrier / LDS buffer reused too early).

Exit status 0 only if every case is exact and no sanitizer or model violation was reported.  A kernel source that has
not passed this command is not launched on a GPU: an out-of-bounds access there faults the card for every job on it.
"""
import argparse
import os
import sys
import tempfile
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--kernel-dir", help="directory with the kernel sources to check (default: STHIP_KERNEL_DIR, else the library's csrc)")
    ap.add_argument("--tsan", action="store_true", help="also run the kernel cases under ThreadSanitizer")
    ap.add_argument("--no-library", action="store_true", help="skip the library-level run (kernel headers only)")
    args = ap.parse_args()
    if args.kernel_dir:
        os.environ["STHIP_KERNEL_DIR"] = args.kernel_dir
    import hostbuild as hb
    if hb.clang() is None:
        print("preflight: no clang++ (set STHIP_HOST_CXX)")
        return 2
    print("preflight: kernel sources from", hb.kernel_dir(), flush=True)
    failures = []
    with tempfile.TemporaryDirectory(prefix="sthip_preflight_") as tmp:
        def stage(label, build, shares):
            t0 = time.time()
            try:
                exe = build()
            except AssertionError as e:
                failures.append(label + ": does not build")
                print("preflight: %s: BUILD FAILED\n%s" % (label, str(e)[-2000:]), flush=True)
                return
            rc, out, err = hb.run_shares(exe, shares=shares)
            lines = [l for l in out.splitlines() if "wrong of" in l]
            bad = [l for l in lines if ": 0 wrong of" not in l]
            problems = []
            if rc != 0: problems.append("exit status %d" % rc)
            if bad: problems.append("%d inexact cases" % len(bad))
            if not lines: problems.append("no case ran")
            if out.count("ALL EXACT") != shares: problems.append("a share of the cases did not finish")
            for word in ("AddressSanitizer", "ThreadSanitizer", "runtime error", "MODEL VIOLATION"):
                if word in err: problems.append(word)
            print("preflight: %s: %d cases, %s (%.0f s)" % (label, len(lines), "; ".join(problems) if problems else "all exact, no violation",
                                                               time.time() - t0), flush=True)
            if problems:
                failures.append(label + ": " + "; ".join(problems))
                print("\n".join(bad[:20]))
                print(err[-3000:])
        stage("kernels (address, alignment, bounds checks; both load timings)", lambda: hb.build_checked(tmp), 4)
        if not args.no_library:
            stage("library through its C ABI", lambda: hb.build_library(tmp, "lib")["library_host.cpp"], 3)
        if args.tsan:
            stage("kernels under ThreadSanitizer", lambda: hb.build_kernels(tmp, "tsan", extra=("-g", "-fsanitize=thread")), 4)
    if failures:
        print("preflight: FAILED\n  " + "\n  ".join(failures))
        return 1
    print("preflight: PASSED")
    return 0


if __name__ == "__main__":
    sys.exit(main())
