"""Builds and runs the vector-instruction issue-rate microbenchmark (issue_rate.hip) on cuda:0.

    python -m adkv_amd.tools.issue_rate            # build if needed, run, print the table
    python -m adkv_amd.tools.issue_rate --all      # plus a survey of 32-bit and scalar-f16 forms at 4 and 8 waves
    python -m adkv_amd.tools.issue_rate --mfma     # matrix-core instructions interleaved with packed vector arithmetic
    python -m adkv_amd.tools.issue_rate --build    # build only (hipcc cross-compiles without a GPU)
"""
from __future__ import annotations

import os
import subprocess
import sys

_DIR = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(_DIR, "issue_rate.hip")
EXE = os.path.join(_DIR, "issue_rate.bin")


def build(force: bool = False) -> str:
    if force or not os.path.exists(EXE) or os.path.getmtime(EXE) < os.path.getmtime(SRC):
        subprocess.check_call([os.environ.get("HIPCC", "hipcc"), "-O3", "--offload-arch=gfx950", "-std=c++17",
                               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                               "-Wno-unused-command-line-argument", "-o", EXE, SRC])
    return EXE


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    exe = build(force="--build" in argv)
    if "--build" in argv:
        print(exe)
        return 0
    return subprocess.call([exe] + [a for a in argv if a in ("--all", "--mfma")])


if __name__ == "__main__":
    sys.exit(main())
