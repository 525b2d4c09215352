"""Builds and runs the many-streams HBM read microbenchmark (hbm_streams.hip) on cuda:0.

    python -m adkv_amd.tools.hbm_streams            # build if needed, run, print the table
    python -m adkv_amd.tools.hbm_streams --build    # build only (hipcc cross-compiles without a GPU)
"""
from __future__ import annotations

import os
import subprocess
import sys

_DIR = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(_DIR, "hbm_streams.hip")
EXE = os.path.join(_DIR, "hbm_streams.bin")


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
    return subprocess.call([exe])


if __name__ == "__main__":
    sys.exit(main())
