"""Builds libadkv_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
from __future__ import annotations

import glob
import os
import subprocess
import sys

_DIR = os.path.dirname(os.path.abspath(__file__))
SOURCES = [os.path.join(_DIR, "csrc", "adkv_kernels.hip"),
           os.path.join(_DIR, "csrc", "adkv_fp32.hip"),
           os.path.join(_DIR, "csrc", "fp16_baseline.hip")]
HEADERS = sorted(glob.glob(os.path.join(_DIR, "csrc", "*.h"))) + \
    [os.path.join(_DIR, "..", "include", "adkv_hip.h")]
LIB_PATH = os.path.join(_DIR, "libadkv_hip.so")

# -ffp-contract=off: the fp16 recurrence needs "q*sc + zp" as two roundings where the reference
#   has two, and one where it has an explicit fma (src/adkv/kernel/gemv.cu:644-645 vs :796).
# -fhip-fp32-correctly-rounded-divide-sqrt: the quantiser divides in IEEE fp32 (gemv.cu:152).
# -packed-fp32-ops off: keep the compiler from forming v_pk_*_f32 from scalar float code.
HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def needs_build() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > t for p in SOURCES + HEADERS)


def build_hip(force: bool = True, verbose: bool = False) -> str:
    """Compile the kernels; returns the library path.  Raises CalledProcessError on failure."""
    if not force and not needs_build():
        return LIB_PATH
    hipcc = os.environ.get("HIPCC", "hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, "-o", LIB_PATH, *SOURCES]
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise subprocess.CalledProcessError(r.returncode, cmd, r.stdout, err)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_hip(force=True, verbose=True))
