"""What the per-head-table decode kernels wait for, measured by taking things away.

Builds the library several times from the committed sources with measurement-only macros
(ADKV_FT_OV_MM=0 / 1: the OV kernel's vector contraction / the matrix one without the add;
adkv_ft_kernels.h:
ADKV_ABLATE_NO_LOOKUP skips the LDS table reads, ADKV_ABLATE_CODE_WINDOW=m
keeps every unit's code prefetch inside its first m+1 supergroups, so the bytes come from L1 / L2 /
the memory-side cache instead of HBM), then runs the cfg2 decode step (B=128, 32 heads x 128,
ctx 4096, 4-bit, checkpoints every 256 tokens) with each build in a process of its own and prints
the stage times.  The variants compute wrong results on purpose; only their timing is of interest.

    python -m adkv_amd.tools.ablate --build     # compile the variants (hipcc cross-compiles, ~1 min each, in parallel)
    python -m adkv_amd.tools.ablate             # run them on cuda:0 and print the table
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys

from .. import build as _build

_DIR = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(_DIR, "_ablate")
VARIANTS = [
    ("as shipped", []),
    ("vector contraction in OV", ["-DADKV_FT_OV_MM=0"]),
    ("OV: matrix contraction of q*sc and zp apart (no add)", ["-DADKV_FT_OV_MM=1"]),
    ("no table lookups", ["-DADKV_ABLATE_NO_LOOKUP"]),
    ("codes from L1 (2 supergroups per unit)", ["-DADKV_ABLATE_CODE_WINDOW=1"]),
    ("codes from L2 (4 per unit)", ["-DADKV_ABLATE_CODE_WINDOW=3"]),
    ("codes from L2 / memory-side cache (16 per unit)", ["-DADKV_ABLATE_CODE_WINDOW=15"]),
    ("codes from the memory-side cache (64 per unit)", ["-DADKV_ABLATE_CODE_WINDOW=63"]),
    ("neither lookups nor HBM", ["-DADKV_ABLATE_NO_LOOKUP", "-DADKV_ABLATE_CODE_WINDOW=1"]),
]


def _path(i: int) -> str:
    return os.path.join(OUT, f"libadkv_hip_v{i}.so")


def build_variants() -> None:
    os.makedirs(OUT, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "hipcc")

    def one(i):
        flags = VARIANTS[i][1]
        subprocess.run([hipcc, *_build.HIPCC_FLAGS, *flags, "-o", _path(i), *_build.SOURCES],
                       check=True, capture_output=True)

    with cf.ThreadPoolExecutor(max_workers=min(8, len(VARIANTS))) as ex:
        list(ex.map(one, range(len(VARIANTS))))


def _measure() -> None:
    """Child process: ADKV_ABLATE_LIB names the library to load."""
    from .. import _lib
    _lib.LIB_PATH = os.environ["ADKV_ABLATE_LIB"]
    import torch
    from .. import synth
    from ..kernel import gemv

    dev = torch.device("cuda:0")
    B, H, D, T, S, NL = 128, 32, 128, 4096, 256, 2
    L = _lib.lib()
    ncap = T // S + 1
    state = torch.zeros(B, H, D, 2, dtype=torch.float16, device=dev)
    layers = []
    for l in range(NL):
        kp = synth.make_params(H, D, seed=3, layer=l).to(dev)
        vp = synth.make_params(H, D, seed=4, layer=l).to(dev)
        kc = synth.alloc_cache(B, H, T + 16, D, dev)
        vc = synth.alloc_cache(B, H, T + 16, D, dev)
        kk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=dev)
        vk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=dev)
        gemv.append_kv(kc, synth.make_k(B, H, T, D, layer=l, dtype=torch.float16, device=dev),
                       *kp.astuple(), 0, state, ckpt=kk, ckpt_interval=S)
        gemv.append_kv(vc, synth.make_v(B, H, T, D, layer=l, dtype=torch.float16, device=dev),
                       *vp.astuple(), 0, state, ckpt=vk, ckpt_interval=S)
        layers.append((kp.astuple(), vp.astuple(), kc, vc, kk, vk))
    q = synth.make_q(B, H, D, device=dev)
    k_new = synth.make_k(B, H, 1, D, seed=11, dtype=torch.float16, device=dev, t0=T)
    v_new = synth.make_v(B, H, 1, D, seed=12, dtype=torch.float16, device=dev)
    ws = torch.empty(gemv.decode_step_workspace_bytes(B, H, H, T, D, ncap, S), dtype=torch.uint8, device=dev)
    arr4 = _lib.C.c_void_p * 4

    def step(l):
        kp, vp, kc, vc, kk, vk = layers[l]
        e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        for x in e:
            x.record()
        L.adkv_set_stage_events(arr4(*[x.cuda_event for x in e]))
        gemv.decode_step(q, kc, vc, k_new, v_new, kp, vp, T, D ** -0.5, k_ckpt=kk, v_ckpt=vk,
                         ckpt_interval=S, workspace=ws)
        L.adkv_set_stage_events(None)
        return e

    for i in range(6):
        step(i % NL)
    torch.cuda.synchronize()
    n = 30
    marks = [step(i % NL) for i in range(n)]
    torch.cuda.synchronize()
    med = lambda a, b: sorted(e[a].elapsed_time(e[b]) for e in marks)[n // 2] * 1e3
    print(f"{med(0, 1):8.1f} {med(1, 2):8.1f} {med(2, 3):8.1f}", flush=True)


def main(argv=None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    if "--child" in argv:
        _measure()
        return 0
    if "--build" in argv:
        build_variants()
        print(OUT)
        return 0
    missing = [i for i, (_, f) in enumerate(VARIANTS) if f and not os.path.exists(_path(i))]
    if missing:
        raise SystemExit("variant libraries missing: run with --build first (on the machine with hipcc)")
    print(f"{'variant':52s} {'qk us':>8s} {'softmax':>8s} {'ov us':>8s}   (medians of 30 steps)")
    for i, (name, flags) in enumerate(VARIANTS + [VARIANTS[0]]):
        env = dict(os.environ)
        env["ADKV_ABLATE_LIB"] = _build.LIB_PATH if not flags else _path(i)
        r = subprocess.run([sys.executable, "-m", "adkv_amd.tools.ablate", "--child"], env=env,
                           capture_output=True, text=True, timeout=300)
        if r.returncode != 0:
            print(r.stderr[-2000:])
            return r.returncode
        print(f"{name:52s} {r.stdout.strip().splitlines()[-1]}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
