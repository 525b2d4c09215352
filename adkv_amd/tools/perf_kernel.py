"""Decode-step latency table in the protocol of the reference's tools/perf_kernel.py:15-119.

One step = forward_qk -> softmax -> forward_ov for 32 heads of dimension 128; the table gives
requests/s at 32 layers, B / (32 * median step time), over a grid of batch sizes and cached
lengths (tools/perf_kernel.py:12-13,91-104).  Timing as there: warm-up steps, then
clamp(2e6 / (B*T), 5, 100) timed steps between device events, median (tools/perf_kernel.py:60-74),
after a burst of copies that lifts the device out of its idle clocks (:83-89).

Two cache modes:

  --cache fill      the reference's set-up (:34-49): every cache byte is 0x5A (codes +2 / -3),
                    zp=0, sc=1, alpha=0.05, beta=0, no checkpoints, so every (batch, head) is one
                    serial replay from token 0 -- the plain drop-in API.
  --cache encoded   synthetic K/V quantised by the encoder with state checkpoints every
                    --ckpt-interval tokens, which lets the decode kernels cut the context into
                    independently replayed segments (the extension this library adds).

--softmax torch keeps the reference's torch.softmax between the two calls; --softmax fused uses
the library's single-launch softmax.

    python -m adkv_amd.tools.perf_kernel --cache fill
"""
from __future__ import annotations

import argparse
import logging
import math

import torch

from adkv_amd import synth
from adkv_amd.kernel import gemv

logger = logging.getLogger("adkv_amd.perf_kernel")

NH, DIM = 32, 128
SCALE_MIN, SCALE_MAX = math.exp(-4.0), math.exp(4.0)
WARMUP = 3


def _fill_case(B: int, T: int, dev):
    n_super = (T + 1 + 7) // 8 + 1
    caches = [torch.full((B, NH, n_super, DIM // 4, 4, 4), 0x5A, dtype=torch.uint8, device=dev)
              for _ in range(2)]
    half = lambda v: torch.full((NH, DIM), v, dtype=torch.float16, device=dev)
    params = (half(0.0), half(1.0), half(0.05), half(0.0), half(3.5))
    return caches, (params, params), (None, None), 0


def _encoded_case(B: int, T: int, dev, interval: int):
    ncap = T // interval + 1
    out, pars, cks = [], [], []
    for i, make in enumerate((synth.make_k, synth.make_v)):
        p = synth.make_params(NH, DIM, seed=3 + i).to(dev)
        x = make(B, NH, T, DIM, dtype=torch.float16, device=dev)
        cache = synth.alloc_cache(B, NH, T + 8, DIM, dev)
        ck = torch.zeros(B, NH, ncap, DIM, 2, dtype=torch.float16, device=dev)
        gemv.encode_kv(cache, x, *p.astuple(), SCALE_MIN, SCALE_MAX, ckpt=ck, ckpt_interval=interval)
        out.append(cache)
        pars.append(p.astuple())
        cks.append(ck)
    return out, tuple(pars), tuple(cks), interval


def bench_step(B: int, T: int, dev, cache_mode: str, softmax: str, interval: int) -> float:
    """Median latency in ms of one decode step over T cached tokens."""
    if cache_mode == "fill":
        (kc, vc), (kp, vp), (kck, vck), S = _fill_case(B, T, dev)
    else:
        (kc, vc), (kp, vp), (kck, vck), S = _encoded_case(B, T, dev, interval)
    g = torch.Generator(device=dev).manual_seed(B * 131 + T)
    new = lambda: torch.randn(B, NH, 1, DIM, generator=g, dtype=torch.float16, device=dev) * 0.5
    q, k_new, v_new = new(), new(), new()

    def step():
        logits = gemv.forward_qk(q, kc, k_new, *kp, T, SCALE_MIN, SCALE_MAX, ckpt=kck, ckpt_interval=S)
        if softmax == "torch":
            attn = torch.softmax(logits, dim=-1)
        else:
            attn = gemv.softmax_scale_mask(logits, 1.0)
        gemv.forward_ov(attn, vc, v_new, *vp, SCALE_MIN, SCALE_MAX, ckpt=vck, ckpt_interval=S)

    # the appended token lands in slot T every time, so all steps do the same work
    for _ in range(WARMUP):
        step()
    torch.cuda.synchronize(dev)
    iters = max(5, min(100, 2_000_000 // (B * T)))
    marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
             for _ in range(iters)]
    for a, b in marks:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize(dev)
    times = sorted(a.elapsed_time(b) for a, b in marks)
    return times[len(times) // 2]


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--cache", choices=["fill", "encoded"], default="fill")
    ap.add_argument("--softmax", choices=["torch", "fused"], default="torch")
    ap.add_argument("--ckpt-interval", type=int, default=256)
    ap.add_argument("--batches", type=int, nargs="+", default=[1, 4, 16, 32, 64, 128, 256, 512])
    ap.add_argument("--seq-lens", type=int, nargs="+", default=[128, 256, 512, 1024, 2048])
    args = ap.parse_args(argv)
    logging.basicConfig(level=logging.INFO)
    torch.manual_seed(0)
    dev = torch.device("cuda:0")

    burn = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(burn)
    for _ in range(20):
        dst.copy_(burn)
    torch.cuda.synchronize(dev)
    del burn, dst
    torch.cuda.empty_cache()

    logger.info("Request throughput at 32 layers (req/s): B / (single-layer step latency * 32)")
    logger.info(f"Step = forward_qk + softmax({args.softmax}) + forward_ov;  nh={NH}, DIM={DIM}, fp16, "
                f"cache={args.cache}" + (f", checkpoints every {args.ckpt_interval}" if args.cache == "encoded" else ""))
    header = "B\\T".ljust(8) + "".join(f"{t:>10}" for t in args.seq_lens)
    logger.info(header)
    logger.info("-" * len(header))
    for B in args.batches:
        row = []
        for T in args.seq_lens:
            try:
                ms = bench_step(B, T, dev, args.cache, args.softmax, args.ckpt_interval)
                row.append(B / (ms * 1e-3 * 32.0))
            except torch.cuda.OutOfMemoryError:
                row.append(float("nan"))
            torch.cuda.empty_cache()
        logger.info(f"{B:<8}" + "".join(f"{v:10.1f}" if v == v else f"{'OOM':>10}" for v in row))
    logger.info("-" * len(header))
    logger.info("requests/s, 32 layers (higher is better)")


if __name__ == "__main__":
    main()
