"""End-to-end generation throughput and peak memory, ADKV cache versus the fp16 cache.

Protocol of the reference's tools/perf_e2e.py:83-113: a batch of equal-length prompts, greedy
``generate`` for a fixed number of new tokens, wall time per repeat and
``torch.cuda.max_memory_allocated``.  Differences forced by running offline: the model is a
random-init Llama of the named geometry (no checkpoint can be fetched), the prompt is random token
ids (no tokenizer), and ADKV parameters come from calibration files when ``--calib_dir`` exists,
else from the synthetic benchmark parameters.

    python -m adkv_amd.tools.perf_e2e --batch_size 64 --kv adkv
    python -m adkv_amd.tools.perf_e2e --batch_size 64 --kv fp16
    python -m adkv_amd.tools.perf_e2e --search        # largest batch of each kind that fits
    python -m adkv_amd.tools.perf_e2e --kv adkv --batch_size 448 --prompt_lenth 3840 --output_length 256 --prefill_slice 8
                                                      # a batch near the memory limit at ctx 4096: the prompt
                                                      # is prefilled slice by slice, then the whole batch decodes
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import threading
import time

import torch

GEOMETRIES = {
    # hidden, intermediate, layers, heads, kv heads, vocab
    "llama-2-7b": (4096, 11008, 32, 32, 32, 32000),
    "llama-2-13b": (5120, 13824, 40, 40, 40, 32000),
    "tiny": (256, 512, 2, 2, 2, 128),
}


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", default="llama-2-7b", choices=sorted(GEOMETRIES))
    ap.add_argument("--layers", type=int, default=0, help="override the layer count (quick runs)")
    ap.add_argument("--calib_dir", default="calib")
    ap.add_argument("--kv", choices=["adkv", "fp16"], default="adkv")
    ap.add_argument("--batch_size", type=int, default=256)
    ap.add_argument("--prompt_lenth", type=int, default=160)   # spelling of the reference's flag
    ap.add_argument("--output_length", type=int, default=338)
    ap.add_argument("--num_repeats", type=int, default=3)
    ap.add_argument("--search", action="store_true",
                    help="print the largest batch the memory model admits for each cache kind")
    ap.add_argument("--hbm_gib", type=float, default=288.0)
    ap.add_argument("--prefill_slice", type=int, default=0,
                    help="prefill the prompt this many sequences at a time into one cache for the whole "
                         "batch, then decode the whole batch greedily (the dense attention and MLP "
                         "activations of a long prompt, not the cache, limit the batch of one prefill call)")
    return ap.parse_args(argv)


def build_model(args, device):
    from transformers import LlamaConfig, LlamaForCausalLM

    from ..calib import load_calibration, synthetic_adkv_config
    from ..hf.llama_adkv import LlamaForCausalLM_ADKV

    hidden, inter, layers, heads, kv_heads, vocab = GEOMETRIES[args.model]
    layers = args.layers or layers
    cfg = LlamaConfig(vocab_size=vocab, hidden_size=hidden, intermediate_size=inter,
                      num_hidden_layers=layers, num_attention_heads=heads,
                      num_key_value_heads=kv_heads, max_position_embeddings=4096,
                      attn_implementation="sdpa")
    torch.manual_seed(0)
    cls = LlamaForCausalLM_ADKV if args.kv == "adkv" else LlamaForCausalLM
    with torch.device(device):
        model = cls(cfg)
    model = model.half().eval()
    if args.kv == "adkv":
        width = kv_heads * (hidden // heads)
        if os.path.isdir(args.calib_dir):
            adkv = load_calibration(args.calib_dir, layers, width)
            source = f"calibration files in {args.calib_dir}"
        else:
            adkv = synthetic_adkv_config(layers, kv_heads, hidden // heads)
            source = "synthetic parameters"
        model.load_adkv_config(adkv)
    else:
        source = "n/a"
    model.generation_config.pad_token_id = 0
    return model, cfg, source


def max_batch(args) -> dict:
    """Largest batch whose weights + KV cache fit in ``--hbm_gib``, by the reference's accounting
    (tools/memory_comparison_fig.py:46-77): fp16 weights, K and V for every layer and token."""
    from ..hf.cache import adkv_cache_bytes, fp16_cache_bytes

    hidden, inter, layers, heads, kv_heads, vocab = GEOMETRIES[args.model]
    d = hidden // heads
    weights = 2 * (2 * vocab * hidden + layers * (4 * hidden * hidden + 3 * hidden * inter + 2 * hidden) + hidden)
    budget = args.hbm_gib * 2 ** 30 - weights
    tokens = args.prompt_lenth + args.output_length
    per_seq = {"adkv": adkv_cache_bytes(1, kv_heads, d, tokens, layers),
               "fp16": fp16_cache_bytes(1, kv_heads, d, tokens, layers)}
    return {"weights_GiB": weights / 2 ** 30, "tokens_per_sequence": tokens,
            **{f"max_batch_{k}": int(budget // v) for k, v in per_seq.items()},
            **{f"cache_MiB_per_sequence_{k}": v / 2 ** 20 for k, v in per_seq.items()}}


def _heartbeat(stop: threading.Event, every: float = 30.0) -> None:
    """A line on stderr every `every` seconds: long generate() calls print nothing by themselves."""
    t0 = time.time()
    while not stop.wait(every):
        print(f"[perf_e2e] running, {time.time() - t0:.0f} s", file=sys.stderr, flush=True)


def sliced_run(args, model, cfg, source, device):
    """Decode phase of a batch near the memory limit (the second number of the reference's
    protocol, tools/perf_e2e.py:75-78 with --batch_size at the largest value that runs).  The
    prompt goes in ``--prefill_slice`` sequences at a time: into views of one ADKV cache reserved
    for the whole batch, or, for the fp16 cache, into per-slice caches concatenated layer by layer
    afterwards.  Then every step feeds one token per sequence to the whole batch."""
    from ..hf.cache import KVCache_ADKV

    B, P, N, bs = args.batch_size, args.prompt_lenth, args.output_length, args.prefill_slice
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(1, cfg.vocab_size, (B, P), generator=g).to(device)
    d = cfg.hidden_size // cfg.num_attention_heads
    first = torch.empty(B, dtype=torch.long, device=device)
    stop = threading.Event()
    threading.Thread(target=_heartbeat, args=(stop,), daemon=True).start()
    torch.cuda.reset_peak_memory_stats()
    with torch.no_grad():
        t0 = time.time()
        if args.kv == "adkv":
            cache = KVCache_ADKV(cfg.num_hidden_layers)
            cache.reserve(B, cfg.num_key_value_heads, d, P + N, device)
            for b0 in range(0, B, bs):
                b1 = min(B, b0 + bs)
                r = model(ids[b0:b1], past_key_values=cache.batch_view(b0, b1), use_cache=True, logits_to_keep=1)
                first[b0:b1] = r.logits[:, -1].argmax(-1)
            cache.commit(P)
        else:
            from transformers import DynamicCache
            # K and V of the whole batch are allocated before any activation exists and filled
            # slice by slice: long-lived cache tensors carved out of freed activation blocks
            # would fragment the allocator's pool by tens of GiB at this size
            shape = (B, cfg.num_key_value_heads, P, d)
            full = [(torch.empty(shape, dtype=torch.float16, device=device),
                     torch.empty(shape, dtype=torch.float16, device=device))
                    for _ in range(cfg.num_hidden_layers)]
            for b0 in range(0, B, bs):
                b1 = min(B, b0 + bs)
                r = model(ids[b0:b1], use_cache=True, logits_to_keep=1)
                first[b0:b1] = r.logits[:, -1].argmax(-1)
                for i, layer in enumerate(r.past_key_values.layers):
                    full[i][0][b0:b1].copy_(layer.keys)
                    full[i][1][b0:b1].copy_(layer.values)
                del r, layer
                torch.cuda.empty_cache()
            cache = DynamicCache()
            for i in range(cfg.num_hidden_layers):
                k, v = full[i]
                full[i] = None
                cache.update(k, v, i)                       # the cache makes its own copy
                del k, v
                torch.cuda.empty_cache()
            del full
        torch.cuda.synchronize()
        prefill_s = time.time() - t0
        print(f"[perf_e2e] prompt done in {prefill_s:.1f} s, "
              f"{torch.cuda.memory_allocated() / 2 ** 30:.1f} GiB allocated", file=sys.stderr, flush=True)
        tok = first
        step_ms = []
        for i in range(N - 1):
            torch.cuda.synchronize()
            t1 = time.time()
            r = model(tok[:, None], past_key_values=cache, use_cache=True)
            tok = r.logits[:, -1].argmax(-1)
            torch.cuda.synchronize()
            step_ms.append((time.time() - t1) * 1e3)
            if i < 3 or i % 32 == 0:
                print(f"[perf_e2e] decode step {i}: {step_ms[-1]:.1f} ms", file=sys.stderr, flush=True)
    stop.set()
    assert cache.get_seq_length() == P + N - 1
    steps = sorted(step_ms)
    decode_s = sum(step_ms) / 1e3
    print(json.dumps({
        "model": args.model, "layers": cfg.num_hidden_layers, "kv": args.kv, "weights": "random init fp16",
        "adkv_params": source, "batch_size": B, "prompt_length": P, "output_length": N,
        "prefill_slice": bs, "prefill_s": prefill_s, "decode_s": decode_s,
        "decode_ms_per_step_median": steps[len(steps) // 2], "decode_ms_per_step_last": step_ms[-1],
        "decode_tokens_per_s": B * (N - 1) / decode_s,
        "peak_mem_GiB": torch.cuda.max_memory_allocated() / 2 ** 30}))


def generate_run(args, device=None) -> dict:
    """One measurement by the protocol above (whole-batch prefill): builds the model, generates four
    tokens untimed, then times ``num_repeats`` greedy ``generate`` calls.  Returns the record that
    ``main`` prints."""
    device = device or torch.device("cuda:0")
    model, cfg, source = build_model(args, device)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(1, cfg.vocab_size, (args.batch_size, args.prompt_lenth), generator=g).to(device)
    mask = torch.ones_like(ids)
    gen = dict(max_new_tokens=args.output_length, min_new_tokens=args.output_length, do_sample=False)
    stop = threading.Event()
    threading.Thread(target=_heartbeat, args=(stop,), daemon=True).start()
    try:
        with torch.no_grad():
            model.generate(ids, attention_mask=mask, max_new_tokens=4, min_new_tokens=4, do_sample=False)
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            t0 = time.time()
            for _ in range(args.num_repeats):
                out = model.generate(ids, attention_mask=mask, **gen)
            torch.cuda.synchronize()
    finally:
        stop.set()
    ms = (time.time() - t0) / args.num_repeats * 1e3
    assert out.shape[1] == args.prompt_lenth + args.output_length
    return {
        "model": args.model, "layers": cfg.num_hidden_layers, "kv": args.kv, "weights": "random init fp16",
        "adkv_params": source, "batch_size": args.batch_size, "prompt_length": args.prompt_lenth,
        "output_length": args.output_length, "used_time_ms": ms,
        "generated_tokens_per_s": args.batch_size * args.output_length / (ms * 1e-3),
        "peak_mem_GiB": torch.cuda.max_memory_allocated() / 2 ** 30}


def main(argv=None):
    args = parse_args(argv)
    if args.search:
        print(json.dumps(max_batch(args)))
        return
    if args.prefill_slice > 0:
        device = torch.device("cuda:0")
        model, cfg, source = build_model(args, device)
        return sliced_run(args, model, cfg, source, device)
    print(json.dumps(generate_run(args)))


if __name__ == "__main__":
    main()
