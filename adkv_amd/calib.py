"""Calibrated ADKV parameters: reading the reference's per-layer checkpoint files.

The reference's calibration writes one ``state_dict`` of its ``ADKVTrainModel`` per layer and per
tensor, ``ckpt_k_{L}.pt`` / ``ckpt_v_{L}.pt`` with the raw (unconstrained) parameters
``init_zp, init_log_sc, alpha, beta, target``; its tools turn them into the five deployment vectors
with ``exp`` / ``sigmoid`` / ``0.1*sigmoid`` (src/adkv/train/train_model.py:127-134, used at
tools/perf_e2e.py:37-60).  ``load_calibration`` does exactly that, on the CPU, with a loader that
executes nothing from the file.
"""
from __future__ import annotations

from pathlib import Path

import torch

from .hf.llama_adkv import ADKVConfig

RAW_FIELDS = ("init_zp", "init_log_sc", "alpha", "beta", "target")


def config_from_state_dict(sd: dict) -> ADKVConfig:
    """Raw calibration parameters -> deployment vectors (train_model.py:127-134)."""
    missing = [k for k in RAW_FIELDS if k not in sd]
    if missing:
        raise KeyError(f"calibration state_dict lacks {missing}")
    f = {k: sd[k].detach().to(torch.float32).reshape(-1) for k in RAW_FIELDS}
    n = f["init_zp"].numel()
    if any(t.numel() != n for t in f.values()):
        raise ValueError("calibration vectors differ in length")
    return ADKVConfig(zp_init=f["init_zp"], scale_init=torch.exp(f["init_log_sc"]),
                      alpha=torch.sigmoid(f["alpha"]), beta=0.1 * torch.sigmoid(f["beta"]),
                      quant_target=f["target"])


def load_calibration(calib_dir, num_layers: int, hidden_size: int | None = None):
    """``[(ADKVConfig for K, ADKVConfig for V)] * num_layers`` from ``ckpt_{k,v}_{L}.pt``; the list
    ``LlamaForCausalLM_ADKV.load_adkv_config`` takes."""
    calib_dir = Path(calib_dir)
    out = []
    for layer in range(num_layers):
        pair = []
        for side in ("k", "v"):
            path = calib_dir / f"ckpt_{side}_{layer}.pt"
            if not path.exists():
                raise FileNotFoundError(path)
            cfg = config_from_state_dict(torch.load(path, map_location="cpu", weights_only=True))
            if hidden_size is not None and cfg.alpha.numel() != hidden_size:
                raise ValueError(f"{path}: {cfg.alpha.numel()} channels, expected {hidden_size}")
            pair.append(cfg)
        out.append(tuple(pair))
    return out


def save_calibration(calib_dir, raw_layers) -> None:
    """Write ``[(k_state_dict, v_state_dict)]`` in the layout ``load_calibration`` reads."""
    calib_dir = Path(calib_dir)
    calib_dir.mkdir(parents=True, exist_ok=True)
    for layer, (k, v) in enumerate(raw_layers):
        for side, sd in (("k", k), ("v", v)):
            torch.save({n: sd[n].detach().cpu() for n in RAW_FIELDS}, calib_dir / f"ckpt_{side}_{layer}.pt")


def synthetic_adkv_config(num_layers: int, heads: int, head_dim: int, seed: int = 3):
    """Deployment vectors drawn like the benchmark's synthetic parameters, for runs without
    calibration files (none ship with the reference)."""
    from . import synth
    out = []
    for layer in range(num_layers):
        pair = []
        for s in (seed, seed + 1):
            p = synth.make_params(heads, head_dim, seed=s, layer=layer)
            pair.append(ADKVConfig(*[t.float().reshape(-1) for t in p.astuple()]))
        out.append(tuple(pair))
    return out
