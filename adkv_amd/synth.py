"""Seeded synthetic K/V, queries and ADKV parameters of the benchmark configurations.

K is post-RoPE-like: N(0,1) per element plus four drifting outlier channels per head (channel
``32*k`` carries ``8*sin(0.01*(k+1)*t)``, k = 0..3); V and q are N(0,1).  Per-(head, channel)
parameters: ``alpha`` and ``scale_init`` uniform in [0.9, 0.999], ``zp_init = 0``,
``beta = 0.02``, ``quant_target = (2^(bits-1)-1)/2`` (the reference's initial target,
src/adkv/train/train_model.py:124).  Everything is generated with explicit ``torch.Generator``
seeds so CPU and GPU runs see identical bits when generated on the CPU.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

SEED_K, SEED_V, SEED_Q, SEED_PARAMS = 0, 1, 2, 3


@dataclass
class ADKVParams:
    """The five per-(head, channel) tensors, each ``[H, D]`` (field order of
    src/adkv/hf/llama_adkv.py:27)."""
    zp_init: torch.Tensor
    scale_init: torch.Tensor
    alpha: torch.Tensor
    beta: torch.Tensor
    quant_target: torch.Tensor

    def astuple(self):
        return (self.zp_init, self.scale_init, self.alpha, self.beta, self.quant_target)

    def to(self, *a, **k):
        return ADKVParams(*[t.to(*a, **k) for t in self.astuple()])


def make_params(H: int, D: int, bits: int = 4, seed: int = SEED_PARAMS, layer: int = 0,
                dtype=torch.float16, device="cpu") -> ADKVParams:
    g = torch.Generator().manual_seed(seed + 1000 * layer)
    u = lambda: 0.9 + 0.099 * torch.rand(H, D, generator=g)
    alpha = u()
    scale = u()
    zp = torch.zeros(H, D)
    beta = torch.full((H, D), 0.02)
    tgt = torch.full((H, D), ((1 << (bits - 1)) - 1) / 2.0)
    return ADKVParams(*[t.to(dtype=dtype, device=device) for t in (zp, scale, alpha, beta, tgt)])


def _outliers(T: int, D: int, t0: int = 0, device="cpu") -> torch.Tensor:
    """[T, D] drift term: channel 32k gets 8*sin(0.01*(k+1)*t)."""
    t = torch.arange(t0, t0 + T, dtype=torch.float32, device=device)
    o = torch.zeros(T, D, dtype=torch.float32, device=device)
    for k in range(4):
        if 32 * k < D:
            o[:, 32 * k] = 8.0 * torch.sin(0.01 * (k + 1) * t)
    return o


def make_k(B: int, H: int, T: int, D: int, seed: int = SEED_K, layer: int = 0,
           dtype=torch.float32, device="cpu", t0: int = 0) -> torch.Tensor:
    """[B, H, T, D] keys: Gaussian + sinusoidal-drift outlier channels."""
    g = torch.Generator(device=device).manual_seed(seed + 1000 * layer)
    k = torch.randn(B, H, T, D, generator=g, dtype=torch.float32, device=device)
    k += _outliers(T, D, t0, device)
    return k.to(dtype)


def make_v(B: int, H: int, T: int, D: int, seed: int = SEED_V, layer: int = 0,
           dtype=torch.float32, device="cpu") -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(seed + 1000 * layer)
    return torch.randn(B, H, T, D, generator=g, dtype=torch.float32, device=device).to(dtype)


def make_q(B: int, H: int, D: int, seed: int = SEED_Q, layer: int = 0,
           dtype=torch.float16, device="cpu") -> torch.Tensor:
    """[B, H, 1, D] single query token."""
    g = torch.Generator(device=device).manual_seed(seed + 1000 * layer)
    return torch.randn(B, H, 1, D, generator=g, dtype=torch.float32, device=device).to(dtype)


def n_super(tokens: int) -> int:
    return (tokens + 7) // 8


def alloc_cache(B: int, H: int, cap_tokens: int, D: int, device, bits: int = 4) -> torch.Tensor:
    """Zero-filled packed cache ``[B, H, n_super, D/4, 4, 4]`` uint8
    (src/adkv/hf/llama_adkv.py:87-94); a supergroup is ``32 // bits`` tokens."""
    tps = 32 // bits
    return torch.zeros((B, H, -(-cap_tokens // tps), D // 4, 4, 4), dtype=torch.uint8, device=device)
