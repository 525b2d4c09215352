"""Forward pass of the reference's fp32 ADKV quantiser (src/adkv/train/train_model.py) on gfx950.

``quant_f32`` is the raw kernel call; ``adkv_chunk_forward`` has the signature and return values of
the reference's ``_adkv_chunk_forward`` (train_model.py:46-86); ``ADKVTrainModel`` keeps the
reference module's parameters, constraints and ``forward`` (train_model.py:89-213).  Only the
forward values are produced: the straight-through / LSQ backward pass (train_model.py:24-43) and
truncated BPTT belong to calibration, which this package does not do.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import _lib
from ..kernel.gemv import _chk, _need_device

_DTYPES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _f32vec(t: torch.Tensor, n: int, name: str) -> torch.Tensor:
    _chk(t.numel() == n, f"{name} must have {n} elements")
    return t.detach().to(torch.float32).contiguous().view(n)


def quant_f32(x: torch.Tensor, alpha: torch.Tensor, beta: torch.Tensor, target: torch.Tensor,
              lower_limit: int, upper_limit: int, sc_min: float, sc_max: float, *,
              zp_state: torch.Tensor | None = None, sc_state: torch.Tensor | None = None,
              zp_init: torch.Tensor | None = None, sc_init: torch.Tensor | None = None,
              out: torch.Tensor | None = None, want_codes: bool = False,
              output_states: bool = False):
    """Fake-quantise ``x [B, T, C]`` (fp32 / fp16 / bf16, channel stride 1) along ``T``.

    State: ``zp_state`` / ``sc_state`` fp32 ``[B, C]`` are updated in place; they are also the
    starting state unless ``zp_init`` / ``sc_init`` ``[C]`` are given.  ``out`` may be ``x`` itself
    (in-place, as the reference's eval cache does).  Returns ``(xhat, codes | None, zp_seq | None,
    sc_seq | None)``.
    """
    _chk(x.dim() == 3 and x.dtype in _DTYPES and x.stride(2) == 1, "x must be [B, T, C] with unit channel stride")
    B, T, C = x.shape
    dev = _need_device(x)
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format) if x.is_contiguous() \
            else torch.empty_strided(x.shape, x.stride(), dtype=x.dtype, device=dev)
    _chk(out.shape == x.shape and out.dtype == x.dtype and out.stride() == x.stride(),
         "out must match x in shape, dtype and strides")
    al, be, tg = (_f32vec(t, C, n) for t, n in ((alpha, "alpha"), (beta, "beta"), (target, "target")))
    zi = si = None
    if zp_init is not None or sc_init is not None:
        _chk(zp_init is not None and sc_init is not None, "zp_init and sc_init go together")
        zi, si = _f32vec(zp_init, C, "zp_init"), _f32vec(sc_init, C, "sc_init")
    if zp_state is None:
        _chk(zi is not None, "either a state or an initial state is required")
        zp_state = torch.empty(B, C, dtype=torch.float32, device=dev)
        sc_state = torch.empty(B, C, dtype=torch.float32, device=dev)
    for t, n in ((zp_state, "zp_state"), (sc_state, "sc_state")):
        _chk(t is not None and t.dtype == torch.float32 and t.is_contiguous() and t.shape == (B, C),
             f"{n} must be contiguous fp32 [B, C]")
    codes = torch.empty(B, T, C, dtype=torch.int8, device=dev) if want_codes else None
    zs = torch.empty(B, T, C, dtype=torch.float32, device=dev) if output_states else None
    ss = torch.empty(B, T, C, dtype=torch.float32, device=dev) if output_states else None
    p = lambda t: None if t is None else t.data_ptr()
    sb = x.stride(0) if B > 1 else T * max(x.stride(1), C)
    st = x.stride(1) if T > 1 else C
    with _lib.device_guard(dev):
        rc = _lib.lib().adkv_quant_f32(
            x.data_ptr(), out.data_ptr(), p(codes), zp_state.data_ptr(), sc_state.data_ptr(),
            p(zi), p(si), al.data_ptr(), be.data_ptr(), tg.data_ptr(), p(zs), p(ss),
            B, T, C, sb, st, _DTYPES[x.dtype], int(lower_limit), int(upper_limit),
            float(sc_min), float(sc_max), _lib.current_stream_ptr(dev))
    _lib.check(rc, "quant_f32")
    return out, codes, zs, ss


def adkv_chunk_forward(kv_cache_chunk, current_zp, current_sc, alpha, beta, target,
                       upper_limit, lower_limit, sc_min, sc_max, output_states):
    """Same contract as the reference's ``_adkv_chunk_forward`` (train_model.py:46-86):
    returns ``(outputs [B,chunk,C], zp [B,C], sc [B,C], zp_seq | None, sc_seq | None)`` and leaves
    its arguments untouched."""
    zp = current_zp.detach().to(torch.float32).clone().contiguous()
    sc = current_sc.detach().to(torch.float32).clone().contiguous()
    out, _, zs, ss = quant_f32(kv_cache_chunk.detach(), alpha, beta, target, lower_limit, upper_limit,
                               sc_min, sc_max, zp_state=zp, sc_state=sc, output_states=bool(output_states))
    return out, zp, sc, zs, ss


class ADKVTrainModel(nn.Module):
    """Parameters and forward pass of the reference's ``ADKVTrainModel`` (train_model.py:89-213)."""

    def __init__(self, num_hidden_states, truncation=32, bits=4, log_sc_min=-4.0, log_sc_max=4.0):
        super().__init__()
        self.num_hidden_states = num_hidden_states
        self.truncation = truncation
        self.bits = bits
        self.upper_limit = 2 ** (bits - 1) - 1
        self.lower_limit = -2 ** (bits - 1)
        self.sc_min = math.exp(log_sc_min)
        self.sc_max = math.exp(log_sc_max)
        self.init_zp = nn.Parameter(torch.zeros(num_hidden_states))
        self.init_log_sc = nn.Parameter(torch.zeros(num_hidden_states))
        self.alpha = nn.Parameter(torch.zeros(num_hidden_states))
        self.beta = nn.Parameter(torch.zeros(num_hidden_states))
        self.target = nn.Parameter(torch.zeros(num_hidden_states))
        self.reset_parameters()

    def reset_parameters(self):
        nn.init.constant_(self.init_zp, 0.0)
        nn.init.constant_(self.init_log_sc, 0.0)
        nn.init.normal_(self.alpha, mean=0.0, std=0.02)
        nn.init.normal_(self.beta, mean=0.0, std=0.02)
        nn.init.constant_(self.target, self.upper_limit / 2)

    # constrained parameters (train_model.py:127-134)
    def get_sc(self):
        return torch.exp(self.init_log_sc)

    def get_alpha(self):
        return torch.sigmoid(self.alpha)

    def get_beta(self):
        return 0.1 * torch.sigmoid(self.beta)

    @torch.no_grad()
    def forward(self, kv_cache, CHUNK=32, output_states=False):
        """``kv_cache [B, T, C]`` -> fake-quantised ``[B, T, C]`` (and the per-token state when
        ``output_states``).  One launch covers all tokens: the reference's chunking and zero padding
        (train_model.py:150-205) only serve its compiler and do not change any value in ``[:T]``."""
        B, T, C = kv_cache.shape
        assert C == self.num_hidden_states
        assert self.truncation % CHUNK == 0
        out, _, zs, ss = quant_f32(kv_cache, self.get_alpha(), self.get_beta(), self.target,
                                   self.lower_limit, self.upper_limit, self.sc_min, self.sc_max,
                                   zp_init=self.init_zp, sc_init=self.get_sc(),
                                   output_states=output_states)
        return (out, zs, ss) if output_states else out
