"""PyTorch-CPU restatement of the reference's fp32 path -- TEST INFRASTRUCTURE ONLY.

This is the "reference PyTorch CPU path" the benchmark's ``cpu_baseline`` leg times on the host:
the eager per-token recurrence over whole ``[B, C]`` tensors (src/adkv/train/train_model.py:8-22,
61-81: about ten small tensor operations per token, unfused, fp32) followed by the single-query
attention over the dequantised tensors (src/adkv/train/llama_attention.py:41-44).  The reference
wraps the 32-token chunk body in ``torch.compile`` (train_model.py:46); here it runs eagerly, like
every CPU test of the reference's module would without a compiler cache.  Only tests and
``bench.py``'s ``cpu_baseline`` leg may import this module.

Pinned by tests/test_oracle_torch_cpu.py: codes, dequantised values and the final state equal
the C oracle's ``adkv_o_quant_f32`` bit for bit (itself pinned by vectors recorded from the
reference's own module), and the attention equals ``adkv_o_attention_f64`` within fp32 accuracy.
"""
from __future__ import annotations

import math

import torch


def quant_stream_f32(x, zp0, sc0, alpha, beta, tgt, bits=4, sc_min=None, sc_max=None, want_codes=False):
    """train_model.py:61-81 over ``x [B, T, C]`` fp32, one token at a time.

    Returns ``(xhat [B,T,C], zp [B,C], sc [B,C], codes [B,T,C] int8 | None)``."""
    B, T, C = x.shape
    qu, ql = float(2 ** (bits - 1) - 1), float(-2 ** (bits - 1))          # train_model.py:96-97
    sc_min = math.exp(-4.0) if sc_min is None else sc_min                 # train_model.py:98-99
    sc_max = math.exp(4.0) if sc_max is None else sc_max
    zp = zp0.reshape(1, C).expand(B, C).clone()                           # train_model.py:163-164
    sc = sc0.reshape(1, C).expand(B, C).clone()
    alpha, beta, tgt = alpha.reshape(1, C), beta.reshape(1, C), tgt.reshape(1, C)
    out = torch.empty_like(x)
    codes = torch.empty(B, T, C, dtype=torch.int8) if want_codes else None
    for t in range(T):
        xt = x[:, t]
        s = torch.clamp(sc, min=1e-8)                                     # train_model.py:9-10
        q = torch.clamp(torch.round((xt - zp) / s), ql, qu)               # :13-14, 70
        xr = q * s                                                        # :17
        out[:, t] = xr + zp                                               # :73
        if want_codes:
            codes[:, t] = q.to(torch.int8)
        zp = zp + alpha * xr                                              # :77
        err = q.abs() - tgt                                               # :78
        sc = torch.clamp(sc + (sc * beta) * err, sc_min, sc_max)          # :79-81
    return out, zp, sc, codes


def single_query_attention(q, khat, vhat, heads, scaling):
    """softmax(scaling * q.K^T) V for one query per (sequence, head), llama_attention.py:41-44
    with the causal mask of a last-position query (it sees every key).
    ``q [B, heads*d]``, ``khat``/``vhat [B, T, heads*d]`` fp32 -> ``[B, heads*d]``."""
    B, T, C = khat.shape
    d = C // heads
    qh = q.view(B, heads, 1, d)
    kh = khat.view(B, T, heads, d).transpose(1, 2)
    vh = vhat.view(B, T, heads, d).transpose(1, 2)
    w = torch.softmax(torch.matmul(qh, kh.transpose(2, 3)) * scaling, dim=-1)
    return torch.matmul(w, vh).reshape(B, C)


def decode_step(q, k, v, kp, vp, heads, scaling, bits=4):
    """One decode-attention step of one layer the way the CPU path has to do it: run the recurrence
    over the whole context of K and of V, then attend.  ``kp`` / ``vp``: the five ``[C]`` vectors
    (zp_init, scale_init, alpha, beta, target)."""
    khat, _, _, _ = quant_stream_f32(k, *kp, bits=bits)
    vhat, _, _, _ = quant_stream_f32(v, *vp, bits=bits)
    return single_query_attention(q, khat, vhat, heads, scaling)
