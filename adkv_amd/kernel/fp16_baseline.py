"""fp16-KV single-query attention: the uncompressed-cache comparator for the ADKV decode path.

Not part of the reference's API (it ships no fp16 kernel; its memory model for the fp16 cache is
tools/memory_comparison_fig.py:46-56).  Exists so that "ADKV versus an fp16 KV cache" is measured
on the same GPU with a kernel that streams K and V once at HBM speed.
"""
from __future__ import annotations

import torch

from .. import _lib
from .gemv import _chk, _need_device


def fp16_decode_attention(q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, scaling: float,
                          workspace: torch.Tensor | None = None) -> torch.Tensor:
    """``softmax(scaling * q K^T) V`` for one query per head.

    q ``[B, H, 1, 128]`` or ``[B, H, 128]``, K and V ``[B, H, T, 128]``, all fp16 and contiguous.
    Returns ``[B, H, 128]`` fp16."""
    dev = _need_device(q, K, V)
    for t, n in ((q, "q"), (K, "K"), (V, "V")):
        _chk(t.dtype == torch.float16 and t.is_contiguous(), f"{n} must be contiguous float16")
    B, H, T, D = K.shape
    _chk(V.shape == K.shape, "K and V shapes differ")
    _chk(q.numel() == B * H * D, "q must hold one query per head")
    L = _lib.lib()
    need = L.adkv_fp16_decode_workspace_bytes(B, H, T)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    _chk(workspace.is_cuda and workspace.numel() * workspace.element_size() >= need,
         "workspace too small")
    out = torch.empty(B, H, D, dtype=torch.float16, device=dev)
    _lib.check(L.adkv_fp16_decode(q.data_ptr(), K.data_ptr(), V.data_ptr(), out.data_ptr(),
                                  workspace.data_ptr(), workspace.numel() * workspace.element_size(),
                                  B, H, T, D, float(scaling), _lib.current_stream_ptr(dev)),
                "adkv_fp16_decode")
    return out
