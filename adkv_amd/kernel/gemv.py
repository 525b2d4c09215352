"""Drop-in for the reference's ``adkv.kernel.gemv`` (src/adkv/kernel/gemv.py:16-132).

Same three functions, same argument order, same tensor layouts and the same error messages as the
reference's C++ bindings (src/adkv/kernel/gemv.cu:368-414, 883-939, 1233-1288); the work is done
by hand-written gfx950 kernels behind ``libadkv_hip.so``.  Differences, all on the safe side:

* launches go to PyTorch's *current* stream (the reference uses legacy stream 0);
* an unsupported head dim raises in ``forward_qk`` / ``forward_ov`` too (the reference's launcher
  silently skips the launch and returns uninitialised memory, gemv.cu:875-878, 1226-1229);
* logits and outputs are accumulated in fp32 and rounded once to fp16 (the reference accumulates in
  fp16); codes written to the cache and the filter state are bit-identical.
"""
from __future__ import annotations

import functools

import torch

from .. import _lib

_TILE = 4
_DIMS = (128, 256, 512)
_GROUPS = (1, 2, 4, 8)   # query heads per KV head


def _chk(cond: bool, msg: str) -> None:
    # TORCH_CHECK surfaces as RuntimeError in Python
    if not cond:
        raise RuntimeError(msg)


def _need_device(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type == "cuda":
        for t in tensors:
            if t.device != dev:
                break
        else:
            return dev
    for t in tensors:
        _chk(t.is_cuda, "ADKV kernels need every tensor on a HIP device; there is no CPU path")
        _chk(t.device == dev, "ADKV kernels need all tensors on the same device")
    return dev


def _params(tensors, names, nh, dim):
    want = nh * dim
    res = []
    for t in tensors:
        if t.dtype != torch.float16 or t.numel() != want:
            break
        res.append(t if t.is_contiguous() else t.contiguous())
    else:
        return res
    for t, n in zip(tensors, names):      # same order of complaints as the reference's checks
        _chk(t.dtype == torch.float16, f"{n} must be float16")
    for t, n in zip(tensors, names):
        _chk(t.numel() == want, f"{n} must have nh*DIM = {want} elements")
    raise AssertionError("unreachable")


@functools.lru_cache(maxsize=4096)
def _row_pitch(n: int) -> int:
    """The library's row pitch for rows of ``n`` elements (a pure function of ``n``)."""
    return int(_lib.lib().adkv_row_pitch(n))


def _pitch(n: int) -> int:
    """Row pitch for a ``[rows, n]`` logits / weights matrix.  Long rows are padded to the library's
    recommended pitch (an odd multiple of 128 elements) so that rows of different heads do not all
    start in one memory channel; short rows stay packed."""
    return _row_pitch(n) if n >= 1024 else n


def _rows_view(t: torch.Tensor):
    """``(tensor, pitch)`` for a ``[B, nh, n]`` matrix whose rows are ``pitch`` elements apart: the
    tensor itself when it is packed or a padded view this module produced, else a packed copy."""
    B, nh, n = t.shape
    if t.is_contiguous():
        return t, n
    if t.stride(2) == 1 and t.stride(1) >= n and t.stride(0) == nh * t.stride(1):
        return t, t.stride(1)
    return t.contiguous(), n


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _ckpt_args(ckpt: torch.Tensor | None, ckpt_interval: int, B: int, nh: int, DIM: int, bits: int = 4):
    """Validates a checkpoint tensor ``[B, nh, n_ckpt_cap, DIM, 2]`` fp16 -> (ptr, cap, interval)."""
    if ckpt is None:
        return None, 0, 0
    _chk(ckpt.dtype == torch.float16 and ckpt.is_contiguous() and ckpt.dim() == 5
         and ckpt.shape[0] == B and ckpt.shape[1] == nh and ckpt.shape[3] == DIM and ckpt.shape[4] == 2
         and ckpt.shape[2] >= 1,
         "ckpt must be contiguous fp16 [B, nh, n_ckpt_cap, DIM, 2]")
    tps = 32 // bits
    _chk(ckpt_interval > 0 and ckpt_interval % tps == 0,
         f"ckpt_interval must be a positive multiple of {tps}")
    return ckpt.data_ptr(), ckpt.shape[2], int(ckpt_interval)


def forward_qk(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    k_new: torch.Tensor,
    k_zp: torch.Tensor,
    k_sc: torch.Tensor,
    k_alpha: torch.Tensor,
    k_beta: torch.Tensor,
    k_t: torch.Tensor,
    T: int,
    scale_min: float,
    scale_max: float,
    *,
    state_out: torch.Tensor | None = None,
    ckpt: torch.Tensor | None = None,
    ckpt_interval: int = 0,
    bits: int = 4,
) -> torch.Tensor:
    """Decode-phase QK^T over the nibble-packed ADKV cache (reference gemv.py:16-55).

    ``o[b,h,t] = sum_c q[b,h,c] * k_deq[b,h,t,c]`` for the ``T`` cached tokens; then ``k_new`` is
    quantised with the filter state after token ``T-1`` and written at position ``T`` in place, and
    its own logit is returned as the last element.

    Args:
        q, k_new: ``[B, nh, 1, DIM]`` float16.
        k_cache:  ``[B, nh, n_super_cap, DIM/4, 4, 4]`` uint8, contiguous, appended in place.
        k_zp, k_sc, k_alpha, k_beta, k_t: ``[nh, DIM]`` float16 ADKV parameters.
        T: number of cached tokens.
        scale_min, scale_max: kept for API compatibility (unused by the fp16 recurrence).
        state_out: optional ``[B, nh, DIM, 2]`` float16, receives (zp, sc) after token ``T-1``
            (extension; not in the reference).
        ckpt, ckpt_interval: optional state checkpoints of this cache, ``[B, nh, n, DIM, 2]`` float16
            with entry ``j`` = state before token ``(j+1)*ckpt_interval`` (extension).  With them
            the time axis is replayed in independent segments; entry ``T/ckpt_interval - 1`` is
            written when token ``T`` opens a new interval.

    Returns ``[B, nh, T+1]`` float16 logits.
    """
    _chk(q.dtype == torch.float16, "q must be float16")
    _chk(k_new.dtype == torch.float16, "k_new must be float16")
    _chk(k_cache.dtype == torch.uint8, "k_cache must be uint8")
    _chk(k_cache.is_contiguous(), "k_cache must be contiguous (appended in place)")
    B, nq = q.shape[0], q.shape[1]
    nh = k_cache.shape[1]          # KV heads; nq is a multiple of it under grouped-query attention
    n_super_cap, n_cgroup = k_cache.shape[2], k_cache.shape[3]
    DIM = n_cgroup * _TILE
    zp, sc, al, be, tg = _params((k_zp, k_sc, k_alpha, k_beta, k_t),
                                 ("k_zp", "k_sc", "k_alpha", "k_beta", "k_t"), nh, DIM)
    _chk(DIM == q.shape[3], "q head dimension does not match k_cache")
    _chk(nq % nh == 0 and nq // nh in _GROUPS, "query heads must be 1, 2, 4 or 8 times the KV heads")
    _chk(nq == nh or DIM == 128, "grouped-query attention needs DIM == 128")
    _chk(T >= 0, "T must be non-negative")
    _chk(bits in (2, 4), "bits must be 2 or 4")
    _chk(bits == 4 or DIM == 128, "2-bit codes need DIM == 128")
    _chk(T // (32 // bits) < n_super_cap, f"k_cache has no free supergroup to append token {T}")
    _chk(DIM in _DIMS, "DIM must be 128, 256 or 512")
    dev = _need_device(q, k_cache, k_new, zp, sc, al, be, tg)

    q_flat = q.contiguous()
    k_new_flat = k_new.reshape(B * nh, DIM).contiguous()
    ld = _pitch(T + 1)
    o = torch.empty((B, nq, ld), dtype=torch.float16, device=dev)
    if state_out is not None:
        _chk(state_out.dtype == torch.float16 and state_out.is_contiguous()
             and state_out.numel() == B * nh * DIM * 2, "state_out must be contiguous fp16 [B,nh,DIM,2]")
    cp, ccap, civ = _ckpt_args(ckpt, ckpt_interval, B, nh, DIM, bits)
    with _lib.device_guard(dev):
        rc = _lib.lib().adkv_forward_qk_gqa(
            q_flat.data_ptr(), k_cache.data_ptr(), k_new_flat.data_ptr(), o.data_ptr(),
            zp.data_ptr(), sc.data_ptr(), al.data_ptr(), be.data_ptr(), tg.data_ptr(),
            B, nq, nh, T, DIM, n_super_cap, bits, ld, _ptr(state_out), cp, ccap, civ,
            _lib.current_stream_ptr(dev))
    _lib.check(rc, "forward_qk")
    return o[:, :, :T + 1]


def forward_ov(
    attn: torch.Tensor,
    v_cache: torch.Tensor,
    v_new: torch.Tensor,
    v_zp: torch.Tensor,
    v_sc: torch.Tensor,
    v_alpha: torch.Tensor,
    v_beta: torch.Tensor,
    v_t: torch.Tensor,
    scale_min: float,
    scale_max: float,
    *,
    state_out: torch.Tensor | None = None,
    ckpt: torch.Tensor | None = None,
    ckpt_interval: int = 0,
    bits: int = 4,
) -> torch.Tensor:
    """Decode-phase OV over the nibble-packed ADKV cache (reference gemv.py:58-97).

    ``o[b,h,c] = sum_t attn[b,h,t] * v_deq[b,h,t,c]`` over the ``T = attn.shape[2]-1`` cached
    tokens plus ``attn[T] * v_deq_new``; ``v_new`` is quantised with the state after token ``T-1``
    and written at position ``T`` in place.

    Returns ``[B, nh, DIM]`` float16.
    """
    _chk(attn.dtype == torch.float16, "attn must be float16")
    _chk(v_new.dtype == torch.float16, "v_new must be float16")
    _chk(v_cache.dtype == torch.uint8, "v_cache must be uint8")
    _chk(v_cache.is_contiguous(), "v_cache must be contiguous (appended in place)")
    B, nq = attn.shape[0], attn.shape[1]
    nh = v_cache.shape[1]
    _chk(attn.shape[2] >= 1, "attn must contain the cached weights plus the self weight")
    T = attn.shape[2] - 1
    n_super_cap, n_cgroup = v_cache.shape[2], v_cache.shape[3]
    DIM = n_cgroup * _TILE
    zp, sc, al, be, tg = _params((v_zp, v_sc, v_alpha, v_beta, v_t),
                                 ("v_zp", "v_sc", "v_alpha", "v_beta", "v_t"), nh, DIM)
    _chk(DIM == v_new.shape[-1], "v_new head dimension does not match v_cache")
    _chk(nq % nh == 0 and nq // nh in _GROUPS, "query heads must be 1, 2, 4 or 8 times the KV heads")
    _chk(nq == nh or DIM == 128, "grouped-query attention needs DIM == 128")
    _chk(T >= 0, "T must be non-negative")
    _chk(bits in (2, 4), "bits must be 2 or 4")
    _chk(bits == 4 or DIM == 128, "2-bit codes need DIM == 128")
    _chk(T // (32 // bits) < n_super_cap, f"v_cache has no free supergroup to append token {T}")
    _chk(DIM in _DIMS, "DIM must be 128, 256 or 512")
    dev = _need_device(attn, v_cache, v_new, zp, sc, al, be, tg)

    attn_flat, ld = _rows_view(attn)
    v_new_flat = v_new.reshape(B * nh, DIM).contiguous()
    o = torch.empty((B * nq, DIM), dtype=torch.float16, device=dev)
    if state_out is not None:
        _chk(state_out.dtype == torch.float16 and state_out.is_contiguous()
             and state_out.numel() == B * nh * DIM * 2, "state_out must be contiguous fp16 [B,nh,DIM,2]")
    cp, ccap, civ = _ckpt_args(ckpt, ckpt_interval, B, nh, DIM, bits)
    L = _lib.lib()
    ws, ws_bytes = None, 0
    if cp is not None:
        ws_bytes = L.adkv_forward_ov_gqa_workspace_bytes(B, nq, nh, T, DIM, ccap, civ)
        if ws_bytes:
            ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=dev)
    with _lib.device_guard(dev):
        rc = L.adkv_forward_ov_gqa(
            attn_flat.data_ptr(), v_cache.data_ptr(), v_new_flat.data_ptr(), o.data_ptr(),
            zp.data_ptr(), sc.data_ptr(), al.data_ptr(), be.data_ptr(), tg.data_ptr(),
            B, nq, nh, T, DIM, n_super_cap, bits, ld, _ptr(state_out), cp, ccap, civ,
            _ptr(ws), ws_bytes, _lib.current_stream_ptr(dev))
    _lib.check(rc, "forward_ov")
    return o.view(attn.shape[0], attn.shape[1], -1)


def encode_kv(
    kv_cache: torch.Tensor,
    kv_new: torch.Tensor,
    kv_zp: torch.Tensor,
    kv_sc: torch.Tensor,
    kv_alpha: torch.Tensor,
    kv_beta: torch.Tensor,
    kv_t: torch.Tensor,
    scale_min: float,
    scale_max: float,
    *,
    state_out: torch.Tensor | None = None,
    ckpt: torch.Tensor | None = None,
    ckpt_interval: int = 0,
) -> torch.Tensor:
    """Prefill: quantise tokens ``[0, T)`` into the uint4-tiled KV cache (reference gemv.py:100-132).

    Replays the ADKV filter from ``(kv_zp, kv_sc)``; token ``t`` goes to byte row ``t/2``, low
    nibble for even ``t`` and high nibble for odd ``t``.  Purely in place; returns ``kv_cache``.
    ``ckpt`` (extension): receives the state before every token ``(j+1)*ckpt_interval <= T``.
    """
    _chk(kv_new.dtype == torch.float16, "kv_new must be float16")
    _chk(kv_cache.dtype == torch.uint8, "kv_cache must be uint8")
    _chk(kv_cache.is_contiguous(), "kv_cache must be contiguous (written in place)")
    B, nh, T, DIM = kv_new.shape
    zp, sc, al, be, tg = _params((kv_zp, kv_sc, kv_alpha, kv_beta, kv_t),
                                 ("kv_zp", "kv_sc", "kv_alpha", "kv_beta", "kv_t"), nh, DIM)
    n_super_cap = kv_cache.shape[2]
    _chk(kv_cache.shape[3] * _TILE == DIM, "kv_cache channel groups do not match kv_new head dim")
    n_super = ((T + 1) // 2 + _TILE - 1) // _TILE
    _chk(n_super <= n_super_cap,
         f"kv_cache capacity too small: need {n_super} supergroups for {T} tokens, have {n_super_cap}")
    _chk(DIM in _DIMS, "DIM must be 128, 256 or 512")
    dev = _need_device(kv_cache, kv_new, zp, sc, al, be, tg)

    kv_new_flat = kv_new.contiguous()
    if state_out is not None:
        _chk(state_out.dtype == torch.float16 and state_out.is_contiguous()
             and state_out.numel() == B * nh * DIM * 2, "state_out must be contiguous fp16 [B,nh,DIM,2]")
    if B * nh * T == 0 and state_out is None:
        return kv_cache
    cp, ccap, civ = _ckpt_args(ckpt, ckpt_interval, B, nh, DIM)
    with _lib.device_guard(dev):
        rc = _lib.lib().adkv_encode_kv_ex(
            kv_cache.data_ptr(), kv_new_flat.data_ptr(),
            zp.data_ptr(), sc.data_ptr(), al.data_ptr(), be.data_ptr(), tg.data_ptr(),
            B, nh, T, DIM, n_super_cap, _ptr(state_out), cp, ccap, civ,
            _lib.current_stream_ptr(dev))
    _lib.check(rc, "encode_kv")
    return kv_cache


def append_kv(
    kv_cache: torch.Tensor,
    kv_new: torch.Tensor,
    kv_zp: torch.Tensor,
    kv_sc: torch.Tensor,
    kv_alpha: torch.Tensor,
    kv_beta: torch.Tensor,
    kv_t: torch.Tensor,
    T0: int,
    state: torch.Tensor,
    *,
    ckpt: torch.Tensor | None = None,
    ckpt_interval: int = 0,
    bits: int = 4,
) -> torch.Tensor:
    """Streaming append (extension; the reference can only append inside forward_qk/forward_ov,
    after an O(T) replay): quantise ``kv_new [B, nh, n, DIM]`` as tokens ``T0 .. T0+n-1``.

    ``state`` ``[B, nh, DIM, 2]`` float16 carries (zp, sc): the state after token ``T0-1`` on entry
    (ignored when ``T0 == 0``), the state after the last new token on return.  The cache ends up
    byte-identical to ``encode_kv`` over all ``T0+n`` tokens.  Returns ``kv_cache``.
    """
    _chk(kv_new.dtype == torch.float16, "kv_new must be float16")
    _chk(kv_cache.dtype == torch.uint8, "kv_cache must be uint8")
    _chk(kv_cache.is_contiguous(), "kv_cache must be contiguous (written in place)")
    B, nh, n, DIM = kv_new.shape
    zp, sc, al, be, tg = _params((kv_zp, kv_sc, kv_alpha, kv_beta, kv_t),
                                 ("kv_zp", "kv_sc", "kv_alpha", "kv_beta", "kv_t"), nh, DIM)
    n_super_cap = kv_cache.shape[2]
    _chk(kv_cache.shape[3] * _TILE == DIM, "kv_cache channel groups do not match kv_new head dim")
    _chk(T0 >= 0, "T0 must be non-negative")
    _chk(bits in (2, 4), "bits must be 2 or 4")
    tps = 32 // bits
    need = (T0 + n + tps - 1) // tps
    _chk(need <= n_super_cap,
         f"kv_cache capacity too small: need {need} supergroups for {T0 + n} tokens, have {n_super_cap}")
    _chk(DIM in _DIMS, "DIM must be 128, 256 or 512")
    _chk(state.dtype == torch.float16 and state.is_contiguous() and state.numel() == B * nh * DIM * 2,
         "state must be contiguous fp16 [B,nh,DIM,2]")
    dev = _need_device(kv_cache, kv_new, zp, sc, al, be, tg, state)
    cp, ccap, civ = _ckpt_args(ckpt, ckpt_interval, B, nh, DIM, bits)
    if n == 0:
        return kv_cache
    x = kv_new.contiguous()
    with _lib.device_guard(dev):
        rc = _lib.lib().adkv_append_kv(
            kv_cache.data_ptr(), x.data_ptr(),
            zp.data_ptr(), sc.data_ptr(), al.data_ptr(), be.data_ptr(), tg.data_ptr(),
            B, nh, T0, n, DIM, n_super_cap, bits, state.data_ptr(), cp, ccap, civ,
            _lib.current_stream_ptr(dev))
    _lib.check(rc, "append_kv")
    return kv_cache


_DT_F16, _DT_BF16 = 1, 2     # ADKV_DT_F16 / ADKV_DT_BF16 of include/adkv_hip.h


def _row_strides(t: torch.Tensor):
    """``(tensor, strides)`` for new rows ``[B, nh, n, DIM]``: ``strides`` is None for a packed
    tensor, a ctypes array of the (batch, head, token) element strides when the library can read
    the rows where they lie (contiguous channels, even strides, 4-byte aligned), else the tensor
    is packed first."""
    if t.is_contiguous():
        return t, None
    sb, sh, st, sc = t.stride()
    if sc == 1 and st >= t.shape[3] and not ((sb | sh | st) & 1) and not (t.data_ptr() & 3) \
            and min(sb, sh) >= 0:
        return t, (_lib.C.c_int64 * 3)(sb, sh, st)
    return t.contiguous(), None


def append_kv_pair(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    k_params,
    v_params,
    T0: int,
    k_state: torch.Tensor,
    v_state: torch.Tensor,
    *,
    k_ckpt: torch.Tensor | None = None,
    v_ckpt: torch.Tensor | None = None,
    ckpt_interval: int = 0,
    bits: int = 4,
) -> None:
    """``append_kv`` for the K and V rows of the same tokens in one launch (the two calls of
    src/adkv/hf/llama_adkv.py:144-153 made together).  Results are byte-identical to two
    ``append_kv`` calls; at small batch the pair takes the time of one tensor because channels are
    the encoder's only parallel axis.  ``k_params`` / ``v_params``: the five ``[nh, DIM]`` fp16
    tensors ``(zp, sc, alpha, beta, quant_target)``.

    ``k_new`` / ``v_new`` ``[B, nh, n, DIM]`` may be float16 or bfloat16 (rounded to fp16 as they
    are read, like the reference's ``.to(torch.float16)``, llama_adkv.py:141-142) and need not be
    packed: a ``[B, n, nh, DIM]`` projection output viewed with the head axis first is read in
    place.
    """
    _chk(k_new.dtype == v_new.dtype and k_new.dtype in (torch.float16, torch.bfloat16),
         "kv_new must be float16 or bfloat16 (K and V alike)")
    _chk(k_cache.dtype == torch.uint8 and v_cache.dtype == torch.uint8, "kv_cache must be uint8")
    _chk(k_cache.is_contiguous() and v_cache.is_contiguous(),
         "kv_cache must be contiguous (written in place)")
    _chk(k_new.shape == v_new.shape and k_cache.shape == v_cache.shape,
         "K and V must have the same shapes")
    B, nh, n, DIM = k_new.shape
    kp = _params(k_params, ("k_zp", "k_sc", "k_alpha", "k_beta", "k_t"), nh, DIM)
    vp = _params(v_params, ("v_zp", "v_sc", "v_alpha", "v_beta", "v_t"), nh, DIM)
    n_super_cap = k_cache.shape[2]
    _chk(k_cache.shape[3] * _TILE == DIM, "kv_cache channel groups do not match kv_new head dim")
    _chk(T0 >= 0, "T0 must be non-negative")
    _chk(bits in (2, 4), "bits must be 2 or 4")
    tps = 32 // bits
    need = (T0 + n + tps - 1) // tps
    _chk(need <= n_super_cap,
         f"kv_cache capacity too small: need {need} supergroups for {T0 + n} tokens, have {n_super_cap}")
    _chk(DIM in _DIMS, "DIM must be 128, 256 or 512")
    for st in (k_state, v_state):
        _chk(st.dtype == torch.float16 and st.is_contiguous() and st.numel() == B * nh * DIM * 2,
             "state must be contiguous fp16 [B,nh,DIM,2]")
    _chk((k_ckpt is None) == (v_ckpt is None), "give both checkpoint tensors or neither")
    dev = _need_device(k_cache, v_cache, k_new, v_new, *kp, *vp, k_state, v_state)
    kc, ccap, civ = _ckpt_args(k_ckpt, ckpt_interval, B, nh, DIM, bits)
    vc, vcap, _ = _ckpt_args(v_ckpt, ckpt_interval, B, nh, DIM, bits)
    _chk(ccap == vcap, "K and V checkpoint tensors must have the same capacity")
    if n == 0:
        return
    xk, ks = _row_strides(k_new)
    xv, vs = _row_strides(v_new)
    arr = _lib.C.c_void_p * 5
    with _lib.device_guard(dev):
        rc = _lib.lib().adkv_append_kv_pair(
            k_cache.data_ptr(), v_cache.data_ptr(), xk.data_ptr(), xv.data_ptr(),
            _DT_BF16 if k_new.dtype == torch.bfloat16 else _DT_F16, ks, vs,
            arr(*[t.data_ptr() for t in kp]), arr(*[t.data_ptr() for t in vp]),
            B, nh, T0, n, DIM, n_super_cap, bits, k_state.data_ptr(), v_state.data_ptr(),
            kc, vc, ccap, civ, _lib.current_stream_ptr(dev))
    _lib.check(rc, "append_kv_pair")


def rope_qk(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor
            ) -> tuple[torch.Tensor, torch.Tensor]:
    """Rotary position embedding of ``q [B, Hq, T, D]`` and ``k [B, H, T, D]`` in one launch.

    Bit-identical to ``transformers``' ``apply_rotary_pos_emb(q, k, cos, sin)`` as the attention
    module calls it (src/adkv/hf/llama_adkv.py:336-337): ``x*cos + rotate_half(x)*sin`` with each
    of the three operations rounded to the tensors' type.  fp16 or bf16, all four tensors of one
    type; ``cos`` / ``sin``: ``[B, T, D]`` (or ``[1, T, D]``).  Any batch / head / token strides with
    contiguous channels are read in place; the results are contiguous.
    """
    _chk(q.dim() == 4 and k.dim() == 4 and cos.dim() == 3 and sin.dim() == 3,
         "q, k must be [B, H, T, D] and cos, sin [B, T, D]")
    B, Hq, T, D = q.shape
    H = k.shape[1]
    _chk(k.shape[0] == B and k.shape[2] == T and k.shape[3] == D, "q and k disagree in shape")
    _chk(q.dtype in (torch.float16, torch.bfloat16), "q must be float16 or bfloat16")
    _chk(k.dtype == q.dtype and cos.dtype == q.dtype and sin.dtype == q.dtype,
         "q, k, cos, sin must share one dtype")
    _chk(cos.shape == sin.shape and cos.shape[1] == T and cos.shape[2] == D and cos.shape[0] in (1, B),
         "cos, sin must be [B, T, D] or [1, T, D]")
    _chk(D % 4 == 0 and B * Hq * T * D > 0, "head dim must be a positive multiple of 4")
    dev = _need_device(q, k, cos, sin)

    def rows(t):        # channels contiguous, even strides, 4-byte aligned base: read in place
        ok = t.stride(-1) == 1 and all(st % 2 == 0 for st in t.stride()[:-1]) and t.data_ptr() % 4 == 0
        return t if ok else t.contiguous()
    q_, k_, c_, s_ = rows(q), rows(k), rows(cos), rows(sin)
    if s_.stride() != c_.stride():
        c_, s_ = c_.contiguous(), s_.contiguous()
    q_out = torch.empty((B, Hq, T, D), dtype=q.dtype, device=dev)
    k_out = torch.empty((B, H, T, D), dtype=q.dtype, device=dev)
    with _lib.device_guard(dev):
        rc = _lib.lib().adkv_rope_qk(
            q_.data_ptr(), k_.data_ptr(), c_.data_ptr(), s_.data_ptr(), q_out.data_ptr(), k_out.data_ptr(),
            B, Hq, H, T, D, q_.stride(0), q_.stride(1), q_.stride(2), k_.stride(0), k_.stride(1), k_.stride(2),
            c_.stride(0) if c_.shape[0] == B and B > 1 else 0, c_.stride(1),
            1 if q.dtype == torch.bfloat16 else 0, _lib.current_stream_ptr(dev))
    _lib.check(rc, "rope_qk")
    return q_out, k_out


def softmax_scale_mask(logits: torch.Tensor, scaling: float,
                       mask: torch.Tensor | None = None) -> torch.Tensor:
    """``softmax(logits.float()*scaling + mask) -> fp16`` in one launch.

    Fuses the element-wise chain the reference runs in torch between the two GEMVs
    (src/adkv/hf/llama_adkv.py:266-271).  ``logits``: fp16 ``[B, nh, n]``; ``mask``: optional
    ``[B, 1, n]`` / ``[B, nh, n]`` / ``[B, 1, 1, n]`` additive mask (any float dtype).
    """
    _chk(logits.dtype == torch.float16, "logits must be float16")
    _chk(logits.dim() == 3, "logits must be [B, nh, n]")
    B, nh, n = logits.shape
    dev = _need_device(logits)
    lg, ld = _rows_view(logits)
    out = torch.empty((B, nh, ld), dtype=torch.float16, device=dev)[:, :, :n]
    rpm, mptr = 1, None
    mk = None
    if mask is not None:
        mk = mask[:, :, 0, :] if mask.dim() == 4 else mask
        _chk(mk.dim() == 3 and mk.shape[0] == B and mk.shape[2] == n and mk.shape[1] in (1, nh),
             "mask must broadcast to [B, nh, n]")
        rpm = nh if mk.shape[1] == 1 else 1
        mk = mk.to(device=dev, dtype=torch.float32).contiguous()
        mptr = mk.data_ptr()
    L = _lib.lib()
    wsb = L.adkv_softmax_workspace_bytes(B * nh, n)
    ws = torch.empty(wsb, dtype=torch.uint8, device=dev) if wsb else None
    with _lib.device_guard(dev):
        rc = L.adkv_softmax_ex(lg.data_ptr(), out.data_ptr(), mptr, B * nh, n, ld, rpm, float(scaling),
                               _ptr(ws), wsb, _lib.current_stream_ptr(dev))
    _lib.check(rc, "softmax_scale_mask")
    return out


def decode_step(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_new: torch.Tensor,
    v_new: torch.Tensor,
    k_params,
    v_params,
    T: int,
    scaling: float,
    mask: torch.Tensor | None = None,
    *,
    k_ckpt: torch.Tensor | None = None,
    v_ckpt: torch.Tensor | None = None,
    ckpt_interval: int = 0,
    bits: int = 4,
    workspace: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """One decode-attention step of a layer through a single library call.

    The body of the reference's ``KVCacheLayer_ADKV.decode`` (src/adkv/hf/llama_adkv.py:245-276):
    ``forward_qk`` -> ``softmax(logits*scaling + mask)`` -> ``forward_ov``, with ``k_new`` / ``v_new``
    appended at slot ``T`` of both caches.  ``k_params`` / ``v_params`` are the five ``[nh, DIM]``
    fp16 tensors ``(zp, sc, alpha, beta, quant_target)``.  Returns ``(out [B,nh,DIM] fp16,
    weights [B,nh,T+1] fp16)``.  ``q``, ``k_new`` and ``v_new`` may all be bfloat16: the kernels
    round them to fp16 as they read them and return ``out`` in bfloat16, with the values of the
    reference's ``.to(torch.float16)`` / ``.to(q.dtype)`` around its kernels
    (llama_adkv.py:248-250, 274) but without those launches.  ``workspace`` (uint8, 256-byte aligned, sized by
    ``decode_step_workspace_bytes``) may be passed to avoid the per-call allocation.
    """
    f16, u8 = torch.float16, torch.uint8
    act = q.dtype            # float16 as in the reference, or bfloat16 (extension; see the docstring)
    if not (act in (f16, torch.bfloat16) and k_new.dtype == act and v_new.dtype == act
            and k_cache.dtype == u8 and v_cache.dtype == u8 and k_cache.is_contiguous()
            and v_cache.is_contiguous()):
        for t, n in ((q, "q"), (k_new, "k_new"), (v_new, "v_new")):
            _chk(t.dtype == (act if act == torch.bfloat16 else f16),
                 f"{n} must be float16" + (" (or bfloat16 like q)" if act == torch.bfloat16 else ""))
        for t, n in ((k_cache, "k_cache"), (v_cache, "v_cache")):
            _chk(t.dtype == u8, f"{n} must be uint8")
            _chk(t.is_contiguous(), f"{n} must be contiguous (appended in place)")
    _chk(k_cache.shape == v_cache.shape, "k_cache and v_cache shapes differ")
    B, nq, nh = q.shape[0], q.shape[1], k_cache.shape[1]
    n_super_cap, DIM = k_cache.shape[2], k_cache.shape[3] * _TILE
    _chk(nq % nh == 0 and nq // nh in _GROUPS, "query heads must be 1, 2, 4 or 8 times the KV heads")
    _chk(nq == nh or DIM == 128, "grouped-query attention needs DIM == 128")
    kp = _params(k_params, ("k_zp", "k_sc", "k_alpha", "k_beta", "k_t"), nh, DIM)
    vp = _params(v_params, ("v_zp", "v_sc", "v_alpha", "v_beta", "v_t"), nh, DIM)
    _chk(DIM == q.shape[-1], "q head dimension does not match k_cache")
    _chk(T >= 0, "T must be non-negative")
    _chk(bits in (2, 4), "bits must be 2 or 4")
    _chk(bits == 4 or DIM == 128, "2-bit codes need DIM == 128")
    if not T // (32 // bits) < n_super_cap:
        raise RuntimeError(f"k_cache has no free supergroup to append token {T}")
    _chk(DIM in _DIMS, "DIM must be 128, 256 or 512")
    dev = _need_device(q, k_cache, v_cache, k_new, v_new, *kp, *vp)
    n = T + 1
    rpm, mptr, mk = 1, None, None
    if mask is not None:
        mk = mask[:, :, 0, :] if mask.dim() == 4 else mask
        _chk(mk.dim() == 3 and mk.shape[0] == B and mk.shape[2] == n and mk.shape[1] in (1, nq),
             "mask must broadcast to [B, nh, n]")
        rpm = nq if mk.shape[1] == 1 else 1
        mk = mk.to(device=dev, dtype=torch.float32).contiguous()
        mptr = mk.data_ptr()
    kcp, ccap, civ = _ckpt_args(k_ckpt, ckpt_interval, B, nh, DIM, bits)
    vcp, vcap, _ = _ckpt_args(v_ckpt, ckpt_interval, B, nh, DIM, bits)
    _chk((k_ckpt is None) == (v_ckpt is None) and ccap == vcap,
         "k_ckpt and v_ckpt must both be given, with the same capacity, or both omitted")
    L = _lib.lib()
    if workspace is None:
        need = L.adkv_decode_step_workspace_bytes(B, nq, nh, T, DIM, ccap, civ)
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    # a caller's workspace is sized against the launch by the library itself ("workspace too small")
    _chk(workspace.dtype == torch.uint8 and workspace.is_cuda, "workspace must be a uint8 device tensor")
    qf = q.contiguous()
    knf = k_new.reshape(B * nh, DIM).contiguous()
    vnf = v_new.reshape(B * nh, DIM).contiguous()
    out = torch.empty((B, nq, DIM), dtype=act, device=dev)
    wld = _row_pitch(n)
    weights = torch.empty((B, nq, wld), dtype=torch.float16, device=dev)
    arr = _lib.C.c_void_p * 5
    with _lib.device_guard(dev):
        rc = L.adkv_decode_step(
            qf.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), knf.data_ptr(), vnf.data_ptr(),
            arr(*[t.data_ptr() for t in kp]), arr(*[t.data_ptr() for t in vp]),
            mptr, rpm, float(scaling), out.data_ptr(), weights.data_ptr(), wld,
            B, nq, nh, T, DIM, n_super_cap, bits, _DT_BF16 if act == torch.bfloat16 else _DT_F16,
            kcp, vcp, ccap, civ,
            workspace.data_ptr(), workspace.numel(), _lib.current_stream_ptr(dev))
    _lib.check(rc, "decode_step")
    return out, weights[:, :, :n]


def decode_step_workspace_bytes(B: int, nq: int, nh: int, T: int, DIM: int, n_ckpt_cap: int = 0,
                                 ckpt_interval: int = 0) -> int:
    """Bytes ``decode_step`` needs for ``nq`` query heads over ``nh`` KV heads."""
    return int(_lib.lib().adkv_decode_step_workspace_bytes(B, nq, nh, T, DIM, n_ckpt_cap,
                                                            ckpt_interval))
