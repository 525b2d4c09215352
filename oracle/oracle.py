"""ctypes/numpy front end of the ADKV CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the bench's cpu_baseline leg may import this module; the shipped
package never does.  fp16 arrays are numpy ``float16`` (or ``uint16`` bit patterns) on this side
and raw 16-bit words on the C side.

Reference lines each call follows are cited in ``adkv_oracle.h`` / ``adkv_oracle.c``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "libadkv_oracle.so")


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_SO) or (
            os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_DIR, "adkv_oracle.c"))):
        subprocess.check_call(["make", "-s", "-B", "-C", _DIR, "libadkv_oracle.so"])
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        u16, i32, f32, f64, vp = C.c_uint16, C.c_int, C.c_float, C.c_double, C.c_void_p
        L.adkv_o_h2f.restype, L.adkv_o_h2f.argtypes = f32, [u16]
        L.adkv_o_f2h.restype, L.adkv_o_f2h.argtypes = u16, [f32]
        L.adkv_o_d2h.restype, L.adkv_o_d2h.argtypes = u16, [f64]
        for n in ("hmul", "hadd", "hsub"):
            f = getattr(L, "adkv_o_" + n)
            f.restype, f.argtypes = u16, [u16, u16]
        L.adkv_o_hfma.restype, L.adkv_o_hfma.argtypes = u16, [u16, u16, u16]
        L.adkv_o_quantize_f16.restype, L.adkv_o_quantize_f16.argtypes = i32, [u16, u16, u16]
        L.adkv_o_omt_f16.restype, L.adkv_o_omt_f16.argtypes = u16, [u16, u16]
        L.adkv_o_update_f16.restype = None
        L.adkv_o_update_f16.argtypes = [i32, C.POINTER(u16), C.POINTER(u16), u16, u16, u16]
        L.adkv_o_dequant2_f16.restype, L.adkv_o_dequant2_f16.argtypes = u16, [i32, u16, u16]
        L.adkv_o_dequant1_f16.restype, L.adkv_o_dequant1_f16.argtypes = u16, [i32, u16, u16]
        L.adkv_o_byte_offset.restype, L.adkv_o_byte_offset.argtypes = C.c_int64, [i32, i32, i32]
        L.adkv_o_get_code.restype, L.adkv_o_get_code.argtypes = i32, [vp, i32, i32, i32]
        L.adkv_o_put_code.restype, L.adkv_o_put_code.argtypes = None, [vp, i32, i32, i32, i32]
        L.adkv_o_encode_kv_f16.restype = None
        L.adkv_o_encode_kv_f16.argtypes = [vp] * 7 + [i32] * 5 + [vp]
        L.adkv_o_replay_f16.restype = None
        L.adkv_o_replay_f16.argtypes = [vp] * 6 + [i32] * 5 + [vp, vp]
        L.adkv_o_forward_qk_f16.restype = None
        L.adkv_o_forward_qk_f16.argtypes = [vp] * 8 + [i32] * 5 + [vp, vp]
        L.adkv_o_forward_ov_f16.restype = None
        L.adkv_o_forward_ov_f16.argtypes = [vp] * 8 + [i32] * 5 + [vp, vp]
        L.adkv_o_quant_f32.restype = None
        L.adkv_o_quant_f32.argtypes = [vp] * 6 + [i32] * 4 + [f32, f32] + [vp] * 6
        L.adkv_o_attention_f64.restype = None
        L.adkv_o_attention_f64.argtypes = [vp] * 3 + [i32] * 4 + [f64, vp, vp]
        _lib = L
    return _lib


# ---------------------------------------------------------------------------------------------
# helpers
# ---------------------------------------------------------------------------------------------

def _h(a) -> np.ndarray:
    """Contiguous uint16 view of an fp16 (or already-uint16) array."""
    a = np.asarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    elif a.dtype != np.uint16:
        a = a.astype(np.float16).view(np.uint16)
    return np.ascontiguousarray(a)


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def get_bits() -> int:
    return lib().adkv_o_get_bits()


class code_bits:
    """``with code_bits(2): ...`` runs the semantics-B functions with 2-bit codes (the default, 4,
    is the reference's format) and restores the previous width afterwards."""

    def __init__(self, bits: int):
        self.bits = bits

    def __enter__(self):
        self.prev = get_bits()
        if lib().adkv_o_set_bits(self.bits) != 0:
            raise ValueError(f"unsupported code width {self.bits}")
        return self

    def __exit__(self, *exc):
        lib().adkv_o_set_bits(self.prev)
        return False


def n_super(tokens: int) -> int:
    """Supergroups (8 tokens each; 16 with 2-bit codes) covering ``tokens`` tokens;
    llama_adkv.py:84-85."""
    tpw = 32 // get_bits()
    return (tokens + tpw - 1) // tpw


def alloc_cache(B: int, H: int, cap_tokens: int, D: int) -> np.ndarray:
    """Zero cache [B,H,n_super,D/4,4,4] uint8; llama_adkv.py:87-94."""
    return np.zeros((B, H, n_super(cap_tokens), D // 4, 4, 4), dtype=np.uint8)


def unpack_codes(cache: np.ndarray, T: int) -> np.ndarray:
    """[B,H,T,D] int8 codes from a packed cache (pure numpy; independent of the C unpacker)."""
    B, H, S, G, _, _ = cache.shape
    D = G * 4
    bits = get_bits()
    per_byte, tpw = 8 // bits, 32 // bits
    c = cache.reshape(B, H, S, D, 4)                      # (.., sg, channel, byte_row)
    fields = [((c >> (bits * i)) & ((1 << bits) - 1)).astype(np.int8) - (1 << (bits - 1))
              for i in range(per_byte)]                   # token tpw*sg + per_byte*br + i
    tok = np.stack(fields, axis=-1).reshape(B, H, S, D, tpw)   # (.., sg, channel, t % tpw)
    tok = tok.transpose(0, 1, 2, 4, 3).reshape(B, H, S * tpw, D)
    return np.ascontiguousarray(tok[:, :, :T])


# ---------------------------------------------------------------------------------------------
# semantics B
# ---------------------------------------------------------------------------------------------

def encode_kv_f16(cache, kv_new, zp, sc, alpha, beta, tgt):
    """In-place prefill encode; returns final state [B,H,D,2] uint16 (zp, sc)."""
    kv = _h(kv_new)
    B, H, T, D = kv.shape
    assert cache.dtype == np.uint8 and cache.flags.c_contiguous
    cap = cache.shape[2]
    assert n_super(T) <= cap and cache.shape[3] * 4 == D
    state = np.zeros((B, H, D, 2), dtype=np.uint16)
    ps = [_h(x) for x in (zp, sc, alpha, beta, tgt)]
    lib().adkv_o_encode_kv_f16(_p(cache), _p(kv), *[_p(x) for x in ps], B, H, T, D, cap, _p(state))
    return state


def replay_f16(cache, zp, sc, alpha, beta, tgt, T, want_khat=True):
    """Returns (khat [B,H,T,D] float16 or None, state [B,H,D,2] uint16)."""
    B, H, cap, G = cache.shape[:4]
    D = G * 4
    khat = np.zeros((B, H, T, D), dtype=np.uint16) if want_khat else None
    state = np.zeros((B, H, D, 2), dtype=np.uint16)
    ps = [_h(x) for x in (zp, sc, alpha, beta, tgt)]
    lib().adkv_o_replay_f16(_p(cache), *[_p(x) for x in ps], B, H, T, D, cap, _p(khat), _p(state))
    return (khat.view(np.float16) if want_khat else None), state


def forward_qk_f16(q, cache, k_new, zp, sc, alpha, beta, tgt, T, refemu=False):
    """Appends k_new at slot T in place.  Returns (logits_exact f64 [B,H,T+1], refemu f16|None)."""
    B, H, cap, G = cache.shape[:4]
    D = G * 4
    qh, kn = _h(q).reshape(B, H, D), _h(k_new).reshape(B, H, D)
    assert T // (32 // get_bits()) < cap
    out = np.zeros((B, H, T + 1), dtype=np.float64)
    emu = np.zeros((B, H, T + 1), dtype=np.uint16) if refemu else None
    ps = [_h(x) for x in (zp, sc, alpha, beta, tgt)]
    lib().adkv_o_forward_qk_f16(_p(qh), _p(cache), _p(kn), *[_p(x) for x in ps],
                                B, H, T, D, cap, _p(out), _p(emu))
    return out, (emu.view(np.float16) if refemu else None)


def forward_ov_f16(attn, cache, v_new, zp, sc, alpha, beta, tgt, refemu=False):
    """Appends v_new at slot T=attn.shape[2]-1.  Returns (out_exact f64 [B,H,D], refemu|None)."""
    B, H, cap, G = cache.shape[:4]
    D = G * 4
    a = _h(attn)
    T = a.shape[2] - 1
    vn = _h(v_new).reshape(B, H, D)
    assert T // (32 // get_bits()) < cap
    out = np.zeros((B, H, D), dtype=np.float64)
    emu = np.zeros((B, H, D), dtype=np.uint16) if refemu else None
    ps = [_h(x) for x in (zp, sc, alpha, beta, tgt)]
    lib().adkv_o_forward_ov_f16(_p(a), _p(cache), _p(vn), *[_p(x) for x in ps],
                                B, H, T, D, cap, _p(out), _p(emu))
    return out, (emu.view(np.float16) if refemu else None)


def decode_step_f16(q, k_cache, v_cache, k_new, v_new, kp, vp, T, scaling, mask=None):
    """One decode-attention step exactly as llama_adkv.py:264-274 composes it, with exact
    (fp64) sums inside the two GEMVs: logits -> fp16 -> fp32*scaling(+mask) -> softmax -> fp16
    weights -> OV.  Returns (out f64 [B,H,D], weights f16 [B,H,T+1], logits f64)."""
    logits, _ = forward_qk_f16(q, k_cache, k_new, *kp, T)
    l16 = logits.astype(np.float16)                        # forward_qk returns fp16
    l32 = l16.astype(np.float32) * np.float32(scaling)
    if mask is not None:
        l32 = l32 + np.asarray(mask, dtype=np.float32)
    m = l32.max(axis=-1, keepdims=True)
    e = np.exp((l32 - m).astype(np.float64))
    w = (e / e.sum(axis=-1, keepdims=True)).astype(np.float32).astype(np.float16)
    out, _ = forward_ov_f16(w, v_cache, v_new, *vp)
    return out, w, logits


# ---------------------------------------------------------------------------------------------
# semantics A
# ---------------------------------------------------------------------------------------------

def quant_f32(x, zp0, sc0, alpha, beta, tgt, bits=4, sc_min=None, sc_max=None, want_seq=False):
    """train_model.py:61-81 on x [B,T,C] fp32.  Returns dict(xhat, codes, zp, sc[, zp_seq, sc_seq])."""
    import math
    x = np.ascontiguousarray(x, dtype=np.float32)
    B, T, Cc = x.shape
    sc_min = np.float32(math.exp(-4.0)) if sc_min is None else np.float32(sc_min)
    sc_max = np.float32(math.exp(4.0)) if sc_max is None else np.float32(sc_max)
    ps = [np.ascontiguousarray(p, dtype=np.float32).reshape(Cc) for p in (zp0, sc0, alpha, beta, tgt)]
    xhat = np.zeros_like(x)
    codes = np.zeros(x.shape, dtype=np.int8)
    zps = np.zeros_like(x) if want_seq else None
    scs = np.zeros_like(x) if want_seq else None
    zpo = np.zeros((B, Cc), dtype=np.float32)
    sco = np.zeros((B, Cc), dtype=np.float32)
    lib().adkv_o_quant_f32(_p(x), *[_p(p) for p in ps], B, T, Cc, bits, float(sc_min), float(sc_max),
                           _p(xhat), _p(codes), _p(zps), _p(scs), _p(zpo), _p(sco))
    r = dict(xhat=xhat, codes=codes, zp=zpo, sc=sco)
    if want_seq:
        r.update(zp_seq=zps, sc_seq=scs)
    return r


def attention_f64(q, K, V, scaling):
    """softmax(scaling * q.K^T) V for one query per (b,h).  q [B,H,D], K/V [B,H,T,D] fp32."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    K = np.ascontiguousarray(K, dtype=np.float32)
    V = np.ascontiguousarray(V, dtype=np.float32)
    B, H, T, D = K.shape
    out = np.zeros((B, H, D), dtype=np.float64)
    w = np.zeros((B, H, T), dtype=np.float64)
    lib().adkv_o_attention_f64(_p(q), _p(K), _p(V), B, H, T, D, float(scaling), _p(out), _p(w))
    return out, w
