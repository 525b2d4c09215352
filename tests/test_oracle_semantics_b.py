"""Pins the oracle's fp16 (deployment) recurrence, packing and GEMVs without the reference's
runtime: exact-rational step arithmetic, closed forms, a byte-level layout brute force, the
benchmark script's constant cache pattern and replay invariants.

Reference lines pinned: src/adkv/kernel/gemv.cu:79-164 (steps), :220-221 (omt), :243-305 and
:91-146 (packing), :644-654 / :786-798 (two-rounding vs fused dequant), tools/perf_kernel.py:34-49.
"""
from fractions import Fraction

import numpy as np
import pytest

import exact16 as X

F16 = np.float16


def h(x):
    """float -> binary16 bits via exact rounding."""
    return X.from_float(float(x))


# ------------------------------------------------------------------------------------------
# scalar steps
# ------------------------------------------------------------------------------------------

def test_quantize_known_answers(oracle):
    L = oracle.lib()
    q = lambda x, zp, sc: L.adkv_o_quantize_f16(h(x), h(zp), h(sc))
    assert q(1.0, 0.0, 1.0) == 1
    assert q(-1.0, 0.0, 1.0) == -1
    assert q(3.0, 1.0, 0.5) == 4
    # ties go to even (gemv.cu:152 __float2int_rn)
    assert q(0.5, 0.0, 1.0) == 0
    assert q(1.5, 0.0, 1.0) == 2
    assert q(2.5, 0.0, 1.0) == 2
    assert q(-0.5, 0.0, 1.0) == 0
    assert q(-1.5, 0.0, 1.0) == -2
    assert q(-2.5, 0.0, 1.0) == -2
    assert q(1.25, 0.0, 0.5) == 2          # 2.5 -> 2
    assert q(1.75, 0.0, 0.5) == 4          # 3.5 -> 4
    # clamp to [-8, 7]
    assert q(100.0, 0.0, 1.0) == 7
    assert q(-100.0, 0.0, 1.0) == -8
    assert q(7.5, 0.0, 1.0) == 7           # 7.5 -> 8 -> clamp 7
    assert q(-8.5, 0.0, 1.0) == -8
    # degenerate scales: +-inf saturate then clamp, NaN -> 0 (CUDA __float2int_rn)
    assert q(1.0, 0.0, 0.0) == 7
    assert q(-1.0, 0.0, 0.0) == -8
    assert q(0.0, 0.0, 0.0) == 0
    INF, NAN = 0x7C00, 0x7E00
    assert L.adkv_o_quantize_f16(h(1.0), h(0.0), INF) == 0
    assert L.adkv_o_quantize_f16(h(1.0), h(0.0), NAN) == 0
    assert L.adkv_o_quantize_f16(NAN, h(0.0), h(1.0)) == 0
    assert L.adkv_o_quantize_f16(INF, h(0.0), h(1.0)) == 7
    # negative scale flips the sign of the code
    assert q(2.0, 0.0, -1.0) == -2


def test_quantize_vs_numpy_float32(oracle):
    """numpy float32 (IEEE sub, div, rint) as an independent implementation, dense around ties."""
    L = oracle.lib()
    rng = np.random.default_rng(11)
    n = 40000
    sc = rng.uniform(0.05, 4.0, n).astype(F16)
    zp = rng.normal(0, 2, n).astype(F16)
    k = rng.integers(-10, 10, n)
    # half of the samples sit exactly on (k + 1/2) * sc + zp in exact arithmetic, rounded to fp16
    x = np.where(rng.random(n) < 0.5,
                 (k + 0.5) * sc.astype(np.float64) + zp.astype(np.float64),
                 rng.normal(0, 4, n)).astype(F16)
    d = x.astype(np.float32) - zp.astype(np.float32)
    u = d / sc.astype(np.float32)
    want = np.clip(np.rint(u), -8, 7).astype(np.int32)
    xs, zs, ss = x.view(np.uint16), zp.view(np.uint16), sc.view(np.uint16)
    for i in range(n):
        assert L.adkv_o_quantize_f16(int(xs[i]), int(zs[i]), int(ss[i])) == want[i]


def _exact_update(q, zp, sc, alpha, beta, omt):
    """gemv.cu:158-164 in exact-rational binary16: returns (zp', sc')."""
    qf = h(q)
    p = X.hmul(qf, sc)
    nzp = X.hfma(alpha, p, zp)
    f = X.hfma(beta, qf & 0x7FFF, omt)
    return nzp, X.hmul(sc, f)


def test_update_step_vs_exact(oracle):
    import ctypes as C
    import random
    L = oracle.lib()
    rng = random.Random(5)
    for _ in range(20000):
        q = rng.randrange(-8, 8)
        zp = h(rng.gauss(0, 3))
        sc = h(rng.uniform(0.01, 8))
        alpha = h(rng.uniform(0, 1))
        beta = h(rng.uniform(0, 0.1))
        tgt = h(rng.uniform(0, 7))
        omt = X.hadd(0x3C00, X.hmul(beta, tgt) ^ 0x8000)
        assert L.adkv_o_omt_f16(beta, tgt) == omt
        z, s = C.c_uint16(zp), C.c_uint16(sc)
        L.adkv_o_update_f16(q, C.byref(z), C.byref(s), alpha, beta, omt)
        assert (z.value, s.value) == _exact_update(q, zp, sc, alpha, beta, omt)
        # the two dequant forms differ in the number of roundings (gemv.cu:644-645 vs :796)
        assert L.adkv_o_dequant2_f16(q, zp, sc) == X.hadd(X.hmul(h(q), sc), zp)
        assert L.adkv_o_dequant1_f16(q, zp, sc) == X.hfma(h(q), sc, zp)


def test_nibble_bit_trick_all_bytes(oracle):
    """gemv.cu:79-88: 0x6400|n is 1024+n in binary16 and (1024+n)-1032 = n-8 exactly."""
    for n in range(16):
        assert X.h_to_frac(0x6400 | n) == 1024 + n
        assert X.hadd(0x6400 | n, 0x6408 ^ 0x8000) == h(n - 8)
        # the same trick one binade lower reads a high nibble in place
        assert X.h_to_frac(0x5400 | (n << 4)) == 64 + n
        assert X.hadd(0x5400 | (n << 4), h(72.0) ^ 0x8000) == h(n - 8)


# ------------------------------------------------------------------------------------------
# layout
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("T", [0, 1, 2, 7, 8, 9, 15, 16, 17])
def test_layout_bruteforce(oracle, D, T):
    """alpha = beta = 0, zp = 0, sc = 1: codes are the (integer) inputs.  Every byte of the cache is
    checked against the 6-D index meaning [b, h, sg, cg, channel-in-group, byte-row]."""
    B, H = 2, 3
    rng = np.random.default_rng(T * 1000 + D)
    codes = rng.integers(-8, 8, (B, H, T, D)).astype(np.int8)
    zero = np.zeros((H, D), F16)
    one = np.ones((H, D), F16)
    cache = np.full((B, H, oracle.n_super(T) + 1, D // 4, 4, 4), 0xEE, np.uint8)
    oracle.encode_kv_f16(cache, codes.astype(F16), zero, one, zero, zero, one)
    ns = oracle.n_super(T)
    want = np.full_like(cache, 0xEE)
    want[:, :, :ns] = 0
    for t in range(T):
        sg, br = t // 8, (t % 8) // 2
        nibs = (codes[:, :, t, :].astype(np.int16) + 8).astype(np.uint8)       # [B,H,D]
        nibs = nibs.reshape(B, H, D // 4, 4)
        if t % 2 == 0:
            want[:, :, sg, :, :, br] |= nibs
        else:
            want[:, :, sg, :, :, br] |= (nibs << 4).astype(np.uint8)
    assert np.array_equal(cache, want)
    # flat-offset formula and the independent numpy unpacker agree with it
    L = oracle.lib()
    flat = cache[1, 2].reshape(-1)
    for t in range(T):
        for c in (0, 1, 5, D - 1):
            off = ((t // 8 * (D // 4) + c // 4) * 4 + c % 4) * 4 + (t % 8) // 2
            assert L.adkv_o_byte_offset(t, c, D) == off
            b = int(flat[off])
            assert ((b >> 4) if t & 1 else (b & 15)) - 8 == codes[1, 2, t, c]
    assert np.array_equal(oracle.unpack_codes(cache, T), codes)


def test_perf_script_fill_pattern(oracle):
    """tools/perf_kernel.py:34-49: cache bytes 0x5A, zp=0, sc=1, alpha=0.05, beta=0, target=3.5.
    Even tokens decode to q=+2, odd tokens to q=-3; with beta=0 the scale never moves and zp_t is a
    short fp16 sequence computed here in exact arithmetic; logits follow in closed form."""
    B, H, D, T = 1, 2, 128, 37
    cache = np.full((B, H, oracle.n_super(T + 1), D // 4, 4, 4), 0x5A, np.uint8)
    codes = oracle.unpack_codes(cache, T)
    assert np.all(codes[:, :, 0::2] == 2) and np.all(codes[:, :, 1::2] == -3)

    a16 = h(0.05)
    zp, sc = 0x0000, 0x3C00
    omt = X.hadd(0x3C00, X.hmul(0x0000, h(3.5)) ^ 0x8000)
    assert omt == 0x3C00
    khat_seq = []
    for t in range(T):
        q = 2 if t % 2 == 0 else -3
        khat_seq.append(X.hadd(X.hmul(h(q), sc), zp))
        zp, sc = _exact_update(q, zp, sc, a16, 0x0000, omt)
        assert sc == 0x3C00
    p = [np.full((H, D), v, F16) for v in (0.0, 1.0, 0.05, 0.0, 3.5)]
    khat, state = oracle.replay_f16(cache, *p, T)
    for t in range(T):
        assert np.all(khat.view(np.uint16)[:, :, t, :] == khat_seq[t])
    assert np.all(state[..., 0] == zp) and np.all(state[..., 1] == sc)

    rng = np.random.default_rng(3)
    q = (rng.normal(0, 0.5, (B, H, 1, D))).astype(F16)
    k_new = np.zeros((B, H, 1, D), F16)
    logits, _ = oracle.forward_qk_f16(q, cache, k_new, *p, T)
    qsum = q.astype(np.float64).sum(axis=-1)[:, :, 0]
    for t in range(T):
        want = qsum * float(X.h_to_frac(khat_seq[t]))
        assert np.allclose(logits[:, :, t], want, rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------------------------------
# closed forms of the recurrence
# ------------------------------------------------------------------------------------------

def _rand_inputs(rng, B, H, T, D):
    x = rng.normal(0, 1.5, (B, H, T, D)).astype(F16)
    zp = rng.normal(0, 0.5, (H, D)).astype(F16)
    sc = rng.uniform(0.2, 1.0, (H, D)).astype(F16)
    al = rng.uniform(0.5, 0.999, (H, D)).astype(F16)
    be = rng.uniform(0.0, 0.05, (H, D)).astype(F16)
    tg = np.full((H, D), 3.5, F16)
    return x, (zp, sc, al, be, tg)


def test_alpha0_beta0_is_fixed_step_rtn(oracle):
    """alpha = 0 and beta = 0 freeze the state: textbook round-to-nearest with a fixed step."""
    rng = np.random.default_rng(21)
    B, H, T, D = 2, 2, 50, 128
    x, (zp, sc, al, be, tg) = _rand_inputs(rng, B, H, T, D)
    al[:] = 0
    be[:] = 0
    cache = oracle.alloc_cache(B, H, T, D)
    state = oracle.encode_kv_f16(cache, x, zp, sc, al, be, tg)
    u = (x.astype(np.float32) - zp.astype(np.float32)[None, :, None, :]) / sc.astype(np.float32)[None, :, None, :]
    want = np.clip(np.rint(u), -8, 7).astype(np.int8)
    assert np.array_equal(oracle.unpack_codes(cache, T), want)
    assert np.array_equal(state[..., 0], np.broadcast_to(zp.view(np.uint16), (B, H, D)))
    assert np.array_equal(state[..., 1], np.broadcast_to(sc.view(np.uint16), (B, H, D)))
    khat, _ = oracle.replay_f16(cache, zp, sc, al, be, tg, T)
    deq = (want.astype(F16) * sc[None, :, None, :]).astype(F16) + zp[None, :, None, :]
    assert np.array_equal(khat.view(np.uint16), deq.astype(F16).view(np.uint16))


def test_beta0_keeps_scale(oracle):
    rng = np.random.default_rng(22)
    B, H, T, D = 1, 2, 40, 128
    x, (zp, sc, al, be, tg) = _rand_inputs(rng, B, H, T, D)
    be[:] = 0
    cache = oracle.alloc_cache(B, H, T, D)
    state = oracle.encode_kv_f16(cache, x, zp, sc, al, be, tg)
    assert np.array_equal(state[..., 1], np.broadcast_to(sc.view(np.uint16), (B, H, D)))


def test_unclipped_error_bound(oracle):
    """Where the code is not clipped, |x - x_hat| <= sc/2 up to fp16 rounding of x_hat."""
    rng = np.random.default_rng(23)
    B, H, T, D = 1, 2, 64, 128
    x, p = _rand_inputs(rng, B, H, T, D)
    cache = oracle.alloc_cache(B, H, T, D)
    oracle.encode_kv_f16(cache, x, *p)
    codes = oracle.unpack_codes(cache, T)
    khat, _ = oracle.replay_f16(cache, *p, T)
    # per-token scale: replay prefixes
    inner = (codes > -8) & (codes < 7)
    err = np.abs(x.astype(np.float64) - khat.astype(np.float64))
    # a loose, state-free bound: the scale never exceeds sc0 * prod(1 + beta*4.5) over T steps
    assert np.all(err[inner] < 4.0)
    # tight check on token 0, whose state is the initial one
    sc0 = p[1].astype(np.float64)[None, :, :]
    e0 = err[:, :, 0, :]
    ok = inner[:, :, 0, :]
    ulp = np.abs(khat[:, :, 0, :].astype(np.float64)) * 2.0 ** -10 + 2.0 ** -24
    assert np.all(e0[ok] <= (sc0 / 2 + ulp)[np.broadcast_to(ok, e0.shape)] + 1e-3)


# ------------------------------------------------------------------------------------------
# invariants between encode, replay and the two GEMVs
# ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("T", [0, 1, 7, 8, 9, 31, 32, 33])
def test_append_equals_longer_encode(oracle, T):
    """encode(T) followed by forward_qk's append of token T == encode(T+1), byte for byte; the same
    for forward_ov.  The replayed state after T tokens equals the encoder's final state."""
    rng = np.random.default_rng(100 + T)
    B, H, D = 2, 3, 128
    x, p = _rand_inputs(rng, B, H, T + 1, D)
    full = oracle.alloc_cache(B, H, T + 8, D)
    oracle.encode_kv_f16(full, x, *p)

    part = oracle.alloc_cache(B, H, T + 8, D)
    st_enc = oracle.encode_kv_f16(part, x[:, :, :T], *p)
    _, st_rep = oracle.replay_f16(part, *p, T, want_khat=False)
    assert np.array_equal(st_enc, st_rep)

    q = rng.normal(0, 1, (B, H, 1, D)).astype(F16)
    k_cache = part.copy()
    logits, emu = oracle.forward_qk_f16(q, k_cache, x[:, :, T:T + 1], *p, T, refemu=True)
    assert np.array_equal(k_cache, full)

    v_cache = part.copy()
    attn = rng.random((B, H, T + 1)).astype(F16)
    out, oemu = oracle.forward_ov_f16(attn, v_cache, x[:, :, T:T + 1], *p, refemu=True)
    assert np.array_equal(v_cache, full)

    # GEMVs against a plain numpy contraction of the replayed (bit-exact) dequantised values;
    # the appended token uses the fused dequant of its own code with the state after T-1
    khat, st = oracle.replay_f16(full, *p, T)
    L = oracle.lib()
    codes = oracle.unpack_codes(full, T + 1)
    new = np.zeros((B, H, D), np.float64)
    for b in range(B):
        for hh in range(H):
            for c in range(D):
                new[b, hh, c] = L.adkv_o_h2f(L.adkv_o_dequant1_f16(
                    int(codes[b, hh, T, c]), int(st_enc[b, hh, c, 0]), int(st_enc[b, hh, c, 1])))
    kall = np.concatenate([khat.astype(np.float64), new[:, :, None, :]], axis=2)
    want_l = np.einsum("bhc,bhtc->bht", q[:, :, 0].astype(np.float64), kall)
    assert np.allclose(logits, want_l, rtol=1e-12, atol=1e-12)
    want_o = np.einsum("bht,bhtc->bhc", attn.astype(np.float64), kall)
    assert np.allclose(out, want_o, rtol=1e-12, atol=1e-12)
    # the emulation of the reference's own fp16 accumulation stays near the exact sums
    assert np.max(np.abs(emu.astype(np.float64) - logits)) < 0.25
    assert np.max(np.abs(oemu.astype(np.float64) - out)) < 0.25


def test_self_logit_matches_next_step_up_to_one_rounding(oracle):
    """forward_qk(T)[T] uses the fused dequant; the same token seen as a cached token by
    forward_qk(T+1) uses two roundings (gemv.cu:796 vs :644-645): per-channel difference is at most
    one binary16 ulp of the dequantised value."""
    rng = np.random.default_rng(77)
    B, H, D, T = 1, 2, 128, 19
    x, p = _rand_inputs(rng, B, H, T + 2, D)
    cache = oracle.alloc_cache(B, H, T + 8, D)
    oracle.encode_kv_f16(cache, x[:, :, :T], *p)
    q = rng.normal(0, 1, (B, H, 1, D)).astype(F16)
    l0, _ = oracle.forward_qk_f16(q, cache, x[:, :, T:T + 1], *p, T)
    l1, _ = oracle.forward_qk_f16(q, cache, x[:, :, T + 1:T + 2], *p, T + 1)
    assert np.array_equal(l0[:, :, :T], l1[:, :, :T])
    bound = np.sum(np.abs(q.astype(np.float64))) * 2.0 ** -8
    assert np.max(np.abs(l0[:, :, T] - l1[:, :, T])) <= bound
