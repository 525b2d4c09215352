"""Pins the oracle's 2-bit mode: the same fp16 recurrence as the 4-bit deployment path
(src/adkv/kernel/gemv.cu:150-164) with the code range [-2, 1] that the reference's train model
uses for bits=2 (src/adkv/train/train_model.py:96-97) and 16 tokens per 32-bit word.  The reference
has no fp16 2-bit kernel, so these checks are closed forms, a byte-level layout brute force and an
exact-rational re-evaluation of whole sequences."""
import numpy as np
import pytest

import exact16 as X

F16 = np.float16


def h(x):
    return X.from_float(float(x))


@pytest.fixture()
def o2(oracle):
    with oracle.code_bits(2):
        yield oracle
    assert oracle.get_bits() == 4


def test_width_switch(oracle):
    assert oracle.get_bits() == 4 and oracle.n_super(17) == 3
    with oracle.code_bits(2):
        assert oracle.get_bits() == 2 and oracle.n_super(17) == 2 and oracle.n_super(16) == 1
    assert oracle.get_bits() == 4
    with pytest.raises(ValueError):
        with oracle.code_bits(3):
            pass
    assert oracle.get_bits() == 4


def test_quantize_clamps_to_two_bits(o2):
    L = o2.lib()
    q = lambda x, zp, sc: L.adkv_o_quantize_f16(h(x), h(zp), h(sc))
    assert [q(v, 0.0, 1.0) for v in (-5.0, -2.0, -1.0, 0.0, 1.0, 2.0, 9.0)] == [-2, -2, -1, 0, 1, 1, 1]
    assert q(0.5, 0.0, 1.0) == 0 and q(1.5, 0.0, 1.0) == 1 and q(-1.5, 0.0, 1.0) == -2   # ties to even, then clamp
    assert q(-2.5, 0.0, 1.0) == -2 and q(0.75, 0.25, 0.5) == 1
    assert q(1.0, 0.0, 0.0) == 1 and q(-1.0, 0.0, 0.0) == -2                              # +-inf saturate


@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("T", [0, 1, 3, 4, 15, 16, 17, 33])
def test_layout_bruteforce_2bit(o2, D, T):
    """alpha = beta = 0, zp = 0, sc = 1: codes are the (integer) inputs; every byte is checked
    against [b, h, sg, cg, channel-in-group, byte-row] with four tokens per byte."""
    B, H = 2, 2
    rng = np.random.default_rng(T * 100 + D)
    codes = rng.integers(-2, 2, (B, H, T, D)).astype(np.int8)
    zero, one = np.zeros((H, D), F16), np.ones((H, D), F16)
    ns = o2.n_super(T)
    assert ns == (T + 15) // 16
    cache = np.full((B, H, ns + 1, D // 4, 4, 4), 0xEE, np.uint8)
    o2.encode_kv_f16(cache, codes.astype(F16), zero, one, zero, zero, one)
    want = np.full_like(cache, 0xEE)
    want[:, :, :ns] = 0
    for t in range(T):
        sg, br, i = t // 16, (t % 16) // 4, t % 4
        f = (codes[:, :, t, :].astype(np.int16) + 2).astype(np.uint8).reshape(B, H, D // 4, 4)
        want[:, :, sg, :, :, br] |= (f << (2 * i)).astype(np.uint8)
    assert np.array_equal(cache, want)
    L = o2.lib()
    flat = cache[1, 1].reshape(-1)
    for t in range(T):
        for c in (0, 3, 6, D - 1):
            off = ((t // 16 * (D // 4) + c // 4) * 4 + c % 4) * 4 + (t % 16) // 4
            assert L.adkv_o_byte_offset(t, c, D) == off
            assert ((int(flat[off]) >> (2 * (t % 4))) & 3) - 2 == codes[1, 1, t, c]
            assert L.adkv_o_get_code(flat.ctypes.data, t, c, D) == codes[1, 1, t, c]
    assert np.array_equal(o2.unpack_codes(cache, T), codes)
    # the word view the kernels use: token 16sg+i of channel c at bits 2i..2i+1 of word (sg, c)
    words = cache.view(np.uint32).reshape(B, H, ns + 1, D)
    for t in range(T):
        assert np.array_equal(((words[:, :, t // 16, :] >> (2 * (t % 16))) & 3).astype(np.int8) - 2,
                              codes[:, :, t, :])


def _exact_sequence(x, zp, sc, alpha, beta, tgt, lo, hi):
    """One channel of the recurrence in exact-rational binary16 (gemv.cu:150-164): returns codes,
    two-rounding dequantised values and the final state."""
    omt = X.hadd(0x3C00, X.hmul(beta, tgt) ^ 0x8000)
    codes, deq = [], []
    for xv in x:
        d = np.float32(float(X.h_to_frac(xv))) - np.float32(float(X.h_to_frac(zp)))
        with np.errstate(divide="ignore", invalid="ignore"):
            u = np.float32(d) / np.float32(float(X.h_to_frac(sc)))
        q = 0 if np.isnan(u) else int(min(max(np.rint(u), lo), hi))
        codes.append(q)
        qf = h(q)
        p = X.hmul(qf, sc)
        deq.append(X.hadd(p, zp))
        zp = X.hfma(alpha, p, zp)
        sc = X.hmul(sc, X.hfma(beta, qf & 0x7FFF, omt))
    return codes, deq, zp, sc


@pytest.mark.parametrize("bits", [2, 4])
def test_sequences_vs_exact_rational(oracle, bits):
    rng = np.random.default_rng(bits)
    B, H, T, D = 1, 1, 40, 128
    x = (rng.standard_normal((B, H, T, D)) * 1.5).astype(F16)
    zp = (rng.standard_normal((H, D)) * 0.2).astype(F16)
    sc = rng.uniform(0.5, 1.5, (H, D)).astype(F16)
    al = rng.uniform(0.5, 1.0, (H, D)).astype(F16)
    be = rng.uniform(0.0, 0.08, (H, D)).astype(F16)
    tg = np.full((H, D), (2 ** (bits - 1) - 1) / 2, F16)
    with oracle.code_bits(bits):
        cache = oracle.alloc_cache(B, H, T, D)
        state = oracle.encode_kv_f16(cache, x, zp, sc, al, be, tg)
        codes = oracle.unpack_codes(cache, T)
        khat, st2 = oracle.replay_f16(cache, zp, sc, al, be, tg, T)
    assert np.array_equal(state, st2)
    u = lambda a: a.view(np.uint16)
    for c in range(0, D, 7):
        cs, deq, z, s = _exact_sequence([int(v) for v in u(x)[0, 0, :, c]], int(u(zp)[0, c]), int(u(sc)[0, c]),
                                        int(u(al)[0, c]), int(u(be)[0, c]), int(u(tg)[0, c]),
                                        -2 ** (bits - 1), 2 ** (bits - 1) - 1)
        assert cs == codes[0, 0, :, c].tolist()
        assert deq == u(khat)[0, 0, :, c].tolist()
        assert (z, s) == (int(state[0, 0, c, 0]), int(state[0, 0, c, 1]))


def test_two_bit_products_are_exact(o2):
    """q in {-2,-1,0,1} only scales by a power of two or flips the sign, so r16(q*sc) is exact and
    the one- and two-rounding dequant forms coincide (unlike 4-bit codes)."""
    L = o2.lib()
    rng = np.random.default_rng(1)
    for _ in range(3000):
        sc, zp = h(rng.uniform(0.01, 30)), h(rng.normal(0, 3))
        for q in (-2, -1, 0, 1):
            assert L.adkv_o_dequant1_f16(q, zp, sc) == L.adkv_o_dequant2_f16(q, zp, sc)


@pytest.mark.parametrize("T", [0, 1, 15, 16, 17, 40])
def test_append_equals_longer_encode_2bit(o2, T):
    rng = np.random.default_rng(T)
    B, H, D = 2, 2, 128
    x = (rng.standard_normal((B, H, T + 1, D)) * 1.2).astype(F16)
    zp = np.zeros((H, D), F16)
    sc = rng.uniform(0.6, 1.2, (H, D)).astype(F16)
    al = rng.uniform(0.8, 1.0, (H, D)).astype(F16)
    be = np.full((H, D), 0.02, F16)
    tg = np.full((H, D), 0.5, F16)
    q = rng.standard_normal((B, H, D)).astype(F16)
    a = o2.alloc_cache(B, H, T + 16, D)
    b = o2.alloc_cache(B, H, T + 16, D)
    if T:
        o2.encode_kv_f16(a, x[:, :, :T], zp, sc, al, be, tg)
    logits, _ = o2.forward_qk_f16(q, a, x[:, :, T:], zp, sc, al, be, tg, T)
    o2.encode_kv_f16(b, x, zp, sc, al, be, tg)
    assert np.array_equal(a, b)
    khat, _ = o2.replay_f16(b, zp, sc, al, be, tg, T + 1)
    want = np.einsum("bhd,bhtd->bht", q.astype(np.float64), khat.astype(np.float64))
    assert np.allclose(logits, want, rtol=0, atol=1e-9)
