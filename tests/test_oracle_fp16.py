"""Pins the oracle's binary16 soft-float against exact rational arithmetic and numpy."""
import random

import numpy as np

import exact16 as X


def _finite(rng):
    while True:
        h = rng.randrange(0, 65536)
        if (h & 0x7C00) != 0x7C00:
            return h


def _special_pool():
    pool = [0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x0401, 0x3C00, 0xBC00, 0x3BFF, 0x3C01,
            0x7BFF, 0xFBFF, 0x7800, 0x4800, 0xC800, 0x6400, 0x6408, 0x5400, 0x2E66, 0x251F]
    return pool


def test_roundtrip_all_bit_patterns(oracle):
    L = oracle.lib()
    for h in range(65536):
        f = X.h_to_frac(h)
        if f is None:
            continue
        assert float(f) == L.adkv_o_h2f(h)
        if f != 0:  # a Fraction cannot carry the sign of zero
            assert L.adkv_o_f2h(float(f)) == h
    assert L.adkv_o_f2h(-0.0) == 0x8000 and L.adkv_o_f2h(0.0) == 0


def test_mul_add_fma_vs_exact(oracle):
    L = oracle.lib()
    rng = random.Random(1234)
    pool = _special_pool()
    for i in range(30000):
        if i % 3 == 0:
            a, b, c = (rng.choice(pool) for _ in range(3))
        else:
            a, b, c = _finite(rng), _finite(rng), _finite(rng)
        assert L.adkv_o_hmul(a, b) == X.hmul(a, b), (hex(a), hex(b))
        assert L.adkv_o_hadd(a, c) == X.hadd(a, c), (hex(a), hex(c))
        assert L.adkv_o_hsub(a, c) == X.hadd(a, c ^ 0x8000), (hex(a), hex(c))
        assert L.adkv_o_hfma(a, b, c) == X.hfma(a, b, c), (hex(a), hex(b), hex(c))


def test_fma_is_single_rounding(oracle):
    """a*b lands exactly on a binary16 tie; a tiny addend must break the tie in its direction.
    A mul-then-add (two roundings) gets the downward case wrong."""
    L = oracle.lib()
    a, b = 0x3C01, 0x3E00                 # (1 + 2^-10) * 1.5 = 1.5 + 2^-10 + 2^-11: a tie
    tiny_p, tiny_n = 0x0001, 0x8001       # +/- 2^-24
    assert L.adkv_o_hmul(a, b) == 0x3E02                  # tie -> even
    assert L.adkv_o_hfma(a, b, 0x0000) == 0x3E02
    assert L.adkv_o_hfma(a, b, tiny_p) == 0x3E02          # just above the tie -> up
    assert L.adkv_o_hfma(a, b, tiny_n) == 0x3E01          # just below the tie -> down
    assert L.adkv_o_hadd(L.adkv_o_hmul(a, b), tiny_n) == 0x3E02   # what two roundings give
    for c in (0x0000, tiny_p, tiny_n):
        assert L.adkv_o_hfma(a, b, c) == X.hfma(a, b, c)


def test_inf_nan_rules(oracle):
    L = oracle.lib()
    INF, NINF, NAN = 0x7C00, 0xFC00, 0x7E00
    assert X.is_nan(L.adkv_o_hmul(INF, 0))
    assert L.adkv_o_hmul(INF, 0xBC00) == NINF
    assert X.is_nan(L.adkv_o_hadd(INF, NINF))
    assert L.adkv_o_hadd(INF, 0x3C00) == INF
    assert X.is_nan(L.adkv_o_hfma(INF, 0x3C00, NINF))
    assert L.adkv_o_hfma(0x3C00, 0x3C00, NINF) == NINF
    assert X.is_nan(L.adkv_o_hfma(NAN, 0, 0))
    assert L.adkv_o_hmul(0x7BFF, 0x4000) == INF       # overflow
    assert L.adkv_o_hadd(0x8000, 0x8000) == 0x8000    # -0 + -0
    assert L.adkv_o_hadd(0x8000, 0x0000) == 0x0000
    assert L.adkv_o_hmul(0x8000, 0x3C00) == 0x8000
    assert L.adkv_o_hfma(0x8000, 0x3C00, 0x0000) == 0x0000


def test_vs_numpy_float16(oracle):
    """numpy's float16 (+,*) is a second independent implementation."""
    L = oracle.lib()
    rng = np.random.default_rng(7)
    a = rng.integers(0, 65536, 20000).astype(np.uint16)
    b = rng.integers(0, 65536, 20000).astype(np.uint16)
    af, bf = a.view(np.float16), b.view(np.float16)
    with np.errstate(all="ignore"):
        mul = (af.astype(np.float32) * bf.astype(np.float32)).astype(np.float16).view(np.uint16)
        add = (af.astype(np.float64) + bf.astype(np.float64)).astype(np.float16).view(np.uint16)
    for i in range(len(a)):
        m, s = L.adkv_o_hmul(int(a[i]), int(b[i])), L.adkv_o_hadd(int(a[i]), int(b[i]))
        assert m == int(mul[i]) or (X.is_nan(m) and X.is_nan(int(mul[i])))
        assert s == int(add[i]) or (X.is_nan(s) and X.is_nan(int(add[i])))
