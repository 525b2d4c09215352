"""Pins the oracle's fp32 (train/eval) recurrence: src/adkv/train/train_model.py:8-22, 61-81.

Independent checks: a vectorised numpy-float32 evaluation in the reference's operation order,
closed forms (alpha = beta = 0 is fixed-step RTN), tie/eps/clamp corner cases with hand-derived
answers.  Whether the reference's torch.compile'd chunk function is bit-identical to eager order
is not decidable without running it: parity unpinned on that point.
"""
import math

import numpy as np
import pytest

F32 = np.float32


def _numpy_ref(x, zp0, sc0, al, be, tg, bits, sc_min, sc_max):
    """train_model.py:65-81, one numpy float32 op per reference op, vectorised over [B, C]."""
    QU, QL = F32(2 ** (bits - 1) - 1), F32(-2 ** (bits - 1))
    B, T, C = x.shape
    zp = np.broadcast_to(zp0, (B, C)).astype(F32).copy()
    sc = np.broadcast_to(sc0, (B, C)).astype(F32).copy()
    xh = np.zeros_like(x)
    qs = np.zeros(x.shape, np.int8)
    for t in range(T):
        s = np.maximum(sc, F32(1e-8))
        r = x[:, t] - zp
        q = np.clip(np.rint(r / s), QL, QU).astype(F32)
        rh = q * s
        xh[:, t] = rh + zp
        qs[:, t] = q.astype(np.int8)
        zp = zp + al * rh
        err = np.abs(q) - tg
        sc = np.clip(sc + (sc * be) * err, F32(sc_min), F32(sc_max))
    return xh, qs, zp, sc


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_vs_numpy_float32(oracle, bits):
    rng = np.random.default_rng(bits)
    B, T, C = 2, 96, 64
    x = rng.normal(0, 1.5, (B, T, C)).astype(F32)
    x[:, :, 0] += (8 * np.sin(0.01 * np.arange(T))).astype(F32)
    zp0 = rng.normal(0, 0.3, C).astype(F32)
    sc0 = rng.uniform(0.3, 1.2, C).astype(F32)
    al = rng.uniform(0.5, 0.999, C).astype(F32)
    be = rng.uniform(0, 0.1, C).astype(F32)
    tg = np.full(C, (2 ** (bits - 1) - 1) / 2, F32)
    smin, smax = F32(math.exp(-4.0)), F32(math.exp(4.0))
    r = oracle.quant_f32(x, zp0, sc0, al, be, tg, bits=bits, want_seq=True)
    xh, qs, zp, sc = _numpy_ref(x, zp0, sc0, al, be, tg, bits, smin, smax)
    assert np.array_equal(r["codes"], qs)
    assert np.array_equal(r["xhat"].view(np.uint32), xh.view(np.uint32))
    assert np.array_equal(r["zp"].view(np.uint32), zp.view(np.uint32))
    assert np.array_equal(r["sc"].view(np.uint32), sc.view(np.uint32))
    # zp_seq/sc_seq hold the state BEFORE each token (train_model.py:66-68)
    assert np.array_equal(r["zp_seq"][:, 0], np.broadcast_to(zp0, (B, C)))
    assert np.array_equal(r["sc_seq"][:, 0], np.broadcast_to(sc0, (B, C)))


def test_alpha0_beta0_fixed_step(oracle):
    rng = np.random.default_rng(9)
    B, T, C = 1, 33, 32
    x = rng.normal(0, 2, (B, T, C)).astype(F32)
    zp0 = rng.normal(0, 0.3, C).astype(F32)
    sc0 = rng.uniform(0.3, 1.2, C).astype(F32)
    z = np.zeros(C, F32)
    r = oracle.quant_f32(x, zp0, sc0, z, z, np.full(C, 3.5, F32))
    want = np.clip(np.rint((x - zp0) / sc0), -8, 7)
    assert np.array_equal(r["codes"], want.astype(np.int8))
    assert np.array_equal(r["xhat"], want.astype(F32) * sc0 + zp0)
    assert np.array_equal(r["zp"][0], zp0) and np.array_equal(r["sc"][0], sc0)


def test_corner_cases(oracle):
    one = np.ones(1, F32)
    z = np.zeros(1, F32)
    run = lambda xs, **k: oracle.quant_f32(np.array(xs, F32).reshape(1, -1, 1), k.get("zp", z),
                                           k.get("sc", one), k.get("al", z), k.get("be", z),
                                           k.get("tg", 3.5 * one), bits=k.get("bits", 4))
    # ties to even, clamp to [-8, 7]
    assert run([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 7.5, 9.0, -8.5, -20.0])["codes"].reshape(-1).tolist() == \
        [0, 2, 2, 0, -2, -2, 7, 7, -8, -8]
    # 2-bit range is [-2, 1]
    assert run([5.0, -5.0, 0.6], bits=2)["codes"].reshape(-1).tolist() == [1, -2, 1]
    # eps guard: a zero scale quantises with 1e-8 but the UPDATE uses the unguarded scale
    r = run([1.0], sc=z, be=0.1 * one)
    assert r["codes"].reshape(-1).tolist() == [7]
    assert r["xhat"][0, 0, 0] == F32(7) * F32(1e-8)
    assert r["sc"][0, 0] == F32(math.exp(-4.0))          # 0 + (0*beta)*err = 0 -> clamped up
    # scale clamp at e^4 and e^-4 (train_model.py:79-81)
    r = run([1000.0] * 400, be=0.1 * one, tg=z)
    assert r["sc"][0, 0] == F32(math.exp(4.0))
    r = run([0.0] * 400, be=0.1 * one, tg=7 * one)
    assert r["sc"][0, 0] == F32(math.exp(-4.0))
    # zero-point tracks: alpha = 1 makes zp the previous reconstruction
    r = oracle.quant_f32(np.array([1.0, 1.0, 1.0], F32).reshape(1, 3, 1), z, one, one, z, 3.5 * one,
                         want_seq=True)
    assert r["zp_seq"].reshape(-1).tolist() == [0.0, 1.0, 1.0]
    assert r["codes"].reshape(-1).tolist() == [1, 0, 0]


def test_attention_f64(oracle):
    rng = np.random.default_rng(4)
    B, H, T, D = 1, 2, 17, 8
    q = rng.normal(size=(B, H, D)).astype(F32)
    K = rng.normal(size=(B, H, T, D)).astype(F32)
    V = rng.normal(size=(B, H, T, D)).astype(F32)
    out, w = oracle.attention_f64(q, K, V, 0.35)
    l = np.einsum("bhd,bhtd->bht", q.astype(np.float64), K.astype(np.float64)) * 0.35
    e = np.exp(l - l.max(-1, keepdims=True))
    ww = e / e.sum(-1, keepdims=True)
    assert np.allclose(w, ww, atol=1e-14)
    assert np.allclose(out, np.einsum("bht,bhtd->bhd", ww, V.astype(np.float64)), atol=1e-13)
