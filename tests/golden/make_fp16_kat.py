"""Writes tests/golden/kat_fp16.json: known-answer vectors for the fp16 (deployment) recurrence.

Everything here is computed with exact rational arithmetic (tests/exact16.py) and plain Python
integers from the step definitions of src/adkv/kernel/gemv.cu:150-164, 220-221 and the cache layout
of src/adkv/hf/llama_adkv.py:47-55 -- no oracle, no GPU, no reference code is run.  The quotient of
the quantise step is evaluated as an exact fraction and rounded half to even, which equals the
reference's fp32 subtract + IEEE divide + rint whenever the fp32 difference is exact (it is, for
the magnitudes used here) and the quotient is not within fp32 rounding distance of a tie (the
generator asserts a safety margin and constructs the ties explicitly).

    python tests/golden/make_fp16_kat.py
"""
import json
import os
import random
import sys
from fractions import Fraction

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import exact16 as X  # noqa: E402

H = X.from_float


def quantize(x, zp, sc, lo, hi):
    """clamp(round_half_even((x - zp) / sc)) on exact values; asserts the fp32 evaluation agrees."""
    d = X.h_to_frac(x) - X.h_to_frac(zp)
    assert d == 0 or abs(d) >= Fraction(1, 1 << 24)          # exact in fp32: both are multiples of 2^-24
    u = d / X.h_to_frac(sc)
    k = u.numerator // u.denominator                             # floor
    frac = u - k
    if frac != Fraction(1, 2):
        assert abs(frac - Fraction(1, 2)) > Fraction(1, 1 << 18) * max(1, abs(u))   # far from a tie in fp32
    n = k + 1 if frac > Fraction(1, 2) else k
    if frac == Fraction(1, 2):
        n = k if k % 2 == 0 else k + 1
    return max(lo, min(hi, n))


def update(q, zp, sc, alpha, beta, omt):
    qf = H(q)
    p = X.hmul(qf, sc)
    return X.hfma(alpha, p, zp), X.hmul(sc, X.hfma(beta, qf & 0x7FFF, omt)), X.hadd(p, zp)


def sequence(xs, zp, sc, alpha, beta, tgt, bits):
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    omt = X.hadd(0x3C00, X.hmul(beta, tgt) ^ 0x8000)
    codes, deq = [], []
    for x in xs:
        q = quantize(x, zp, sc, lo, hi)
        codes.append(q)
        zp, sc, kh = update(q, zp, sc, alpha, beta, omt)
        deq.append(kh)
    return codes, deq, zp, sc


def pack(codes_tc, D, bits):
    """codes_tc[t][c] -> bytes of one (b, h) block [n_super, D/4, 4, 4]."""
    tpw = 32 // bits
    T = len(codes_tc)
    ns = -(-T // tpw)
    words = [[0] * D for _ in range(ns)]
    for t in range(T):
        for c in range(D):
            words[t // tpw][c] |= ((codes_tc[t][c] + (1 << (bits - 1))) & ((1 << bits) - 1)) << (bits * (t % tpw))
    out = bytearray()
    for sg in range(ns):
        for c in range(D):                                       # (cg, channel in group) = channel order
            out += words[sg][c].to_bytes(4, "little")            # byte row br = bits 8br..8br+7
    return bytes(out)


def main():
    rng = random.Random(2024)
    kat = {"update": [], "quantize": [], "sequences": []}
    for _ in range(400):
        q = rng.randrange(-8, 8)
        zp, sc = H(rng.gauss(0, 3)), H(rng.uniform(0.01, 8))
        al, be, tg = H(rng.uniform(0, 1)), H(rng.uniform(0, 0.1)), H(rng.uniform(0, 7))
        omt = X.hadd(0x3C00, X.hmul(be, tg) ^ 0x8000)
        nzp, nsc, kh = update(q, zp, sc, al, be, omt)
        kat["update"].append([q, zp, sc, al, be, tg, omt, nzp, nsc, kh])
    for bits in (4, 2):
        lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
        for sc in (0.25, 0.5, 1.0, 1.5, 3.0):
            for k in range(-11, 11):
                for off in (0.0, 0.5):                            # integers and exact ties
                    x, z = (k + off) * sc, 0.0
                    kat["quantize"].append([bits, H(x), H(z), H(sc), quantize(H(x), H(z), H(sc), lo, hi)])
    for bits, T, D, seed in ((4, 19, 128, 1), (2, 37, 128, 2), (4, 9, 256, 3)):
        r = random.Random(seed)
        par = [[H(r.gauss(0, 0.2)) for _ in range(D)], [H(r.uniform(0.6, 1.4)) for _ in range(D)],
               [H(r.uniform(0.6, 1.0)) for _ in range(D)], [H(r.uniform(0.0, 0.06)) for _ in range(D)],
               [H(((1 << (bits - 1)) - 1) / 2)] * D]
        x = [[H(r.gauss(0, 1.5)) for _ in range(D)] for _ in range(T)]
        codes = [[0] * D for _ in range(T)]
        deq = [[0] * D for _ in range(T)]
        state = []
        for c in range(D):
            cs, dq, z, s = sequence([x[t][c] for t in range(T)], par[0][c], par[1][c], par[2][c], par[3][c],
                                    par[4][c], bits)
            for t in range(T):
                codes[t][c], deq[t][c] = cs[t], dq[t]
            state.append([z, s])
        kat["sequences"].append({"bits": bits, "T": T, "D": D, "params": par, "x": x, "codes": codes,
                                 "dequant": deq, "state": state, "packed_hex": pack(codes, D, bits).hex()})
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat_fp16.json")
    with open(dst, "w") as f:
        json.dump(kat, f, separators=(",", ":"))
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()
