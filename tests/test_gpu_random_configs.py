"""Seeded sweep over random shapes of the whole path (stream append in two cuts, forward_qk,
forward_ov) against the CPU oracle: code widths, head dims, grouped queries, odd head counts,
ragged lengths around every supergroup / interval boundary, with and without checkpoints.  The
hand-picked cases of test_gpu_parity.py name the corners; this file guards the combinations."""
import random

import numpy as np
import pytest
import torch

from adkv_amd import synth
from adkv_amd.kernel import gemv

pytestmark = pytest.mark.gpu

LENGTHS = [0, 1, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 100, 255, 256, 257, 511, 700, 1023, 1100]


def _np16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.float16)


def _ulp16(v):
    a = np.maximum(np.abs(v), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - 10)


def _config(seed):
    rng = random.Random(seed)
    bits = rng.choice([4, 4, 2])
    D = 128 if bits == 2 else rng.choice([128, 128, 256, 512])
    G = rng.choice([1, 1, 2, 4, 8]) if D == 128 else 1
    B, Hkv = rng.randint(1, 3), rng.randint(1, 5)
    T = rng.choice(LENGTHS)
    tps = 32 // bits
    S = rng.choice([0, 0, tps, 2 * tps, 64, 256])
    return bits, D, G, B, Hkv, T, S, rng.randint(0, T)


@pytest.mark.parametrize("seed", range(48))
def test_random_config(gpu, oracle, seed):
    bits, D, G, B, Hkv, T, S, cut = _config(seed)
    tps, Hq = 32 // bits, Hkv * G
    g = torch.Generator().manual_seed(1000 + seed)
    p = synth.make_params(Hkv, D, bits=bits, seed=seed)
    p.zp_init = (0.3 * torch.randn(Hkv, D, generator=g)).half()
    p.beta = (0.05 * torch.rand(Hkv, D, generator=g)).half()
    x = synth.make_k(B, Hkv, T + 1, D, seed=seed, dtype=torch.float16)
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    attn = torch.softmax(2.0 * torch.randn(B, Hq, T + 1, generator=g), dim=-1).half()
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    ncap = (T + tps) // S + 1 if S else 0
    what = f"bits={bits} D={D} G={G} B={B} Hkv={Hkv} T={T} S={S} cut={cut}"

    with oracle.code_bits(bits):
        want = oracle.alloc_cache(B, Hkv, T + tps, D)
        if T:
            oracle.encode_kv_f16(want, _np16(x)[:, :, :T], *pn)
        cache = synth.alloc_cache(B, Hkv, T + tps, D, gpu, bits=bits)
        st = torch.zeros(B, Hkv, D, 2, dtype=torch.float16, device=gpu)
        ck = torch.zeros(B, Hkv, ncap, D, 2, dtype=torch.float16, device=gpu) if S else None
        for a, b in ((0, cut), (cut, T)):
            gemv.append_kv(cache, x[:, :, a:b].to(gpu), *pg, a, st, ckpt=ck, ckpt_interval=S, bits=bits)
        torch.cuda.synchronize()
        assert np.array_equal(cache.cpu().numpy(), want), what
        xn = _np16(x)[:, :, T:T + 1]
        wl, wo = np.zeros((B, Hq, T + 1)), np.zeros((B, Hq, D))
        qn, an = _np16(q).reshape(B, Hkv, G, D), _np16(attn).reshape(B, Hkv, G, T + 1)
        for j in range(G):
            c = want.copy()
            l, _ = oracle.forward_qk_f16(qn[:, :, j], c, xn, *pn, T)
            wl.reshape(B, Hkv, G, T + 1)[:, :, j] = l
            c2 = want.copy()
            o, _ = oracle.forward_ov_f16(an[:, :, j], c2, xn, *pn)
            wo.reshape(B, Hkv, G, D)[:, :, j] = o
    kc, vc = cache.clone(), cache.clone()
    ckv = ck.clone() if ck is not None else None
    logits = gemv.forward_qk(q.to(gpu), kc, x[:, :, T:].to(gpu), *pg, T, 0.0, 1.0,
                             ckpt=ck, ckpt_interval=S, bits=bits)
    out = gemv.forward_ov(attn.to(gpu), vc, x[:, :, T:].to(gpu), *pg, 0.0, 1.0,
                          ckpt=ckv, ckpt_interval=S, bits=bits)
    torch.cuda.synchronize()
    assert np.array_equal(kc.cpu().numpy(), c) and np.array_equal(vc.cpu().numpy(), c2), what
    lg, og = _np16(logits).astype(np.float64), _np16(out).astype(np.float64)
    assert np.all(np.abs(lg - wl) <= _ulp16(wl) + 1e-3), what
    assert np.all(np.abs(og - wo) <= _ulp16(wo) + 1e-3), what
    if S:
        assert torch.equal(ck.view(torch.int16), ckv.view(torch.int16)), what


def _softmax_config(seed):
    rng = random.Random(1000 + seed)
    # row lengths spread over every kernel of the softmax: a wave per row, a workgroup per row in
    # its six shapes, rows held in registers as fp16, the chunked pair
    n = int(round(2.0 ** rng.uniform(0.0, 17.2)))
    near = rng.choice([None, None, 2048, 5120, 6144, 8192, 12288, 16384, 24576, 73728, 139264])
    if near is not None:
        n = max(1, near + rng.randint(-2, 2))
    B = rng.randint(1, 3)
    H = rng.randint(1, max(1, min(48, 6_000_000 // (B * n))))
    if n > 24576 and rng.random() < 0.5:
        H = max(H, (128 + B - 1) // B) if B * n * 130 <= 40_000_000 else H   # enough rows for registers
    mask_mode = rng.choice([None, None, "b1", "bh"])
    scaling = rng.choice([0.0884, 0.0884, 1.0, 0.125, -0.05])
    return B, H, n, mask_mode, scaling


@pytest.mark.parametrize("seed", range(40))
def test_softmax_random_shapes(gpu, seed):
    B, H, n, mask_mode, scaling = _softmax_config(seed)
    g = torch.Generator().manual_seed(seed)
    l = (torch.randn(B, H, n, generator=g) * 6).half()
    mask = None
    if mask_mode == "b1":
        mask = torch.zeros(B, 1, 1, n)
        mask[0, 0, 0, : n // 3] = float("-inf")
    elif mask_mode == "bh":
        mask = torch.randn(B, H, n, generator=g)
    w = gemv.softmax_scale_mask(l.to(gpu), scaling, None if mask is None else mask.to(gpu))
    ref = l.double() * scaling
    if mask is not None:
        ref = ref + (mask[:, :, 0, :] if mask.dim() == 4 else mask).double()
    ref = torch.softmax(ref, -1)
    assert w.shape == (B, H, n)
    err = torch.max(torch.abs(w.cpu().double() - ref)).item()
    assert err < 6e-4, (B, H, n, mask_mode, scaling, err)
