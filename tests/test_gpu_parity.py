"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on identical seeded inputs.

Bar: codes written to the cache and the fp16 filter state are bit-exact; logits and attention
outputs are fp16 roundings of fp32-accumulated sums and must sit within one binary16 ulp of the
oracle's exact sums (plus 1e-3 absolute for cancellation), i.e. well inside the 2e-3 end-to-end
tolerance on attention outputs, which is asserted separately on the full decode step.
"""
import math

import numpy as np
import pytest
import torch

from adkv_amd import synth
from adkv_amd.kernel import gemv

pytestmark = pytest.mark.gpu

SMIN, SMAX = math.exp(-4.0), math.exp(4.0)

SHAPES = [  # (B, H, T, D)
    (1, 2, 1, 128), (2, 3, 7, 128), (2, 3, 8, 128), (1, 5, 9, 128), (1, 4, 65, 128),
    (3, 1, 130, 128), (2, 2, 1024, 128), (1, 2, 40, 256), (1, 3, 17, 256), (1, 3, 33, 512),
    (2, 1, 8, 512),
]


def _np16(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.float16)


def _inputs(B, H, T, D, seed=0, bits=4):
    p = synth.make_params(H, D, bits=bits, seed=3 + seed)
    # spread the parameters more than the benchmark does, to exercise the recurrence
    g = torch.Generator().manual_seed(100 + seed)
    p.zp_init = (0.3 * torch.randn(H, D, generator=g)).half()
    p.beta = (0.05 * torch.rand(H, D, generator=g)).half()
    x = synth.make_k(B, H, T, D, seed=seed, dtype=torch.float16)
    return x, p


def _ulp16(v):
    a = np.maximum(np.abs(v), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - 10)


@pytest.mark.parametrize("B,H,T,D", SHAPES)
def test_encode_bit_exact(gpu, oracle, B, H, T, D):
    x, p = _inputs(B, H, T, D, seed=T)
    pn = [_np16(t) for t in p.astuple()]
    want = np.full((B, H, synth.n_super(T) + 2, D // 4, 4, 4), 0xA5, np.uint8)
    st_want = oracle.encode_kv_f16(want, _np16(x), *pn)

    cache = torch.full(want.shape, 0xA5, dtype=torch.uint8, device=gpu)
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    r = gemv.encode_kv(cache, x.to(gpu), *[t.to(gpu) for t in p.astuple()], SMIN, SMAX, state_out=st)
    assert r is cache
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), want)
    assert np.array_equal(_np16(st).view(np.uint16), st_want)


@pytest.mark.parametrize("B,H,T,D", SHAPES + [(2, 2, 0, 128)])
def test_forward_qk_and_ov(gpu, oracle, B, H, T, D):
    x, p = _inputs(B, H, T + 1, D, seed=7 * T + D)
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    xn = _np16(x)
    base = oracle.alloc_cache(B, H, T + 9, D)
    oracle.encode_kv_f16(base, xn[:, :, :T], *pn)
    _, st_want = oracle.replay_f16(base, *pn, T, want_khat=False)

    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, H, 1, D, generator=g).half()
    attn = torch.softmax(torch.randn(B, H, T + 1, generator=g) * 2, -1).half()

    # --- QK
    k_want = base.copy()
    l_want, l_emu = oracle.forward_qk_f16(_np16(q), k_want, xn[:, :, T:T + 1], *pn, T, refemu=(D == 128))
    k_cache = torch.from_numpy(base.copy()).to(gpu)
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    logits = gemv.forward_qk(q.to(gpu), k_cache, x[:, :, T:T + 1].to(gpu), *pg, T, SMIN, SMAX,
                             state_out=st)
    torch.cuda.synchronize()
    assert logits.shape == (B, H, T + 1) and logits.dtype == torch.float16
    assert np.array_equal(k_cache.cpu().numpy(), k_want), "appended K codes differ"
    assert np.array_equal(_np16(st).view(np.uint16), st_want), "replayed K state differs"
    got = _np16(logits).astype(np.float64)
    assert np.all(np.abs(got - l_want) <= _ulp16(l_want) + 1e-3)
    if l_emu is not None and T > 0:
        # informational: our error vs exact is no worse than the reference's own fp16 accumulation
        assert np.max(np.abs(got - l_want)) <= np.max(np.abs(l_emu.astype(np.float64) - l_want)) + 1e-3

    # --- OV
    v_want = base.copy()
    o_want, _ = oracle.forward_ov_f16(_np16(attn), v_want, xn[:, :, T:T + 1], *pn)
    v_cache = torch.from_numpy(base.copy()).to(gpu)
    st2 = torch.zeros_like(st)
    out = gemv.forward_ov(attn.to(gpu), v_cache, x[:, :, T:T + 1].to(gpu), *pg, SMIN, SMAX,
                          state_out=st2)
    torch.cuda.synchronize()
    assert out.shape == (B, H, D) and out.dtype == torch.float16
    assert np.array_equal(v_cache.cpu().numpy(), v_want), "appended V codes differ"
    assert np.array_equal(_np16(st2).view(np.uint16), st_want), "replayed V state differs"
    goto = _np16(out).astype(np.float64)
    assert np.all(np.abs(goto - o_want) <= _ulp16(o_want) + 1e-3)


@pytest.mark.parametrize("rows,n,mask_mode", [(6, 1, None), (6, 130, None), (8, 4097, "b1"), (8, 257, "bh"),
                                              (4, 5121, None), (6, 20000, "b1"), (2, 131073, "bh"),
                                              # long unmasked rows: four chunks per workgroup in the first
                                              # pass (all inside the row / last group ragged / one group only)
                                              (4, 131073, None), (2, 60000, None), (2, 49152, None),
                                              (2, 49153, None),
                                              # one workgroup per row, its shape chosen by the length:
                                              # first and last length of each shape, then the
                                              # shortest chunked row
                                              (4, 2049, None), (4, 5120, "b1"), (4, 6144, None),
                                              (4, 6145, "bh"), (4, 8192, None), (4, 8193, "b1"),
                                              (4, 12288, None), (4, 12289, "b1"), (2, 16384, None),
                                              (2, 16385, "bh"), (2, 24576, None), (2, 24577, "bh"),
                                              # long unmasked rows kept in registers as fp16 (one
                                              # 1024-thread workgroup per row): shortest, a full
                                              # 9-vector row, the longest; one element more goes
                                              # back to the chunked kernels
                                              (2, 24577, None), (2, 73728, None), (2, 73729, None),
                                              (128, 131073, None), (130, 139264, None),
                                              (130, 139265, None)])
def test_softmax(gpu, rows, n, mask_mode):
    g = torch.Generator().manual_seed(n)
    B, H = 2, rows // 2
    l = (torch.randn(B, H, n, generator=g) * 8).half()
    mask = None
    if mask_mode == "b1":
        mask = torch.zeros(B, 1, 1, n)
        mask[0, 0, 0, : n // 3] = float("-inf")
    elif mask_mode == "bh":
        mask = torch.randn(B, H, n, generator=g)
    w = gemv.softmax_scale_mask(l.to(gpu), 0.0884, None if mask is None else mask.to(gpu))
    ref = l.float() * 0.0884
    if mask is not None:
        ref = ref + (mask[:, :, 0, :] if mask.dim() == 4 else mask)
    ref = torch.softmax(ref.double(), -1)
    assert torch.max(torch.abs(w.cpu().double() - ref)) < 6e-4  # half an fp16 ulp at 1.0 + eps


@pytest.mark.parametrize("n", [4097, 30000, 70000])
@pytest.mark.parametrize("scaling", [-0.05, 0.0])
def test_softmax_negative_and_zero_scaling(gpu, n, scaling):
    """The register-resident long-row kernel pads a row with the infinity that the scaling turns
    into -inf; a negative scaling flips it and a zero scaling must take another kernel."""
    g = torch.Generator().manual_seed(n)
    l = (torch.randn(1, 2, n, generator=g) * 8).half()
    w = gemv.softmax_scale_mask(l.to(gpu), scaling)
    ref = torch.softmax(l.double() * scaling, -1)
    assert torch.max(torch.abs(w.cpu().double() - ref)) < 6e-4
    assert torch.all(torch.isfinite(w.cpu().float()))


@pytest.mark.parametrize("B,H,T,D", [(1, 32, 1024, 128), (2, 4, 257, 128), (1, 2, 100, 256)])
def test_decode_step_within_tolerance(gpu, oracle, B, H, T, D):
    """One whole decode-attention step (QK -> softmax -> OV, as llama_adkv.py:264-274) against the
    oracle's exact-sum evaluation of the same chain: max-abs-error <= 2e-3 on the fp16 output."""
    kp = synth.make_params(H, D, seed=3)
    vp = synth.make_params(H, D, seed=4)
    k = synth.make_k(B, H, T + 1, D, dtype=torch.float16)
    v = synth.make_v(B, H, T + 1, D, dtype=torch.float16)
    q = synth.make_q(B, H, D)
    scaling = D ** -0.5
    kpn = [_np16(t) for t in kp.astuple()]
    vpn = [_np16(t) for t in vp.astuple()]
    kc = oracle.alloc_cache(B, H, T + 8, D)
    vc = oracle.alloc_cache(B, H, T + 8, D)
    oracle.encode_kv_f16(kc, _np16(k)[:, :, :T], *kpn)
    oracle.encode_kv_f16(vc, _np16(v)[:, :, :T], *vpn)
    kg, vg = torch.from_numpy(kc.copy()).to(gpu), torch.from_numpy(vc.copy()).to(gpu)
    want, w_want, _ = oracle.decode_step_f16(_np16(q), kc, vc, _np16(k)[:, :, T:], _np16(v)[:, :, T:],
                                             kpn, vpn, T, scaling)

    logits = gemv.forward_qk(q.to(gpu), kg, k[:, :, T:].to(gpu), *[t.to(gpu) for t in kp.astuple()],
                             T, SMIN, SMAX)
    weights = gemv.softmax_scale_mask(logits, scaling)
    out = gemv.forward_ov(weights, vg, v[:, :, T:].to(gpu), *[t.to(gpu) for t in vp.astuple()],
                          SMIN, SMAX)
    torch.cuda.synchronize()
    err = np.max(np.abs(_np16(out).astype(np.float64) - want))
    assert err <= 2e-3, err
    assert np.array_equal(kg.cpu().numpy(), kc) and np.array_equal(vg.cpu().numpy(), vc)
    # same chain with torch's softmax in the middle, exactly as the reference composes it
    w2 = torch.softmax(logits.float() * scaling, dim=-1).to(torch.float16)
    assert torch.max(torch.abs(w2.float() - weights.float())) < 1e-3


def test_full_size_invariants(gpu, oracle):
    """B=128, 32 heads, d=128, ctx 4096 (the headline shape).  Size-independent properties:
    (1) decode replay reproduces the encoder's final state bit-for-bit for every channel;
    (2) encode(T) + in-kernel append of token T == encode(T+1), byte for byte;
    (3) logits/outputs of sampled heads match the oracle run on just those heads."""
    B, H, T, D = 128, 32, 4096, 128
    p = synth.make_params(H, D).to(gpu)
    x = synth.make_k(B, H, T + 1, D, dtype=torch.float16, device=gpu)
    full = synth.alloc_cache(B, H, T + 8, D, gpu)
    gemv.encode_kv(full, x, *p.astuple(), SMIN, SMAX)
    part = synth.alloc_cache(B, H, T + 8, D, gpu)
    st_enc = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    gemv.encode_kv(part, x[:, :, :T].contiguous(), *p.astuple(), SMIN, SMAX, state_out=st_enc)

    q = synth.make_q(B, H, D, device=gpu)
    st_qk = torch.zeros_like(st_enc)
    k_cache = part.clone()
    logits = gemv.forward_qk(q, k_cache, x[:, :, T:].contiguous(), *p.astuple(), T, SMIN, SMAX,
                             state_out=st_qk)
    assert torch.equal(st_qk.view(torch.int16), st_enc.view(torch.int16))
    assert torch.equal(k_cache, full)

    weights = gemv.softmax_scale_mask(logits, D ** -0.5)
    st_ov = torch.zeros_like(st_enc)
    v_cache = part.clone()
    out = gemv.forward_ov(weights, v_cache, x[:, :, T:].contiguous(), *p.astuple(), SMIN, SMAX,
                          state_out=st_ov)
    assert torch.equal(st_ov.view(torch.int16), st_enc.view(torch.int16))
    assert torch.equal(v_cache, full)
    s = weights.float().sum(-1)
    assert torch.all(torch.abs(s - 1) < 5e-3)

    pn = [_np16(t) for t in p.astuple()]
    for (b, h) in [(0, 0), (77, 13), (127, 31)]:
        ph = [a[h:h + 1] for a in pn]
        sub = part[b:b + 1, h:h + 1].cpu().numpy().copy()
        lw, _ = oracle.forward_qk_f16(_np16(q[b:b + 1, h:h + 1]), sub.copy(),
                                      _np16(x[b:b + 1, h:h + 1, T:]), *ph, T)
        got = _np16(logits[b:b + 1, h:h + 1]).astype(np.float64)
        assert np.all(np.abs(got - lw) <= _ulp16(lw) + 1e-3)
        ow, _ = oracle.forward_ov_f16(_np16(weights[b:b + 1, h:h + 1]), sub.copy(),
                                      _np16(x[b:b + 1, h:h + 1, T:]), *ph)
        goto = _np16(out[b:b + 1, h:h + 1]).astype(np.float64)
        assert np.max(np.abs(goto - ow)) <= 2e-3


def _oracle_ckpts(oracle, cache_np, pn, T, S, ncap):
    """Checkpoints the oracle way: entry j = replayed state after (j+1)*S tokens."""
    B, H = cache_np.shape[:2]
    D = cache_np.shape[3] * 4
    ck = np.zeros((B, H, ncap, D, 2), np.uint16)
    for j in range(ncap):
        if (j + 1) * S <= T:
            _, st = oracle.replay_f16(cache_np, *pn, (j + 1) * S, want_khat=False)
            ck[:, :, j] = st
    return ck


@pytest.mark.parametrize("B,H,T,D,S", [
    (1, 2, 100, 128, 16), (2, 3, 64, 128, 16), (1, 2, 63, 128, 8), (1, 1, 257, 128, 64),
    (2, 2, 48, 256, 16), (1, 2, 40, 512, 8), (3, 2, 15, 128, 16), (1, 2, 1024, 128, 256),
    (1, 3, 100, 128, 16), (1, 5, 70, 128, 8),   # odd head counts: a wave's second half is padding
    (24, 32, 41, 128, 8),    # 3840 units: past the two-channel-per-lane shape, still 4-wave workgroups
    (9, 32, 20, 128, 16),    # 576 units: two channels per lane with every SIMD of a few CUs busy
])
def test_checkpointed_segments(gpu, oracle, B, H, T, D, S):
    """Encoder checkpoints are the oracle's replayed states; decode over independently replayed
    segments gives the same appended codes, final state and (up to fp32 summation order) the same
    logits/outputs as one sequential replay; a checkpoint is recorded when T closes an interval."""
    x, p = _inputs(B, H, T + 1, D, seed=3 * T + S)
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    xn = _np16(x)
    ncap = T // S + 2
    base = oracle.alloc_cache(B, H, T + 9, D)
    oracle.encode_kv_f16(base, xn[:, :, :T], *pn)
    ck_want = _oracle_ckpts(oracle, base, pn, T, S, ncap)

    cache = synth.alloc_cache(B, H, T + 9, D, gpu)
    ck = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
    gemv.encode_kv(cache, x[:, :, :T].contiguous().to(gpu), *pg, SMIN, SMAX, ckpt=ck, ckpt_interval=S)
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), base)
    n_have = T // S
    assert np.array_equal(_np16(ck).view(np.uint16)[:, :, :n_have], ck_want[:, :, :n_have])
    assert not ck[:, :, n_have:].any()

    g = torch.Generator().manual_seed(9)
    q = torch.randn(B, H, 1, D, generator=g).half()
    attn = torch.softmax(torch.randn(B, H, T + 1, generator=g) * 2, -1).half()
    _, st_want = oracle.replay_f16(base, *pn, T, want_khat=False)

    k_want = base.copy()
    l_want, _ = oracle.forward_qk_f16(_np16(q), k_want, xn[:, :, T:T + 1], *pn, T)
    kc, ckk = cache.clone(), ck.clone()
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    logits = gemv.forward_qk(q.to(gpu), kc, x[:, :, T:T + 1].to(gpu), *pg, T, SMIN, SMAX,
                             state_out=st, ckpt=ckk, ckpt_interval=S)
    torch.cuda.synchronize()
    assert np.array_equal(kc.cpu().numpy(), k_want)
    assert np.array_equal(_np16(st).view(np.uint16), st_want)
    assert np.all(np.abs(_np16(logits).astype(np.float64) - l_want) <= _ulp16(l_want) + 1e-3)
    got_ck = _np16(ckk).view(np.uint16)
    if T % S == 0:
        assert np.array_equal(got_ck[:, :, T // S - 1], st_want), "closing checkpoint not recorded"
    assert np.array_equal(got_ck[:, :, :n_have], ck_want[:, :, :n_have])

    v_want = base.copy()
    o_want, _ = oracle.forward_ov_f16(_np16(attn), v_want, xn[:, :, T:T + 1], *pn)
    vc, ckv = cache.clone(), ck.clone()
    st2 = torch.zeros_like(st)
    out = gemv.forward_ov(attn.to(gpu), vc, x[:, :, T:T + 1].to(gpu), *pg, SMIN, SMAX,
                          state_out=st2, ckpt=ckv, ckpt_interval=S)
    torch.cuda.synchronize()
    assert np.array_equal(vc.cpu().numpy(), v_want)
    assert np.array_equal(_np16(st2).view(np.uint16), st_want)
    assert np.all(np.abs(_np16(out).astype(np.float64) - o_want) <= _ulp16(o_want) + 1e-3)
    if T % S == 0:
        assert np.array_equal(_np16(ckv).view(np.uint16)[:, :, T // S - 1], st_want)


def test_full_size_segmented_matches_sequential(gpu, oracle):
    """Headline shape with checkpoints every 256 tokens, the launch the benchmark times (per-head
    table, 16-wave workgroups, segments summed inside the workgroup): it appends the same codes and
    state as the sequential launch, its logits/outputs agree with that launch, and on sampled
    (sequence, head) pairs they are held to the oracle directly."""
    from adkv_amd import _lib
    B, H, T, D, S = 128, 32, 4096, 128, 256
    name = _lib.lib().adkv_decode_kernel_name(B, H, H, T, D, 4, T // S + 1, S).decode()
    assert name.startswith("ft_kernel"), name      # the kernels bench.py's headline runs
    p = synth.make_params(H, D).to(gpu)
    x = synth.make_k(B, H, T + 1, D, dtype=torch.float16, device=gpu)
    cache = synth.alloc_cache(B, H, T + 8, D, gpu)
    ck = torch.zeros(B, H, T // S + 1, D, 2, dtype=torch.float16, device=gpu)
    gemv.encode_kv(cache, x[:, :, :T].contiguous(), *p.astuple(), SMIN, SMAX, ckpt=ck, ckpt_interval=S)
    q = synth.make_q(B, H, D, device=gpu)
    xn = x[:, :, T:].contiguous()
    c1, c2 = cache.clone(), cache.clone()
    s1 = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    s2 = torch.zeros_like(s1)
    l1 = gemv.forward_qk(q, c1, xn, *p.astuple(), T, SMIN, SMAX, state_out=s1)
    l2 = gemv.forward_qk(q, c2, xn, *p.astuple(), T, SMIN, SMAX, state_out=s2, ckpt=ck, ckpt_interval=S)
    assert torch.equal(c1, c2) and torch.equal(s1.view(torch.int16), s2.view(torch.int16))
    # the two launches may run different kernels (shared or per-head table) that add the 32 lanes'
    # fp32 partials of a token in different orders: the fp16 logits sit at most one ulp apart
    dl = torch.abs(l1.float() - l2.float())
    assert torch.all(dl <= 2.0 ** -10 * torch.clamp(l1.float().abs(), min=2.0 ** -4))
    assert torch.equal(ck[:, :, T // S - 1].view(torch.int16), s1.view(torch.int16))
    w = gemv.softmax_scale_mask(l1, D ** -0.5)
    c1, c2 = cache.clone(), cache.clone()
    o1 = gemv.forward_ov(w, c1, xn, *p.astuple(), SMIN, SMAX)
    o2 = gemv.forward_ov(w, c2, xn, *p.astuple(), SMIN, SMAX, ckpt=ck, ckpt_interval=S)
    assert torch.equal(c1, c2)
    # fp32 partial sums are added in a different order: at most one fp16 ulp apart
    d = torch.abs(o1.float() - o2.float())
    assert torch.all(d <= 2.0 ** -10 * torch.clamp(o1.float().abs(), min=2.0 ** -4))

    # the checkpointed launch against the oracle: logits within one fp16 ulp + 1e-3 of the exact
    # sums, outputs (from the launch's own weights) within 2e-3, appended codes byte for byte
    w2 = gemv.softmax_scale_mask(l2, D ** -0.5)
    c3 = cache.clone()
    o3 = gemv.forward_ov(w2, c3, xn, *p.astuple(), SMIN, SMAX, ckpt=ck, ckpt_interval=S)
    pn = [_np16(t) for t in p.astuple()]
    for (b, h) in [(0, 0), (1, 31), (77, 13), (127, 31)]:
        ph = [a[h:h + 1] for a in pn]
        sub = cache[b:b + 1, h:h + 1].cpu().numpy().copy()
        ksub = sub.copy()
        lw, _ = oracle.forward_qk_f16(_np16(q[b:b + 1, h:h + 1]), ksub, _np16(xn[b:b + 1, h:h + 1]), *ph, T)
        got = _np16(l2[b:b + 1, h:h + 1]).astype(np.float64)
        assert np.all(np.abs(got - lw) <= _ulp16(lw) + 1e-3), (b, h)
        assert np.array_equal(c2[b:b + 1, h:h + 1].cpu().numpy(), ksub), (b, h)
        vsub = sub.copy()
        ow, _ = oracle.forward_ov_f16(_np16(w2[b:b + 1, h:h + 1]), vsub, _np16(xn[b:b + 1, h:h + 1]), *ph)
        goto = _np16(o3[b:b + 1, h:h + 1]).astype(np.float64)
        assert np.max(np.abs(goto - ow)) <= 2e-3, (b, h)
        assert np.array_equal(c3[b:b + 1, h:h + 1].cpu().numpy(), vsub), (b, h)


def test_full_size_decode_step_in_one_launch(gpu, oracle):
    """adkv_decode_step at the headline shape with checkpoints every 256 tokens, run as ONE launch
    (adkv_set_fused_step(1)).  Against the same step as three launches, the call the benchmark
    times: appended K and V codes and checkpoints byte for byte, weights and outputs within an
    fp16 ulp; on sampled (sequence, head) pairs the weights and outputs are held to the oracle's
    exact-sum chain (llama_adkv.py:264-274), output max-abs-error <= 2e-3."""
    from adkv_amd import _lib
    L = _lib.lib()
    B, H, T, D, S = 128, 32, 4096, 128, 256
    ncap = T // S + 1
    kp, vp = synth.make_params(H, D, seed=3).to(gpu), synth.make_params(H, D, seed=4).to(gpu)
    k = synth.make_k(B, H, T + 1, D, dtype=torch.float16, device=gpu)
    v = synth.make_v(B, H, T + 1, D, dtype=torch.float16, device=gpu)
    q = synth.make_q(B, H, D, device=gpu)
    scaling = D ** -0.5
    kc0, vc0 = synth.alloc_cache(B, H, T + 8, D, gpu), synth.alloc_cache(B, H, T + 8, D, gpu)
    kk0 = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
    vk0 = torch.zeros_like(kk0)
    gemv.encode_kv(kc0, k[:, :, :T].contiguous(), *kp.astuple(), SMIN, SMAX, ckpt=kk0, ckpt_interval=S)
    gemv.encode_kv(vc0, v[:, :, :T].contiguous(), *vp.astuple(), SMIN, SMAX, ckpt=vk0, ckpt_interval=S)

    def step():
        bufs = (kc0.clone(), vc0.clone(), kk0.clone(), vk0.clone())
        out, w = gemv.decode_step(q, bufs[0], bufs[1], k[:, :, T:], v[:, :, T:], kp.astuple(), vp.astuple(), T,
                                   scaling, None, k_ckpt=bufs[2], v_ckpt=bufs[3], ckpt_interval=S)
        torch.cuda.synchronize()
        return (out.clone(), w.clone()) + bufs

    three = step()
    L.adkv_set_fused_step(1)
    try:
        assert L.adkv_decode_step_is_fused(B, H, H, T, D, 4, ncap, S, 0) == 1
        one = step()
    finally:
        L.adkv_set_fused_step(0)
    for a, b, what in zip(one[2:], three[2:], ("K cache", "V cache", "K checkpoints", "V checkpoints")):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), what
    assert not torch.equal(one[2], kc0)                                   # the token was appended
    for got, ref in ((one[1], three[1]), (one[0], three[0])):
        d = torch.abs(got.float() - ref.float())
        assert torch.all(d <= 2.0 ** -10 * torch.clamp(ref.float().abs(), min=2.0 ** -6)), d.max()
    assert torch.all(torch.isfinite(one[0].float()))
    kpn, vpn = [_np16(t) for t in kp.astuple()], [_np16(t) for t in vp.astuple()]
    for (b, h) in [(0, 0), (127, 31), (66, 17)]:
        kph, vph = [a[h:h + 1] for a in kpn], [a[h:h + 1] for a in vpn]
        ks, vs = kc0[b:b + 1, h:h + 1].cpu().numpy().copy(), vc0[b:b + 1, h:h + 1].cpu().numpy().copy()
        want, w_want, _ = oracle.decode_step_f16(_np16(q[b:b + 1, h:h + 1]), ks, vs, _np16(k[b:b + 1, h:h + 1, T:]),
                                                 _np16(v[b:b + 1, h:h + 1, T:]), kph, vph, T, scaling)
        assert np.max(np.abs(_np16(one[0][b:b + 1, h:h + 1]).astype(np.float64) - want)) <= 2e-3, (b, h)
        assert np.max(np.abs(_np16(one[1][b:b + 1, h:h + 1]).astype(np.float64) - w_want.astype(np.float64))) < 6e-4
        assert np.array_equal(one[2][b:b + 1, h:h + 1].cpu().numpy(), ks), (b, h)
        assert np.array_equal(one[3][b:b + 1, h:h + 1].cpu().numpy(), vs), (b, h)


@pytest.mark.parametrize("B,H,D,cuts", [
    (2, 3, 128, [0, 5, 6, 8, 19, 40, 41, 64, 100]),     # resumes inside, at and across supergroups
    (1, 2, 256, [0, 16, 17, 33]),
    (1, 1, 512, [0, 3, 24]),
    (2, 2, 128, [3, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18]),  # token by token
])
def test_streaming_append_equals_one_shot_encode(gpu, oracle, B, H, D, cuts):
    """append_kv over any split of the stream == encode_kv over the whole stream: cache bytes,
    carried state and checkpoints (interval 16) are identical."""
    T, S = cuts[-1], 16
    x, p = _inputs(B, H, T, D, seed=T + D)
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    want = oracle.alloc_cache(B, H, T + 8, D)
    st_want = oracle.encode_kv_f16(want, _np16(x), *pn)
    ncap = T // S + 1
    ck_want = _oracle_ckpts(oracle, want, pn, T, S, ncap)

    cache = synth.alloc_cache(B, H, T + 8, D, gpu)
    ck = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
    state = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    xg = x.to(gpu)
    t0 = 0
    for t1 in cuts:
        r = gemv.append_kv(cache, xg[:, :, t0:t1].contiguous(), *pg, t0, state, ckpt=ck, ckpt_interval=S)
        assert r is cache
        t0 = t1
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), want)
    assert np.array_equal(_np16(state).view(np.uint16), st_want)
    assert np.array_equal(_np16(ck).view(np.uint16)[:, :, :T // S], ck_want[:, :, :T // S])


# ------------------------------------------------------------------ fp16-KV comparator kernel
@pytest.mark.gpu
@pytest.mark.parametrize("B,H,T", [(1, 2, 1), (2, 3, 17), (2, 4, 512), (1, 4, 513), (2, 2, 1500)])
def test_fp16_comparator_matches_fp32_attention(gpu, B, H, T):
    """The uncompressed-cache comparator is ordinary attention: check it against fp32 torch math
    (tolerance 2e-3 absolute on outputs of magnitude <= 1, the bar used for the ADKV outputs)."""
    import torch
    from adkv_amd.kernel.fp16_baseline import fp16_decode_attention

    g = torch.Generator().manual_seed(100 + T)
    q = torch.randn(B, H, 128, generator=g).half().cuda()
    K = torch.randn(B, H, T, 128, generator=g).half().cuda()
    V = torch.randn(B, H, T, 128, generator=g).half().cuda()
    scaling = 128 ** -0.5
    out = fp16_decode_attention(q, K, V, scaling)
    torch.cuda.synchronize()
    w = torch.softmax(torch.einsum("bhd,bhtd->bht", q.float(), K.float()) * scaling, dim=-1)
    ref = torch.einsum("bht,bhtd->bhd", w, V.float())
    assert (out.float() - ref).abs().max().item() <= 2e-3


@pytest.mark.gpu
def test_fp16_comparator_rejects_other_head_dims(gpu):
    import torch
    from adkv_amd.kernel.fp16_baseline import fp16_decode_attention

    q = torch.zeros(1, 1, 256, dtype=torch.float16, device="cuda")
    K = torch.zeros(1, 1, 8, 256, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        fp16_decode_attention(q, K, K, 1.0)


# ------------------------------------------------------------------ single-call decode step
@pytest.mark.gpu
@pytest.mark.parametrize("B,H,T,D,S,masked", [
    (2, 4, 257, 128, 0, False), (2, 3, 530, 128, 64, True), (1, 2, 100, 256, 16, False),
    (1, 2, 0, 128, 0, False)])
def test_decode_step_equals_three_calls(gpu, B, H, T, D, S, masked):
    """adkv_decode_step is the three entry points chained inside the library: outputs, weights,
    appended codes and checkpoints must equal the separate calls bit for bit."""
    kp = [t.to(gpu) for t in synth.make_params(H, D, seed=3).astuple()]
    vp = [t.to(gpu) for t in synth.make_params(H, D, seed=4).astuple()]
    k = synth.make_k(B, H, T + 1, D, dtype=torch.float16).to(gpu)
    v = synth.make_v(B, H, T + 1, D, dtype=torch.float16).to(gpu)
    q = synth.make_q(B, H, D).to(gpu)
    scaling = D ** -0.5
    ncap = (T + 8) // S + 1 if S else 0
    mask = None
    if masked:
        mask = torch.zeros(B, 1, 1, T + 1)
        mask[:, :, :, :5] = torch.finfo(torch.float32).min
        mask = mask.to(gpu)

    def fresh():
        kc, vc = synth.alloc_cache(B, H, T + 8, D, gpu), synth.alloc_cache(B, H, T + 8, D, gpu)
        kk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu) if S else None
        vk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu) if S else None
        if T:
            gemv.encode_kv(kc, k[:, :, :T].contiguous(), *kp, SMIN, SMAX, ckpt=kk, ckpt_interval=S)
            gemv.encode_kv(vc, v[:, :, :T].contiguous(), *vp, SMIN, SMAX, ckpt=vk, ckpt_interval=S)
        return kc, vc, kk, vk

    kc, vc, kk, vk = fresh()
    logits = gemv.forward_qk(q, kc, k[:, :, T:], *kp, T, SMIN, SMAX, ckpt=kk, ckpt_interval=S)
    w = gemv.softmax_scale_mask(logits, scaling, mask)
    out = gemv.forward_ov(w, vc, v[:, :, T:], *vp, SMIN, SMAX, ckpt=vk, ckpt_interval=S)

    kc2, vc2, kk2, vk2 = fresh()
    out2, w2 = gemv.decode_step(q, kc2, vc2, k[:, :, T:], v[:, :, T:], kp, vp, T, scaling, mask,
                                 k_ckpt=kk2, v_ckpt=vk2, ckpt_interval=S)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    assert torch.equal(w.view(torch.int16), w2.view(torch.int16))
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)
    if S:
        assert torch.equal(kk.view(torch.int16), kk2.view(torch.int16))
        assert torch.equal(vk.view(torch.int16), vk2.view(torch.int16))


@pytest.mark.parametrize("B,H,T,S,lanes", [
    (16, 2, 300, 32, 16), (5, 3, 257, 32, 16), (21, 2, 263, 32, 16),      # uneven segments; whole / half-empty waves / two workgroups per head
    (8, 2, 127, 32, 32), (3, 2, 120, 32, 32), (19, 2, 127, 32, 32),       # four even segments (too few checkpoints for uneven ones)
])
def test_decode_step_in_one_launch(gpu, oracle, B, H, T, S, lanes):
    """Where forward_qk and forward_ov both cut every sequence into four segments inside one
    workgroup, adkv_decode_step can run forward_qk, the softmax and forward_ov as ONE launch
    (adkv_set_fused_step; the kernels forced here on small shapes through the kernel knob).
    Against the three launches: appended codes and checkpoints identical, weights and outputs
    within an fp16 ulp (the softmax sums in another order); against the oracle's exact-sum chain: output max-abs-error <= 2e-3.  Replays are
    bit-identical; with a mask the step falls back to three launches."""
    from adkv_amd import _lib
    L = _lib.lib()
    D = 128
    kp, vp = synth.make_params(H, D, seed=3), synth.make_params(H, D, seed=4)
    kpg, vpg = [t.to(gpu) for t in kp.astuple()], [t.to(gpu) for t in vp.astuple()]
    k = synth.make_k(B, H, T + 1, D, dtype=torch.float16)
    v = synth.make_v(B, H, T + 1, D, dtype=torch.float16)
    q = synth.make_q(B, H, D)
    scaling = D ** -0.5
    ncap = (T + 8) // S + 1
    kpn, vpn = [_np16(t) for t in kp.astuple()], [_np16(t) for t in vp.astuple()]
    kc, vc = oracle.alloc_cache(B, H, T + 8, D), oracle.alloc_cache(B, H, T + 8, D)
    oracle.encode_kv_f16(kc, _np16(k)[:, :, :T], *kpn)
    oracle.encode_kv_f16(vc, _np16(v)[:, :, :T], *vpn)
    want, w_want, _ = oracle.decode_step_f16(_np16(q), kc.copy(), vc.copy(), _np16(k)[:, :, T:], _np16(v)[:, :, T:],
                                             kpn, vpn, T, scaling)
    kg, vg, qg = k.to(gpu), v.to(gpu), q.to(gpu)

    def fresh():
        a, b = synth.alloc_cache(B, H, T + 8, D, gpu), synth.alloc_cache(B, H, T + 8, D, gpu)
        kk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
        vk = torch.zeros_like(kk)
        gemv.encode_kv(a, kg[:, :, :T].contiguous(), *kpg, SMIN, SMAX, ckpt=kk, ckpt_interval=S)
        gemv.encode_kv(b, vg[:, :, :T].contiguous(), *vpg, SMIN, SMAX, ckpt=vk, ckpt_interval=S)
        return a, b, kk, vk

    def step(bufs, mask=None):
        out, w = gemv.decode_step(qg, bufs[0], bufs[1], kg[:, :, T:], vg[:, :, T:], kpg, vpg, T, scaling, mask,
                                   k_ckpt=bufs[2], v_ckpt=bufs[3], ckpt_interval=S)
        torch.cuda.synchronize()
        return out.clone(), w.clone()

    L.adkv_set_mha_kernel(3 if lanes == 16 else 4)
    try:
        assert L.adkv_decode_step_is_fused(B, H, H, T, D, 4, ncap, S, 0) == 0   # off unless asked for
        L.adkv_set_fused_step(1)
        assert L.adkv_decode_step_is_fused(B, H, H, T, D, 4, ncap, S, 0) == 1
        assert L.adkv_decode_step_is_fused(B, H, H, T, D, 4, ncap, S, 1) == 0
        one = fresh()
        assert np.array_equal(one[0].cpu().numpy(), kc) and np.array_equal(one[1].cpu().numpy(), vc)
        out1, w1 = step(one)
        again = fresh()
        out1b, w1b = step(again)
        L.adkv_set_fused_step(0)
        assert L.adkv_decode_step_is_fused(B, H, H, T, D, 4, ncap, S, 0) == 0
        three = fresh()
        out3, w3 = step(three)
    finally:
        L.adkv_set_fused_step(0)
        L.adkv_set_mha_kernel(-1)
    assert torch.equal(out1.view(torch.int16), out1b.view(torch.int16)) and torch.equal(w1.view(torch.int16), w1b.view(torch.int16))
    for a, b, what in zip(one, three, ("K cache", "V cache", "K checkpoints", "V checkpoints")):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), what
    for got, ref in ((w1, w3), (out1, out3)):
        d = torch.abs(got.float() - ref.float())
        assert torch.all(d <= 2.0 ** -10 * torch.clamp(ref.float().abs(), min=2.0 ** -6)), d.max()
    assert torch.all(torch.isfinite(out1.float())) and torch.all(torch.isfinite(w1.float()))
    assert np.max(np.abs(_np16(out1).astype(np.float64) - want)) <= 2e-3
    assert np.max(np.abs(_np16(w1).astype(np.float64) - w_want.astype(np.float64))) < 6e-4


@pytest.mark.parametrize("H,Hq,T,S,bits", [(4, 4, 300, 64, 4), (2, 8, 530, 64, 4), (2, 8, 200, 32, 2)])
def test_decode_step_replays_from_a_captured_graph(gpu, H, Hq, T, S, bits):
    """The library never allocates, clears memory or synchronises, so a decode step can be captured
    in a HIP graph by a serving loop.  Every replay (with eager work and synchronisations between
    replays) must reproduce the eager step: outputs, weights and the caches with the appended token."""
    B, D = 2, 128
    tps = 32 // bits
    kp = [t.to(gpu) for t in synth.make_params(H, D, seed=3, bits=bits).astuple()]
    vp = [t.to(gpu) for t in synth.make_params(H, D, seed=4, bits=bits).astuple()]
    k = synth.make_k(B, H, T + 1, D, dtype=torch.float16).to(gpu)
    v = synth.make_v(B, H, T + 1, D, dtype=torch.float16).to(gpu)
    q = synth.make_q(B, Hq, D).to(gpu)
    scaling = D ** -0.5
    ncap = (T + tps) // S + 1

    def fresh():
        kc = synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits)
        vc = synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits)
        kk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
        vk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
        ks = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
        vs = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
        gemv.append_kv_pair(kc, vc, k[:, :, :T], v[:, :, :T], kp, vp, 0, ks, vs,
                            k_ckpt=kk, v_ckpt=vk, ckpt_interval=S, bits=bits)
        return kc, vc, kk, vk

    ws_bytes = gemv.decode_step_workspace_bytes(B, Hq, H, T, D, ncap, S)
    ws = torch.empty(ws_bytes + 256, dtype=torch.uint8, device=gpu)
    ws = ws[(-ws.data_ptr()) % 256:][:ws_bytes]

    def step(kc, vc, kk, vk):
        return gemv.decode_step(q, kc, vc, k[:, :, T:], v[:, :, T:], kp, vp, T, scaling, None,
                                 k_ckpt=kk, v_ckpt=vk, ckpt_interval=S, bits=bits, workspace=ws)

    e = fresh()
    out_e, w_e = step(*e)
    torch.cuda.synchronize()
    out_e, w_e = out_e.clone(), w_e.clone()

    gbuf = fresh()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(*gbuf)                                  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g, w_g = step(*gbuf)
    for rep in range(4):
        out_g.zero_()
        w_g.zero_()
        graph.replay()
        junk = (k.float() * 1.5).sum()               # the program's own eager work between replays
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
        assert torch.equal(out_g.view(torch.int16), out_e.view(torch.int16)), rep
        assert torch.equal(w_g.view(torch.int16), w_e.view(torch.int16)), rep
        for a, b in zip(gbuf, e):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), rep


@pytest.mark.parametrize("B,H,Hq,T,S,bits", [
    (2, 4, 4, 257, 0, 4),        # vector kernels, one segment
    (2, 3, 3, 530, 64, 4),       # vector kernels, a few segments (narrow partial-sum kernel)
    (1, 2, 2, 2100, 64, 4),      # many segments (wide partial-sum kernel)
    (40, 32, 32, 300, 64, 4),    # enough units for four channels per lane
    (2, 2, 8, 530, 64, 4),       # matrix-core kernels, 4 query heads per KV head
    (1, 2, 16, 200, 32, 2),      # 2-bit codes, 8 query heads per KV head
    (3, 2, -2, 530, 64, 4),      # the per-head-table kernels (forced, 32 lanes per head), a few segments
    (5, 3, -3, 257, 0, 4),       # the per-head-table kernels (forced, 32 lanes per head), one segment
    (3, 2, -102, 530, 64, 4),    # the per-head-table kernels (forced, 16 lanes per head), a few segments
    (5, 3, -103, 257, 0, 4),     # the per-head-table kernels (forced, 16 lanes per head), one segment
])
def test_decode_step_takes_bfloat16_activations(gpu, B, H, Hq, T, S, bits):
    """q, k_new, v_new in bfloat16: the kernels round them to fp16 on the way in and the result to
    bfloat16 on the way out.  Everything equals the fp16 call on `.to(float16)` inputs followed by
    `.to(bfloat16)`: output bits, weights, appended codes, checkpoints.  (A negative Hq means
    -Hq query heads with the per-head-table kernels forced, -100 - Hq those with 16 lanes per head.)"""
    from adkv_amd import _lib
    if Hq < -100:
        Hq = -Hq - 100
        _lib.lib().adkv_set_mha_kernel(3)
    elif Hq < 0:
        Hq = -Hq
        _lib.lib().adkv_set_mha_kernel(4)
    try:
        _bf16_case(gpu, B, H, Hq, T, S, bits)
    finally:
        _lib.lib().adkv_set_mha_kernel(-1)


def _bf16_case(gpu, B, H, Hq, T, S, bits):
    D = 128
    tps = 32 // bits
    kp = [t.to(gpu) for t in synth.make_params(H, D, seed=3, bits=bits).astuple()]
    vp = [t.to(gpu) for t in synth.make_params(H, D, seed=4, bits=bits).astuple()]
    k = synth.make_k(B, H, T, D, dtype=torch.float16).to(gpu)
    v = synth.make_v(B, H, T, D, dtype=torch.float16).to(gpu)
    g = torch.Generator().manual_seed(T)
    qb, kb, vb = [(1.01 * torch.randn(B, h, 1, D, generator=g)).to(torch.bfloat16).to(gpu)
                  for h in (Hq, H, H)]
    ncap = (T + tps) // S + 1 if S else 0

    def fresh():
        kc = synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits)
        vc = synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits)
        kk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu) if S else None
        vk = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu) if S else None
        ks = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
        vs = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
        gemv.append_kv_pair(kc, vc, k, v, kp, vp, 0, ks, vs, k_ckpt=kk, v_ckpt=vk, ckpt_interval=S, bits=bits)
        return kc, vc, kk, vk

    a = fresh()
    out_a, w_a = gemv.decode_step(qb.half(), a[0], a[1], kb.half(), vb.half(), kp, vp, T, D ** -0.5, None,
                                   k_ckpt=a[2], v_ckpt=a[3], ckpt_interval=S, bits=bits)
    b = fresh()
    out_b, w_b = gemv.decode_step(qb, b[0], b[1], kb, vb, kp, vp, T, D ** -0.5, None,
                                   k_ckpt=b[2], v_ckpt=b[3], ckpt_interval=S, bits=bits)
    torch.cuda.synchronize()
    assert out_a.dtype == torch.float16 and out_b.dtype == torch.bfloat16
    assert torch.equal(out_a.to(torch.bfloat16).view(torch.int16), out_b.view(torch.int16))
    assert torch.equal(w_a.view(torch.int16), w_b.view(torch.int16))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    if S:
        assert torch.equal(a[2].view(torch.int16), b[2].view(torch.int16))
        assert torch.equal(a[3].view(torch.int16), b[3].view(torch.int16))


# ------------------------------------------------------------------ grouped-query / matrix-core kernels
def _gqa_case(gpu, oracle, B, Hkv, G, T, S, seed=0, bits=4):
    """One QK + OV pass with G query heads per KV head against the oracle run once per group member
    on a copy of the same cache (query head j reads KV head j // G)."""
    D = 128
    Hq = Hkv * G
    tps = 32 // bits
    x, p = _inputs(B, Hkv, T + 1, D, seed=seed, bits=bits)
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    g = torch.Generator().manual_seed(50 + seed)
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    attn = torch.softmax(2.0 * torch.randn(B, Hq, T + 1, generator=g), dim=-1).half()
    xn = _np16(x)[:, :, T:T + 1]
    want_l = np.zeros((B, Hq, T + 1))
    want_o = np.zeros((B, Hq, D))
    qn, an = _np16(q).reshape(B, Hkv, G, D), _np16(attn).reshape(B, Hkv, G, T + 1)
    ncap = (T + tps) // S + 1 if S else 0
    ck = None
    with oracle.code_bits(bits):
        cache0 = oracle.alloc_cache(B, Hkv, T + tps, D)
        if T:
            oracle.encode_kv_f16(cache0, _np16(x)[:, :, :T], *pn)
        if S:
            ck = torch.from_numpy(_oracle_ckpts(oracle, cache0, pn, T, S, ncap).view(np.int16)) \
                .view(torch.float16).to(gpu)
        for j in range(G):
            c = cache0.copy()
            l, _ = oracle.forward_qk_f16(qn[:, :, j], c, xn, *pn, T)
            want_l.reshape(B, Hkv, G, T + 1)[:, :, j] = l
            c2 = cache0.copy()
            o, _ = oracle.forward_ov_f16(an[:, :, j], c2, xn, *pn)
            want_o.reshape(B, Hkv, G, D)[:, :, j] = o
        _, st_want = oracle.replay_f16(cache0, *pn, T, want_khat=False)
    kc = torch.from_numpy(cache0.copy()).to(gpu)
    vc = torch.from_numpy(cache0.copy()).to(gpu)
    ckv = ck.clone() if ck is not None else None
    st_k = torch.zeros(B, Hkv, D, 2, dtype=torch.float16, device=gpu)
    logits = gemv.forward_qk(q.to(gpu), kc, x[:, :, T:T + 1].to(gpu), *pg, T, SMIN, SMAX,
                             state_out=st_k, ckpt=ck, ckpt_interval=S, bits=bits)
    out = gemv.forward_ov(attn.to(gpu), vc, x[:, :, T:T + 1].to(gpu), *pg, SMIN, SMAX,
                          ckpt=ckv, ckpt_interval=S, bits=bits)
    torch.cuda.synchronize()
    assert logits.shape == (B, Hq, T + 1) and out.shape == (B, Hq, D)
    assert np.array_equal(kc.cpu().numpy(), c) and np.array_equal(vc.cpu().numpy(), c2)
    assert np.array_equal(st_k.cpu().view(torch.int16).numpy().view(np.uint16), st_want)
    lg, og = _np16(logits).astype(np.float64), _np16(out).astype(np.float64)
    assert np.all(np.abs(lg - want_l) <= _ulp16(want_l) + 1e-3), np.abs(lg - want_l).max()
    assert np.all(np.abs(og - want_o) <= _ulp16(want_o) + 1e-3), np.abs(og - want_o).max()
    if S:
        assert torch.equal(ck.view(torch.int16), ckv.view(torch.int16))


@pytest.mark.parametrize("bits,B,H,D,cuts,S", [
    (4, 2, 3, 128, (0, 5, 8, 19, 64, 100), 16),   # one channel per lane (few channels)
    (4, 1, 2, 512, (0, 3, 24), 0),
    (4, 16, 32, 128, (0, 40), 8),                 # 65 536 channels per tensor: still one per lane
    (4, 64, 32, 128, (0, 17), 0),                 # 262 144 channels per tensor: two per lane
    (2, 2, 2, 128, (0, 33, 34, 64, 150), 32),
])
def test_paired_append_equals_oracle(gpu, oracle, bits, B, H, D, cuts, S):
    """K and V rows of the same tokens quantised in one launch: both caches, both carried states
    and both checkpoint tensors equal the oracle's for each tensor on its own."""
    T = cuts[-1]
    tps = 32 // bits
    ncap = T // S + 1 if S else 0
    data, want = [], []
    for i in range(2):
        x, p = _inputs(B, H, T, D, seed=11 + i, bits=bits)
        pn = [_np16(t) for t in p.astuple()]
        with oracle.code_bits(bits):
            c = oracle.alloc_cache(B, H, T + tps, D)
            st = oracle.encode_kv_f16(c, _np16(x), *pn)
            ck = _oracle_ckpts(oracle, c, pn, T, S, ncap) if S else None
        data.append((x.to(gpu), [t.to(gpu) for t in p.astuple()]))
        want.append((c, st, ck))
    caches = [synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits) for _ in range(2)]
    states = [torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu) for _ in range(2)]
    cks = [torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu) if S else None
           for _ in range(2)]
    for a, b in zip(cuts[:-1], cuts[1:]):
        gemv.append_kv_pair(caches[0], caches[1], data[0][0][:, :, a:b], data[1][0][:, :, a:b],
                            data[0][1], data[1][1], a, states[0], states[1],
                            k_ckpt=cks[0], v_ckpt=cks[1], ckpt_interval=S, bits=bits)
    torch.cuda.synchronize()
    for i in range(2):
        assert np.array_equal(caches[i].cpu().numpy(), want[i][0]), i
        assert np.array_equal(_np16(states[i]).view(np.uint16), want[i][1]), i
        if S:
            n = T // S
            assert np.array_equal(_np16(cks[i]).view(np.uint16)[:, :, :n], want[i][2][:, :, :n]), i


@pytest.mark.parametrize("B,Hkv,G,T,S", [
    (1, 2, 4, 0, 0), (2, 2, 4, 5, 0), (1, 3, 2, 8, 0), (2, 2, 4, 71, 0), (1, 2, 8, 40, 0),
    (2, 3, 4, 530, 64), (1, 2, 2, 256, 64), (1, 1, 8, 200, 16), (1, 5, 4, 1025, 0), (1, 3, 4, 200, 16)])
def test_grouped_query_kernels(gpu, oracle, B, Hkv, G, T, S):
    _gqa_case(gpu, oracle, B, Hkv, G, T, S, seed=T % 7)


@pytest.mark.parametrize("dtype,strided,bits,B,H,D,cuts", [
    (torch.float16, True, 4, 2, 3, 128, (0, 5, 8, 19, 64, 100)),
    (torch.bfloat16, False, 4, 2, 3, 128, (0, 7, 40)),
    (torch.bfloat16, True, 4, 1, 2, 256, (0, 16, 17, 33)),
    (torch.bfloat16, True, 2, 2, 2, 128, (0, 33, 34, 64, 150)),
    (torch.bfloat16, True, 4, 48, 32, 128, (0, 21)),        # 196 608 channels per tensor: two per lane
])
def test_paired_append_reads_projection_outputs_in_place(gpu, oracle, dtype, strided, bits, B, H, D, cuts):
    """The K/V rows as an attention module has them: bfloat16 or float16, laid out [B, T, H, D] and
    viewed head-first.  The paired append rounds bf16 to fp16 (nearest even) and follows the
    strides itself; the result equals the oracle on a packed fp16 copy."""
    T = cuts[-1]
    tps = 32 // bits
    caches = [synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits) for _ in range(2)]
    states = [torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu) for _ in range(2)]
    rows, pars, want = [], [], []
    for i in range(2):
        x, p = _inputs(B, H, T, D, seed=21 + i, bits=bits)
        x = (x.float() * 1.01).to(dtype)                      # values that are not fp16 numbers in bf16
        if strided:
            xg = x.permute(0, 2, 1, 3).contiguous().to(gpu).permute(0, 2, 1, 3)   # memory [B, T, H, D]
            assert not xg.is_contiguous()
        else:
            xg = x.to(gpu)
        rows.append(xg)
        pars.append([t.to(gpu) for t in p.astuple()])
        pn = [_np16(t) for t in p.astuple()]
        with oracle.code_bits(bits):
            c = oracle.alloc_cache(B, H, T + tps, D)
            st = oracle.encode_kv_f16(c, _np16(x.to(torch.float16)), *pn)
        want.append((c, st))
    for a, b in zip(cuts[:-1], cuts[1:]):
        gemv.append_kv_pair(caches[0], caches[1], rows[0][:, :, a:b], rows[1][:, :, a:b],
                            pars[0], pars[1], a, states[0], states[1], bits=bits)
    torch.cuda.synchronize()
    for i in range(2):
        assert np.array_equal(caches[i].cpu().numpy(), want[i][0]), i
        assert np.array_equal(_np16(states[i]).view(np.uint16), want[i][1]), i


@pytest.mark.parametrize("G,bits", [(4, 4), (8, 4), (2, 2), (4, 2), (8, 2)])
def test_grouped_query_kernels_in_16_wave_workgroups(gpu, oracle, G, bits):
    """A launch big enough for the 16-wave workgroups (128 KV heads x 64 segments = 8192 units):
    the instantiations the small cases above never reach, including the eight-head QK kernel
    that runs them with spilled registers.  The GPU does the whole problem; the oracle (far too
    slow for all of it) replays three sampled (sequence, KV head) pairs from the GPU-encoded cache."""
    B, Hkv, D, S = 16, 8, 128, 16
    T = 64 * S + 5
    Hq = Hkv * G
    tps = 32 // bits
    x, p = _inputs(B, Hkv, T + 1, D, seed=G, bits=bits)
    pg = [t.to(gpu) for t in p.astuple()]
    g = torch.Generator().manual_seed(50 + G)
    q = torch.randn(B, Hq, 1, D, generator=g).half()
    attn = torch.softmax(2.0 * torch.randn(B, Hq, T + 1, generator=g), dim=-1).half()
    ncap = (T + tps) // S + 1
    cache = synth.alloc_cache(B, Hkv, T + tps, D, gpu, bits=bits)
    st = torch.zeros(B, Hkv, D, 2, dtype=torch.float16, device=gpu)
    ck = torch.zeros(B, Hkv, ncap, D, 2, dtype=torch.float16, device=gpu)
    gemv.append_kv(cache, x[:, :, :T].to(gpu), *pg, 0, st, ckpt=ck, ckpt_interval=S, bits=bits)
    torch.cuda.synchronize()
    cache0 = cache.cpu().numpy()
    kc, vc, ckv = cache.clone(), cache.clone(), ck.clone()
    xnew = x[:, :, T:T + 1].to(gpu)
    logits = gemv.forward_qk(q.to(gpu), kc, xnew, *pg, T, SMIN, SMAX, ckpt=ck, ckpt_interval=S, bits=bits)
    out = gemv.forward_ov(attn.to(gpu), vc, xnew, *pg, SMIN, SMAX, ckpt=ckv, ckpt_interval=S, bits=bits)
    torch.cuda.synchronize()
    lg = _np16(logits).astype(np.float64).reshape(B, Hkv, G, T + 1)
    og = _np16(out).astype(np.float64).reshape(B, Hkv, G, D)
    qn, an = _np16(q).reshape(B, Hkv, G, D), _np16(attn).reshape(B, Hkv, G, T + 1)
    for (b, h) in [(0, 0), (B - 1, Hkv - 1), (7, 3)]:
        pn = [_np16(t)[h:h + 1] for t in p.astuple()]
        xn = _np16(x)[b:b + 1, h:h + 1, T:T + 1]
        with oracle.code_bits(bits):
            want = oracle.alloc_cache(1, 1, T + tps, D)
            oracle.encode_kv_f16(want, _np16(x)[b:b + 1, h:h + 1, :T], *pn)
            assert np.array_equal(cache0[b:b + 1, h:h + 1], want), (b, h)
            for j in range(G):
                c = want.copy()
                l, _ = oracle.forward_qk_f16(qn[b:b + 1, h:h + 1, j], c, xn, *pn, T)
                c2 = want.copy()
                o, _ = oracle.forward_ov_f16(an[b:b + 1, h:h + 1, j], c2, xn, *pn)
                assert np.all(np.abs(lg[b, h, j] - l[0, 0]) <= _ulp16(l[0, 0]) + 1e-3), (b, h, j)
                assert np.all(np.abs(og[b, h, j] - o[0, 0]) <= _ulp16(o[0, 0]) + 1e-3), (b, h, j)
        assert np.array_equal(kc[b:b + 1, h:h + 1].cpu().numpy(), c), (b, h)
        assert np.array_equal(vc[b:b + 1, h:h + 1].cpu().numpy(), c2), (b, h)
    assert torch.equal(ck.view(torch.int16), ckv.view(torch.int16))


@pytest.mark.parametrize("B,H,T,S", [
    (2, 3, 0, 0), (1, 2, 7, 0), (3, 2, 8, 0), (2, 2, 130, 0),          # nothing cached / tail only / one word
    (3, 2, 100, 16), (1, 2, 63, 8), (5, 2, 257, 64), (2, 3, 530, 64),  # odd batches: half-empty waves
    (2, 2, 1024, 256), (33, 3, 72, 8),                                 # several workgroups per head
    (40, 2, 300, 0),                                                   # no checkpoints, 20 waves per head
    (4, 2, 40, 32), (2, 2, 64, 32), (5, 3, 100, 32), (9, 2, 127, 32),  # two / four segments (ragged last one):
                                                                       # partial outputs added in the workgroup
    (4, 8, 300, 8),                                                    # four groups of four uneven segments in one
                                                                       # round of workgroups: with 16 lanes forward_ov
                                                                       # takes them too, through the workspace
])
@pytest.mark.parametrize("lanes", [32, 16])
def test_per_head_table_kernels(gpu, oracle, B, H, T, S, lanes):
    """The decode kernels that keep a per-head (code, channel pair) -> (q, scale multiplier) table
    and reduce logits with masked DPP adds, forced for shapes far smaller than the ones that
    take them by default, with a head over 32 lanes (two sequences per wave) and over 16 (four
    sequences per wave, two passes per supergroup): appended codes, replayed state and recorded
    checkpoints bit-exact, logits and outputs within an fp16 ulp of the oracle's exact sums."""
    from adkv_amd import _lib
    _lib.lib().adkv_set_mha_kernel(3 if lanes == 16 else 4)
    try:
        _gqa_case(gpu, oracle, B, H, 1, T, S, seed=5)
    finally:
        _lib.lib().adkv_set_mha_kernel(-1)


@pytest.mark.parametrize("B,H,T,S,mode", [
    (34, 64, 203, 8, 4),     # 32 lanes per head: two groups, 256 workgroups of three virtual ones
    (50, 64, 203, 8, 4),     # one group, two virtual workgroups per workgroup
    (67, 64, 203, 8, 3),     # 16 lanes per head: two groups, three virtual workgroups, a wave with three sequences
    (100, 64, 203, 8, 3),    # one group, two virtual workgroups per workgroup
])
def test_virtual_workgroups_with_uneven_segments(gpu, oracle, B, H, T, S, mode):
    """The per-head-table kernels on a plan that only big launches get by themselves: segments of
    unequal length (the four wave slots of a SIMD get unequal shares), several virtual workgroups
    walked through by each launched workgroup, partial outputs through the workspace.  Forced on
    a mid-sized shape.  Appended codes equal a one-shot encode of T+1 tokens; state, checkpoints,
    logits and outputs equal those of the shared-table kernels (which cut the context evenly);
    sampled (sequence, head) pairs are held to the oracle."""
    from adkv_amd import _lib
    import ctypes
    L = _lib.lib()
    D = 128
    x, p = _inputs(B, H, T + 1, D, seed=21)
    pg = [t.to(gpu) for t in p.astuple()]
    xg = x.to(gpu)
    ncap = (T + 8) // S + 1
    full = synth.alloc_cache(B, H, T + 9, D, gpu)
    gemv.encode_kv(full, xg, *pg, SMIN, SMAX)
    cache = synth.alloc_cache(B, H, T + 9, D, gpu)
    ck = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
    st_enc = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    gemv.encode_kv(cache, xg[:, :, :T].contiguous(), *pg, SMIN, SMAX, state_out=st_enc, ckpt=ck, ckpt_interval=S)
    g = torch.Generator().manual_seed(4)
    q = torch.randn(B, H, 1, D, generator=g).half().to(gpu)
    attn = torch.softmax(2.0 * torch.randn(B, H, T + 1, generator=g), dim=-1).half().to(gpu)
    xn = xg[:, :, T:].contiguous()

    def run(mode):
        L.adkv_set_mha_kernel(mode)
        try:
            kc, vc, ckk, ckv = cache.clone(), cache.clone(), ck.clone(), ck.clone()
            sk, sv = torch.zeros_like(st_enc), torch.zeros_like(st_enc)
            lg = gemv.forward_qk(q, kc, xn, *pg, T, SMIN, SMAX, state_out=sk, ckpt=ckk, ckpt_interval=S)
            o = gemv.forward_ov(attn, vc, xn, *pg, SMIN, SMAX, state_out=sv, ckpt=ckv, ckpt_interval=S)
            torch.cuda.synchronize()
            return lg, o, kc, vc, ckk, ckv, sk, sv
        finally:
            L.adkv_set_mha_kernel(-1)

    L.adkv_set_mha_kernel(mode)
    try:
        b = (ctypes.c_int * 80)()
        info = (ctypes.c_int * 2)()
        n = L.adkv_decode_segments(B, H, H, T, D, 4, ncap, S, b, 80, info)
        name = L.adkv_decode_kernel_name(B, H, H, T, D, 4, ncap, S).decode()
    finally:
        L.adkv_set_mha_kernel(-1)
    assert "uneven" in name and n in (4, 8) and info[1] >= 2, (name, n, list(info))
    lens = [b[i + 1] - b[i] for i in range(n)]
    assert len(set(lens)) > 2, lens                                     # really uneven

    assert ("16 lanes" in name) == (mode == 3), name
    got, want = run(mode), run(0)
    for a, w, what in zip(got[2:], want[2:], ("K cache", "V cache", "K checkpoints", "V checkpoints", "K state", "V state")):
        assert torch.equal(a.view(torch.uint8), w.view(torch.uint8)), what
    assert torch.equal(got[2], full) and torch.equal(got[3], full)
    assert torch.equal(got[6].view(torch.int16), st_enc.view(torch.int16))
    for a, w in ((got[0], want[0]), (got[1], want[1])):                  # summation order differs: one ulp
        d = torch.abs(a.float() - w.float())
        assert torch.all(d <= 2.0 ** -10 * torch.clamp(w.float().abs(), min=2.0 ** -4))
    pn = [_np16(t) for t in p.astuple()]
    for (bb, h) in [(0, 0), (B - 1, H - 1), (B // 2, 17), (7, 40), (B - 2, 1), (B - 3, 63)]:
        ph = [a[h:h + 1] for a in pn]
        sub = cache[bb:bb + 1, h:h + 1].cpu().numpy().copy()
        lw, _ = oracle.forward_qk_f16(_np16(q[bb:bb + 1, h:h + 1]), sub.copy(), _np16(xn[bb:bb + 1, h:h + 1]), *ph, T)
        gl = _np16(got[0][bb:bb + 1, h:h + 1]).astype(np.float64)
        assert np.all(np.abs(gl - lw) <= _ulp16(lw) + 1e-3), (bb, h)
        ow, _ = oracle.forward_ov_f16(_np16(attn[bb:bb + 1, h:h + 1]), sub.copy(), _np16(xn[bb:bb + 1, h:h + 1]), *ph)
        go = _np16(got[1][bb:bb + 1, h:h + 1]).astype(np.float64)
        assert np.all(np.abs(go - ow) <= _ulp16(ow) + 1e-3), (bb, h)


@pytest.mark.parametrize("B,H,T,S", [(2, 3, 0, 0), (1, 2, 7, 0), (2, 2, 130, 0), (2, 3, 530, 64)])
def test_matrix_core_kernels_for_equal_heads(gpu, oracle, B, H, T, S):
    """The same matrix-core kernels with one query head per KV head (selected by the tuning knob)
    meet the bar of the vector kernels."""
    from adkv_amd import _lib
    _lib.lib().adkv_set_mha_kernel(1)
    try:
        _gqa_case(gpu, oracle, B, H, 1, T, S, seed=3)
    finally:
        _lib.lib().adkv_set_mha_kernel(-1)


# ------------------------------------------------------------------ 2-bit codes
@pytest.mark.parametrize("B,H,T", [(1, 2, 1), (2, 3, 15), (2, 3, 16), (1, 5, 17), (1, 4, 100), (2, 2, 1024)])
def test_encode_2bit_bit_exact(gpu, oracle, B, H, T):
    """2-bit prompt quantisation (append from token 0): codes and final state equal the oracle's."""
    D = 128
    x, p = _inputs(B, H, T, D, seed=T % 5, bits=2)
    pn = [_np16(t) for t in p.astuple()]
    with oracle.code_bits(2):
        want = oracle.alloc_cache(B, H, T + 16, D)
        st_want = oracle.encode_kv_f16(want, _np16(x), *pn)
    cache = synth.alloc_cache(B, H, T + 16, D, gpu, bits=2)
    assert cache.shape == want.shape
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    gemv.append_kv(cache, x.to(gpu), *[t.to(gpu) for t in p.astuple()], 0, st, bits=2)
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), want)
    assert np.array_equal(st.cpu().view(torch.int16).numpy().view(np.uint16), st_want)


@pytest.mark.parametrize("cuts,S", [((0, 5, 16, 17, 40, 41, 90), 0), ((0, 33, 34, 64, 150), 32)])
def test_streaming_append_2bit(gpu, oracle, cuts, S):
    B, H, D = 2, 2, 128
    T = cuts[-1]
    x, p = _inputs(B, H, T, D, seed=2, bits=2)
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    ncap = T // S + 1 if S else 0
    with oracle.code_bits(2):
        want = oracle.alloc_cache(B, H, T + 16, D)
        st_want = oracle.encode_kv_f16(want, _np16(x), *pn)
        ck_want = _oracle_ckpts(oracle, want, pn, T, S, ncap) if S else None
    cache = synth.alloc_cache(B, H, T + 16, D, gpu, bits=2)
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    ck = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu) if S else None
    for a, b in zip(cuts[:-1], cuts[1:]):
        gemv.append_kv(cache, x[:, :, a:b].to(gpu), *pg, a, st, ckpt=ck, ckpt_interval=S, bits=2)
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), want)
    assert np.array_equal(st.cpu().view(torch.int16).numpy().view(np.uint16), st_want)
    if S:
        assert np.array_equal(ck.cpu().view(torch.int16).numpy().view(np.uint16), ck_want)


@pytest.mark.parametrize("B,Hkv,G,T,S", [
    (1, 2, 1, 0, 0), (2, 2, 1, 7, 0), (1, 3, 1, 16, 0), (2, 2, 4, 9, 0), (1, 2, 4, 31, 0), (2, 3, 4, 77, 0),
    (1, 2, 8, 40, 0), (2, 3, 4, 530, 64), (1, 2, 2, 256, 64), (1, 1, 1, 200, 16), (1, 5, 4, 1033, 0)])
def test_decode_kernels_2bit(gpu, oracle, B, Hkv, G, T, S):
    _gqa_case(gpu, oracle, B, Hkv, G, T, S, seed=T % 7, bits=2)


def test_non_finite_inputs_and_runaway_state(gpu, oracle):
    """Parameters that make the scale run away to infinity or zero within a few tokens, large
    inputs and a few infinite / NaN elements: codes, the carried state (NaN in the same places)
    and the state replayed by the decode kernel still equal the oracle's."""
    B, H, D, T = 1, 2, 128, 200
    p = synth.make_params(H, D, seed=1)
    g = torch.Generator().manual_seed(0)
    p.beta = (0.9 * torch.rand(H, D, generator=g)).half()
    p.alpha = (2.0 * torch.rand(H, D, generator=g)).half()
    x = (50.0 * torch.randn(B, H, T + 1, D, generator=g)).half()
    x[0, 0, 5, 3] = float("inf")
    x[0, 1, 9, 7] = float("nan")
    x[0, 1, 30, 8] = -float("inf")
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    want = oracle.alloc_cache(B, H, T + 8, D)
    st_want = oracle.encode_kv_f16(want, _np16(x)[:, :, :T], *pn)
    wf = st_want.view(np.float16).astype(np.float32)
    assert np.isinf(wf).any() and np.isnan(wf).any() and (wf[..., 1] == 0).any()   # it did run away

    def same(a, b):
        nan = np.isnan(a.view(np.float16).astype(np.float32)) & np.isnan(b.view(np.float16).astype(np.float32))
        return np.array_equal(np.where(nan, 0, a), np.where(nan, 0, b))

    cache = synth.alloc_cache(B, H, T + 8, D, gpu)
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    gemv.append_kv(cache, x[:, :, :T].to(gpu), *pg, 0, st)
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), want)
    assert same(_np16(st).view(np.uint16), st_want)

    q = torch.randn(B, H, 1, D, generator=g).half()
    kc, st2 = cache.clone(), torch.zeros_like(st)
    gemv.forward_qk(q.to(gpu), kc, x[:, :, T:].to(gpu), *pg, T, SMIN, SMAX, state_out=st2)
    torch.cuda.synchronize()
    assert same(_np16(st2).view(np.uint16), st_want)
    kw = want.copy()
    oracle.forward_qk_f16(_np16(q), kw, _np16(x)[:, :, T:T + 1], *pn, T)
    assert np.array_equal(kc.cpu().numpy(), kw)


def _fclass(a):
    """0 finite, 1 +inf, 2 -inf, 3 NaN."""
    a = np.asarray(a, dtype=np.float64)
    return np.where(np.isnan(a), 3, np.where(np.isposinf(a), 1, np.where(np.isneginf(a), 2, 0)))


@pytest.mark.parametrize("kernels", ["default", "per_head_table", "per_head_table_16_lanes"])
def test_non_finite_values_in_logits_and_outputs(gpu, oracle, kernels):
    """What the decode kernels return when the replayed state (and with it the dequantised values)
    turns infinite or NaN part of the way through the context.

    Logits, every kernel: finite where the oracle's exact sum is finite (and then within the usual
    bar), and +inf / -inf / NaN exactly where the oracle's is: a sum's class does not depend on the
    order of its terms.

    Outputs, vector contraction (the default dispatch of a launch this small: two channels per
    lane): the same, channel by channel.  Outputs, per-head-table kernel: the contraction runs on
    the matrix cores with explicit zeros in one operand, so a non-finite dequantised value reaches
    BOTH channels of its channel pair as NaN (0 * inf); the reference (gemv.cu:1087) and the vector
    form confine it to its own channel.  Pinned here as the accepted difference: a channel whose
    pair holds no non-finite value equals the oracle; a channel whose own column is non-finite is
    non-finite; a finite channel next to a non-finite partner comes back NaN."""
    from adkv_amd import _lib
    B, H, D, T = 2, 2, 128, 200
    p = synth.make_params(H, D, seed=1)
    g = torch.Generator().manual_seed(0)
    p.beta = (0.02 * torch.rand(H, D, generator=g)).half()
    p.alpha = (0.5 * torch.rand(H, D, generator=g)).half()
    # a few channels with an unstable filter (alpha = 2, a large scale multiplier) and large
    # inputs: their state runs away to infinity / NaN within the context
    hot = [(0, 3), (0, 64), (1, 7), (1, 126)]
    for h, c in hot:
        p.beta[h, c] = 0.9
        p.alpha[h, c] = 2.0
    x = (2.0 * torch.randn(B, H, T + 1, D, generator=g)).half()
    for h, c in hot:
        x[:, h, :, c] *= 25
    x[0, 0, 50, 10] = float("inf")        # non-finite inputs saturate the code and leave the state finite
    x[1, 1, 90, 33] = float("nan")
    pn = [_np16(t) for t in p.astuple()]
    pg = [t.to(gpu) for t in p.astuple()]
    base = oracle.alloc_cache(B, H, T + 8, D)
    oracle.encode_kv_f16(base, _np16(x)[:, :, :T], *pn)
    khat, _ = oracle.replay_f16(base, *pn, T)
    bad = ~np.isfinite(khat.astype(np.float32)).all(axis=2)               # [B, H, D]: channel has a non-finite value
    assert bad.any() and not bad.all()
    q = torch.randn(B, H, 1, D, generator=g).half()
    attn = torch.softmax(torch.randn(B, H, T + 1, generator=g), -1).half()
    lw, _ = oracle.forward_qk_f16(_np16(q), base.copy(), _np16(x)[:, :, T:T + 1], *pn, T)
    ow, _ = oracle.forward_ov_f16(_np16(attn), base.copy(), _np16(x)[:, :, T:T + 1], *pn)
    assert (_fclass(lw) != 0).any() and (_fclass(ow) != 0).any() and (_fclass(ow) == 0).any()

    S = 64
    ck = None
    if kernels != "default":
        _lib.lib().adkv_set_mha_kernel(3 if kernels.endswith("16_lanes") else 4)
        ck = torch.zeros(B, H, T // S + 1, D, 2, dtype=torch.float16, device=gpu)
    try:
        cache = synth.alloc_cache(B, H, T + 8, D, gpu)
        st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
        gemv.append_kv(cache, x[:, :, :T].to(gpu), *pg, 0, st, ckpt=ck, ckpt_interval=S if ck is not None else 0)
        torch.cuda.synchronize()
        assert np.array_equal(cache.cpu().numpy(), base)
        kw = dict(ckpt=ck, ckpt_interval=S) if ck is not None else {}
        logits = gemv.forward_qk(q.to(gpu), cache.clone(), x[:, :, T:].to(gpu), *pg, T, SMIN, SMAX, **kw)
        out = gemv.forward_ov(attn.to(gpu), cache.clone(), x[:, :, T:].to(gpu), *pg, SMIN, SMAX, **kw)
        torch.cuda.synchronize()
    finally:
        _lib.lib().adkv_set_mha_kernel(-1)

    def check(got, want, where):
        got = got.astype(np.float64)
        # fp16 results: an exact sum beyond the fp16 range comes back infinite
        w16 = want.astype(np.float32).astype(np.float16).astype(np.float64)
        near_overflow = np.abs(want) > 6.0e4
        cls_ok = (_fclass(got) == _fclass(w16)) | near_overflow
        assert np.all(cls_ok[where]), "finite / inf / NaN pattern differs from the oracle"
        fin = where & (_fclass(w16) == 0) & ~near_overflow
        assert np.all(np.abs(got[fin] - want[fin]) <= _ulp16(want[fin]) + 1e-3)

    check(_np16(logits), lw, np.ones_like(lw, dtype=bool))
    got_o = _np16(out)
    if kernels == "default":
        check(got_o, ow, np.ones_like(ow, dtype=bool))
    else:
        partner_bad = bad.reshape(B, H, D // 2, 2)[..., ::-1].reshape(B, H, D)
        check(got_o, ow, ~partner_bad)                                   # pair clean, or only this channel bad
        spill = partner_bad & ~bad                                        # finite channel, non-finite partner
        assert spill.any()
        assert np.all(np.isnan(got_o.astype(np.float32)[spill])), "documented pair-wide NaN of the matrix-core contraction"
        assert np.all(_fclass(ow)[spill] == 0)


@pytest.mark.parametrize("bits", [4, 2])
def test_encode_rounding_boundaries(gpu, oracle, bits):
    """Inputs on and next to the quantiser's rounding boundaries: (x - zp) / sc = k + 1/2 exactly
    (ties go to even), one fp16 step to either side, and scales that are not powers of two.  The
    encoder decides most elements with a reciprocal multiply and must fall back to the exact
    divide for these; codes have to match the oracle bit for bit."""
    B, H, D, T = 1, 2, 128, 96
    g = torch.Generator().manual_seed(11 + bits)
    sc_choices = torch.tensor([0.25, 0.5, 1.0, 2.0, 0.75, 1.5, 3.0, 0.3330078125])
    sc = sc_choices[torch.randint(0, len(sc_choices), (H, D), generator=g)].half()
    k = torch.randint(-11, 11, (B, H, T, D), generator=g).float()
    x = ((k + 0.5) * sc.float()[None, :, None, :]).half()                      # exact ties where representable
    nudge = torch.randint(-1, 2, (B, H, T, D), generator=g).to(torch.int16)    # -1, 0, +1 fp16 steps
    x = (x.view(torch.int16) + nudge).view(torch.float16)
    zero = torch.zeros(H, D).half()
    tgt = torch.full((H, D), 3.5 if bits == 4 else 0.5).half()
    params = (zero, sc, zero, zero, tgt)                                       # alpha = beta = 0: state stays put
    pn = [_np16(t) for t in params]
    with oracle.code_bits(bits):
        want = oracle.alloc_cache(B, H, T, D)
        oracle.encode_kv_f16(want, _np16(x), *pn)
    cache = synth.alloc_cache(B, H, T, D, gpu, bits=bits)
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    gemv.append_kv(cache, x.to(gpu), *[t.to(gpu) for t in params], 0, st, bits=bits)
    torch.cuda.synchronize()
    assert np.array_equal(cache.cpu().numpy(), want)


def test_long_context_grouped_query_full_size(gpu, oracle):
    """B=16, 32 query heads over 8 KV heads, d=128, ctx 131072, 2-bit codes, bfloat16 activations:
    the whole step through decode_step at its real size (the 16-wave matrix-core kernels with
    four query heads per KV head, 64 segments, chunked softmax).  Size-independent properties over
    the whole tensor, and two sampled (sequence, KV head) pairs against the oracle:
    (1) encode(T) + the in-kernel append of token T == encode(T+1), byte for byte, K and V;
    (2) the replayed state after T-1 == the encoder's, and it is recorded as the closing checkpoint;
    (3) attention weights sum to one; outputs and weights of the samples within tolerance."""
    B, H, G, D, T, S, bits = 16, 8, 4, 128, 131072, 256, 2
    Hq, tps = H * G, 16
    bf = torch.bfloat16
    kp = synth.make_params(H, D, bits=bits, seed=3).to(gpu)
    vp = synth.make_params(H, D, bits=bits, seed=4).to(gpu)
    caches, fulls, states, ckpts, news = [], [], [], [], []
    samples = [(0, 0), (B - 1, H - 1)]
    rows = {bh: [] for bh in samples}                       # the sampled heads' input rows, for the oracle
    for make, p, seed in ((synth.make_k, kp, 0), (synth.make_v, vp, 1)):
        x = make(B, H, T + 1, D, seed=seed, dtype=torch.float16, device=gpu)
        x[:, :, T] = x[:, :, T].to(bf).to(torch.float16)        # the new token arrives as bfloat16
        ncap = (T + tps) // S + 1
        part = synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits)
        full = synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits)
        st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
        st_full = torch.zeros_like(st)
        ck = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
        gemv.append_kv(part, x[:, :, :T], *p.astuple(), 0, st, ckpt=ck, ckpt_interval=S, bits=bits)
        gemv.append_kv(full, x, *p.astuple(), 0, st_full, bits=bits)
        caches.append(part); fulls.append(full); states.append(st); ckpts.append(ck)
        news.append(x[:, :, T:T + 1].to(bf))
        for (b, h) in samples:
            rows[(b, h)].append(_np16(x[b:b + 1, h:h + 1]))
        del x
    torch.cuda.empty_cache()
    q = synth.make_q(B, Hq, D, dtype=bf, device=gpu)
    kc, vc = caches[0].clone(), caches[1].clone()
    out, w = gemv.decode_step(q, kc, vc, news[0], news[1], kp.astuple(), vp.astuple(), T, D ** -0.5,
                               k_ckpt=ckpts[0], v_ckpt=ckpts[1], ckpt_interval=S, bits=bits)
    torch.cuda.synchronize()
    assert out.dtype == bf and out.shape == (B, Hq, D) and w.shape == (B, Hq, T + 1)
    assert torch.equal(kc, fulls[0]) and torch.equal(vc, fulls[1])                                 # (1)
    for ck, st in zip(ckpts, states):                                                              # (2)
        assert torch.equal(ck[:, :, T // S - 1].view(torch.int16), st.view(torch.int16))
    st_qk = torch.zeros_like(states[0])
    gemv.forward_qk(q.to(torch.float16), caches[0].clone(), news[0].to(torch.float16), *kp.astuple(), T,
                    SMIN, SMAX, state_out=st_qk, ckpt=ckpts[0], ckpt_interval=S, bits=bits)
    assert torch.equal(st_qk.view(torch.int16), states[0].view(torch.int16))
    assert torch.all(torch.abs(w.float().sum(-1) - 1) < 2e-2)                                      # (3)
    qn = _np16(q.to(torch.float16)).reshape(B, H, G, D)
    got = out.float().cpu().numpy().reshape(B, H, G, D)
    kpn, vpn = [_np16(t) for t in kp.astuple()], [_np16(t) for t in vp.astuple()]
    with oracle.code_bits(bits):
        for (b, h) in samples:
            xk, xv = rows[(b, h)]
            ko, vo = oracle.alloc_cache(1, 1, T + tps, D), oracle.alloc_cache(1, 1, T + tps, D)
            oracle.encode_kv_f16(ko, xk[:, :, :T], *[a[h:h + 1] for a in kpn])
            oracle.encode_kv_f16(vo, xv[:, :, :T], *[a[h:h + 1] for a in vpn])
            assert np.array_equal(caches[0][b:b + 1, h:h + 1].cpu().numpy(), ko), (b, h)
            assert np.array_equal(caches[1][b:b + 1, h:h + 1].cpu().numpy(), vo), (b, h)
            for j in (0, G - 1):
                want, w_want, _ = oracle.decode_step_f16(
                    qn[b:b + 1, h:h + 1, j], ko.copy(), vo.copy(), xk[:, :, T:], xv[:, :, T:],
                    [a[h:h + 1] for a in kpn], [a[h:h + 1] for a in vpn], T, D ** -0.5)
                # fp16 result rounded to bf16: half a bf16 ulp on top of the 2e-3 of the fp16 path
                tol = 2e-3 + 2.0 ** -8 * np.abs(want[0, 0])
                assert np.all(np.abs(got[b, h, j] - want[0, 0]) <= tol), (b, h, j)
                # the fp16 logit may sit one ulp from the oracle's (fp32 sums in another order):
                # a factor exp(ulp * scaling) on the weight, below 1 %
                wg = _np16(w[b, h * G + j]).astype(np.float64)
                ww = w_want[0, 0].astype(np.float64)
                assert np.all(np.abs(wg - ww) <= 0.02 * ww + 1e-7), (b, h, j)


def test_streaming_quantiser_full_size(gpu, oracle):
    """B=8, 32 heads, d=128: prefill-quantise 32768 tokens with checkpoints every 256 (one channel
    per lane, 128 checkpoints), then 256 single-token appends with the carried state.  The stream
    equals a one-shot encode of all 33024 tokens byte for byte (whole tensor), two sampled heads
    equal the oracle's codes and final state, and sampled checkpoints equal the oracle's state
    after that many tokens."""
    B, H, D, T, n_app, S = 8, 32, 128, 32768, 256, 256
    p = synth.make_params(H, D).to(gpu)
    x = synth.make_k(B, H, T + n_app, D, dtype=torch.float16, device=gpu)
    ncap = (T + n_app) // S + 1
    cache = synth.alloc_cache(B, H, T + n_app + 8, D, gpu)
    ck = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    gemv.append_kv(cache, x[:, :, :T], *p.astuple(), 0, st, ckpt=ck, ckpt_interval=S)
    st_prefill = st.clone()
    for i in range(n_app):
        gemv.append_kv(cache, x[:, :, T + i:T + i + 1], *p.astuple(), T + i, st, ckpt=ck, ckpt_interval=S)
    once = synth.alloc_cache(B, H, T + n_app + 8, D, gpu)
    ck1 = torch.zeros_like(ck)
    st1 = torch.zeros_like(st)
    gemv.encode_kv(once, x, *p.astuple(), SMIN, SMAX, state_out=st1, ckpt=ck1, ckpt_interval=S)
    torch.cuda.synchronize()
    assert torch.equal(cache, once)
    assert torch.equal(st.view(torch.int16), st1.view(torch.int16))
    assert torch.equal(ck.view(torch.int16), ck1.view(torch.int16))
    assert ck[:, :, (T + n_app) // S - 1].any() and not ck[:, :, (T + n_app) // S:].any()
    assert torch.equal(ck[:, :, T // S - 1].view(torch.int16), st_prefill.view(torch.int16))
    pn = [_np16(t) for t in p.astuple()]
    for (b, h) in [(0, 0), (B - 1, H - 1)]:
        ph = [a[h:h + 1] for a in pn]
        xs = _np16(x[b:b + 1, h:h + 1])
        want = oracle.alloc_cache(1, 1, T + n_app + 8, D)
        st_want = oracle.encode_kv_f16(want, xs, *ph)
        assert np.array_equal(cache[b:b + 1, h:h + 1].cpu().numpy(), want), (b, h)
        assert np.array_equal(_np16(st[b:b + 1, h:h + 1]).view(np.uint16), st_want), (b, h)
        for j in (0, 1, 63, 127, 128):                       # state before token (j+1)*S
            scratch = oracle.alloc_cache(1, 1, (j + 1) * S, D)
            sj = oracle.encode_kv_f16(scratch, xs[:, :, :(j + 1) * S], *ph)
            assert np.array_equal(_np16(ck[b:b + 1, h:h + 1, j]).view(np.uint16), sj), (b, h, j)
