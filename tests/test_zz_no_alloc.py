"""The entry point that allocates nothing, adkv_forward_ov_noalloc, against adkv_forward_ov_gqa.

Both run the same kernels; the only difference is where the fp32 partial sums of a segmented
launch live (the library's static device array instead of a caller workspace), so outputs, appended
codes, recorded checkpoints and the state must be bit-identical.  Two calls in a row share the
array, the second with a smaller problem, which must not see anything the first one left behind.
"""
import ctypes
import math

import numpy as np
import pytest
import torch

from adkv_amd import _lib, synth
from adkv_amd.kernel import gemv

pytestmark = pytest.mark.gpu

SMIN, SMAX = math.exp(-4.0), math.exp(4.0)


def _case(gpu, B, H, G, T, S, bits, seed):
    """A cache of T tokens with checkpoints every S, weights for Hq = H*G query heads, one new row."""
    D = 128
    tps = 32 // bits
    p = synth.make_params(H, D, bits=bits, seed=seed).to(gpu)
    x = synth.make_v(B, H, T + 1, D, seed=seed, dtype=torch.float16, device=gpu)
    cache = synth.alloc_cache(B, H, T + tps, D, gpu, bits=bits)
    ncap = (T + tps) // S + 1
    ck = torch.zeros(B, H, ncap, D, 2, dtype=torch.float16, device=gpu)
    st = torch.zeros(B, H, D, 2, dtype=torch.float16, device=gpu)
    gemv.append_kv(cache, x[:, :, :T].contiguous(), *p.astuple(), 0, st, ckpt=ck, ckpt_interval=S, bits=bits)
    g = torch.Generator().manual_seed(seed)
    attn = torch.softmax(2.0 * torch.randn(B, H * G, T + 1, generator=g), dim=-1).half().to(gpu)
    return dict(B=B, H=H, Hq=H * G, T=T, D=D, S=S, bits=bits, p=p, cache=cache, ck=ck, ncap=ncap,
                attn=attn, v_new=x[:, :, T].contiguous())


def _run(L, c, noalloc):
    """One forward_ov through the C ABI on copies of the case's cache and checkpoints."""
    dev = c["cache"].device
    cache, ck = c["cache"].clone(), c["ck"].clone()
    out = torch.full((c["B"], c["Hq"], c["D"]), float("nan"), dtype=torch.float16, device=dev)
    st = torch.zeros(c["B"], c["H"], c["D"], 2, dtype=torch.float16, device=dev)
    pp = [t.data_ptr() for t in c["p"].astuple()]
    head = [c["attn"].data_ptr(), cache.data_ptr(), c["v_new"].data_ptr(), out.data_ptr(), *pp,
            c["B"], c["Hq"], c["H"], c["T"], c["D"], cache.shape[2], c["bits"], 0,
            st.data_ptr(), ck.data_ptr(), c["ncap"], c["S"]]
    stream = _lib.current_stream_ptr(dev)
    if noalloc:
        rc = L.adkv_forward_ov_noalloc(*head, stream)
    else:
        need = L.adkv_forward_ov_gqa_workspace_bytes(c["B"], c["Hq"], c["H"], c["T"], c["D"], c["ncap"], c["S"])
        assert need > 0, "the case must run several segments, or no scratch is exercised"
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        rc = L.adkv_forward_ov_gqa(*head, ws.data_ptr(), need, stream)
    assert rc == 0, L.adkv_strerror(rc)
    torch.cuda.synchronize()
    return out, cache, ck, st


def test_noalloc_forward_ov_equals_workspace_variant_twice_in_a_row(gpu):
    L = _lib.lib()
    assert L.adkv_static_scratch_bytes() == 32 << 20
    assert L.adkv_init() == 0
    big = _case(gpu, B=3, H=4, G=1, T=1031, S=64, bits=4, seed=5)       # 17 segments, vector kernels
    small = _case(gpu, B=1, H=2, G=4, T=200, S=32, bits=2, seed=6)      # matrix-core kernels, 2-bit
    for c in (big, small):                                              # the second call is the smaller one
        got = _run(L, c, noalloc=True)
        want = _run(L, c, noalloc=False)
        for a, b, name in zip(got, want, ("out", "cache", "checkpoints", "state")):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name
    # a second round over the same array, big problem again after the small one
    got = _run(L, big, noalloc=True)
    want = _run(L, big, noalloc=False)
    assert torch.equal(got[0].view(torch.int16), want[0].view(torch.int16))


def test_noalloc_rejects_launches_beyond_the_static_scratch(gpu):
    """A segment costs B*Hq*D*4 bytes: 96 sequences x 64 query heads over a 131072-token context
    plan 32 segments = 96 MiB > 32 MiB.  The rejection happens on the host, before any pointer
    is used (the pointers here are not device memory)."""
    L = _lib.lib()
    one = ctypes.c_void_p(256)
    need = L.adkv_forward_ov_gqa_workspace_bytes(96, 64, 8, 131072, 128, 513, 256)
    assert need > L.adkv_static_scratch_bytes()
    rc = L.adkv_forward_ov_noalloc(*([one] * 9), 96, 64, 8, 131072, 128, 8200, 4, 0, None, one, 513, 256, None)
    assert rc == -8 and b"static" in L.adkv_strerror(rc)
    # the largest benchmark shape (16 sequences, 32 query heads over 8 KV heads, 131072 tokens) fits
    assert L.adkv_forward_ov_gqa_workspace_bytes(16, 32, 8, 131072, 128, 513, 256) <= L.adkv_static_scratch_bytes()


def test_noalloc_call_is_capturable_in_a_graph(gpu):
    """Stream capture fails on any allocation, so capturing one adkv_forward_ov_noalloc call (after
    adkv_init() has resolved the array's address) shows that the call allocates nothing; every
    replay, with the program's own eager work between replays, reproduces the eager result."""
    L = _lib.lib()
    assert L.adkv_init() == 0
    c = _case(gpu, B=3, H=4, G=1, T=1031, S=64, bits=4, seed=7)         # 17 segments through the array
    want = _run(L, c, noalloc=False)
    dev = c["cache"].device
    cache0, ck0 = c["cache"].clone(), c["ck"].clone()
    cache, ck = cache0.clone(), ck0.clone()
    out = torch.zeros((c["B"], c["Hq"], c["D"]), dtype=torch.float16, device=dev)
    st = torch.zeros(c["B"], c["H"], c["D"], 2, dtype=torch.float16, device=dev)
    pp = [t.data_ptr() for t in c["p"].astuple()]
    head = [c["attn"].data_ptr(), cache.data_ptr(), c["v_new"].data_ptr(), out.data_ptr(), *pp,
            c["B"], c["Hq"], c["H"], c["T"], c["D"], cache.shape[2], c["bits"], 0,
            st.data_ptr(), ck.data_ptr(), c["ncap"], c["S"]]

    def call():
        rc = L.adkv_forward_ov_noalloc(*head, _lib.current_stream_ptr(dev))
        assert rc == 0, L.adkv_strerror(rc)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()                                          # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        out.zero_()
        st.zero_()
        cache.copy_(cache0)
        ck.copy_(ck0)
        graph.replay()
        junk = (c["attn"].float() * 1.5).sum()          # eager work between replays
        torch.cuda.synchronize()
        assert torch.isfinite(junk)
        for a, b, name in zip((out, cache, ck, st), want, ("out", "cache", "checkpoints", "state")):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), (rep, name)


@pytest.mark.parametrize("mode", [4, 3])
def test_noalloc_accepts_launches_that_sum_their_segments_in_the_workgroup(gpu, mode):
    """The per-head-table kernel adds two or four segments inside its workgroups and touches no
    scratch: such a launch is never refused for its size.  Forced here on a small shape (the
    kernels take it by themselves only for launches of hundreds of workgroups), with a head over
    32 lanes (mode 4) and over 16 (mode 3)."""
    L = _lib.lib()
    c = _case(gpu, B=4, H=2, G=1, T=40, S=32, bits=4, seed=8)           # two segments
    L.adkv_set_mha_kernel(mode)
    try:
        got = _run(L, c, noalloc=True)
    finally:
        L.adkv_set_mha_kernel(-1)
    # the same launch through the shared-table kernels and a workspace: same codes, state and
    # checkpoints; outputs one fp16 ulp apart at most (different summation order)
    want = _run(L, c, noalloc=False)
    for a, b, name in zip(got[1:], want[1:], ("cache", "checkpoints", "state")):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name
    d = (got[0].float() - want[0].float()).abs()
    assert torch.all(d <= 2.0 ** -10 * torch.clamp(want[0].float().abs(), min=2.0 ** -4))
