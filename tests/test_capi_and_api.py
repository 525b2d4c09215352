"""CPU-only checks of the boundary: the C-ABI library loads and exports every symbol the public
header declares, and the Python drop-in raises the reference's error messages
(src/adkv/kernel/gemv.cu:375-398, 892-912, 1241-1266) before touching a device."""
import ctypes
import math
import os
import re

import pytest
import torch

from adkv_amd import _lib
from adkv_amd.kernel import gemv

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SMIN, SMAX = math.exp(-4.0), math.exp(4.0)


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "adkv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(adkv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert {"adkv_encode_kv", "adkv_forward_qk", "adkv_forward_ov", "adkv_softmax"} <= set(names)
    L = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/adkv_hip.h but not exported"
    assert set(names) == set(_lib.PROTOTYPES), "ctypes prototypes out of sync with the header"


def test_abi_version_and_strerror():
    L = _lib.lib()
    assert L.adkv_abi_version() == _lib.ABI_VERSION
    assert L.adkv_strerror(0) == b"ok"
    assert b"128, 256 or 512" in L.adkv_strerror(-2)


def test_argument_validation_in_c_abi_needs_no_device():
    """NULL pointers, bad dims and capacity are rejected on the host before any launch."""
    L = _lib.lib()
    one = ctypes.c_void_p(16)
    args = lambda D, T, cap: [one] * 7 + [1, 1, T, D, cap, 0.0, 1.0, None, None]
    assert L.adkv_encode_kv(*([None] + args(128, 8, 1)[1:])) == -1
    assert L.adkv_encode_kv(*args(64, 8, 1)) == -2
    assert L.adkv_encode_kv(*args(128, 9, 1)) == -4
    assert L.adkv_encode_kv(*args(128, -1, 1)) == -3
    qk = [one] * 9 + [1, 1, 8, 128, 1, 0.0, 1.0, None, None]
    assert L.adkv_forward_qk(*qk) == -4          # slot 8 needs a second supergroup
    qk[12] = 96
    assert L.adkv_forward_qk(*qk) == -2
    # checkpoint arguments: interval must be a positive multiple of 8; a multi-segment OV needs workspace
    ex = [one] * 9 + [1, 1, 64, 128, 16, None, one, 8, 12, None]
    assert L.adkv_forward_qk_ex(*ex) == -3
    assert L.adkv_forward_ov_workspace_bytes(1, 1, 64, 128, 8, 16) == 4 * 1 * 1 * 128 * 4
    ov = [one] * 9 + [1, 1, 64, 128, 16, None, one, 8, 16, None, 0, None]
    assert L.adkv_forward_ov_ex(*ov) == -7
    # the headline shape: forward_qk is cut into four uneven segments under the per-head-table plan,
    # forward_ov into two even ones; the size covers either plan, whichever kernel family is selected
    assert L.adkv_forward_ov_workspace_bytes(128, 32, 4096, 128, 17, 256) == 4 * 128 * 32 * 128 * 4


def test_paired_append_and_fused_decode_validation_needs_no_device():
    """The newer entry points reject bad dtypes, strides and NULL parameter arrays on the host."""
    L = _lib.lib()
    one = ctypes.c_void_p(16)
    arr5 = (ctypes.c_void_p * 5)(*[16] * 5)
    st3 = lambda b, h, t: (ctypes.c_int64 * 3)(b, h, t)
    pair = lambda dtype, ks, vs, params=arr5: [one, one, one, one, dtype, ks, vs, params, params,
                                               1, 1, 0, 8, 128, 1, 4, one, one, None, None, 0, 0, None]
    assert L.adkv_append_kv_pair(*pair(0, None, None)) == -6               # fp32 rows are not taken
    assert L.adkv_append_kv_pair(*pair(1, None, None, None)) == -1         # no parameter arrays
    assert L.adkv_append_kv_pair(*pair(1, st3(1024, 128, 127), None)) == -3   # token stride below D
    assert L.adkv_append_kv_pair(*pair(2, st3(1025, 128, 128), None)) == -3   # odd stride: rows unaligned
    fused = [one] * 5 + [arr5, arr5, None, 1, 1.0, one, None, 0, 1, 1, 1, 8, 128, 2, 4, 0,
             None, None, 0, 0, one, 1 << 20, None]
    assert L.adkv_decode_step(*fused) == -6                                # activation dtype must be f16 / bf16


def test_segment_plans_cut_at_checkpoints_and_cover_the_context():
    """adkv_decode_segments: boundaries start at 0, end at T, increase strictly, inner ones lie on
    checkpoints that exist (index below n_ckpt_cap); uneven plans give the oldest wave slot of a
    SIMD the longest segment of its group of four.  Host logic only."""
    L = _lib.lib()
    for (B, Hq, H, T, D, bits, S) in [(128, 32, 32, 4096, 128, 4, 256), (64, 32, 32, 4096, 128, 4, 256),
                                      (352, 32, 32, 4096, 128, 4, 256), (32, 32, 32, 4097, 128, 4, 128),
                                      (34, 32, 32, 3000, 128, 4, 64), (128, 32, 32, 640, 128, 4, 256),
                                      (16, 32, 8, 131072, 128, 2, 256), (1, 32, 32, 32768, 128, 4, 256),
                                      (128, 32, 32, 4096, 128, 4, 0), (3, 5, 5, 1000, 256, 4, 8)]:
        ncap = T // S + 1 if S else 0
        b = (ctypes.c_int * 600)()
        info = (ctypes.c_int * 2)()
        n = L.adkv_decode_segments(B, Hq, H, T, D, bits, ncap, S, b, 600, info)
        assert n >= 1, (B, T)
        bounds = list(b[:n + 1])
        assert bounds[0] == 0 and bounds[-1] == T
        assert all(x < y for x, y in zip(bounds, bounds[1:])), bounds
        for x in bounds[1:-1]:
            assert S and x % S == 0 and x // S - 1 < ncap, (bounds, S)
        name = L.adkv_decode_kernel_name(B, Hq, H, T, D, bits, ncap, S).decode()
        if "uneven" in name:
            assert n % 4 == 0 and info[0] > 0 and info[1] >= 1
            for g in range(n // 4):
                lens = [bounds[4 * g + k + 1] - bounds[4 * g + k] for k in range(4)]
                assert lens[3] + S > lens[2] >= lens[1] >= lens[0], lens       # the last holds the ragged tail
    assert L.adkv_decode_segments(1, 3, 2, 10, 128, 4, 0, 0, None, 0, None) == -1        # 3 query heads over 2
    # the headline shape: shares 7 : 5 : 2 : 2 of 16 intervals, the oldest wave slot's (7) last in time; 16 lanes per head (four sequences per
    # wave) fill the device with 256 workgroups of one virtual workgroup each, 32 lanes per head walk two
    n = L.adkv_decode_segments(128, 32, 32, 4096, 128, 4, 17, 256, b, 600, info)
    assert n == 4 and list(b[:5]) == [0, 512, 1024, 2304, 4096] and list(info) == [256, 1]
    assert b"16 lanes per head" in L.adkv_decode_kernel_name(128, 32, 32, 4096, 128, 4, 17, 256)
    L.adkv_set_mha_kernel(4)
    try:
        n = L.adkv_decode_segments(128, 32, 32, 4096, 128, 4, 17, 256, b, 600, info)
        assert n == 4 and list(b[:5]) == [0, 512, 1024, 2304, 4096] and list(info) == [256, 2]
        assert b"16 lanes" not in L.adkv_decode_kernel_name(128, 32, 32, 4096, 128, 4, 17, 256)
    finally:
        L.adkv_set_mha_kernel(-1)
    # lane width follows a model of the two plans (rounds x virtual workgroups x longest segment): 100 sequences
    # fill 224 workgroups once with 16 lanes and twice with 32; 8 sequences over 65536 tokens would leave half of
    # the 16-lane waves as padding; groups of fewer than 16 checkpoint intervals keep 32 lanes
    assert b"16 lanes per head" in L.adkv_decode_kernel_name(100, 32, 32, 4096, 128, 4, 17, 256)
    assert b"16 lanes" not in L.adkv_decode_kernel_name(8, 32, 32, 65536, 128, 4, 257, 256)
    assert b"16 lanes" not in L.adkv_decode_kernel_name(64, 32, 32, 4096, 128, 4, 17, 256)
    # groups and workgroups are chosen together: 40 sequences over 8192 tokens take three groups in 256
    # workgroups of two virtual ones (two groups by occupancy alone would fill 160)
    n = L.adkv_decode_segments(40, 32, 32, 8192, 128, 4, 33, 256, b, 600, info)
    assert n == 12 and list(info) == [256, 2]
    # a batch too small for that keeps 32 lanes per head unless told otherwise
    assert b"16 lanes" not in L.adkv_decode_kernel_name(34, 32, 32, 3000, 128, 4, 47, 64)
    L.adkv_set_mha_kernel(3)
    try:
        assert b"16 lanes per head" in L.adkv_decode_kernel_name(34, 32, 32, 3000, 128, 4, 47, 64)
    finally:
        L.adkv_set_mha_kernel(-1)


def test_segment_plans_of_random_shapes_stay_inside_the_checkpoints():
    """Seeded sweep of batch sizes, head counts, context lengths, checkpoint intervals and capacities,
    under the library's own choice of kernels and with every kernel family forced: every plan covers
    [0, T] with increasing boundaries, every inner boundary lies on a checkpoint that exists (a
    segment starts from checkpoint boundary / interval - 1, which must be below the capacity), uneven
    plans come in groups of four, and the workspace the library asks for holds the partial sums of
    that many segments (forward_qk's plan; forward_ov's own may have fewer).  Host logic only."""
    import random
    L = _lib.lib()
    rng = random.Random(7)
    cap = 1 << 15
    b = (ctypes.c_int * cap)()
    info = (ctypes.c_int * 2)()
    try:
        for it in range(400):
            mode = rng.choice([-1, -1, 0, 1, 2, 3, 4])
            H = rng.choice([1, 2, 5, 8, 32, 40, 64])
            gq = rng.choice([1, 1, 1, 2, 4, 8]) if mode in (-1, 1) else 1
            Hq = H * gq
            bits = rng.choice([4, 4, 2]) if mode in (-1, 1) else 4
            B = rng.choice([1, 2, 3, 5, 8, 13, 16, 24, 40, 64, 100, 128, 200, 352, 500])
            S = rng.choice([8, 16, 64, 128, 256, 512]) * (2 if bits == 2 else 1)
            T = rng.choice([0, 1, 7, 63, 64, 65, 255, 1000, 4095, 4096, 4097, 8192, 20000, 32768, 131072, 200001])
            full = T // S + 1
            ncap = rng.choice([full, full, full + 3, max(1, full // 2), 1])
            L.adkv_set_mha_kernel(mode)
            n = L.adkv_decode_segments(B, Hq, H, T, 128, bits, ncap, S, b, cap, info)
            case = (mode, B, Hq, H, T, bits, ncap, S)
            assert 1 <= n <= max(1, (T + S - 1) // S) and n < cap, case
            bounds = list(b[:n + 1])
            assert bounds[0] == 0 and bounds[-1] == T, case
            assert all(x < y for x, y in zip(bounds, bounds[1:])) or T == 0, (case, bounds)
            for x in bounds[1:-1]:
                assert x % S == 0 and 0 <= x // S - 1 < ncap, (case, bounds)
            name = L.adkv_decode_kernel_name(B, Hq, H, T, 128, bits, ncap, S).decode()
            if "uneven" in name:
                assert n % 4 == 0, (case, name)
            if info[0]:
                assert info[1] >= 1 and info[0] % H == 0, (case, list(info))
            if gq == 1 and bits == 4:
                need = L.adkv_forward_ov_workspace_bytes(B, H, T, 128, ncap, S)    # equal heads, 4-bit codes
                assert need >= 4 * 128 * B * H * n or n == 1 or (info[0] and n in (2, 4)), (case, need, n)
                assert L.adkv_decode_step_workspace_bytes(B, Hq, H, T, 128, ncap, S) >= need, case
    finally:
        L.adkv_set_mha_kernel(-1)


def test_static_scratch_entry_points_return_a_code_without_a_device():
    """adkv_init() and adkv_forward_ov_noalloc resolve the address of the library's static device
    array with HIP calls.  Where no GPU is present those calls fail; the library must hand that
    back as ADKV_E_DEVICE (with the HIP code kept for adkv_last_hip_error), never abort.  On a
    machine with a GPU adkv_init() succeeds and this test has nothing to show."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: adkv_init() succeeds here")
    L = _lib.lib()
    rc = L.adkv_init()
    assert rc == -9 and b"device" in L.adkv_strerror(rc).lower()
    assert L.adkv_last_hip_error() != 0
    one = ctypes.c_void_p(256)
    # a launch that fits the static array: the size check passes, the address lookup reports the failure
    rc = L.adkv_forward_ov_noalloc(*([one] * 9), 1, 2, 2, 600, 128, 80, 4, 0, None, one, 10, 64, None)
    assert rc == -9
    # one that does not fit is refused before any HIP call
    rc = L.adkv_forward_ov_noalloc(*([one] * 9), 96, 64, 8, 131072, 128, 8200, 4, 0, None, one, 513, 256, None)
    assert rc == -8


def test_rotary_embedding_validation_needs_no_device():
    """adkv_rope_qk rejects NULL pointers, head dims that are no multiple of 4, unaligned bases and
    odd strides on the host, before any launch."""
    L = _lib.lib()
    one = ctypes.c_void_p(16)
    rope = lambda ptrs=None, D=128, strides=None: (ptrs or [one] * 6) + [2, 4, 2, 1, D] + \
        (strides or [4 * D, D, 4 * D, 2 * D, D, 2 * D, D, D]) + [0, None]
    assert L.adkv_rope_qk(*rope(ptrs=[one, None, one, one, one, one])) == -1
    assert L.adkv_rope_qk(*rope(D=126)) == -3
    assert L.adkv_rope_qk(*rope(ptrs=[ctypes.c_void_p(18)] + [one] * 5)) == -5
    assert L.adkv_rope_qk(*rope(strides=[513, 128, 512, 256, 128, 256, 128, 128])) == -5


def test_row_strides_of_projection_outputs():
    """A [B, T, H, D] projection output viewed head-first is handed over with its strides; layouts
    the library cannot read in place (odd strides, channel stride 2) are packed first."""
    from adkv_amd.kernel.gemv import _row_strides
    x = torch.zeros(2, 5, 3, 128, dtype=torch.bfloat16)
    t, s = _row_strides(x.permute(0, 2, 1, 3))
    assert t.data_ptr() == x.data_ptr() and list(s) == [5 * 3 * 128, 128, 3 * 128]
    t, s = _row_strides(x.permute(0, 2, 1, 3).contiguous())
    assert s is None
    odd = torch.zeros(2, 3, 5, 129, dtype=torch.float16)[..., :128]         # token stride 129
    t, s = _row_strides(odd)
    assert s is None and t.is_contiguous()
    every_other = torch.zeros(2, 3, 5, 256, dtype=torch.float16)[..., ::2]
    t, s = _row_strides(every_other)
    assert s is None and t.is_contiguous()


def _p(nh, D, dtype=torch.float16):
    return [torch.zeros(nh, D, dtype=dtype) for _ in range(5)]


def _cache(B, nh, cap, D):
    return torch.zeros(B, nh, cap, D // 4, 4, 4, dtype=torch.uint8)


def _h(*s):
    return torch.zeros(*s, dtype=torch.float16)


def test_forward_qk_errors():
    B, nh, D = 1, 2, 128
    ok = dict(q=_h(B, nh, 1, D), c=_cache(B, nh, 2, D), k=_h(B, nh, 1, D))
    call = lambda q=None, c=None, k=None, p=None, T=3: gemv.forward_qk(
        ok["q"] if q is None else q, ok["c"] if c is None else c, ok["k"] if k is None else k,
        *(_p(nh, D) if p is None else p), T, SMIN, SMAX)
    with pytest.raises(RuntimeError, match="q must be float16"):
        call(q=torch.zeros(B, nh, 1, D))
    with pytest.raises(RuntimeError, match="k_new must be float16"):
        call(k=torch.zeros(B, nh, 1, D))
    with pytest.raises(RuntimeError, match="k_cache must be uint8"):
        call(c=_cache(B, nh, 2, D).to(torch.int8))
    with pytest.raises(RuntimeError, match="k_cache must be contiguous"):
        call(c=_cache(B, nh, 4, D)[:, :, ::2])
    with pytest.raises(RuntimeError, match="k_alpha must be float16"):
        p = _p(nh, D)
        p[2] = p[2].float()
        call(p=p)
    with pytest.raises(RuntimeError, match="q head dimension does not match k_cache"):
        call(q=_h(B, nh, 1, 256))
    with pytest.raises(RuntimeError, match="T must be non-negative"):
        call(T=-1)
    with pytest.raises(RuntimeError, match="k_cache has no free supergroup to append token 16"):
        call(T=16)
    with pytest.raises(RuntimeError, match="DIM must be 128, 256 or 512"):
        gemv.forward_qk(_h(B, nh, 1, 64), _cache(B, nh, 2, 64), _h(B, nh, 1, 64), *_p(nh, 64), 3, SMIN, SMAX)
    # everything valid but on the CPU: loud failure, no fallback
    with pytest.raises(RuntimeError, match="HIP device"):
        call()


def test_forward_ov_errors():
    B, nh, D = 1, 2, 128
    call = lambda a=None, c=None, v=None: gemv.forward_ov(
        _h(B, nh, 4) if a is None else a, _cache(B, nh, 2, D) if c is None else c,
        _h(B, nh, 1, D) if v is None else v, *_p(nh, D), SMIN, SMAX)
    with pytest.raises(RuntimeError, match="attn must be float16"):
        call(a=torch.zeros(B, nh, 4))
    with pytest.raises(RuntimeError, match="v_cache must be uint8"):
        call(c=_cache(B, nh, 2, D).float())
    with pytest.raises(RuntimeError, match="attn must contain the cached weights plus the self weight"):
        call(a=_h(B, nh, 0))
    with pytest.raises(RuntimeError, match="v_new head dimension does not match v_cache"):
        call(v=_h(B, nh, 1, 256))
    with pytest.raises(RuntimeError, match="v_cache has no free supergroup to append token 16"):
        call(a=_h(B, nh, 17))
    with pytest.raises(RuntimeError, match="HIP device"):
        call()


def test_encode_kv_errors():
    B, nh, D = 1, 2, 128
    call = lambda c=None, x=None: gemv.encode_kv(
        _cache(B, nh, 2, D) if c is None else c, _h(B, nh, 9, D) if x is None else x,
        *_p(nh, D), SMIN, SMAX)
    with pytest.raises(RuntimeError, match="kv_new must be float16"):
        call(x=torch.zeros(B, nh, 9, D))
    with pytest.raises(RuntimeError, match="kv_cache must be contiguous \\(written in place\\)"):
        call(c=_cache(B, nh, 4, D)[:, :, ::2])
    with pytest.raises(RuntimeError, match="kv_cache channel groups do not match kv_new head dim"):
        call(c=_cache(B, nh, 2, 256))
    with pytest.raises(RuntimeError,
                       match="kv_cache capacity too small: need 3 supergroups for 17 tokens, have 2"):
        call(x=_h(B, nh, 17, D))
    with pytest.raises(RuntimeError, match="HIP device"):
        call()


def test_missing_library_is_loud(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.ADKVLibraryError, match="no CPU fallback"):
        _lib.lib()
