"""Oracle and GPU kernels against tests/golden/kat_fp16.json, the exact-rational known-answer
vectors of the fp16 recurrence (made by tests/golden/make_fp16_kat.py from the step definitions of
src/adkv/kernel/gemv.cu:150-164, 220-221 and the layout of src/adkv/hf/llama_adkv.py:47-55)."""
import ctypes as C
import json
import os

import numpy as np
import pytest

KAT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kat_fp16.json")


@pytest.fixture(scope="module")
def kat():
    with open(KAT) as f:
        return json.load(f)


def test_update_vectors(oracle, kat):
    L = oracle.lib()
    assert len(kat["update"]) == 400
    for q, zp, sc, al, be, tg, omt, nzp, nsc, kh in kat["update"]:
        assert L.adkv_o_omt_f16(be, tg) == omt
        z, s = C.c_uint16(zp), C.c_uint16(sc)
        L.adkv_o_update_f16(q, C.byref(z), C.byref(s), al, be, omt)
        assert (z.value, s.value) == (nzp, nsc)
        assert L.adkv_o_dequant2_f16(q, zp, sc) == kh


def test_quantize_vectors(oracle, kat):
    L = oracle.lib()
    for bits in (4, 2):
        with oracle.code_bits(bits):
            rows = [r for r in kat["quantize"] if r[0] == bits]
            assert len(rows) == 220
            for _, x, zp, sc, want in rows:
                assert L.adkv_o_quantize_f16(x, zp, sc) == want


def _arrays(s):
    D, T = s["D"], s["T"]
    par = [np.array(p, np.uint16).reshape(1, D) for p in s["params"]]
    x = np.array(s["x"], np.uint16).reshape(1, 1, T, D)
    packed = np.frombuffer(bytes.fromhex(s["packed_hex"]), np.uint8)
    state = np.array(s["state"], np.uint16).reshape(1, 1, D, 2)
    return par, x, packed, state


def test_sequences_oracle(oracle, kat):
    for s in kat["sequences"]:
        par, x, packed, state = _arrays(s)
        with oracle.code_bits(s["bits"]):
            cache = oracle.alloc_cache(1, 1, s["T"], s["D"])
            st = oracle.encode_kv_f16(cache, x.view(np.float16), *[p.view(np.float16) for p in par])
            assert np.array_equal(cache.reshape(-1), packed)
            assert np.array_equal(st, state)
            assert np.array_equal(oracle.unpack_codes(cache, s["T"])[0, 0], np.array(s["codes"], np.int8))
            khat, _ = oracle.replay_f16(cache, *[p.view(np.float16) for p in par], s["T"])
            assert np.array_equal(khat.view(np.uint16)[0, 0], np.array(s["dequant"], np.uint16))


@pytest.mark.gpu
def test_sequences_gpu(gpu, kat):
    """The GPU encoder writes the fixture's bytes and final state; the decode kernels, given a
    one-hot query / weight, return the fixture's dequantised values."""
    import torch
    from adkv_amd import synth
    from adkv_amd.kernel import gemv
    for s in kat["sequences"]:
        if s["bits"] == 2 and s["D"] != 128:
            continue
        par, x, packed, state = _arrays(s)
        T, D, bits = s["T"], s["D"], s["bits"]
        tps = 32 // bits
        f16 = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.float16).to(gpu)
        pg = [f16(p) for p in par]
        cache = synth.alloc_cache(1, 1, T + tps, D, gpu, bits=bits)
        st = torch.zeros(1, 1, D, 2, dtype=torch.float16, device=gpu)
        gemv.append_kv(cache, f16(x), *pg, 0, st, bits=bits)
        torch.cuda.synchronize()
        n = len(packed)
        assert np.array_equal(cache.cpu().numpy().reshape(-1)[:n], packed)
        assert np.array_equal(st.cpu().view(torch.int16).numpy().view(np.uint16), state)
        # logits with q = e_c pick channel c of every dequantised token
        deq = np.array(s["dequant"], np.uint16).view(np.float16).astype(np.float32)      # [T, D]
        for c in (0, 5, D - 1):
            q = torch.zeros(1, 1, 1, D, dtype=torch.float16, device=gpu)
            q[..., c] = 1.0
            kc = cache.clone()
            logits = gemv.forward_qk(q, kc, f16(x)[:, :, :1], *pg, T, 0.0, 1.0, bits=bits)
            got = logits[0, 0, :T].float().cpu().numpy()
            assert np.array_equal(got, deq[:, c]), c
