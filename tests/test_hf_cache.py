"""Host-side cache object and HF integration (counterparts of src/adkv/hf/llama_adkv.py:44-462)."""
import math

import numpy as np
import pytest
import torch

from adkv_amd import synth
from adkv_amd.hf import cache as C
from adkv_amd.hf.cache import KVCache_ADKV, KVCacheLayer_ADKV


def _np16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.float16)


def _flat(p):
    return [t.reshape(-1) for t in p.astuple()]


# ----------------------------------------------------------------------------- CPU: host logic
def test_cache_storage_management_cpu():
    c = KVCacheLayer_ADKV()
    assert c.get_seq_length() == 0 and c.key_states is None
    c._init_buffers(2, 3, 128, torch.device("cpu"))
    assert c.key_states.shape == (2, 3, 8, 32, 4, 4) and c.key_states.dtype == torch.uint8
    assert c._cap_len == 64 and not c.key_states.any()
    c._key_buf[0, 0, 0, 0, 0, 0] = 7
    c._key_ckpt[0, 0, 0, 0, 0] = 1.5
    c._cap_buffers(64)                       # fits: nothing happens
    assert c._cap_len == 64
    c._cap_buffers(65)                       # grows geometrically, in CAP_LEN steps, keeps content
    assert c._cap_len == 128 and c.key_states.shape[2] == 16
    assert c._key_buf[0, 0, 0, 0, 0, 0] == 7 and c._key_ckpt[0, 0, 0, 0, 0] == 1.5
    assert not c._key_buf[:, :, 8:].any()    # new slots are zero (the append is a read-modify-write)
    c._cap_buffers(1000)
    assert c._cap_len == 1024 and c._key_ckpt.shape[2] == 1024 // C.CKPT_INTERVAL + 1
    assert c.get_mask_sizes(torch.arange(3)) == (3, 0)
    assert KVCacheLayer_ADKV()._n_super(0) == 0 and KVCacheLayer_ADKV()._n_super(9) == 2
    assert KVCacheLayer_ADKV(bits=2)._n_super(17) == 2


def test_cache_errors_cpu():
    p = synth.make_params(2, 128)
    kp = _flat(p)
    c = KVCacheLayer_ADKV()
    with pytest.raises(ValueError, match="head_dim in \\(128, 256, 512\\)"):
        c.prefill(torch.zeros(1, 2, 4, 64), torch.zeros(1, 2, 4, 64), *kp, *kp)
    c = KVCacheLayer_ADKV()
    with pytest.raises(ValueError, match="key/value shapes differ"):
        c.prefill(torch.zeros(1, 2, 4, 128), torch.zeros(1, 2, 5, 128), *kp, *kp)
    c.prefill(torch.zeros(1, 2, 0, 128), torch.zeros(1, 2, 0, 128), *kp, *kp)   # T == 0: allocate only
    assert c.get_seq_length() == 0 and c.key_states is not None
    with pytest.raises(ValueError, match="different \\(B, H, C\\)"):
        c.prefill(torch.zeros(2, 2, 4, 128), torch.zeros(2, 2, 4, 128), *kp, *kp)
    q = torch.zeros(1, 2, 1, 128)
    with pytest.raises(ValueError, match="exactly one query/key/value token"):
        c.decode(torch.zeros(1, 2, 2, 128), q, q, *kp, *kp)
    with pytest.raises(ValueError, match="query heads per KV head"):
        c.decode(torch.zeros(1, 6, 1, 128), q, q, *kp, *kp)     # 3 query heads per KV head
    c._quant_len, c._state_valid = 3, False      # as after decode steps: the carried state is gone
    with pytest.raises(NotImplementedError, match="chunked prefill is not supported"):
        c.prefill(torch.zeros(1, 2, 4, 128), torch.zeros(1, 2, 4, 128), *kp, *kp)
    kv = KVCache_ADKV(3)
    assert len(kv) == 3 and kv.get_seq_length(1) == 0
    # no device => loud failure from the kernel layer, never a CPU fallback
    c2 = KVCacheLayer_ADKV()
    with pytest.raises(RuntimeError, match="HIP device"):
        c2.prefill(torch.zeros(1, 2, 4, 128), torch.zeros(1, 2, 4, 128), *kp, *kp)


def test_memory_model():
    """Same accounting as tools/memory_comparison_fig.py:46-56 for B=32, T=4096, hidden 4096."""
    a = C.adkv_cache_bytes(32, 32, 128, 4096, layers=1, ckpt_interval=0)
    assert a == 2 * 32 * 4096 * 4096 // 2 + 10 * 4096 * 2
    f = C.fp16_cache_bytes(32, 32, 128, 4096, layers=1)
    assert 3.9 < f / a < 4.0
    with_ck = C.adkv_cache_bytes(32, 32, 128, 4096, layers=1, ckpt_interval=256)
    assert 1.03 < with_ck / a < 1.04


# ----------------------------------------------------------------------------- GPU
@pytest.mark.gpu
@pytest.mark.parametrize("interval", [0, 16, 256])
def test_prefill_then_decode_steps_match_oracle(gpu, oracle, monkeypatch, interval):
    """Prompt of 50 tokens, then 30 single-token steps that cross capacity growth (64 -> 128 slots)
    and several checkpoint boundaries; codes bit-exact and outputs within 2e-3 at every step."""
    monkeypatch.setattr(C, "CKPT_INTERVAL", interval)
    B, H, D, T0, steps = 2, 3, 128, 50, 30
    kp, vp = synth.make_params(H, D, seed=3), synth.make_params(H, D, seed=4)
    k = synth.make_k(B, H, T0 + steps, D, dtype=torch.float16)
    v = synth.make_v(B, H, T0 + steps, D, dtype=torch.float16)
    g = torch.Generator().manual_seed(1)
    scaling = D ** -0.5
    kpn, vpn = [_np16(t) for t in kp.astuple()], [_np16(t) for t in vp.astuple()]
    ko, vo = oracle.alloc_cache(B, H, T0 + steps + 8, D), oracle.alloc_cache(B, H, T0 + steps + 8, D)
    oracle.encode_kv_f16(ko, _np16(k)[:, :, :T0], *kpn)
    oracle.encode_kv_f16(vo, _np16(v)[:, :, :T0], *vpn)

    layer = KVCacheLayer_ADKV()
    kg, vg = _flat(kp.to(gpu)), _flat(vp.to(gpu))
    # the prompt arrives in two chunks (cut inside a supergroup)
    layer.prefill(k[:, :, :21].to(gpu), v[:, :, :21].to(gpu), *kg, *vg)
    layer.prefill(k[:, :, 21:T0].to(gpu), v[:, :, 21:T0].to(gpu), *kg, *vg)
    assert layer.get_seq_length() == T0
    for s in range(steps):
        T = T0 + s
        q = torch.randn(B, H, 1, D, generator=g).half()
        mask = None
        if s % 3 == 1:                        # additive mask that hides a few cached tokens
            mask = torch.zeros(B, 1, 1, T + 1)
            mask[:, :, :, 3:9] = float("-inf")
        out, w = layer.decode(q.to(gpu), k[:, :, T:T + 1].to(gpu), v[:, :, T:T + 1].to(gpu), *kg, *vg,
                              attention_mask=None if mask is None else mask.to(gpu), scaling=scaling)
        want, w_want, _ = oracle.decode_step_f16(_np16(q), ko, vo, _np16(k)[:, :, T:T + 1],
                                                 _np16(v)[:, :, T:T + 1], kpn, vpn, T, scaling,
                                                 mask=None if mask is None else mask[:, :, 0, :].numpy())
        assert out.shape == (B, H, D) and w.shape == (B, H, T + 1) and out.dtype == torch.float16
        assert np.max(np.abs(_np16(out).astype(np.float64) - want)) <= 2e-3, s
        assert layer.get_seq_length() == T + 1
    n = oracle.n_super(T0 + steps)
    assert np.array_equal(layer.key_states.cpu().numpy()[:, :, :n], ko[:, :, :n])
    assert np.array_equal(layer.value_states.cpu().numpy()[:, :, :n], vo[:, :, :n])
    assert layer._cap_len == 128


@pytest.mark.gpu
def test_tiny_llama_generate(gpu):
    """Random-init 2-layer Llama (2 heads of 128) decodes greedily through the ADKV cache; with
    near-lossless parameters (tiny scale) its tokens match the dense fp32 model's."""
    transformers = pytest.importorskip("transformers")
    from transformers import LlamaConfig, LlamaForCausalLM
    from adkv_amd.hf.llama_adkv import ADKVConfig, LlamaForCausalLM_ADKV

    cfg = LlamaConfig(vocab_size=128, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                      num_attention_heads=2, num_key_value_heads=2, max_position_embeddings=256,
                      attn_implementation="eager")
    torch.manual_seed(0)
    dense = LlamaForCausalLM(cfg).to(gpu).eval()
    model = LlamaForCausalLM_ADKV(cfg).to(gpu).eval()
    model.load_state_dict(dense.state_dict())
    n = 2 * 128
    # delta coding with alpha = 1 and an adaptive scale tracks smooth-ish activations closely
    mk = lambda: ADKVConfig(zp_init=torch.zeros(n), scale_init=torch.full((n,), 0.05),
                            alpha=torch.full((n,), 0.95), beta=torch.full((n,), 0.05),
                            quant_target=torch.full((n,), 3.5))
    model.load_adkv_config([(mk(), mk()) for _ in range(2)])
    ids = torch.randint(0, 128, (2, 12), generator=torch.Generator().manual_seed(3)).to(gpu)
    with torch.no_grad():
        out = model.generate(ids, max_new_tokens=8, do_sample=False)
        ref = dense.generate(ids, max_new_tokens=8, do_sample=False)
    assert out.shape == (2, 20)
    assert torch.equal(out[:, :12], ids)
    # the first generated token comes from the dense prefill path: identical by construction
    assert torch.equal(out[:, 12], ref[:, 12])


@pytest.mark.gpu
def test_tiny_llama_follow_up_chunk_equals_single_token_steps(gpu):
    """A second multi-token call on top of a cache that already holds codes (a follow-up turn):
    the module takes it as successive decode steps, so the cache ends up byte-identical to
    feeding the same tokens one call at a time and the logits agree (the projections run as one
    GEMM instead of five, hence a small tolerance)."""
    pytest.importorskip("transformers")
    from transformers import LlamaConfig
    from adkv_amd.hf.llama_adkv import ADKVConfig, LlamaForCausalLM_ADKV

    cfg = LlamaConfig(vocab_size=128, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                      num_attention_heads=2, num_key_value_heads=2, max_position_embeddings=256,
                      attn_implementation="eager")
    torch.manual_seed(0)
    model = LlamaForCausalLM_ADKV(cfg).to(gpu).half().eval()
    n = 2 * 128
    mk = lambda: ADKVConfig(zp_init=torch.zeros(n), scale_init=torch.full((n,), 0.05),
                            alpha=torch.full((n,), 0.95), beta=torch.full((n,), 0.05),
                            quant_target=torch.full((n,), 3.5))
    model.load_adkv_config([(mk(), mk()) for _ in range(2)])
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, 128, (2, 12), generator=g).to(gpu)
    more = torch.randint(0, 128, (2, 5), generator=g).to(gpu)
    with torch.no_grad():
        a = model(prompt, use_cache=True)
        chunk = model(more, past_key_values=a.past_key_values, use_cache=True)
        b = model(prompt, use_cache=True)
        singles = []
        cache = b.past_key_values
        for i in range(5):
            r = model(more[:, i:i + 1], past_key_values=cache, use_cache=True)
            cache = r.past_key_values
            singles.append(r.logits)
    assert chunk.past_key_values.get_seq_length() == 17 and cache.get_seq_length() == 17
    for la, lb in zip(chunk.past_key_values, cache):
        assert torch.equal(la._key_buf, lb._key_buf) and torch.equal(la._value_buf, lb._value_buf)
    got, want = chunk.logits.float(), torch.cat(singles, dim=1).float()
    assert got.shape == want.shape == (2, 5, 128)
    assert torch.allclose(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("interval", [0, 16])
def test_cache_save_and_restore_continues_identically(gpu, tmp_path, monkeypatch, interval):
    """A cache saved after prefill + decode steps and restored from the file continues exactly like
    the original: same outputs, same codes, same checkpoints; a cache saved right after prefill
    also keeps its carried state and accepts another prompt chunk."""
    monkeypatch.setattr(C, "CKPT_INTERVAL", interval)
    B, H, D, T0 = 2, 2, 128, 41
    kp, vp = synth.make_params(H, D, seed=3), synth.make_params(H, D, seed=4)
    kg, vg = _flat(kp.to(gpu)), _flat(vp.to(gpu))
    k = synth.make_k(B, H, T0 + 40, D, dtype=torch.float16).to(gpu)
    v = synth.make_v(B, H, T0 + 40, D, dtype=torch.float16).to(gpu)
    q = torch.randn(B, H, 1, D, generator=torch.Generator().manual_seed(5)).half().to(gpu)

    def step(layer, t):
        return layer.decode(q, k[:, :, t:t + 1], v[:, :, t:t + 1], *kg, *vg, scaling=D ** -0.5)

    cache = KVCache_ADKV(1)
    cache[0].prefill(k[:, :, :T0], v[:, :, :T0], *kg, *vg)
    cache.save(tmp_path / "prefill.pt")
    for t in range(T0, T0 + 3):
        step(cache[0], t)
    cache.save(tmp_path / "decoded.pt")

    again = KVCache_ADKV.load(tmp_path / "decoded.pt", gpu)
    assert again[0].get_seq_length() == T0 + 3 and not again[0]._state_valid
    for t in range(T0 + 3, T0 + 30):              # crosses capacity growth in both
        o1, w1 = step(cache[0], t)
        o2, w2 = step(again[0], t)
        assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))
        assert torch.equal(w1.view(torch.int16), w2.view(torch.int16))
    n = cache[0]._n_super(T0 + 30)
    assert torch.equal(cache[0].key_states[:, :, :n], again[0].key_states[:, :, :n])
    assert torch.equal(cache[0].value_states[:, :, :n], again[0].value_states[:, :, :n])
    with pytest.raises(NotImplementedError):
        again[0].prefill(k[:, :, :4], v[:, :, :4], *kg, *vg)

    # restored right after prefill: the carried state survives, so a second chunk is accepted
    chunked = KVCache_ADKV.load(tmp_path / "prefill.pt", gpu)
    chunked[0].prefill(k[:, :, T0:T0 + 9], v[:, :, T0:T0 + 9], *kg, *vg)
    whole = KVCacheLayer_ADKV()
    whole.prefill(k[:, :, :T0 + 9], v[:, :, :T0 + 9], *kg, *vg)
    n = whole._n_super(T0 + 9)
    assert torch.equal(chunked[0].key_states[:, :, :n], whole.key_states[:, :, :n])
    assert torch.equal(chunked[0].value_states[:, :, :n], whole.value_states[:, :, :n])


@pytest.mark.gpu
@pytest.mark.parametrize("bits,G,dtype", [(2, 1, torch.float16), (4, 4, torch.bfloat16), (2, 4, torch.bfloat16)])
def test_cache_layer_grouped_queries_two_bit_and_bf16(gpu, oracle, bits, G, dtype):
    """The cache object with 2-bit codes, 4 query heads per KV head and bf16 activations: prompt in
    two chunks, then steps across a capacity growth; codes bit-exact, outputs within 2e-3 of the
    oracle evaluated per query head (query head j reads KV head j // G)."""
    B, H, D, T0, steps = 2, 2, 128, 45, 25
    Hq = H * G
    kp, vp = synth.make_params(H, D, bits=bits, seed=3), synth.make_params(H, D, bits=bits, seed=4)
    k = synth.make_k(B, H, T0 + steps, D, dtype=torch.float16)
    v = synth.make_v(B, H, T0 + steps, D, dtype=torch.float16)
    if dtype == torch.bfloat16:          # values a bf16 model would hand over: exact in fp16 as well
        k, v = k.to(dtype).to(torch.float16), v.to(dtype).to(torch.float16)
    gq = torch.Generator().manual_seed(2)
    scaling = D ** -0.5
    kpn, vpn = [_np16(t) for t in kp.astuple()], [_np16(t) for t in vp.astuple()]
    layer = KVCacheLayer_ADKV(bits=bits)
    kg, vg = _flat(kp.to(gpu)), _flat(vp.to(gpu))
    layer.prefill(k[:, :, :19].to(gpu).to(dtype), v[:, :, :19].to(gpu).to(dtype), *kg, *vg)
    layer.prefill(k[:, :, 19:T0].to(gpu).to(dtype), v[:, :, 19:T0].to(gpu).to(dtype), *kg, *vg)
    with oracle.code_bits(bits):
        ko, vo = oracle.alloc_cache(B, H, T0 + steps + 16, D), oracle.alloc_cache(B, H, T0 + steps + 16, D)
        oracle.encode_kv_f16(ko, _np16(k)[:, :, :T0], *kpn)
        oracle.encode_kv_f16(vo, _np16(v)[:, :, :T0], *vpn)
        for s in range(steps):
            T = T0 + s
            q = torch.randn(B, Hq, 1, D, generator=gq).to(dtype)
            out, w = layer.decode(q.to(gpu), k[:, :, T:T + 1].to(gpu).to(dtype), v[:, :, T:T + 1].to(gpu).to(dtype),
                                  *kg, *vg, scaling=scaling)
            assert out.dtype == dtype and out.shape == (B, Hq, D) and w.shape == (B, Hq, T + 1)
            qn = _np16(q.to(torch.float16)).reshape(B, H, G, D)
            got = out.float().cpu().numpy().reshape(B, H, G, D)
            for j in range(G):
                kc, vc = ko.copy(), vo.copy()
                want, _, _ = oracle.decode_step_f16(qn[:, :, j], kc, vc, _np16(k)[:, :, T:T + 1],
                                                    _np16(v)[:, :, T:T + 1], kpn, vpn, T, scaling)
                tol = 2e-3 if dtype == torch.float16 else 2e-3 + 2.0 ** -8 * np.abs(want)
                assert np.all(np.abs(got[:, :, j] - want) <= tol), (s, j)
            ko, vo = kc, vc
        n = oracle.n_super(T0 + steps)
    assert np.array_equal(layer.key_states.cpu().numpy()[:, :, :n], ko[:, :, :n])
    assert np.array_equal(layer.value_states.cpu().numpy()[:, :, :n], vo[:, :, :n])
