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


def _tiny_cfg(heads, kv_heads):
    from transformers import LlamaConfig
    return LlamaConfig(vocab_size=128, hidden_size=128 * heads, intermediate_size=512, num_hidden_layers=2,
                       num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=128,
                       max_position_embeddings=256, attn_implementation="eager")


def _rope(x, cos, sin):
    """Rotary embedding written out (x [B, H, T, d]; cos, sin [B, T, d]): the textbook form,
    x*cos + rotate_half(x)*sin with rotate_half(x) = (-x[d/2:], x[:d/2])."""
    d = x.shape[-1]
    rot = torch.cat((-x[..., d // 2:], x[..., :d // 2]), dim=-1)
    return x * cos[:, None] + rot * sin[:, None]


class _AttentionTap:
    """Records, for every call of every attention module, what went in (hidden states, rotary
    tables, mask) and what reached o_proj, so a test can recompute the step without the module."""

    def __init__(self, model):
        self.calls = []            # dicts: layer, hidden, cos, sin, mask, ctx (input of o_proj), out
        self.cache = None          # the cache object the model made for itself
        self._handles = []
        for i, layer in enumerate(model.model.layers):
            att = layer.self_attn
            self._handles.append(att.register_forward_pre_hook(self._pre(i), with_kwargs=True))
            self._handles.append(att.o_proj.register_forward_pre_hook(self._ctx))
            self._handles.append(att.register_forward_hook(self._post))

    def _pre(self, i):
        def hook(mod, args, kwargs):
            cos, sin = kwargs["position_embeddings"]
            m = kwargs.get("attention_mask")
            self.cache = kwargs.get("past_key_values")
            self.calls.append(dict(layer=i, hidden=kwargs["hidden_states"].detach().clone(),
                                   cos=cos.detach().clone(), sin=sin.detach().clone(),
                                   mask=None if m is None else m.detach().clone()))
        return hook

    def _ctx(self, mod, args):
        self.calls[-1]["ctx"] = args[0].detach().clone()

    def _post(self, mod, args, out):
        self.calls[-1]["out"] = out[0].detach().clone()

    def close(self):
        for h in self._handles:
            h.remove()


def _check_decode_calls_against_oracle(oracle, model, calls, params16, pad, prompt_len):
    """Every single-token call of every attention module, recomputed from the hidden states that
    entered it: projections and rotary embedding here, quantised attention by the oracle (its own
    caches, filled from the prompt call's K/V), query head j reading KV head j // G, scaling
    head_dim**-0.5, the additive mask rebuilt from the known left padding.  The context that
    reached o_proj must agree within 2e-3 and the module's output with o_proj of the oracle's."""
    cfg = model.config
    Hq, H, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    G = Hq // H
    scaling = D ** -0.5
    caches, T = {}, {}
    worst = 0.0
    n_decode = 0
    for c in calls:
        att = model.model.layers[c["layer"]].self_attn
        hs = c["hidden"].float()
        B, Tq, _ = hs.shape
        w = lambda lin: lin.weight.detach().float()
        split = lambda x, n: x.view(B, Tq, n, D).transpose(1, 2)
        q = _rope(split(hs @ w(att.q_proj).T, Hq), c["cos"].float(), c["sin"].float())
        k = _rope(split(hs @ w(att.k_proj).T, H), c["cos"].float(), c["sin"].float())
        v = split(hs @ w(att.v_proj).T, H)
        kpn, vpn = params16[c["layer"]]
        if c["layer"] not in caches:                       # the prompt: quantise, nothing to compare
            assert Tq == prompt_len
            ko = oracle.alloc_cache(B, H, 256, D)
            vo = oracle.alloc_cache(B, H, 256, D)
            oracle.encode_kv_f16(ko, _np16(k.half()), *kpn)
            oracle.encode_kv_f16(vo, _np16(v.half()), *vpn)
            caches[c["layer"]], T[c["layer"]] = (ko, vo), Tq
            continue
        assert Tq == 1
        ko, vo = caches[c["layer"]]
        t = T[c["layer"]]
        mask = np.zeros((B, 1, t + 1), np.float32)
        for b in range(B):
            mask[b, 0, :pad[b]] = -np.inf
        ctx = np.zeros((B, Hq, D))
        qn = _np16(q.half()).reshape(B, H, G, D)
        for j in range(G):                                  # query head h*G + j reads KV head h
            kc, vc = ko.copy(), vo.copy()
            o, _, _ = oracle.decode_step_f16(qn[:, :, j], kc, vc, _np16(k.half()), _np16(v.half()),
                                             kpn, vpn, t, scaling, mask=mask)
            ctx.reshape(B, H, G, D)[:, :, j] = o
        caches[c["layer"]], T[c["layer"]] = (kc, vc), t + 1
        got_ctx = c["ctx"].float().cpu().numpy().reshape(B, Hq, D)
        err = float(np.max(np.abs(got_ctx - ctx)))
        worst = max(worst, err)
        assert err <= 2e-3, (c["layer"], t, err)
        want_out = torch.from_numpy(ctx.reshape(B, 1, Hq * D)).float().to(hs.device) @ w(att.o_proj).T
        assert torch.allclose(c["out"].float(), want_out, atol=2e-3, rtol=0), (c["layer"], t)
        n_decode += 1
    return caches, T, worst, n_decode


def _reference_greedy(oracle, dense, params16, ids, amask, pad, new):
    """Greedy decoding of the tiny Llama written out layer by layer from the dense model's weights
    (fp32): the prompt with ordinary causal attention, every later token with the oracle's quantised
    decode attention over its own caches.  Shares no code with the ADKV modules or the cache object.
    Returns (tokens [B, new], logits of each step [new][B, V])."""
    cfg = dense.config
    Hq, H, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    G, scaling = Hq // H, D ** -0.5
    m = dense.model
    B, P = ids.shape
    dev = ids.device
    pos = (amask.long().cumsum(-1) - 1).masked_fill(amask == 0, 1)        # positions skip the padding
    caches = [None] * len(m.layers)
    toks, step_logits = [], []
    cur, cur_pos, t = ids, pos, P
    for step in range(new):
        h = m.embed_tokens(cur)
        cos, sin = m.rotary_emb(h, cur_pos)
        Tq = cur.shape[1]
        for L, layer in enumerate(m.layers):
            att = layer.self_attn
            x = layer.input_layernorm(h)
            split = lambda y, n: y.view(B, Tq, n, D).transpose(1, 2)
            q = _rope(split(att.q_proj(x), Hq), cos, sin)
            k = _rope(split(att.k_proj(x), H), cos, sin)
            v = split(att.v_proj(x), H)
            kpn, vpn = params16[L]
            if step == 0:
                ko, vo = oracle.alloc_cache(B, H, 256, D), oracle.alloc_cache(B, H, 256, D)
                oracle.encode_kv_f16(ko, _np16(k.half()), *kpn)
                oracle.encode_kv_f16(vo, _np16(v.half()), *vpn)
                caches[L] = (ko, vo)
                kr, vr = k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1)
                sc = torch.matmul(q, kr.transpose(2, 3)) * scaling
                allow = torch.tril(torch.ones(P, P, dtype=torch.bool, device=dev))[None, None] \
                    & (amask[:, None, None, :] != 0)
                sc = sc.masked_fill(~allow, float("-inf"))
                # a padded query row sees nothing; its output is never used, keep it finite
                sc = torch.where(allow.any(-1, keepdim=True), sc, torch.zeros_like(sc))
                ctx = torch.matmul(torch.softmax(sc, dim=-1), vr)
            else:
                mask = np.zeros((B, 1, t + 1), np.float32)
                for b in range(B):
                    mask[b, 0, :pad[b]] = -np.inf
                ko, vo = caches[L]
                qn = _np16(q.half()).reshape(B, H, G, D)
                out = np.zeros((B, H, G, D))
                for j in range(G):
                    kc, vc = ko.copy(), vo.copy()
                    o, _, _ = oracle.decode_step_f16(qn[:, :, j], kc, vc, _np16(k.half()), _np16(v.half()),
                                                     kpn, vpn, t, scaling, mask=mask)
                    out[:, :, j] = o
                caches[L] = (kc, vc)
                ctx = torch.from_numpy(out.reshape(B, Hq, 1, D)).float().to(dev)
            h = h + att.o_proj(ctx.transpose(1, 2).reshape(B, Tq, Hq * D))
            h = h + layer.mlp(layer.post_attention_layernorm(h))
        logits = dense.lm_head(m.norm(h))[:, -1]
        step_logits.append(logits)
        nxt = logits.argmax(-1)
        toks.append(nxt)
        if step > 0:
            t += 1
        cur = nxt[:, None]
        cur_pos = cur_pos[:, -1:] + 1
    return torch.stack(toks, dim=1), step_logits


def _tiny_raw_calibration(layers, n, seed):
    """Raw (unconstrained) calibration parameters as the reference's trainer stores them."""
    g = torch.Generator().manual_seed(seed)
    mk = lambda: {"init_zp": 0.05 * torch.randn(n, generator=g),
                  "init_log_sc": math.log(0.03) + 0.2 * torch.randn(n, generator=g),
                  "alpha": 2.5 + 0.5 * torch.randn(n, generator=g),       # sigmoid -> ~0.92
                  "beta": -0.5 + 0.5 * torch.randn(n, generator=g),       # 0.1*sigmoid -> ~0.04
                  "target": 3.5 + 0.1 * torch.randn(n, generator=g)}
    return [(mk(), mk()) for _ in range(layers)]


def _deployment_params16(raw, H, D):
    """exp / sigmoid / 0.1*sigmoid of the raw values (train_model.py:127-134) in numpy, rounded to
    fp16 as the module's fp16 buffers do: what the oracle is fed."""
    out = []
    for pair in raw:
        both = []
        for sd in pair:
            f = {k: v.numpy().astype(np.float32) for k, v in sd.items()}
            sig = lambda a: (1.0 / (1.0 + np.exp(-a.astype(np.float64)))).astype(np.float32)
            vals = (f["init_zp"], np.exp(f["init_log_sc"].astype(np.float64)).astype(np.float32),
                    sig(f["alpha"]), (0.1 * sig(f["beta"]).astype(np.float64)).astype(np.float32), f["target"])
            both.append([a.astype(np.float16).reshape(H, D) for a in vals])
        out.append(tuple(both))
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("heads,kv_heads", [(2, 2), (4, 2)])
def test_tiny_llama_decode_path_matches_oracle_and_dense_model(gpu, oracle, tmp_path, heads, kv_heads):
    """Random-init 2-layer Llama, a left-padded batch of two prompts, 8 greedy steps through the
    ADKV cache with parameters read from calibration files (ckpt_{k,v}_{L}.pt -> load_calibration
    -> load_adkv_config, the route of tools/perf_e2e.py:37-60).  Every decode-path call of every
    attention module is recomputed with the oracle (see _check_decode_calls_against_oracle); the
    packed caches at the end are the oracle's byte for byte; and all generated tokens and the
    logits behind them equal those of a greedy loop written out in the test from the dense
    model's weights with the oracle as its decode attention (_reference_greedy).  The first
    token, which comes from the dense prompt pass, is also the dense model's; later ones need not
    be: 4-bit K/V codes perturb a random-init model's near-flat logits enough to change an argmax."""
    pytest.importorskip("transformers")
    from transformers import LlamaForCausalLM
    from adkv_amd import calib
    from adkv_amd.hf.llama_adkv import LlamaForCausalLM_ADKV

    cfg = _tiny_cfg(heads, kv_heads)
    torch.manual_seed(0)
    dense = LlamaForCausalLM(cfg).to(gpu).eval()
    model = LlamaForCausalLM_ADKV(cfg).to(gpu).eval()
    model.load_state_dict(dense.state_dict())
    H, D = kv_heads, 128
    raw = _tiny_raw_calibration(2, H * D, seed=11)
    calib.save_calibration(tmp_path, raw)
    model.load_adkv_config(calib.load_calibration(tmp_path, 2, hidden_size=H * D))
    params16 = _deployment_params16(raw, H, D)
    for L, layer in enumerate(model.model.layers):          # the buffers hold exactly those fp16 values
        for side, pn in zip(("key", "value"), params16[L]):
            for name, a in zip(("zp_init", "scale_init", "alpha", "beta", "quant_target"), pn):
                assert np.array_equal(_np16(getattr(layer.self_attn, f"{side}_{name}")).view(np.uint16),
                                      a.reshape(-1).view(np.uint16)), (L, side, name)

    P, new = 12, 8
    pad = [0, 3]                                             # the second prompt is 3 tokens shorter
    ids = torch.randint(1, 128, (2, P), generator=torch.Generator().manual_seed(3))
    amask = torch.ones(2, P, dtype=torch.long)
    for b, n in enumerate(pad):
        ids[b, :n] = 0
        amask[b, :n] = 0
    ids, amask = ids.to(gpu), amask.to(gpu)
    tap = _AttentionTap(model)
    with torch.no_grad():
        gen = model.generate(ids, attention_mask=amask, max_new_tokens=new, do_sample=False, pad_token_id=0,
                             output_logits=True, return_dict_in_generate=True)
        out = gen.sequences
        tap.close()
        ref = dense.generate(ids, attention_mask=amask, max_new_tokens=new, do_sample=False, pad_token_id=0)
        want_toks, want_logits = _reference_greedy(oracle, dense, params16, ids, amask, pad, new)
    assert out.shape == (2, P + new) and torch.equal(out[:, :P], ids)
    caches, T, worst, n_decode = _check_decode_calls_against_oracle(oracle, model, tap.calls, params16, pad, P)
    assert n_decode == 2 * (new - 1) and all(t == P + new - 1 for t in T.values())
    cache = tap.cache                                      # the cache generate() worked on
    assert cache is not None and cache.get_seq_length() == P + new - 1
    n = oracle.n_super(P + new - 1)
    for L in range(2):
        assert np.array_equal(cache[L].key_states.cpu().numpy()[:, :, :n], caches[L][0][:, :, :n]), L
        assert np.array_equal(cache[L].value_states.cpu().numpy()[:, :, :n], caches[L][1][:, :, :n]), L
    assert torch.equal(out[:, P], ref[:, P])               # the dense prompt pass decides the first token
    assert torch.equal(out[:, P:], want_toks), (out[:, P:].tolist(), want_toks.tolist())
    # Across layers the two runs drift a little apart: a context vector that differs in its last
    # bits can move a K/V value of the next layer across a rounding boundary of the quantiser, so
    # whole-model logits get a looser bound than the 2e-3 each layer meets on its own inputs.
    for i, (got, want) in enumerate(zip(gen.logits, want_logits)):
        err = float((got.float() - want.float()).abs().max())
        assert err <= 2e-2, (i, err)


def _check_decode_calls_in_model_dtype(oracle, model, calls, params16, pad, prompt_len):
    """_check_decode_calls_against_oracle for a model whose weights are fp16 or bf16: the
    projections are the module's own linear layers applied to the recorded hidden states and the
    rotary embedding is the textbook expression evaluated in the model's dtype (each product and
    the sum rounded to that dtype, as torch's elementwise kernels do), so q, k and v carry exactly
    the bits the module hands to its cache; they are rounded to fp16 (a no-op for an fp16 model,
    torch's .to(float16) for a bf16 one: llama_adkv.py:248-250) and given to the oracle.
    Tolerance on the context that reached o_proj: 2e-3, plus half a bf16 ulp of the value for a
    bf16 model (the kernel's fp16 result is rounded to bf16 on the way out, llama_adkv.py:274)."""
    cfg = model.config
    Hq, H, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    G = Hq // H
    scaling = D ** -0.5
    dt = model.dtype
    caches, T = {}, {}
    n_decode = 0
    for c in calls:
        att = model.model.layers[c["layer"]].self_attn
        hs = c["hidden"]
        assert hs.dtype == dt
        B, Tq, _ = hs.shape
        split = lambda x, n: x.view(B, Tq, n, D).transpose(1, 2)
        with torch.no_grad():
            q = _rope(split(att.q_proj(hs), Hq), c["cos"], c["sin"])
            k = _rope(split(att.k_proj(hs), H), c["cos"], c["sin"])
            v = split(att.v_proj(hs), H)
        assert q.dtype == dt and k.dtype == dt
        q16, k16, v16 = (_np16(t.to(torch.float16)) for t in (q, k, v))
        kpn, vpn = params16[c["layer"]]
        if c["layer"] not in caches:
            assert Tq == prompt_len
            ko = oracle.alloc_cache(B, H, 256, D)
            vo = oracle.alloc_cache(B, H, 256, D)
            oracle.encode_kv_f16(ko, k16, *kpn)
            oracle.encode_kv_f16(vo, v16, *vpn)
            caches[c["layer"]], T[c["layer"]] = (ko, vo), Tq
            continue
        assert Tq == 1
        ko, vo = caches[c["layer"]]
        t = T[c["layer"]]
        mask = np.zeros((B, 1, t + 1), np.float32)
        for b in range(B):
            mask[b, 0, :pad[b]] = -np.inf
        ctx = np.zeros((B, Hq, D))
        qn = q16.reshape(B, H, G, D)
        for j in range(G):
            kc, vc = ko.copy(), vo.copy()
            o, _, _ = oracle.decode_step_f16(qn[:, :, j], kc, vc, k16, v16, kpn, vpn, t, scaling, mask=mask)
            ctx.reshape(B, H, G, D)[:, :, j] = o
        caches[c["layer"]], T[c["layer"]] = (kc, vc), t + 1
        got_ctx = c["ctx"].float().cpu().numpy().reshape(B, Hq, D)
        tol = 2e-3 + (2.0 ** -9 * np.abs(ctx) if dt == torch.bfloat16 else 0.0)
        assert np.all(np.abs(got_ctx - ctx) <= tol), (c["layer"], t, float(np.max(np.abs(got_ctx - ctx))))
        want_out = torch.from_numpy(ctx.reshape(B, 1, Hq * D)).float().to(hs.device) @ att.o_proj.weight.detach().float().T
        assert torch.allclose(c["out"].float(), want_out, atol=5e-3, rtol=2.0 ** -7), (c["layer"], t)
        n_decode += 1
    return caches, T, n_decode


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,heads,kv_heads", [(torch.float16, 2, 2), (torch.float16, 4, 2),
                                                  (torch.bfloat16, 2, 2)])
def test_tiny_llama_half_precision_decode_path_matches_oracle(gpu, oracle, tmp_path, monkeypatch, dtype,
                                                              heads, kv_heads):
    """The attention module on the route a half-precision model takes: the one-launch rotary
    embedding (adkv_rope_qk) and the branch of KVCacheLayer_ADKV.decode that hands q, k, v to the
    kernels without a conversion.  Same tiny random-init Llama, left-padded batch and calibration
    files as the fp32 test above; every decode call of every attention module is recomputed from
    its input hidden states with the oracle as the attention, and the packed caches at the end
    are the oracle's byte for byte."""
    pytest.importorskip("transformers")
    from adkv_amd import calib
    from adkv_amd.hf import llama_adkv as M

    cfg = _tiny_cfg(heads, kv_heads)
    torch.manual_seed(0)
    model = M.LlamaForCausalLM_ADKV(cfg).to(gpu).to(dtype).eval()
    H, D = kv_heads, 128
    raw = _tiny_raw_calibration(2, H * D, seed=11)
    calib.save_calibration(tmp_path, raw)
    model.load_adkv_config(calib.load_calibration(tmp_path, 2, hidden_size=H * D))
    params16 = _deployment_params16(raw, H, D)

    fused_calls = []
    real_rope = M.rope_qk
    monkeypatch.setattr(M, "rope_qk", lambda *a, **k: (fused_calls.append(1), real_rope(*a, **k))[1])

    P, new = 12, 8
    pad = [0, 3]
    ids = torch.randint(1, 128, (2, P), generator=torch.Generator().manual_seed(3))
    amask = torch.ones(2, P, dtype=torch.long)
    for b, n in enumerate(pad):
        ids[b, :n] = 0
        amask[b, :n] = 0
    ids, amask = ids.to(gpu), amask.to(gpu)
    tap = _AttentionTap(model)
    with torch.no_grad():
        out = model.generate(ids, attention_mask=amask, max_new_tokens=new, do_sample=False, pad_token_id=0)
    tap.close()
    assert out.shape == (2, P + new)
    assert len(fused_calls) == 2 * new                   # every attention call took the fused rotary embedding
    caches, T, n_decode = _check_decode_calls_in_model_dtype(oracle, model, tap.calls, params16, pad, P)
    assert n_decode == 2 * (new - 1) and all(t == P + new - 1 for t in T.values())
    cache = tap.cache
    assert cache is not None and cache.get_seq_length() == P + new - 1
    n = oracle.n_super(P + new - 1)
    for L in range(2):
        assert np.array_equal(cache[L].key_states.cpu().numpy()[:, :, :n], caches[L][0][:, :, :n]), L
        assert np.array_equal(cache[L].value_states.cpu().numpy()[:, :, :n], caches[L][1][:, :, :n]), L


def test_parameter_buffers_stay_fp16_when_the_model_changes_dtype():
    """model.to(torch.bfloat16) casts floating-point buffers; the ten ADKV parameter buffers of an
    attention module must keep fp16 and their exact values (the kernels take fp16 parameters only,
    and bfloat16 would drop three mantissa bits of a calibrated value)."""
    pytest.importorskip("transformers")
    from adkv_amd.hf.llama_adkv import LlamaForCausalLM_ADKV
    model = LlamaForCausalLM_ADKV(_tiny_cfg(2, 2))
    att = model.model.layers[0].self_attn
    att.key_alpha.fill_(0.9501953125)            # not representable in bfloat16
    att.value_beta.fill_(0.0400390625)
    model = model.to(torch.bfloat16)
    assert att.q_proj.weight.dtype == torch.bfloat16
    assert att.key_alpha.dtype == torch.float16 and float(att.key_alpha[0]) == 0.9501953125
    model = model.float().half()
    assert att.value_beta.dtype == torch.float16 and float(att.value_beta[3]) == 0.0400390625


def test_rotary_embedding_keeps_gradients(monkeypatch):
    """Under autograd the attention module must not take the fused rotary-embedding kernel (it has
    no backward pass): the differentiable expression runs and q_proj / k_proj receive gradients.
    Checked on the CPU by making the fused path look eligible and failing the test if it is called."""
    pytest.importorskip("transformers")
    from adkv_amd.hf import llama_adkv as M

    def boom(*a, **k):
        raise AssertionError("fused rotary embedding called while gradients are recorded")

    monkeypatch.setattr(M, "rope_qk", boom)
    cfg = _tiny_cfg(2, 2)
    torch.manual_seed(0)
    model = M.LlamaForCausalLM_ADKV(cfg).to(torch.bfloat16).train()
    att = model.model.layers[0].self_attn

    ids = torch.randint(1, 128, (1, 6))
    # `is_cuda` decides the branch; pretend the projections live on a GPU for that test only
    real_forward = M.LlamaAttention_ADKV.forward
    seen = []

    def forward(self, hidden_states, *a, **k):
        seen.append(torch.is_grad_enabled() and hidden_states.requires_grad)
        return real_forward(self, hidden_states, *a, **k)

    monkeypatch.setattr(M.LlamaAttention_ADKV, "forward", forward)
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: True))
    try:
        loss = model(ids, use_cache=False).logits.float().pow(2).mean()
    finally:
        monkeypatch.undo()
    loss.backward()
    assert seen and all(seen)
    for lin in (att.q_proj, att.k_proj, att.v_proj, att.o_proj):
        assert lin.weight.grad is not None and float(lin.weight.grad.float().abs().sum()) > 0.0


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


def test_batch_views_share_storage_cpu():
    c = KVCache_ADKV(2)
    c.reserve(6, 2, 128, 300, "cpu")
    assert c[0]._cap_len == 320 and c[1].key_states.shape == (6, 2, 40, 32, 4, 4)
    v = c.batch_view(2, 5)
    assert len(v) == 2 and v[0].key_states.shape[0] == 3 and v[0].key_states.is_contiguous()
    v[1]._key_buf[0, 0, 0, 0, 0, 0] = 9
    v[1]._key_state[1, 1, 7, 0] = 2.5
    assert c[1]._key_buf[2, 0, 0, 0, 0, 0] == 9 and c[1]._key_state[3, 1, 7, 0] == 2.5
    with pytest.raises(RuntimeError, match="cannot grow"):
        v[0]._cap_buffers(1000)
    with pytest.raises(ValueError, match="inside its batch"):
        c[0].batch_view(4, 7)
    c.commit(10)
    assert c.get_seq_length() == 10
    with pytest.raises(ValueError, match="more tokens"):
        c[0].commit(1000)


@pytest.mark.gpu
def test_prompt_in_batch_slices_equals_one_prefill(gpu):
    """A cache reserved for the whole batch and filled through batch views, slice by slice, holds
    the same codes, checkpoints and carried state as one prefill of the whole batch, and decodes
    to the same outputs."""
    B, H, D, T0 = 5, 2, 128, 300
    kp, vp = synth.make_params(H, D, seed=3), synth.make_params(H, D, seed=4)
    kg, vg = _flat(kp.to(gpu)), _flat(vp.to(gpu))
    k = synth.make_k(B, H, T0 + 1, D, dtype=torch.float16).to(gpu)
    v = synth.make_v(B, H, T0 + 1, D, dtype=torch.float16).to(gpu)
    whole = KVCacheLayer_ADKV()
    whole.prefill(k[:, :, :T0], v[:, :, :T0], *kg, *vg)
    sliced = KVCacheLayer_ADKV()
    sliced.reserve(B, H, D, T0 + 8, gpu)
    for b0, b1 in ((0, 2), (2, 5)):
        sliced.batch_view(b0, b1).prefill(k[b0:b1, :, :T0], v[b0:b1, :, :T0], *kg, *vg)
    sliced.commit(T0)
    n = whole._n_super(T0)
    assert torch.equal(sliced.key_states[:, :, :n], whole.key_states[:, :, :n])
    assert torch.equal(sliced.value_states[:, :, :n], whole.value_states[:, :, :n])
    nck = T0 // C.CKPT_INTERVAL
    assert torch.equal(sliced._key_ckpt[:, :, :nck].view(torch.int16), whole._key_ckpt[:, :, :nck].view(torch.int16))
    assert torch.equal(sliced._key_state.view(torch.int16), whole._key_state.view(torch.int16))
    q = torch.randn(B, H, 1, D, generator=torch.Generator().manual_seed(5)).half().to(gpu)
    o1, _ = whole.decode(q, k[:, :, T0:], v[:, :, T0:], *kg, *vg, scaling=D ** -0.5)
    o2, _ = sliced.decode(q, k[:, :, T0:], v[:, :, T0:], *kg, *vg, scaling=D ** -0.5)
    assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))


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


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,Hq,H,T,D,shared_table", [(3, 4, 2, 1, 128, False), (2, 8, 8, 5, 64, True),
                                                     (1, 2, 1, 33, 256, False), (130, 32, 32, 1, 128, False),
                                                     (1, 1, 1, 65537, 8, True)])
def test_rope_equals_transformers_bit_for_bit(gpu, dtype, B, Hq, H, T, D, shared_table):
    """The one-launch rotary embedding returns the very bits of transformers' apply_rotary_pos_emb
    (what the reference's attention module calls, llama_adkv.py:336-337) on the same device and
    type: projection-shaped inputs read through their head-first views, values spread over the
    type's range so that products land on rounding ties, small and subnormal results included."""
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb
    from adkv_amd.kernel import gemv
    g = torch.Generator().manual_seed(B * 1000 + T * 10 + D)
    scale = torch.tensor([1.0, 37.5, 2.0 ** -9, 2.0 ** -13])[torch.randint(0, 4, (B, T, 1), generator=g)]
    qp = (torch.randn(B, T, Hq * D, generator=g) * scale).to(dtype).to(gpu)
    kp = (torch.randn(B, T, H * D, generator=g) * scale).to(dtype).to(gpu)
    q = qp.view(B, T, Hq, D).transpose(1, 2)
    k = kp.view(B, T, H, D).transpose(1, 2)
    pos = torch.rand(1 if shared_table else B, T, 1, generator=g) * 4000.0
    inv = 10000.0 ** (-torch.arange(0, D, 2).float() / D)
    ang = torch.cat([pos * inv, pos * inv], dim=-1)
    cos, sin = ang.cos().to(dtype).to(gpu), ang.sin().to(dtype).to(gpu)
    want_q, want_k = apply_rotary_pos_emb(q, k, cos, sin)
    got_q, got_k = gemv.rope_qk(q, k, cos, sin)
    assert got_q.is_contiguous() and got_k.is_contiguous()
    as_bits = lambda t: t.contiguous().view(torch.int16).cpu()
    assert torch.equal(as_bits(got_q), as_bits(want_q))
    assert torch.equal(as_bits(got_k), as_bits(want_k))
    # packed inputs and a table that is a slice (odd storage offset in bytes / 4 is fine, strides even)
    got_q2, _ = gemv.rope_qk(q.contiguous(), k.contiguous(), cos, sin)
    assert torch.equal(as_bits(got_q2), as_bits(want_q))
