"""Accuracy-evaluation flavour of the ADKV cache: values are fake-quantised on write in fp32 and
kept dequantised, attention is the regular dense one.

Counterpart of the reference's ``adkv.hf.llama_adkv_eval`` (src/adkv/hf/llama_adkv_eval.py): same
class names, ``update`` signature and state fields (``key_dc``, ``key_scale``, ...).  The Triton
kernel of the reference (llama_adkv_eval.py:34-118) is replaced by the gfx950 fp32 quantiser
(``adkv_quant_f32``), which walks every newly appended token of K and of V in one launch each
instead of 32-token tiles, in place on the cache buffer.
"""
from __future__ import annotations

import math

import torch
from torch import nn
from transformers.models.llama.modeling_llama import (
    LlamaAttention,
    LlamaDecoderLayer,
    LlamaForCausalLM,
    LlamaModel,
    apply_rotary_pos_emb,
    eager_attention_forward,
)
from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

from ..train.train_model import quant_f32
from .llama_adkv import ADKV_PARAM_FIELDS, ADKVConfig  # noqa: F401

SCALE_MIN = math.exp(-4.0)
SCALE_MAX = math.exp(4.0)
BITS = 4
QUANT_UPPER = 2 ** (BITS - 1) - 1
QUANT_LOWER = -2 ** (BITS - 1)

INIT_SEQ_LEN = 128   # reference llama_adkv_eval.py:129-130
CAP_LEN = 128
GROWTH = 1.5


class KVCacheLayer_ADKV:
    """Dequantised K/V of one layer, ``[B, T, C]`` with ``C = heads * head_dim``, plus the fp32
    filter state per (batch, channel)."""

    def __init__(self):
        self.key_dc = None
        self.key_scale = None
        self.value_dc = None
        self.value_scale = None
        self._key_buf = None
        self._value_buf = None
        self._quant_len = 0
        self._recent_len = 0

    def get_seq_length(self) -> int:
        return self._recent_len

    def get_mask_sizes(self, cache_position) -> tuple[int, int]:
        q_len = cache_position if isinstance(cache_position, int) else cache_position.shape[0]
        return self.get_seq_length() + q_len, 0

    def _init_buffers(self, B: int, C: int, device, dtype):
        self._key_buf = torch.empty(B, INIT_SEQ_LEN, C, device=device, dtype=dtype)
        self._value_buf = torch.empty(B, INIT_SEQ_LEN, C, device=device, dtype=dtype)
        self._recent_len = 0
        self._quant_len = 0

    def _cap_buffers(self, T: int):
        B, max_len, C = self._key_buf.shape
        need = self._recent_len + T
        if need <= max_len:
            return
        new_len = max(need, int(max_len * GROWTH))
        new_len = -(-new_len // CAP_LEN) * CAP_LEN
        for name in ("_key_buf", "_value_buf"):
            old = getattr(self, name)
            new = torch.empty(B, new_len, C, device=old.device, dtype=old.dtype)
            new[:, :self._recent_len] = old[:, :self._recent_len]
            setattr(self, name, new)

    def _append_tokens(self, key_states, value_states):
        T = key_states.shape[1]
        self._key_buf[:, self._recent_len:self._recent_len + T] = key_states
        self._value_buf[:, self._recent_len:self._recent_len + T] = value_states
        self._recent_len += T

    def _quantize_new_tokens(self, key_alpha, key_beta, key_quant_target,
                             value_alpha, value_beta, value_quant_target):
        """Quantise on write: every token appended since the last call, in place."""
        a, b = self._quant_len, self._recent_len
        if b == a:
            return
        for buf, dc, scale, al, be, tg in (
                (self._key_buf, self.key_dc, self.key_scale, key_alpha, key_beta, key_quant_target),
                (self._value_buf, self.value_dc, self.value_scale, value_alpha, value_beta,
                 value_quant_target)):
            view = buf[:, a:b]
            quant_f32(view, al, be, tg, QUANT_LOWER, QUANT_UPPER, SCALE_MIN, SCALE_MAX,
                      zp_state=dc, sc_state=scale, out=view)
        self._quant_len = b

    @property
    def key_states(self):
        return None if self._recent_len == 0 else self._key_buf[:, :self._recent_len]

    @property
    def value_states(self):
        return None if self._recent_len == 0 else self._value_buf[:, :self._recent_len]

    def update(self, key_states, value_states,
               key_zp_init, key_scale_init, key_alpha, key_beta, key_quant_target,
               value_zp_init, value_scale_init, value_alpha, value_beta, value_quant_target):
        """Append ``[B, T, C]`` keys/values, quantise them, return the whole dequantised cache."""
        B, T, C = key_states.shape
        if self._key_buf is None:
            self._init_buffers(B, C, key_states.device, key_states.dtype)
        if self.key_dc is None:
            f = lambda p: p.detach().to(torch.float32).reshape(1, C).repeat(B, 1).contiguous()
            self.key_dc, self.key_scale = f(key_zp_init), f(key_scale_init)
            self.value_dc, self.value_scale = f(value_zp_init), f(value_scale_init)
        self._cap_buffers(T)
        self._append_tokens(key_states, value_states)
        self._quantize_new_tokens(key_alpha, key_beta, key_quant_target,
                                  value_alpha, value_beta, value_quant_target)
        return self.key_states, self.value_states


class KVCache_ADKV(list):
    def __init__(self, num_layers):
        super().__init__(KVCacheLayer_ADKV() for _ in range(num_layers))

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self[layer_idx].get_seq_length()

    def get_mask_sizes(self, cache_position, layer_idx: int) -> tuple[int, int]:
        return self[layer_idx].get_mask_sizes(cache_position)

    def get_query_offset(self, layer_idx: int = 0) -> int:
        return self.get_seq_length(layer_idx)

    def get_max_length(self) -> int:
        return -1

    is_sliding = [False]
    is_compileable = False


class LlamaAttention_ADKV(LlamaAttention):
    """Llama attention over the fake-quantised cache (reference llama_adkv_eval.py:289-424).

    ``prefill_full_precision=True``: a multi-token call attends with the K/V it just computed and
    only writes the cache; ``False``: it reads K/V back from the cache, so quantisation error also
    reaches prefill.  Single-token calls always read the cache.
    """

    _FP32_BUFFERS = frozenset(f"{side}_{name}" for side in ("key", "value") for name in ADKV_PARAM_FIELDS)

    def __init__(self, config, layer_idx: int):
        super().__init__(config, layer_idx)
        n = config.num_key_value_heads * self.head_dim
        for name in self._FP32_BUFFERS:
            self.register_buffer(name, torch.empty(n, dtype=torch.float32), persistent=False)

    def _apply(self, fn, recurse=True):
        # the quantiser state is fp32 whatever dtype the model is cast to
        saved = {name: self._buffers.pop(name) for name in self._FP32_BUFFERS}
        super()._apply(fn, recurse=recurse)
        for name, buf in saved.items():
            if buf is not None:
                buf = fn(buf)
                if buf.dtype != torch.float32:
                    buf = buf.to(torch.float32)
            self._buffers[name] = buf
        return self

    def _adkv_params(self, side: str):
        return tuple(getattr(self, f"{side}_{name}") for name in ADKV_PARAM_FIELDS)

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None,
                past_key_values=None, cache_position=None, use_cache: bool = True,
                prefill_full_precision: bool = True, **kwargs):
        lead = hidden_states.shape[:-1]
        shape = (*lead, -1, self.head_dim)
        q = self.q_proj(hidden_states).view(shape).transpose(1, 2)
        k = self.k_proj(hidden_states).view(shape).transpose(1, 2)
        v = self.v_proj(hidden_states).view(shape).transpose(1, 2)
        cos, sin = position_embeddings
        q, k = apply_rotary_pos_emb(q, k, cos, sin)

        if past_key_values is not None:
            if not isinstance(past_key_values, KVCache_ADKV):
                raise TypeError("ADKV attention requires a KVCache_ADKV, got "
                                f"{type(past_key_values).__name__}")
            layer = past_key_values[self.layer_idx]
            B, H, T, C = k.shape
            dt = k.dtype
            hist = layer.get_seq_length()
            layer.update(k.transpose(1, 2).reshape(B, T, H * C).float(),
                         v.transpose(1, 2).reshape(B, T, H * C).float(),
                         *self._adkv_params("key"), *self._adkv_params("value"))
            heads = lambda t, n: t.view(B, n, H, C).transpose(1, 2).to(dt)
            if T > 1 and prefill_full_precision:
                if hist:
                    k = torch.cat([heads(layer.key_states[:, :hist], hist), k], dim=2)
                    v = torch.cat([heads(layer.value_states[:, :hist], hist), v], dim=2)
            else:
                n = layer.get_seq_length()
                k, v = heads(layer.key_states, n), heads(layer.value_states, n)

        attend = eager_attention_forward
        if self.config._attn_implementation != "eager":
            attend = ALL_ATTENTION_FUNCTIONS[self.config._attn_implementation]
        out, weights = attend(self, q, k, v, attention_mask,
                              dropout=0.0 if not self.training else self.attention_dropout,
                              scaling=self.scaling, **kwargs)
        out = self.o_proj(out.reshape(*lead, -1).contiguous())
        return out, weights


class LlamaDecoderLayer_ADKV(LlamaDecoderLayer):
    def __init__(self, config, layer_idx: int):
        super().__init__(config, layer_idx)
        self.self_attn = LlamaAttention_ADKV(config=config, layer_idx=layer_idx)


class LlamaModel_ADKV(LlamaModel):
    _no_split_modules = ["LlamaDecoderLayer_ADKV"]

    def __init__(self, config):
        super().__init__(config)
        self.layers = nn.ModuleList(LlamaDecoderLayer_ADKV(config, i)
                                    for i in range(config.num_hidden_layers))
        self.post_init()

    def forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None,
                inputs_embeds=None, cache_position=None, use_cache=None, **kwargs):
        if use_cache is None:
            use_cache = getattr(self.config, "use_cache", True)
        if use_cache and past_key_values is None:
            past_key_values = KVCache_ADKV(self.config.num_hidden_layers)
        return super().forward(input_ids=input_ids, attention_mask=attention_mask,
                               position_ids=position_ids, past_key_values=past_key_values,
                               inputs_embeds=inputs_embeds, cache_position=cache_position,
                               use_cache=use_cache, **kwargs)


class LlamaForCausalLM_ADKV(LlamaForCausalLM):
    _no_split_modules = ["LlamaDecoderLayer_ADKV"]

    def __init__(self, config):
        super().__init__(config)
        self.model = LlamaModel_ADKV(config)
        self.tie_weights()

    def forward(self, *args, prefill_full_precision: bool | None = None, **kwargs):
        if prefill_full_precision is None:
            prefill_full_precision = getattr(self.config, "prefill_full_precision", True)
        return super().forward(*args, prefill_full_precision=prefill_full_precision, **kwargs)

    def load_adkv_config(self, adkv_config):
        """Fill the per-layer K/V parameters from ``(ADKVConfig, ADKVConfig)`` pairs."""
        for layer_idx, pair in enumerate(adkv_config):
            attn = self.model.layers[layer_idx].self_attn
            for side, cfg in zip(("key", "value"), pair):
                for name in ADKV_PARAM_FIELDS:
                    getattr(attn, f"{side}_{name}").copy_(getattr(cfg, name))

    def _prepare_cache_for_generation(self, *args, **kwargs):
        # the ADKV cache is created lazily by LlamaModel_ADKV.forward
        return None
