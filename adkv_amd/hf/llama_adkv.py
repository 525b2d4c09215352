"""Hugging Face Llama with the ADKV quantised KV cache on MI355X.

Counterpart of the reference's ``adkv.hf.llama_adkv`` (src/adkv/hf/llama_adkv.py:291-462): same
class names, same buffer names on the attention module (``key_zp_init`` ... ``value_quant_target``),
same ``load_adkv_config`` entry point, so a script written for the reference only changes its
import.  Prefill runs the regular dense attention and also quantises the prompt into the cache;
a single-token step goes through ``KVCacheLayer_ADKV.decode`` (llama_adkv.py:347-356 in the
reference).
"""
from __future__ import annotations

from dataclasses import dataclass

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

from ..kernel.gemv import rope_qk
from .cache import (CAP_LEN, INIT_SEQ_LEN, SCALE_MAX, SCALE_MIN, KVCache_ADKV,  # noqa: F401
                    KVCacheLayer_ADKV)

# the five per-(head, channel) quantities, for K and for V (reference llama_adkv.py:27)
ADKV_PARAM_FIELDS = ("zp_init", "scale_init", "alpha", "beta", "quant_target")


@dataclass
class ADKVConfig:
    """Calibrated parameters of one tensor (K or V) of one layer, each of ``H * head_dim`` values."""
    zp_init: torch.Tensor
    scale_init: torch.Tensor
    alpha: torch.Tensor
    beta: torch.Tensor
    quant_target: torch.Tensor


class LlamaAttention_ADKV(LlamaAttention):
    """Llama attention whose single-token steps read the packed ADKV cache."""

    def __init__(self, config, layer_idx: int):
        super().__init__(config, layer_idx)
        width = config.num_key_value_heads * self.head_dim
        for side in ("key", "value"):
            for name in ADKV_PARAM_FIELDS:
                # fp16 because the deployment recurrence is fp16; filled by load_adkv_config()
                self.register_buffer(f"{side}_{name}", torch.empty(width, dtype=torch.float16),
                                     persistent=False)

    def _adkv_params(self, side: str) -> tuple[torch.Tensor, ...]:
        return tuple(getattr(self, f"{side}_{name}") for name in ADKV_PARAM_FIELDS)

    def _apply(self, fn, recurse=True):
        # model.to(torch.bfloat16) / .half() casts every floating-point buffer.  The recurrence is
        # fp16 whatever the weights are (the kernels take fp16 parameters only, as the reference's
        # do: gemv.cu:375-382), and a round trip through bfloat16 would drop three mantissa bits of
        # the calibrated values: these ten buffers follow the module's device, never its dtype.
        names = [f"{side}_{name}" for side in ("key", "value") for name in ADKV_PARAM_FIELDS]
        kept = {n: self._buffers[n] for n in names if self._buffers.get(n) is not None}
        super()._apply(fn, recurse)
        for n, old in kept.items():
            new = self._buffers[n]
            if new.dtype != torch.float16:
                self._buffers[n] = old.to(device=new.device)
        return self

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None,
                past_key_values=None, cache_position=None, use_cache: bool = True, **kwargs):
        lead = hidden_states.shape[:-1]
        split = (*lead, -1, self.head_dim)
        q = self.q_proj(hidden_states).view(split).transpose(1, 2)
        k = self.k_proj(hidden_states).view(split).transpose(1, 2)
        v = self.v_proj(hidden_states).view(split).transpose(1, 2)
        cos, sin = position_embeddings
        wants_grad = torch.is_grad_enabled() and (q.requires_grad or k.requires_grad)
        if (q.is_cuda and q.dtype in (torch.float16, torch.bfloat16) and cos.dtype == q.dtype
                and cos.dim() == 3 and self.head_dim % 4 == 0 and not wants_grad):
            # one launch instead of apply_rotary_pos_emb's ten, same values bit for bit.  The
            # kernel has no backward pass: whenever autograd is recording, the differentiable
            # expression the reference calls (llama_adkv.py:336-337) runs instead.
            q, k = rope_qk(q, k, cos, sin)
        else:
            q, k = apply_rotary_pos_emb(q, k, cos, sin)

        layer_cache = None
        if use_cache and past_key_values is not None:
            if not isinstance(past_key_values, KVCache_ADKV):
                raise TypeError("ADKV attention requires a KVCache_ADKV, got "
                                f"{type(past_key_values).__name__}")
            layer_cache = past_key_values[self.layer_idx]

        if layer_cache is not None and q.shape[2] == 1:
            ctx, weights = layer_cache.decode(
                q, k, v, *self._adkv_params("key"), *self._adkv_params("value"),
                attention_mask=attention_mask, scaling=self.scaling)
            return self.o_proj(ctx.reshape(*lead, -1).contiguous()), weights

        if layer_cache is not None and layer_cache.get_seq_length() > 0:
            # Several new tokens on top of a cache that already holds codes (a follow-up turn, a
            # prompt fed in pieces).  The earlier tokens exist only as codes, so the new ones are
            # taken one decode step at a time: token i attends over the cache and the new tokens
            # before it, exactly as if they had arrived singly.  (The reference refuses this call,
            # llama_adkv.py:195-197; the first prompt still goes through the dense path below.)
            past = layer_cache.get_seq_length()
            key_p, value_p = self._adkv_params("key"), self._adkv_params("value")
            steps = []
            for i in range(q.shape[2]):
                mask = None
                if attention_mask is not None:
                    mask = attention_mask[:, :, i:i + 1, :past + i + 1]
                o, _ = layer_cache.decode(q[:, :, i:i + 1], k[:, :, i:i + 1], v[:, :, i:i + 1],
                                          *key_p, *value_p, attention_mask=mask, scaling=self.scaling)
                steps.append(o)
            ctx = torch.stack(steps, dim=1)                      # [B, Tq, Hq, C]
            return self.o_proj(ctx.reshape(*lead, -1)), None

        if layer_cache is not None:
            layer_cache.prefill(k, v, *self._adkv_params("key"), *self._adkv_params("value"))

        attend = eager_attention_forward
        if self.config._attn_implementation != "eager":
            attend = ALL_ATTENTION_FUNCTIONS[self.config._attn_implementation]
        ctx, weights = attend(self, q, k, v, attention_mask,
                              dropout=0.0 if not self.training else self.attention_dropout,
                              scaling=self.scaling, **kwargs)
        return self.o_proj(ctx.reshape(*lead, -1).contiguous()), weights


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
        self.post_init()  # the replaced layers need the config's initialisation too

    def forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None,
                inputs_embeds=None, cache_position=None, use_cache=None, **kwargs):
        if use_cache is None:
            use_cache = getattr(self.config, "use_cache", True)
        if use_cache and past_key_values is None:
            # created here so that HF never substitutes its DynamicCache
            # config.adkv_bits = 2 selects the 2-bit code format (extension; default 4 as the reference)
            past_key_values = KVCache_ADKV(self.config.num_hidden_layers,
                                           bits=getattr(self.config, "adkv_bits", 4))
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

    def load_adkv_config(self, adkv_config: list[tuple[ADKVConfig, ADKVConfig]]):
        """Copy per-layer (K, V) parameter sets into the attention modules' fp16 buffers."""
        for layer, pair in zip(self.model.layers, adkv_config):
            for side, cfg in zip(("key", "value"), pair):
                for name in ADKV_PARAM_FIELDS:
                    getattr(layer.self_attn, f"{side}_{name}").copy_(getattr(cfg, name))

    def _prepare_cache_for_generation(self, *args, **kwargs):
        # generate() must not install a DynamicCache; LlamaModel_ADKV makes the ADKV cache itself
        return None
