"""Per-layer packed ADKV KV cache: the host-side owner of the code buffers.

Counterpart of the reference's ``KVCacheLayer_ADKV`` / ``KVCache_ADKV``
(src/adkv/hf/llama_adkv.py:44-288) with the same public names, method signatures, buffer layout
``[B, H, n_super, C // 4, 4, 4]`` uint8 and error behaviour, so code written against the
reference's cache object works unchanged.  What differs is underneath:

* the three kernels are the gfx950 ones (``adkv_amd.kernel.gemv``), launched on the current stream;
* the scale/mask/softmax chain between QK and OV is one fused launch instead of five torch ops;
* capacity grows geometrically (the reference reallocates and copies both caches every 64 tokens,
  llama_adkv.py:104-123);
* next to each code buffer lives a small checkpoint tensor holding the exact fp16 filter state
  every ``CKPT_INTERVAL`` tokens (4 bytes per channel per checkpoint, ~3 % of the codes at 256).
  The kernels keep it up to date and use it to replay the time axis in independent segments;
* the filter state after the last prompt token is carried, so a prompt may be prefilled in chunks
  (the reference refuses: llama_adkv.py:195-197).
"""
from __future__ import annotations

import math

import torch

from ..kernel.gemv import append_kv_pair, decode_step, decode_step_workspace_bytes

SCALE_MIN = math.exp(-4.0)  # kept for API parity; the fp16 recurrence never clamps
SCALE_MAX = math.exp(4.0)

INIT_SEQ_LEN = 64    # token slots of a fresh cache (reference llama_adkv.py:40)
CAP_LEN = 64         # capacity granularity in tokens (reference llama_adkv.py:41)
GROWTH = 1.5         # geometric growth factor once the initial capacity is exceeded
CKPT_INTERVAL = 256  # tokens between state checkpoints (multiple of 8); 0 disables them

_HEAD_DIMS = (128, 256, 512)

# Scratch for the fused decode call (logits + partial sums), one per (device, stream): every layer's
# step on a stream runs after the previous one, so they can share it.
_workspaces: dict[tuple, torch.Tensor] = {}


def _workspace(dev: torch.device, need: int) -> torch.Tensor:
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1) * 5 // 4, dtype=torch.uint8, device=dev)
        _workspaces[key] = ws
    return ws


class KVCacheLayer_ADKV:
    """Quantised K/V store of one attention layer."""

    def __init__(self, bits: int = 4):
        if bits not in (2, 4):
            raise ValueError("ADKV code width must be 2 or 4 bits")
        # 4 = the reference's format; 2 = the same recurrence over codes in [-2, 1], 16 tokens per
        # supergroup (head_dim 128 only), an extension the reference does not have
        self._bits = bits
        self._key_buf: torch.Tensor | None = None
        self._value_buf: torch.Tensor | None = None
        self._key_ckpt: torch.Tensor | None = None
        self._value_ckpt: torch.Tensor | None = None
        # (zp, sc) after the last quantised token, [B, H, C, 2] fp16; lets a prompt arrive in chunks.
        # A decode step appends inside the attention kernels and leaves these stale.
        self._key_state: torch.Tensor | None = None
        self._value_state: torch.Tensor | None = None
        self._state_valid = False
        self._quant_len = 0
        self._cap_len = 0
        self._B = self._H = self._C = 0
        self._device = None
        self._ckpt_interval = CKPT_INTERVAL
        self._views: dict = {}    # id(parameter) -> (parameter, its [H, C] view)
        self._shares_storage = False   # a batch_view(): its buffers belong to another layer object

    # ------------------------------------------------------------------ HF cache protocol
    def get_seq_length(self) -> int:
        return self._quant_len

    def get_mask_sizes(self, cache_position) -> tuple[int, int]:
        """(kv_length, kv_offset) for mask construction.  ``cache_position`` is the query's position
        tensor (transformers 5.3, the version the reference pins) or the query length as an int
        (later 5.x releases)."""
        q_len = cache_position if isinstance(cache_position, int) else cache_position.shape[0]
        return self._quant_len + q_len, 0

    @property
    def key_states(self) -> torch.Tensor | None:
        """Packed uint8 K codes (None before the first token)."""
        return self._key_buf

    @property
    def value_states(self) -> torch.Tensor | None:
        """Packed uint8 V codes (None before the first token)."""
        return self._value_buf

    # ------------------------------------------------------------------ storage
    def _n_super(self, tokens: int) -> int:
        return -(-tokens // (32 // self._bits))

    def _n_ckpt(self, cap_tokens: int) -> int:
        return cap_tokens // self._ckpt_interval + 1 if self._ckpt_interval else 0

    def _new_buffers(self, cap_tokens: int):
        ns = self._n_super(cap_tokens)
        shape = (self._B, self._H, ns, self._C // 4, 4, 4)
        mk = lambda: torch.zeros(shape, dtype=torch.uint8, device=self._device)
        ck = (lambda: torch.zeros((self._B, self._H, self._n_ckpt(ns * (32 // self._bits)), self._C, 2),
                                  dtype=torch.float16, device=self._device)) \
            if self._ckpt_interval else (lambda: None)
        return ns * (32 // self._bits), mk(), mk(), ck(), ck()

    def _init_buffers(self, B: int, H: int, C: int, device: torch.device):
        if C not in _HEAD_DIMS:
            raise ValueError(f"ADKV kernels support head_dim in (128, 256, 512), got {C}")
        if self._bits == 2 and C != 128:
            raise ValueError("2-bit ADKV codes need head_dim 128")
        self._B, self._H, self._C, self._device = B, H, C, device
        self._quant_len = 0
        (self._cap_len, self._key_buf, self._value_buf,
         self._key_ckpt, self._value_ckpt) = self._new_buffers(INIT_SEQ_LEN)
        mk = lambda: torch.zeros((B, H, C, 2), dtype=torch.float16, device=device)
        self._key_state, self._value_state, self._state_valid = mk(), mk(), True

    def _cap_buffers(self, T: int):
        """Make room for ``T`` tokens.  New slots are zero, as the append kernels expect."""
        if T <= self._cap_len:
            return
        if self._shares_storage:
            raise RuntimeError("a batch view cannot grow: reserve() the parent cache for the whole context")
        want = max(T, int(self._cap_len * GROWTH))
        want = -(-want // CAP_LEN) * CAP_LEN
        cap, key, value, kck, vck = self._new_buffers(want)
        old = self._key_buf.shape[2]
        key[:, :, :old].copy_(self._key_buf)
        value[:, :, :old].copy_(self._value_buf)
        if kck is not None:
            n = self._key_ckpt.shape[2]
            kck[:, :, :n].copy_(self._key_ckpt)
            vck[:, :, :n].copy_(self._value_ckpt)
        self._key_buf, self._value_buf, self._key_ckpt, self._value_ckpt = key, value, kck, vck
        self._cap_len = cap

    # ------------------------------------------------------------------ big batches, prompt in slices
    def reserve(self, B: int, H: int, C: int, tokens: int, device) -> None:
        """Allocate for a known batch and context up front: no growth copies later, and the
        prompt of a batch too big for one dense prefill can be quantised slice by slice
        through ``batch_view`` (the dense attention of a long prompt, not the cache, is what
        limits the batch of a single prefill call)."""
        self._init_buffers(B, H, C, torch.device(device))
        self._cap_buffers(tokens)

    def batch_view(self, b0: int, b1: int) -> "KVCacheLayer_ADKV":
        """A layer object over sequences ``b0 .. b1-1`` of this one, sharing its storage (the batch
        axis is the outermost, so the slices are contiguous).  Quantise a slice of the prompt
        through it, then ``commit`` the parent."""
        if self._key_buf is None or not 0 <= b0 < b1 <= self._B:
            raise ValueError("batch_view needs a reserved cache and a slice inside its batch")
        v = KVCacheLayer_ADKV(self._bits)
        v._B, v._H, v._C, v._device = b1 - b0, self._H, self._C, self._device
        v._ckpt_interval, v._cap_len, v._quant_len = self._ckpt_interval, self._cap_len, self._quant_len
        v._key_buf, v._value_buf = self._key_buf[b0:b1], self._value_buf[b0:b1]
        if self._key_ckpt is not None:
            v._key_ckpt, v._value_ckpt = self._key_ckpt[b0:b1], self._value_ckpt[b0:b1]
        v._key_state, v._value_state = self._key_state[b0:b1], self._value_state[b0:b1]
        v._state_valid, v._shares_storage = self._state_valid, True
        return v

    def commit(self, tokens: int) -> None:
        """Declare that every sequence now holds ``tokens`` quantised tokens (all slices prefilled)."""
        if tokens > self._cap_len:
            raise ValueError("more tokens than the cache holds")
        self._quant_len, self._state_valid = tokens, True

    def _check_geometry(self, B: int, H: int, C: int, device: torch.device):
        if self._key_buf is None:
            self._init_buffers(B, H, C, device)
        elif (B, H, C) != (self._B, self._H, self._C):
            raise ValueError("cache was created for a different (B, H, C)")

    @staticmethod
    def _rows(x: torch.Tensor) -> torch.Tensor:
        # fp16 and bf16 rows go to the encoder as they are (it rounds bf16 to fp16 and follows the
        # strides of a [B, T, H, C] projection output itself); anything else is converted first
        return x if x.dtype in (torch.float16, torch.bfloat16) else x.to(torch.float16)

    def _view(self, p: torch.Tensor) -> torch.Tensor:
        # the module passes the same parameter buffers at every step: keep their [H, C] views
        hit = self._views.get(id(p))
        if hit is not None and hit[0] is p:
            return hit[1]
        v = p.view(self._H, self._C)
        if len(self._views) > 64:
            self._views.clear()
        self._views[id(p)] = (p, v)
        return v

    # ------------------------------------------------------------------ quantise
    def _append_tokens(self, key_states, value_states,
                       key_zp_init, key_scale_init, key_alpha, key_beta, key_quant_target,
                       value_zp_init, value_scale_init, value_alpha, value_beta, value_quant_target):
        """Quantise ``[B, H, T, C]`` keys/values as tokens ``quant_len ..`` of the stream."""
        v = self._view
        S = self._ckpt_interval
        append_kv_pair(
            self._key_buf, self._value_buf,
            self._rows(key_states), self._rows(value_states),
            (v(key_zp_init), v(key_scale_init), v(key_alpha), v(key_beta), v(key_quant_target)),
            (v(value_zp_init), v(value_scale_init), v(value_alpha), v(value_beta),
             v(value_quant_target)),
            self._quant_len, self._key_state, self._value_state,
            k_ckpt=self._key_ckpt, v_ckpt=self._value_ckpt, ckpt_interval=S, bits=self._bits)
        self._quant_len += key_states.shape[2]

    def prefill(self, key_states, value_states,
                key_zp_init, key_scale_init, key_alpha, key_beta, key_quant_target,
                value_zp_init, value_scale_init, value_alpha, value_beta, value_quant_target):
        """Quantise the prompt into the cache.  No attention is computed here."""
        B, H, T, C = key_states.shape
        if value_states.shape != key_states.shape:
            raise ValueError("key/value shapes differ")
        self._check_geometry(B, H, C, key_states.device)
        if T == 0:
            return
        if self._quant_len != 0 and not self._state_valid:
            # The reference refuses every second prefill (llama_adkv.py:195-197).  Here a prompt may
            # arrive in chunks because the filter state is carried; only after single-token decode
            # steps, which append inside the attention kernels, is that state gone.
            raise NotImplementedError(
                "ADKV prefill encodes from token 0; chunked prefill is not supported by the kernel")
        self._cap_buffers(self._quant_len + T)
        self._append_tokens(key_states, value_states,
                            key_zp_init, key_scale_init, key_alpha, key_beta, key_quant_target,
                            value_zp_init, value_scale_init, value_alpha, value_beta,
                            value_quant_target)

    # ------------------------------------------------------------------ decode
    def decode(self, query_states, key_states, value_states,
               key_zp_init, key_scale_init, key_alpha, key_beta, key_quant_target,
               value_zp_init, value_scale_init, value_alpha, value_beta, value_quant_target,
               attention_mask: torch.Tensor | None = None,
               scaling: float = 1.0) -> tuple[torch.Tensor, torch.Tensor]:
        """One causal decode step: attend over the cached tokens and the new one, append the new
        K/V codes, return ``(output [B,H,C] in the query's dtype, weights [B,H,ctx+1] fp16)``."""
        B, Hq, Tq, C = query_states.shape
        H, Tk = key_states.shape[1], key_states.shape[2]
        if Tq != 1 or Tk != 1:
            raise ValueError("decode expects exactly one query/key/value token")
        if Hq % H or Hq // H not in (1, 2, 4, 8) or (Hq != H and C != 128):
            # the reference only takes Hq == H (llama_adkv.py:235-238); grouped queries are an extension
            raise ValueError("ADKV decode supports 1, 2, 4 or 8 query heads per KV head "
                             "(more than one only with head_dim 128)")
        self._check_geometry(B, H, C, query_states.device)
        ctx = self._quant_len
        self._cap_buffers(ctx + 1)

        # fp16 and bf16 activations go in as they are; the kernels convert (see decode_step)
        same = query_states.dtype in (torch.float16, torch.bfloat16) \
            and key_states.dtype == query_states.dtype == value_states.dtype
        f16 = (lambda t: t.contiguous()) if same else (lambda t: t.to(torch.float16).contiguous())
        v = self._view
        S = self._ckpt_interval
        dev = query_states.device
        ncap = self._key_ckpt.shape[2] if S else 0
        ws = _workspace(dev, decode_step_workspace_bytes(B, Hq, H, ctx, C, ncap, S))
        out, weights = decode_step(
            f16(query_states), self._key_buf, self._value_buf, f16(key_states), f16(value_states),
            (v(key_zp_init), v(key_scale_init), v(key_alpha), v(key_beta), v(key_quant_target)),
            (v(value_zp_init), v(value_scale_init), v(value_alpha), v(value_beta),
             v(value_quant_target)),
            ctx, scaling, attention_mask,
            k_ckpt=self._key_ckpt, v_ckpt=self._value_ckpt, ckpt_interval=S, bits=self._bits,
            workspace=ws)
        self._quant_len = ctx + 1
        self._state_valid = False
        return (out if out.dtype == query_states.dtype else out.to(query_states.dtype)), weights

    # ------------------------------------------------------------------ save / restore
    def state_dict(self) -> dict:
        """Everything needed to continue decoding elsewhere: the used part of the code buffers, the
        state checkpoints that go with them and, while it is still valid, the carried filter state.
        Plain tensors and ints, so ``torch.save`` / ``torch.load(weights_only=True)`` round-trip it."""
        if self._key_buf is None:
            return {"quant_len": 0}
        ns = self._n_super(self._quant_len)
        nck = self._quant_len // self._ckpt_interval if self._ckpt_interval else 0
        sd = {"quant_len": self._quant_len, "ckpt_interval": self._ckpt_interval, "bits": self._bits,
              "geometry": (self._B, self._H, self._C),
              "key_codes": self._key_buf[:, :, :ns].contiguous(),
              "value_codes": self._value_buf[:, :, :ns].contiguous()}
        if self._ckpt_interval:
            sd["key_ckpt"] = self._key_ckpt[:, :, :nck].contiguous()
            sd["value_ckpt"] = self._value_ckpt[:, :, :nck].contiguous()
        if self._state_valid:
            sd["key_state"], sd["value_state"] = self._key_state.clone(), self._value_state.clone()
        return sd

    def load_state_dict(self, sd: dict, device=None) -> None:
        """Rebuild the layer from ``state_dict()`` output on ``device`` (default: where the saved
        tensors live).  Slots past the saved tokens are zero, as the append kernels expect."""
        if sd.get("quant_len", 0) == 0 and "key_codes" not in sd:
            self.__init__(self._bits)
            return
        self._bits = int(sd.get("bits", 4))
        B, H, C = sd["geometry"]
        dev = torch.device(device) if device is not None else sd["key_codes"].device
        T = int(sd["quant_len"])
        self._ckpt_interval = int(sd["ckpt_interval"])
        self._init_buffers(B, H, C, dev)
        self._cap_buffers(T)
        ns = self._n_super(T)
        if tuple(sd["key_codes"].shape) != (B, H, ns, C // 4, 4, 4):
            raise ValueError("saved code tensor does not match its geometry")
        self._key_buf[:, :, :ns].copy_(sd["key_codes"])
        self._value_buf[:, :, :ns].copy_(sd["value_codes"])
        if self._ckpt_interval:
            nck = T // self._ckpt_interval
            if sd["key_ckpt"].shape[2] != nck:
                raise ValueError("saved checkpoints do not cover the saved tokens")
            self._key_ckpt[:, :, :nck].copy_(sd["key_ckpt"])
            self._value_ckpt[:, :, :nck].copy_(sd["value_ckpt"])
        self._quant_len = T
        self._state_valid = "key_state" in sd
        if self._state_valid:
            self._key_state.copy_(sd["key_state"])
            self._value_state.copy_(sd["value_state"])

    # ------------------------------------------------------------------ accounting
    def nbytes(self) -> int:
        """Device bytes held by this layer (codes + checkpoints)."""
        ts = (self._key_buf, self._value_buf, self._key_ckpt, self._value_ckpt)
        return sum(t.numel() * t.element_size() for t in ts if t is not None)


class KVCache_ADKV(list):
    """One ``KVCacheLayer_ADKV`` per decoder layer (reference llama_adkv.py:279-288)."""

    def __init__(self, num_layers: int, bits: int = 4):
        super().__init__(KVCacheLayer_ADKV(bits) for _ in range(num_layers))

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self[layer_idx].get_seq_length()

    def reserve(self, B: int, H: int, C: int, tokens: int, device) -> None:
        for layer in self:
            layer.reserve(B, H, C, tokens, device)

    def batch_view(self, b0: int, b1: int) -> "KVCache_ADKV":
        view = KVCache_ADKV(0)
        view.extend(layer.batch_view(b0, b1) for layer in self)
        return view

    def commit(self, tokens: int) -> None:
        for layer in self:
            layer.commit(tokens)

    def get_mask_sizes(self, cache_position, layer_idx: int) -> tuple[int, int]:
        return self[layer_idx].get_mask_sizes(cache_position)

    # the rest is what newer transformers releases ask of a cache object during generate()
    def get_query_offset(self, layer_idx: int = 0) -> int:
        return self.get_seq_length(layer_idx)

    def get_max_length(self) -> int:
        return -1

    is_sliding = [False]
    is_compileable = False

    def save(self, path) -> None:
        """Write all layers to one file (tensors moved to the CPU)."""
        cpu = lambda v: v.cpu() if isinstance(v, torch.Tensor) else v
        torch.save([{k: cpu(v) for k, v in layer.state_dict().items()} for layer in self], path)

    @classmethod
    def load(cls, path, device) -> "KVCache_ADKV":
        layers = torch.load(path, map_location="cpu", weights_only=True)
        cache = cls(len(layers))
        for layer, sd in zip(cache, layers):
            layer.load_state_dict(sd, device)
        return cache


def adkv_cache_bytes(B: int, H: int, C: int, tokens: int, layers: int, bits: int = 4,
                     ckpt_interval: int = CKPT_INTERVAL) -> int:
    """Bytes of a full ADKV cache: K and V codes plus fp16 (zp, sc) checkpoints.  Same accounting
    as the reference's memory model (tools/memory_comparison_fig.py:46-56) with
    ``ckpt_num = tokens // ckpt_interval``; the ten parameter vectors per layer are added once."""
    codes = B * H * (-(-tokens // 8) * 8) * C * bits // 8
    ckpt = (B * H * (tokens // ckpt_interval) * C * 2 * 2) if ckpt_interval else 0
    params = 10 * H * C * 2
    return layers * (2 * (codes + ckpt) + params)


def fp16_cache_bytes(B: int, H: int, C: int, tokens: int, layers: int) -> int:
    return layers * 2 * B * H * tokens * C * 2
