"""Decode-side model glue around the retrieval cache: the part of the reference's ``model_hub/LLM.py``
(``layer_decode`` :157-198, ``decode_forward`` :228-243) and ``model_hub/qwen.py`` (``wqkv`` :327-340, ``wo`` :343-346,
``mlp`` :365-383, ``layernorm`` :395-407, ``head_rmsnorm`` :410-431, rotary embedding :434-498) that a decode loop of a
random-initialised Qwen3-shaped model needs, and nothing else: no checkpoint loading, tokenizer, prefill through the
model or sampling beyond arg-max.

The dense projections are plain library GEMMs (``F.linear``); the layer norms and the SiLU gate are torch ops; the
per-head q/k norms and the rotary embedding of a decode token are one HIP launch (``ops.qk_norm_rope``; the torch
forms below remain for other shapes and as the checked restatement); the attention of a decode step is
``attn_hub.polar_decode_attn`` on the cache, exactly as in the reference.  The reference uses flashinfer for the norms
and the activation, which is CUDA only.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from .. import ops, ranges
from ..attn_hub import polar_decode_attn


@dataclass
class QwenConfig:
    """Shape of the model.  The defaults are Qwen3-8B's."""
    hidden_size: int = 4096
    num_layers: int = 36
    num_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 12288
    vocab_size: int = 151936
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1.0e6
    qk_norm: bool = True        # Qwen3 normalises every query / key head (q_norm, k_norm)


class QwenLayer:
    """Weights of one decoder layer (reference ``QwenLayer``, qwen.py:14-70), random-initialised."""

    def __init__(self, cfg: QwenConfig, device, dtype, gen: torch.Generator):
        h, q, kv, inter = cfg.hidden_size, cfg.num_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim, cfg.intermediate_size

        def w(rows, cols):  # ~ N(0, 1/cols): activations keep unit scale through the layer
            return (torch.randn(rows, cols, generator=gen, device=device, dtype=torch.float32) / math.sqrt(cols)).to(dtype)

        self.wqkv = w(q + 2 * kv, h)
        self.bqkv = None
        self.wo = w(h, q)
        self.gate_up_proj = w(2 * inter, h)
        self.down_proj = w(h, inter)
        ones = lambda n: torch.ones(n, device=device, dtype=dtype)
        self.input_layernorm_weight = ones(h)
        self.post_attention_layernorm_weight = ones(h)
        self.input_layernorm_variance_epsilon = cfg.rms_norm_eps
        self.post_attention_layernorm_variance_epsilon = cfg.rms_norm_eps
        self.q_norm_weight = ones(cfg.head_dim) if cfg.qk_norm else None
        self.k_norm_weight = ones(cfg.head_dim) if cfg.qk_norm else None
        self.q_norm_variance_epsilon = self.k_norm_variance_epsilon = cfg.rms_norm_eps


class QwenModel:
    """Random-initialised decoder with the reference's decode call structure.  ``kv_cache`` is a ``polar_cache``
    (either variant) that already holds the prompt; :meth:`decode_forward` runs one token per sequence."""

    def __init__(self, cfg: QwenConfig, kv_cache, device="cuda:0", dtype=torch.bfloat16, max_positions: int = 1 << 20,
                 seed: int = 0):
        self.cfg, self.kv_cache, self.device, self.dtype = cfg, kv_cache, torch.device(device), dtype
        self.num_layers, self.hidden_size = cfg.num_layers, cfg.hidden_size
        self.num_heads, self.num_key_value_heads, self.head_dim = cfg.num_heads, cfg.num_key_value_heads, cfg.head_dim
        gen = torch.Generator(device=self.device).manual_seed(seed)
        self.layers = [QwenLayer(cfg, self.device, dtype, gen) for _ in range(cfg.num_layers)]
        self.embed_tokens = (torch.randn(cfg.vocab_size, cfg.hidden_size, generator=gen, device=self.device,
                                         dtype=torch.float32)).to(dtype)
        self.lm_head = (torch.randn(cfg.vocab_size, cfg.hidden_size, generator=gen, device=self.device, dtype=torch.float32)
                        / math.sqrt(cfg.hidden_size)).to(dtype)
        self.norm_weight = torch.ones(cfg.hidden_size, device=self.device, dtype=dtype)
        self.norm_variance_epsilon = cfg.rms_norm_eps
        # rotary tables for every position the run can reach (reference keeps a cos_sin_cache, qwen.py:434-489)
        inv_freq = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, device=self.device, dtype=torch.float32) / cfg.head_dim))
        ang = torch.arange(max_positions, device=self.device, dtype=torch.float32)[:, None] * inv_freq[None, :]
        self.cos_cache, self.sin_cache = ang.cos().to(dtype), ang.sin().to(dtype)
        self._position = 0

    # ------------------------------------------------------------------ pieces (reference names)
    def word_embedding(self, inputs_id):
        return F.embedding(inputs_id, self.embed_tokens)

    def lm(self, hidden_states):
        return F.linear(hidden_states, self.lm_head).float()

    def layernorm(self, hidden_states, epsilon, weight):
        return F.rms_norm(hidden_states, (hidden_states.shape[-1],), weight, epsilon)

    def head_rmsnorm(self, states, weight, epsilon, num_heads):
        if weight is None:
            return states
        shape = states.shape
        return F.rms_norm(states.reshape(*shape[:-1], num_heads, self.head_dim), (self.head_dim,), weight, epsilon).reshape(shape)

    def wqkv(self, hidden_states, layer):
        qkv = F.linear(hidden_states, layer.wqkv, layer.bqkv)
        q_dim, kv_dim = self.num_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        q, k, v = qkv.split([q_dim, kv_dim, kv_dim], dim=-1)
        q = self.head_rmsnorm(q, layer.q_norm_weight, layer.q_norm_variance_epsilon, self.num_heads)
        k = self.head_rmsnorm(k, layer.k_norm_weight, layer.k_norm_variance_epsilon, self.num_key_value_heads)
        return q, k, v

    def position_embedd(self, query_states, key_states):
        """Rotary embedding (rotate-half form) at the positions of the step's tokens.  The reference reads the position
        from ``kv_cache.context`` in every layer (qwen.py:494), which layer 0's cache update has already advanced
        when layers > 0 get there; here the position is fixed once per step, before layer 0."""
        bsz, seq_len, _ = key_states.shape
        pos = self._position
        cos, sin = self.cos_cache[pos:pos + seq_len], self.sin_cache[pos:pos + seq_len]   # [seq, D/2]

        def rot(x, heads):
            x = x.reshape(bsz, seq_len, heads, self.head_dim)
            x1, x2 = x[..., :self.head_dim // 2], x[..., self.head_dim // 2:]
            c, s = cos[None, :, None, :], sin[None, :, None, :]
            return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)

        return rot(query_states, self.num_heads), rot(key_states, self.num_key_value_heads)

    def wo(self, hidden_states, layer, bsz, seq_len, dim):
        return F.linear(hidden_states.reshape(bsz, seq_len, dim), layer.wo)

    def mlp(self, hidden_states, layer):
        gu = F.linear(hidden_states, layer.gate_up_proj)
        inter = gu.shape[-1] // 2
        return F.linear(F.silu(gu[..., :inter]) * gu[..., inter:], layer.down_proj)

    def decode_attention(self, query_states, key_states, value_states, layer_idx):
        return polar_decode_attn(query_states, key_states, value_states, layer_idx, self.kv_cache)

    # ------------------------------------------------------------------ decode (LLM.py:157-198, 228-243)
    def layer_decode(self, layer_idx, hidden_states):
        residual = hidden_states
        bsz, seq_len, _ = hidden_states.shape
        layer = self.layers[layer_idx]
        hidden_states = self.layernorm(hidden_states, layer.input_layernorm_variance_epsilon, layer.input_layernorm_weight)
        if seq_len == 1 and self.dtype == torch.bfloat16 and self.head_dim == 128 and layer.bqkv is None:
            # one token per sequence: head norms and rotary embedding of q and k in one launch
            qkv = F.linear(hidden_states, layer.wqkv)
            pos = self._position
            q, k = ops.qk_norm_rope(qkv, self.num_heads, self.num_key_value_heads, layer.q_norm_weight, layer.k_norm_weight,
                                    layer.q_norm_variance_epsilon or 0.0, self.cos_cache[pos], self.sin_cache[pos])
            v = qkv[..., (self.num_heads + self.num_key_value_heads) * self.head_dim:]
        else:
            q, k, v = self.wqkv(hidden_states, layer)
            q, k = self.position_embedd(q, k)
            q = q.view(bsz, -1, self.num_heads, self.head_dim)
            k = k.view(bsz, -1, self.num_key_value_heads, self.head_dim)
        v = v.reshape(bsz, -1, self.num_key_value_heads, self.head_dim)
        ranges.push("decode_update_kv_cache")
        k, v = self.kv_cache.decode_update_kv_cache(k, v, layer_idx)
        ranges.pop()
        ranges.push("decode_attention")
        attn_out = self.decode_attention(q, k, v, layer_idx)
        ranges.pop()
        attn_out_dim = attn_out.shape[-2] * attn_out.shape[-1]
        hidden_states = residual + self.wo(attn_out, layer, bsz, seq_len, attn_out_dim)
        residual = hidden_states
        hidden_states = self.layernorm(hidden_states, layer.post_attention_layernorm_variance_epsilon,
                                       layer.post_attention_layernorm_weight)
        return residual + self.mlp(hidden_states, layer)

    def _attention_block(self, layer_idx, normed):
        """QKV projection, head norms + rotary embedding, cache update and decode attention, output projection."""
        layer = self.layers[layer_idx]
        bsz, seq_len, _ = normed.shape
        qkv = F.linear(normed, layer.wqkv)
        pos = self._position
        # where this layer's step will retrieve, its vote table is built by the same launch that finishes the queries
        target = self.kv_cache.query_table_target(layer_idx) if hasattr(self.kv_cache, "query_table_target") else None
        # ... and it writes the token's K/V rows into the cache as well, where the cache's append is nothing more
        slot_rows = (self.kv_cache.fused_append_target(layer_idx)
                     if target is not None and hasattr(self.kv_cache, "fused_append_target") else None)
        q, k = ops.qk_norm_rope(qkv, self.num_heads, self.num_key_value_heads, layer.q_norm_weight, layer.k_norm_weight,
                                layer.q_norm_variance_epsilon or 0.0, self.cos_cache[pos], self.sin_cache[pos],
                                table_for=target, append=slot_rows)
        v = qkv[..., (self.num_heads + self.num_key_value_heads) * self.head_dim:].reshape(bsz, -1, self.num_key_value_heads,
                                                                                             self.head_dim)
        ranges.push("decode_update_kv_cache")  # the reference's ranges of the same names, model_hub/LLM.py:173-183
        if slot_rows is not None:
            k, v = self.kv_cache.decode_update_kv_cache(k, v, layer_idx, appended=True)
        else:
            k, v = self.kv_cache.decode_update_kv_cache(k, v, layer_idx)
        ranges.pop()
        ranges.push("decode_attention")
        attn_out = self.decode_attention(q, k, v, layer_idx)
        ranges.pop()
        return self.wo(attn_out, layer, bsz, seq_len, attn_out.shape[-2] * attn_out.shape[-1])

    def decode_forward(self, inputs_ids):
        """inputs_ids [bs, 1] -> logits [bs, 1, vocab] (fp32)."""
        hidden_states = self.word_embedding(inputs_ids)
        self._position = self.kv_cache.context
        fused = (hidden_states.shape[1] == 1 and self.dtype == torch.bfloat16 and self.head_dim == 128 and
                 self.hidden_size % 8 == 0 and self.hidden_size <= 16384 and all(ly.bqkv is None for ly in self.layers))
        if not fused:
            for ldx in range(self.num_layers):
                hidden_states = self.layer_decode(ldx, hidden_states)
            hidden_states = self.layernorm(hidden_states[:, -1:, :], self.norm_variance_epsilon, self.norm_weight)
            return self.lm(hidden_states)
        # One token per sequence in bf16: the same arithmetic with each residual add folded into the norm that follows
        # it (also across the layer boundary) and the MLP gate in one launch.
        x, pending = hidden_states.contiguous(), None   # residual stream, and what is still to be added to it
        for ldx, layer in enumerate(self.layers):
            x, normed = ops.add_rmsnorm(pending if pending is not None else x, x if pending is not None else None,
                                        layer.input_layernorm_weight, layer.input_layernorm_variance_epsilon)
            x, normed = ops.add_rmsnorm(self._attention_block(ldx, normed), x, layer.post_attention_layernorm_weight,
                                        layer.post_attention_layernorm_variance_epsilon)
            pending = F.linear(ops.silu_mul(F.linear(normed, layer.gate_up_proj)), layer.down_proj)
        _, normed = ops.add_rmsnorm(pending, x, self.norm_weight, self.norm_variance_epsilon, want_sum=False)
        return self.lm(normed)
