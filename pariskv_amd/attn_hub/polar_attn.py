"""Attention entry points of the PolarANN path (reference: ``attn_hub/polar_attn.py:8-62``)."""
import torch
import torch.nn.functional as F


def polar_prefill_attn(query_states, key_states, value_states, causal):
    """Dense prefill attention.  [bs, S, Hq, D] x [bs, S, Hkv, D] -> [bs, S, Hq, D].
    The reference calls flash-attn here; this build uses torch's fused SDPA."""
    q = query_states.transpose(1, 2)
    k = key_states.transpose(1, 2)
    v = value_states.transpose(1, 2)
    out = F.scaled_dot_product_attention(q, k, v, is_causal=bool(causal), enable_gqa=q.shape[1] != k.shape[1])
    return out.transpose(1, 2).contiguous()


def polar_decode_attn(query_states, key_states, value_states, layer_idx, kv_cache):
    """Decode attention through the cache's retrieval path: ``kv_cache.compute(q, layer_idx)``."""
    if kv_cache is None or not hasattr(kv_cache, "compute") or not callable(getattr(kv_cache, "compute")):
        raise TypeError(
            "polar_decode_attn expects kv_cache to provide a callable compute(query_states, layer_idx), "
            f"but got {type(kv_cache).__module__}.{type(kv_cache).__name__}.")
    return kv_cache.compute(query_states.contiguous(), layer_idx)
