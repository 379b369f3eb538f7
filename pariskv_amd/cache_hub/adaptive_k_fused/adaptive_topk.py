"""Adaptive top-k selection (value-weighted), call surface of the reference's
``cache_hub/adaptive_k_fused/adaptive_topk.py:331-405``.

For every (batch, kv-head): benefit_i = exp(l_i - max l) * ||v_i||; the candidates are
ordered by benefit and the shortest prefix whose benefit, together with the dense
(sink/local/buffer) tokens', reaches ``threshold`` of the total is kept."""
from __future__ import annotations

from typing import Any, Tuple

import torch

from ... import _lib, ops


def load_kernel_module(path=None, name=None, **_ignored) -> Any:
    return _lib.lib()


def adaptive_topk_cuda(query_avg: torch.Tensor, sink_local_keys: torch.Tensor, sl_vnorm: torch.Tensor,
                       cand_scores: torch.Tensor, cand_indices: torch.Tensor, cand_vnorm: torch.Tensor,
                       attn_scale: float, threshold: float, topk_cap: int, kernel: Any = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (adaptive_k int64 [bs,H], topk_indices int64 [bs,H,min(topk_cap,C)]): the first
    adaptive_k[b,h] entries are the kept candidates in descending benefit order (ties: candidate
    position ascending; the reference leaves tie order open)."""
    bs, kv_heads, head_dim = query_avg.shape
    sl_len = sink_local_keys.shape[2]
    cand_len = cand_scores.shape[-1]
    K_out = min(topk_cap, cand_len)
    assert query_avg.dtype == torch.bfloat16, f"query_avg dtype: expected bf16, got {query_avg.dtype}"
    assert sink_local_keys.dtype == torch.bfloat16, f"sink_local_keys dtype: expected bf16, got {sink_local_keys.dtype}"
    assert sl_vnorm.dtype == torch.float32, f"sl_vnorm dtype: expected fp32, got {sl_vnorm.dtype}"
    assert cand_scores.dtype == torch.bfloat16, f"cand_scores dtype: expected bf16, got {cand_scores.dtype}"
    assert cand_indices.dtype == torch.int64, f"cand_indices dtype: expected int64, got {cand_indices.dtype}"
    assert cand_vnorm.dtype == torch.float32, f"cand_vnorm dtype: expected fp32, got {cand_vnorm.dtype}"
    for name, t in [("query_avg", query_avg), ("sink_local_keys", sink_local_keys), ("sl_vnorm", sl_vnorm),
                    ("cand_scores", cand_scores), ("cand_indices", cand_indices), ("cand_vnorm", cand_vnorm)]:
        assert t.is_cuda, f"{name} must be on CUDA, got {t.device}"
        assert t.is_contiguous(), f"{name} must be contiguous"
    assert sink_local_keys.shape == (bs, kv_heads, sl_len, head_dim)
    assert sl_vnorm.shape == (bs, kv_heads, sl_len)
    assert cand_scores.shape == cand_indices.shape == cand_vnorm.shape == (bs, kv_heads, cand_len)
    assert 0.0 < threshold <= 1.0, f"threshold must be in (0, 1], got {threshold}"
    assert topk_cap > 0, f"topk_cap must be > 0, got {topk_cap}"
    assert attn_scale > 0, f"attn_scale must be > 0, got {attn_scale}"
    # logits of the dense tokens (reference :383-386: einsum + cast + scale, four launches): one launch of
    # pkv_dense_logits; a [bs,H,D] mean query is a query group of one head
    sl_logits = ops.dense_logits(query_avg, sink_local_keys, sl_len, float(attn_scale))
    return ops.adaptive_topk(sl_logits, sl_vnorm, cand_scores, float(attn_scale), cand_indices, float(threshold),
                             int(K_out), cand_vnorm=cand_vnorm)
