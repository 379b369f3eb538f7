"""4-bit RaBitQ-style rerank, call surface of the reference's
``cache_hub/rerank/rerank.py:172-263``."""
from __future__ import annotations

import torch

from ... import _lib, ops


def load_kernel_module(path=None, name=None, **_ignored):
    """Ahead-of-time build: returns the loaded shared library (reference: JIT, ``:172-211``)."""
    return _lib.lib()


def query_blocks_to_f32(q_blocks: torch.Tensor, q_norm: torch.Tensor):
    bs, H = q_blocks.shape[:2]
    return (q_blocks.reshape(bs, H, 128).to(torch.float32).contiguous(),
            q_norm.reshape(bs, H).to(torch.float32).contiguous())


def partial_rerank_cuda(coarse_indices, key_4bit, key_block_weight, q_blocks, q_norm, mag_centers, B, m, kernel=None,
                        return_v4b: bool = True) -> tuple:
    """Gather + unpack + score the candidates.

    Same arguments as the reference (``q_blocks`` / ``q_norm`` / ``mag_centers``
    may be bf16 or fp32).  Returns ``(approx_scores [bs,H,C], v4b)``; the scores
    are fp32 evaluated in one fixed order rather than bf16 rounded after every
    operation (``rerank.cu:85,127-134``), and within 1e-5 relative of the fp32
    value of the same expression.  ``v4b`` is the unpacked bf16 values
    ``[bs,H,B,C,m]`` as in the reference (skipped with ``return_v4b=False``;
    ``polar_cache`` never reads it)."""
    if B != 16 or m != 8:
        raise RuntimeError("only support B = 16")  # rerank.cu:203-214
    assert coarse_indices.dtype == torch.int64, f"coarse_indices must be int64, got {coarse_indices.dtype}"
    assert coarse_indices.is_contiguous()
    assert key_4bit.stride(-1) == 1
    qhat, qn = query_blocks_to_f32(q_blocks, q_norm)
    centers = mag_centers.to(torch.float32).contiguous()
    scores, v4b = ops.rerank4(coarse_indices, key_4bit, key_block_weight, qhat, qn, centers, want_v4b=return_v4b)
    return scores, v4b


def _coarse_filter_truncate(cache_cnt: torch.Tensor, candidate_ratio: float) -> tuple:
    """Top ``ceil(kv_len * candidate_ratio)`` keys by vote count (reference ``:119-124``).  Returns
    ``(coarse_indices int64 [bs,H,C], C)``; fixed order: counts above the threshold by ascending key, then the
    ties at the threshold by ascending key."""
    import math

    bs, H, kv_len = cache_cnt.shape
    n_cand = max(1, int(math.ceil(kv_len * candidate_ratio)))
    idx = ops.bucket_topk(cache_cnt.reshape(bs * H, kv_len), n_cand)
    return idx.view(bs, H, n_cand), n_cand


def rerank_rabitq_fused(cache_cnt, key_4bit, key_block_weight, q_blocks, q_norm, mag_centers, candidate_ratio: float,
                        final_topk: int, B: int, m: int) -> tuple:
    """Coarse filter by vote count, 4-bit rerank, final top-k (reference ``:266-293``).  Returns
    ``(final_indices [bs,H,final_topk], approx_scores, v4b)``; the last two are ``None`` when the candidate set is
    not larger than ``final_topk``."""
    coarse_indices, max_candidates = _coarse_filter_truncate(cache_cnt, candidate_ratio)
    if max_candidates <= final_topk:
        return coarse_indices[:, :, :final_topk], None, None
    approx_scores, v4b = partial_rerank_cuda(coarse_indices, key_4bit, key_block_weight, q_blocks, q_norm, mag_centers, B, m)
    bs, H, C = approx_scores.shape
    final = ops.topk_f32(approx_scores.view(bs * H, C), final_topk, ids=coarse_indices.view(bs * H, C))
    final_indices = final[0] if isinstance(final, tuple) else final
    return final_indices.view(bs, H, final_topk), approx_scores, v4b
