"""UVA gather of selected K/V rows out of pinned host memory, call surface of
the reference's ``cache_hub/gather_trans/trans_h2d.py:65-105``."""
from __future__ import annotations

import torch

from ... import ops


def h2d_gather_kv(src_k_caches, src_v_caches, selected_indices, dst_k_caches, dst_v_caches) -> None:
    """src [bs,heads,kv_len,128] pinned CPU bf16; selected_indices int64 [bs,heads,topk] on the
    GPU; dst [bs,heads,>=topk,128] on the GPU.  dst[b,h,i] = src[b,h,idx[b,h,i]]."""
    bs, heads, kv_len, dim = src_k_caches.shape
    assert src_k_caches.shape == src_v_caches.shape
    _, _, topk = selected_indices.shape
    assert dst_k_caches.shape == dst_v_caches.shape
    assert dst_k_caches.shape[-2] >= topk
    assert dim == 128
    assert src_k_caches.is_cpu and src_v_caches.is_cpu
    assert src_k_caches.is_pinned() and src_v_caches.is_pinned()
    assert dst_k_caches.is_cuda and dst_v_caches.is_cuda
    assert src_k_caches.dtype == src_v_caches.dtype == dst_k_caches.dtype == dst_v_caches.dtype
    assert src_k_caches.dtype == torch.bfloat16
    assert src_k_caches.is_contiguous() and dst_k_caches.is_contiguous()
    assert src_v_caches.is_contiguous() and dst_v_caches.is_contiguous()
    ops.gather_uva(src_k_caches, src_v_caches, selected_indices.contiguous(), dst_k_caches, dst_v_caches)
