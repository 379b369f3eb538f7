"""Legacy single-tier collision count, call surface of the reference's
``cache_hub/collision/collision.py:87-98``."""
from __future__ import annotations

import torch

from ... import ops


def update_cache_cnt_cuda(sorted_cluster_ids, topk_cluster_cnt, codebook) -> torch.Tensor:
    """sorted_cluster_ids int32 [bs,H,B,K], topk_cluster_cnt int32 [bs,H,B],
    codebook int32 [bs,H,B,kv_len] -> int32 [bs,H,kv_len]: the number of
    subspaces whose code is among the first ``topk_cluster_cnt`` ranked clusters."""
    return ops.update_cache_cnt_legacy(sorted_cluster_ids.contiguous(), topk_cluster_cnt.contiguous(),
                                       codebook.contiguous())
