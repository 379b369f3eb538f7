"""Tiered collision vote, same call surface as the reference's
``cache_hub/collision_fused/collison_interface.py:60-86`` (module name spelled as
there).  The work is done by ``pkv_update_cache_cnt`` in libpariskv_hip.so."""
from __future__ import annotations

import torch

from ... import _lib, ops


def load_kernel_module(path=None, name=None, **_ignored):
    """The reference JIT-compiles its extension here (``:19-57``); this build is
    compiled ahead of time, so loading just returns the shared library."""
    return _lib.lib()


def update_cache_cnt_cuda_interface(sorted_cluster_ids, cluster_key_counts, codebook, tier_counts) -> torch.Tensor:
    """Per-key collision counts.

    Args:
        sorted_cluster_ids: int64 [bs, kv_heads, B, num_clusters], best cluster first
        cluster_key_counts: int32 [bs, kv_heads, B, num_clusters], keys per cluster
        codebook: uint8 [bs, kv_heads, B, kv_len], cluster id per key per subspace
            (any strides: the reference requires stride(3) == 1, key-major views work too)
        tier_counts: list of 1 or 6 cumulative key thresholds
    Returns:
        cache_cnt: int32 [bs, kv_heads, kv_len]
    """
    return ops.update_cache_cnt(sorted_cluster_ids, cluster_key_counts, codebook, list(tier_counts))
