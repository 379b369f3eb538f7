"""Host-side KV gather, call surface of the reference's
``cache_hub/gather/cpp_gather.py:10-41`` / ``gather_cpu.cpp:116-174``."""
from __future__ import annotations

from functools import lru_cache

import torch

from ... import ops


class _GatherExt:
    @staticmethod
    def gather_kv_out_cpu(src: torch.Tensor, index: torch.Tensor, out: torch.Tensor) -> None:
        """src [B,H,N,D] (CPU), index int64 [B,H,K] (CPU), out [B,H,K,D] (CPU, preallocated)."""
        ops.gather_cpu(src, index, out, n_threads=torch.get_num_threads())


@lru_cache()
def load_gather_ext(verbose: bool = False):
    return _GatherExt()
