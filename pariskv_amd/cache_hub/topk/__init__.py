"""Top-k selections with the reference's call surface
(``cache_hub/topk/__init__.py:23-155``; extension functions
``radix_topk.cu:385-401``): ``load_radix_topk_ext()`` returns an object with
``bucket_topk``, ``bucket_topk_3d``, ``radix_topk``, ``radix_topk_3d``.

Differences that stay inside the reference's contract: results come in a fixed
order with a fixed tie rule (the reference's order and tie choice depend on
atomic timing), and ``radix_topk`` on floats is an exact top-k in descending
order (the reference bins floats to 8 bits and picks arbitrarily inside the
threshold bin)."""
from __future__ import annotations

from functools import lru_cache

import torch

from ... import ops


class _TopkExt:
    @staticmethod
    def bucket_topk(input: torch.Tensor, k: int) -> torch.Tensor:
        if input.dim() != 2:
            raise RuntimeError("input must be 2D [B, L]")
        return ops.bucket_topk(input, int(k))

    @staticmethod
    def bucket_topk_3d(input: torch.Tensor, k: int) -> torch.Tensor:
        if input.dim() != 3:
            raise RuntimeError("input must be 3D [bs, kv_heads, kv_len]")
        bs, h, n = input.shape
        return ops.bucket_topk(input.reshape(bs * h, n), int(k)).reshape(bs, h, int(k))

    @staticmethod
    def radix_topk(input: torch.Tensor, k: int) -> torch.Tensor:
        if input.dim() != 2:
            raise RuntimeError("input must be 2D [B, L]")
        if not input.is_cuda:
            raise RuntimeError("input must be on CUDA")
        if input.dtype in (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8):
            return ops.bucket_topk(input, int(k))  # the hot call: collision counts (polar_cache.py:1241)
        return ops.topk_f32(input, int(k))

    @staticmethod
    def radix_topk_3d(input: torch.Tensor, k: int) -> torch.Tensor:
        if input.dim() != 3:
            raise RuntimeError("input must be 3D [bs, kv_heads, kv_len]")
        bs, h, n = input.shape
        return _TopkExt.radix_topk(input.reshape(bs * h, n), int(k)).reshape(bs, h, int(k))


@lru_cache()
def load_radix_topk_ext(verbose: bool = False):
    return _TopkExt()


def bucket_topk(input: torch.Tensor, k: int) -> torch.Tensor:
    assert input.is_cuda, "input must be on CUDA"
    assert k > 0, f"k must be positive, got {k}"
    ext = load_radix_topk_ext()
    if input.dim() == 2:
        return ext.bucket_topk(input, k)
    if input.dim() == 3:
        return ext.bucket_topk_3d(input, k)
    raise ValueError(f"input must be 2D or 3D, got {input.dim()}D")


def radix_topk(input: torch.Tensor, k: int) -> torch.Tensor:
    assert input.is_cuda, "input must be on CUDA"
    assert k > 0, f"k must be positive, got {k}"
    ext = load_radix_topk_ext()
    if input.dim() == 2:
        return ext.radix_topk(input, k)
    if input.dim() == 3:
        return ext.radix_topk_3d(input, k)
    raise ValueError(f"input must be 2D or 3D, got {input.dim()}D")


def fast_topk(input: torch.Tensor, k: int) -> torch.Tensor:
    if input.dtype in (torch.int32, torch.int64, torch.int16, torch.int8):
        return bucket_topk(input.int(), k)
    return radix_topk(input, k)


def fast_topk_with_ratio(input: torch.Tensor, ratio: float) -> torch.Tensor:
    if input.dim() not in (2, 3):
        raise ValueError(f"input must be 2D or 3D, got {input.dim()}D")
    return fast_topk(input, max(1, int(input.size(-1) * ratio)))
