"""Library-routine restatements of the reference's torch expressions.

These follow the *structure* of the reference's own torch code (vector_norm,
bucketize, gather/cumsum/compare, topk, argsort, bincount ...) on CPU tensors,
with the Hadamard transform taken as the textbook ``x @ H_128``
(``scipy.linalg.hadamard``).  They exist to pin the C oracle: a dropped term, a
wrong sign or a transposed index in the oracle disagrees with these.  Summation
order inside torch reductions is backend-defined, so comparisons that depend on
the last ulp are made as match *rates*, everything else exactly.
"""
from __future__ import annotations

import math

import numpy as np
import scipy.linalg
import torch

H128 = torch.from_numpy(scipy.linalg.hadamard(128).astype(np.float32))
SCALE = 1.0 / math.sqrt(128)

MAG_THRESHOLDS = [0.0843, 0.1698, 0.2578, 0.3499, 0.4487, 0.5585, 0.6901]  # polar_cache.py:189
MAG_CENTERS = [0.0420, 0.1266, 0.2130, 0.3025, 0.3973, 0.5001, 0.6169, 0.7633]  # polar_cache.py:192


def hadamard_transform(x: torch.Tensor, scale: float) -> torch.Tensor:
    """Contract of fast_hadamard_transform.hadamard_transform: fp32 inside,
    result in the input dtype."""
    return ((x.float() @ H128) * scale).to(x.dtype)


def pack_4bit(signs, magnitudes):  # polar_cache.py:887-893
    v4 = (signs.to(torch.uint8) << 3) | magnitudes
    return ((v4[..., 1::2] << 4) | v4[..., 0::2]).to(torch.uint8).contiguous()


def unpack_4bit(packed, m=8):  # polar_cache.py:895-903
    v_even = packed & 0x0F
    v_odd = (packed >> 4) & 0x0F
    v4 = torch.stack([v_even, v_odd], dim=-1).view(*packed.shape[:-1], m)
    s_sign = (2 * ((v4 >> 3) & 1).to(torch.int16) - 1).to(torch.int8)
    return s_sign, (v4 & 0x7).to(torch.int64)


def batch_encode(Y: torch.Tensor, signs: torch.Tensor):
    """polar_cache.py:924-978 on a [..., seq, 128] CPU tensor (fp32 or bf16).
    Returns key-major codes [...,seq,16], packed [...,seq,16,4], weight [...,seq,16] (bf16)."""
    dt = Y.dtype
    thr = torch.tensor(MAG_THRESHOLDS, dtype=torch.bfloat16).to(dt)
    cen = torch.tensor(MAG_CENTERS, dtype=torch.bfloat16).to(dt)
    shifts = (1 << torch.arange(8)).to(torch.uint8)
    key_norm = torch.linalg.vector_norm(Y, ord=2, dim=-1, keepdim=True)
    Yn = Y / key_norm.clamp(min=1e-8)
    key_norm = key_norm.squeeze(-1)
    Yr = hadamard_transform(Yn * signs.to(dt), SCALE)
    Yb = Yr.view(*Y.shape[:-1], 16, 8)
    bits = Yb >= 0
    codes = (bits * shifts).sum(dim=-1, dtype=torch.uint8)
    radii = torch.linalg.vector_norm(Yb, ord=2, dim=-1)
    directions = Yb / radii.unsqueeze(-1).clamp(min=1e-8)
    abs_u = directions.abs()
    t_codes = torch.bucketize(abs_u, thr)
    a_vals = cen[t_codes]
    packed = pack_4bit(bits, t_codes.to(torch.uint8))
    alpha = (a_vals * abs_u).sum(dim=-1, dtype=torch.float32).clamp(min=1e-6)
    weight = ((radii / alpha) * key_norm.unsqueeze(-1)).to(torch.bfloat16)
    return codes, packed, weight


def encode_query(q_heads: torch.Tensor, signs: torch.Tensor):
    """polar_cache.py:1027-1031 + 905-922.  q_heads [G,128] -> (qhat [128], qnorm)."""
    dt = q_heads.dtype
    q = q_heads.mean(dim=0)
    qn = torch.linalg.vector_norm(q, ord=2, dim=-1, keepdim=True)
    y = hadamard_transform((q / qn.clamp(min=1e-8)) * signs.to(dt), SCALE)
    return y, qn


def centroid_scores(qhat: torch.Tensor):
    """polar_cache.py:1216: q_blocks @ V^T with the enumeration codebook."""
    V = torch.tensor([[1.0 if (c >> j) & 1 else -1.0 for j in range(8)] for c in range(256)]).to(qhat.dtype)
    return torch.matmul(qhat.view(16, 8), V.T)


def update_cache_cnt_overall(sorted_cluster_ids, cluster_key_counts, codebook, tier_ratios, kv_len, collision_ratio):
    """Structure of collision_fused/collision_test.py:56-98 (gather -> cumsum ->
    exclusive -> threshold mask -> per-tier membership sum); tensors are
    [.., B, K] / [.., B, N] with any leading dims."""
    sorted_key_counts = torch.gather(cluster_key_counts, dim=-1, index=sorted_cluster_ids.long())
    before = torch.cumsum(sorted_key_counts, dim=-1) - sorted_key_counts
    total = None
    K = sorted_cluster_ids.shape[-1]
    for ratio in tier_ratios:
        target = math.ceil(kv_len * collision_ratio * ratio)
        n_sel = (before < target).sum(dim=-1)  # clusters in this tier
        sel = sorted_cluster_ids.clone()
        sel[torch.arange(K).expand_as(sel) >= n_sel.unsqueeze(-1)] = -1
        member = torch.zeros(*sel.shape[:-1], K + 1, dtype=torch.int32)
        member.scatter_(-1, torch.where(sel < 0, torch.full_like(sel, K), sel).long(), 1)
        member = member[..., :K]
        tier_cnt = torch.gather(member, -1, codebook.long()).sum(dim=-2)
        total = tier_cnt if total is None else total + tier_cnt
    return total.to(torch.int32)


def rerank_scores(coarse_indices, key_4bit, key_block_weight, q_blocks, q_norm, mag_centers):
    """polar_cache.py:1281-1298 for one row: key_4bit [16,N,4], weight [16,N],
    q_blocks [16,8], indices [C]."""
    B = 16
    idx_code = coarse_indices.unsqueeze(0).expand(B, -1)
    cand_weight = torch.gather(key_block_weight, dim=1, index=idx_code)
    idx_4bit = coarse_indices.view(1, -1, 1).expand(B, -1, key_4bit.shape[-1])
    cand_4bit = torch.gather(key_4bit, dim=1, index=idx_4bit)
    s_sign, t_codes = unpack_4bit(cand_4bit.reshape(-1, 4))
    s_sign = s_sign.view(B, -1, 8)
    t_codes = t_codes.view(B, -1, 8)
    v4b = mag_centers[t_codes] * s_sign.to(mag_centers.dtype)
    per_block = (q_blocks.unsqueeze(1) * v4b).sum(dim=-1)
    return (per_block * cand_weight).sum(dim=0) * q_norm


def adaptive_topk(logits_sl, sl_vnorm, logits_cand, cand_indices, cand_vnorm, threshold, topk_cap):
    """adaptive_k_fused/adaptive_topk.py:282-311 from the logits on (one row, fp32)."""
    K_out = min(topk_cap, logits_cand.shape[-1])
    joint_max = torch.cat([logits_sl, logits_cand], dim=-1).amax(dim=-1, keepdim=True)
    exp_sl = torch.exp(logits_sl - joint_max)
    exp_cand = torch.exp(logits_cand - joint_max)
    sl_benefit = (exp_sl * sl_vnorm).sum(dim=-1, keepdim=True)
    cand_benefit = exp_cand * cand_vnorm
    top, perm = torch.topk(cand_benefit, k=K_out, dim=-1, largest=True, sorted=True)
    cumsum = torch.cumsum(top, dim=-1)
    total = sl_benefit + cand_benefit.sum(dim=-1, keepdim=True)
    reached = sl_benefit + cumsum >= threshold * total
    k = int(reached.long().argmax(dim=-1)) + 1
    if not bool(reached.any()):
        k = K_out
    if float(total) <= 0:
        k = 1
    return k, cand_indices[perm], cand_benefit
