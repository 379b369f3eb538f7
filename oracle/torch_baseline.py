"""Torch-CPU restatement of one layer's retrieval for a decode step, batched over every (batch, kv-head) row.

TEST INFRASTRUCTURE / REPORTED BASELINE ONLY: timed by the ``cpu_baseline`` leg of ``bench.py`` on the host's own
cores and compared with the C oracle in ``tests/``.  The product package never imports this module.

It follows the structure of the reference's torch code on its own subspace-major tensors
(``cache_hub/polar_cache.py:288-307``): query prep (:1027-1031, :905-922), centroid scores by matmul and ``argsort``
(:1216-1217), tiered collision vote (``collision_fused/collision_test.py:56-98``: gather the cluster sizes in ranked
order, exclusive cumsum, threshold masks; the six membership masks are summed into one vote table before the per-key
gather, which changes no result), candidate ``topk`` (:1239-1241), 4-bit rerank (:1281-1298), final ``topk`` +
``gather`` (:1300-1302) and the host row gather (``gather_trans/trans_h2d.py:129-139``).  The Hadamard transform is
the textbook ``x @ H_128`` (the reference's third-party kernel is not installed).  Ties are broken by torch, not by
the build's fixed rule, so index sets can differ from the oracle's where votes or scores tie.
"""
from __future__ import annotations

import math

import numpy as np
import scipy.linalg
import torch

_H128 = torch.from_numpy(scipy.linalg.hadamard(128).astype(np.float32))
_SCALE = 1.0 / math.sqrt(128)
_V = torch.tensor([[1.0 if (c >> j) & 1 else -1.0 for j in range(8)] for c in range(256)])
MAG_CENTERS = [0.0420, 0.1266, 0.2130, 0.3025, 0.3973, 0.5001, 0.6169, 0.7633]  # polar_cache.py:192


def retrieve_layer(q, signs, codebook, key_4bit, key_block_weight, cluster_key_counts, tier_counts, n_cand, k,
                   keys_cpu=None, values_cpu=None):
    """q [bs,1,Hq,128]; codebook u8 [bs,H,16,N]; key_4bit u8 [bs,H,16,N,4]; key_block_weight bf16 [bs,H,16,N];
    cluster_key_counts int32 [bs,H,16,256]; tier_counts: 6 cumulative key budgets.  Returns (final ids int64 [bs,H,k],
    gathered K, gathered V or None)."""
    bs, H, B, N = codebook.shape
    dt = q.dtype
    G = q.shape[2] // H
    # query prep
    q_avg = q.view(bs, H, G, 128).mean(dim=2)
    q_norm = torch.linalg.vector_norm(q_avg, ord=2, dim=-1, keepdim=True)
    q_unit = (q_avg / q_norm.clamp(min=1e-8)) * signs.to(dt)
    q_hat = ((q_unit.float() @ _H128) * _SCALE).to(dt)
    q_blocks = q_hat.view(bs, H, B, 8)
    # centroid ranking
    scores = torch.matmul(q_blocks, _V.to(dt).T)                       # [bs,H,16,256]
    sorted_ids = torch.argsort(scores, dim=-1, descending=True)
    # tiered vote table: weight[c] = number of tiers whose key budget is not exhausted at c's rank
    sorted_counts = torch.gather(cluster_key_counts, -1, sorted_ids)
    before = torch.cumsum(sorted_counts, dim=-1) - sorted_counts
    votes_ranked = torch.zeros_like(before, dtype=torch.int32)
    for t in tier_counts:
        votes_ranked += (before < int(t)).to(torch.int32)
    lut = torch.zeros_like(votes_ranked)
    lut.scatter_(-1, sorted_ids, votes_ranked)
    # collision count per key
    cache_cnt = torch.gather(lut, -1, codebook.long()).sum(dim=-2)     # [bs,H,N]
    # candidates
    coarse = torch.topk(cache_cnt.float(), n_cand, dim=-1).indices     # [bs,H,C]
    # 4-bit rerank
    idx = coarse.unsqueeze(2).expand(bs, H, B, n_cand)
    cand_w = torch.gather(key_block_weight, 3, idx)
    cand_4 = torch.gather(key_4bit, 3, idx.unsqueeze(-1).expand(bs, H, B, n_cand, 4))
    v4 = torch.stack([cand_4 & 0x0F, (cand_4 >> 4) & 0x0F], dim=-1).view(bs, H, B, n_cand, 8)
    sign = (2 * ((v4 >> 3) & 1).to(torch.int16) - 1).to(dt)
    centers = torch.tensor(MAG_CENTERS, dtype=torch.bfloat16).to(dt)
    v4b = centers[(v4 & 0x7).long()] * sign
    per_block = (q_blocks.unsqueeze(3) * v4b).sum(dim=-1)              # [bs,H,16,C]
    approx = (per_block * cand_w).sum(dim=2) * q_norm                  # [bs,H,C]
    # final top-k
    top = torch.topk(approx, min(k, n_cand), dim=-1).indices
    final = torch.gather(coarse, -1, top)
    gk = gv = None
    if keys_cpu is not None:
        gi = final.unsqueeze(-1).expand(bs, H, final.shape[-1], 128)
        gk, gv = torch.gather(keys_cpu, 2, gi), torch.gather(values_cpu, 2, gi)
    return final, gk, gv
