"""Seeded synthetic workloads shared by the GPU parity tests, smoke() and bench.py.

Keys ~N(0,1) with four fixed outlier channels x10, queries = key mean + N(0,0.5)
(one per q-head), encoded on the CPU by the oracle.  Everything is numpy; the
callers move what they need to the GPU.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np

from oracle import pkv_oracle as O


@dataclass
class Workload:
    name: str
    bs: int
    H: int
    G: int
    N: int
    C: int
    K: int
    dtype: int  # O.F32 / O.BF16
    collision_ratio: float
    signs: np.ndarray
    keys: np.ndarray      # [R, N, 128] f32 (bf16-representable when dtype == BF16)
    values: np.ndarray    # [R, N, 128] f32
    queries: np.ndarray   # [bs, H*G, 128] f32
    codes: np.ndarray     # [R, N, 16] u8
    nib: np.ndarray       # [R, N, 16, 4] u8
    weight: np.ndarray    # [R, N, 16] f32 (bf16 values)
    cluster_counts: np.ndarray  # [R, 16, 256] i32
    tiers: list = field(default_factory=list)

    @property
    def R(self):
        return self.bs * self.H


def make_workload(name, bs, H, G, N, C, K, dtype, collision_ratio, seed0=0, drift=0.0, with_values=True) -> Workload:
    signs = O.srht_signs(42)
    R = bs * H
    bf = dtype == O.BF16
    keys = np.empty((R, N, 128), np.float32)
    values = np.empty((R, N, 128), np.float32) if with_values else np.zeros((0, 0, 128), np.float32)
    queries = np.empty((bs, H * G, 128), np.float32)
    codes = np.empty((R, N, 16), np.uint8)
    nib = np.empty((R, N, 16, 4), np.uint8)
    weight = np.empty((R, N, 16), np.float32)
    cc = np.zeros((R, 16, 256), np.int32)
    for b in range(bs):
        for h in range(H):
            r = b * H + h
            seed = (seed0 + b) * 1000 + h  # independent seed per sequence and head
            keys[r] = O.synth_keys(N, seed, bf16=bf, drift_deg_per_1k=drift)
            if with_values:
                rng = np.random.default_rng(seed + 77)
                v = rng.standard_normal((N, 128), dtype=np.float32)
                values[r] = O.bf16_round(v) if bf else v
            queries[b, h * G:(h + 1) * G] = O.synth_queries(keys[r], G, seed, bf16=bf)
            codes[r], nib[r], weight[r] = O.encode(keys[r], signs, dtype)
            O.count_cluster_keys(codes[r], cc[r])
    tiers = O.tier_counts(N, collision_ratio)
    return Workload(name, bs, H, G, N, C, K, dtype, collision_ratio, signs, keys, values, queries, codes, nib, weight, cc,
                    tiers)


def oracle_stages(w: Workload, row: int):
    """Every intermediate of the retrieval for one row, from the oracle."""
    b, h = divmod(row, w.H)
    q = w.queries[b, h * w.G:(h + 1) * w.G]
    qhat, qn = O.query_prep(q, w.signs, w.dtype)
    ids = O.rank_centroids(qhat, w.dtype)
    lut = O.tier_lut(ids, w.cluster_counts[row], w.tiers)
    cnt = O.collision_count(w.codes[row], lut)
    cand, theta = O.select_candidates(cnt, w.C)
    scores = O.rerank(cand, w.nib[row], w.weight[row], qhat, qn)
    final, pos = O.topk_f32(scores, cand, min(w.K, w.C))
    return dict(qhat=qhat, qnorm=qn, sorted_ids=ids, lut=lut, cnt=cnt, cand=cand, theta=theta, scores=scores,
                final=final, final_scores=scores[pos])


# BASELINE.json configs (1-3) at their stated shapes
def cfg1():
    return make_workload("cfg1", 1, 8, 4, 8192, 1024, 256, O.F32, 0.3, seed0=0)


def cfg2():
    return make_workload("cfg2", 1, 8, 4, 32768, 2048, 512, O.BF16, 0.2, seed0=0)


def cfg3(with_values=True):
    return make_workload("cfg3", 4, 8, 4, 131072, 4096, 1024, O.BF16, 0.2, seed0=0, with_values=with_values)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 array of bf16-representable values -> uint16 bit patterns."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def to_device(w: Workload, device, torch):
    """Key-major GPU tensors of a workload: dict(signs, centers, cluster_counts, codes_km, nib_km, w_km,
    queries (dtype of the workload))."""
    tdt = torch.bfloat16 if w.dtype == O.BF16 else torch.float32
    R, N = w.R, w.N
    codes = torch.from_numpy(w.codes.reshape(w.bs, w.H, N, 16)).to(device)
    nib = torch.from_numpy(w.nib.reshape(w.bs, w.H, N, 64)).to(device)
    wt = torch.from_numpy(f32_to_bf16_bits(w.weight).view(np.int16).reshape(w.bs, w.H, N, 16)).to(device).view(torch.bfloat16)
    return dict(
        signs=torch.from_numpy(w.signs).to(device),
        centers=torch.from_numpy(O.mag_constants()[1]).to(device),
        cluster_counts=torch.from_numpy(w.cluster_counts.reshape(w.bs, w.H, 16, 256)).to(device),
        codes_km=codes, nib_km=nib, w_km=wt,
        queries=torch.from_numpy(w.queries).to(tdt).to(device).view(w.bs, 1, w.H * w.G, 128),
    )
