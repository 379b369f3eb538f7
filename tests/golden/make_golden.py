#!/usr/bin/env python3
"""Writes tests/golden/retrieval_small.npz: seeded inputs and every intermediate of one small retrieval
(2 rows x 1024 keys, bf16 chain), computed by the CPU oracle AFTER its pin tests pass (tests/test_oracle_*.py).
The file freezes the pinned oracle: a later edit that shifts the oracle and the kernels together still fails
against it.  Run from the repository root:  python tests/golden/make_golden.py"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests")]

import workloads as W  # noqa: E402
from oracle import pkv_oracle as O  # noqa: E402


def small_workload():
    return W.make_workload("golden_small", 1, 2, 4, 1024, 128, 32, O.BF16, 0.5, seed0=5)


def main():
    O.build()
    w = small_workload()
    # keys: only the first 128 of every row (enough to pin the encoder); K/V rows: only the selected ones
    out = dict(signs=w.signs, keys_head_bf16=W.f32_to_bf16_bits(w.keys[:, :128]), queries_bf16=W.f32_to_bf16_bits(w.queries),
               codes=w.codes, nib=w.nib, weight_bf16=W.f32_to_bf16_bits(w.weight), cluster_counts=w.cluster_counts,
               tiers=np.asarray(w.tiers, np.int64), n_cand=np.int64(w.C), k=np.int64(w.K))
    for r in range(w.R):
        st = W.oracle_stages(w, r)
        for name in ("qhat", "sorted_ids", "lut", "cnt", "cand", "scores", "final", "final_scores"):
            out[f"row{r}_{name}"] = np.asarray(st[name])
        out[f"row{r}_qnorm"] = np.float32(st["qnorm"])
        out[f"row{r}_theta"] = np.int64(st["theta"])
        b, h = divmod(r, w.H)
        sel = st["final"]
        out[f"row{r}_sel_k_bf16"] = W.f32_to_bf16_bits(w.keys[r][sel])
        out[f"row{r}_sel_v_bf16"] = W.f32_to_bf16_bits(w.values[r][sel])
        out[f"row{r}_attn"] = O.attention(w.queries[b, h * w.G:(h + 1) * w.G], w.keys[r][sel], w.values[r][sel])
    np.savez_compressed(os.path.join(HERE, "retrieval_small.npz"), **out)
    print("wrote", os.path.join(HERE, "retrieval_small.npz"))


if __name__ == "__main__":
    main()
