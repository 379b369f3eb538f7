"""The frozen fixture tests/golden/retrieval_small.npz (written by tests/golden/make_golden.py from the pinned
oracle): the oracle must still reproduce it (CPU), and the HIP path must reproduce it through the C ABI (GPU)."""
import os

import numpy as np
import pytest

from oracle import pkv_oracle as O

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "retrieval_small.npz")
BS, H, G, N = 1, 2, 4, 1024


def _bf16(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


@pytest.fixture(scope="module")
def fx():
    return np.load(FIX)


def test_oracle_reproduces_the_fixture(fx):
    signs = fx["signs"]
    assert np.array_equal(signs, O.srht_signs(42))
    q = _bf16(fx["queries_bf16"])
    tiers = [int(t) for t in fx["tiers"]]
    assert tiers == O.tier_counts(N, 0.5)
    n_cand, k = int(fx["n_cand"]), int(fx["k"])
    weight = _bf16(fx["weight_bf16"])
    for r in range(BS * H):
        ec, en, ew = O.encode(_bf16(fx["keys_head_bf16"][r]), signs, O.BF16)
        assert np.array_equal(ec, fx["codes"][r, :128]) and np.array_equal(en, fx["nib"][r, :128])
        assert np.array_equal(ew, weight[r, :128])
        assert np.array_equal(O.count_cluster_keys(fx["codes"][r]), fx["cluster_counts"][r])
        qh, qn = O.query_prep(q[0, r * G:(r + 1) * G], signs, O.BF16)
        assert np.array_equal(qh.view(np.uint32), fx[f"row{r}_qhat"].view(np.uint32)) and np.float32(qn) == fx[f"row{r}_qnorm"]
        ids = O.rank_centroids(qh, O.BF16)
        assert np.array_equal(ids, fx[f"row{r}_sorted_ids"])
        lut = O.tier_lut(ids, fx["cluster_counts"][r], tiers)
        assert np.array_equal(lut, fx[f"row{r}_lut"])
        cnt = O.collision_count(fx["codes"][r], lut)
        assert np.array_equal(cnt, fx[f"row{r}_cnt"])
        cand, theta = O.select_candidates(cnt, n_cand)
        assert np.array_equal(cand, fx[f"row{r}_cand"]) and theta == int(fx[f"row{r}_theta"])
        sc = O.rerank(cand, fx["nib"][r], weight[r], qh, qn)
        assert np.array_equal(sc.view(np.uint32), fx[f"row{r}_scores"].view(np.uint32))
        final, pos = O.topk_f32(sc, cand, k)
        assert np.array_equal(final, fx[f"row{r}_final"])
        assert np.array_equal(O.retrieve_row(q[0, r * G:(r + 1) * G], signs, O.BF16, fx["codes"][r], fx["nib"][r], weight[r],
                                             fx["cluster_counts"][r], tiers, n_cand, k), fx[f"row{r}_final"])
        att = O.attention(q[0, r * G:(r + 1) * G], _bf16(fx[f"row{r}_sel_k_bf16"]), _bf16(fx[f"row{r}_sel_v_bf16"]))
        np.testing.assert_allclose(att, fx[f"row{r}_attn"], rtol=0, atol=1e-6)


@pytest.mark.gpu
def test_hip_path_reproduces_the_fixture(fx):
    import torch

    from pariskv_amd import ops

    dev = "cuda:0"
    print("golden fixture through the C ABI", flush=True)
    n_cand, k = int(fx["n_cand"]), int(fx["k"])
    tiers = [int(t) for t in fx["tiers"]]
    signs = torch.from_numpy(fx["signs"]).to(dev)
    to_bf = lambda bits: torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)
    q = to_bf(fx["queries_bf16"]).view(BS, 1, H * G, 128)
    codes = torch.from_numpy(fx["codes"]).view(BS, H, N, 16).to(dev)
    nib = torch.from_numpy(fx["nib"].reshape(BS, H, N, 64)).to(dev)
    w = to_bf(fx["weight_bf16"]).view(BS, H, N, 16)
    cc = torch.from_numpy(fx["cluster_counts"]).view(BS, H, 16, 256).to(dev)
    # encoder on the stored head of every row
    ck, nk, wk, cb, k4, kw = ops.alloc_keymajor(BS, H, 128, dev)
    ops.encode_append(to_bf(fx["keys_head_bf16"]).view(BS, H, 128, 128), signs, cb, k4, kw, None)
    assert torch.equal(ck, codes[:, :, :128]) and torch.equal(nk, nib[:, :, :128]) and torch.equal(wk, w[:, :, :128])
    # whole retrieval
    plan = ops.RetrievePlan(BS, H, G, N, dev, N, n_cand, k)
    sc_out = torch.empty(BS, H, k, device=dev)
    out = plan.run(q, signs, ops.mag_centers(dev), cc, codes, nib, w, 0, N, tiers, n_cand, k, out_scores=sc_out)
    torch.cuda.synchronize()
    cand = plan.view("cand", N, n_cand, k, torch.int64).view(H, n_cand).cpu().numpy()
    scores = plan.view("scores", N, n_cand, k, torch.float32).view(H, n_cand).cpu().numpy()
    lut = plan.view("lut", N, n_cand, k, torch.uint8).view(H, 16, 256).cpu().numpy()
    cnt = plan.view("cnt_u8", N, n_cand, k, torch.uint8).view(H, -1)[:, :N].cpu().numpy()
    att = ops.DecodeAttention(BS, H, G, k, dev)
    sel_k = torch.stack([to_bf(fx[f"row{r}_sel_k_bf16"]) for r in range(H)]).view(BS, H, k, 128)
    sel_v = torch.stack([to_bf(fx[f"row{r}_sel_v_bf16"]) for r in range(H)]).view(BS, H, k, 128)
    a = att.run(q, [(sel_k, sel_v, 0, k)]).float().cpu().numpy().reshape(H, G, 128)
    for r in range(H):
        assert np.array_equal(lut[r], fx[f"row{r}_lut"]) and np.array_equal(cnt[r], fx[f"row{r}_cnt"].astype(np.uint8))
        assert np.array_equal(cand[r], fx[f"row{r}_cand"])
        np.testing.assert_allclose(scores[r], fx[f"row{r}_scores"], rtol=1e-5, atol=1e-5 * np.abs(fx[f"row{r}_scores"]).max())
        assert np.array_equal(out[0, r].cpu().numpy(), fx[f"row{r}_final"])
        assert np.array_equal(sc_out[0, r].cpu().numpy(), fx[f"row{r}_final_scores"])
        assert np.abs(a[r] - fx[f"row{r}_attn"]).max() <= 2e-2  # bf16 output, tolerance of the attention row
