"""Pins the oracle's decode-step path (centroid ranking, tiered collision vote,
candidate select, 4-bit rerank, final top-k, gather, adaptive-k) against the
reference's own seeded recipes restated with library routines, closed forms and
brute force.  CPU only."""
import math

import numpy as np
import pytest
import torch

import refforms


def test_rank_centroids_matches_stable_argsort(oracle, signs):
    keys = oracle.synth_keys(256, seed=2)
    for dtype, tdt in ((oracle.F32, torch.float32), (oracle.BF16, torch.bfloat16)):
        q = oracle.synth_queries(keys, 4, seed=9, bf16=dtype == oracle.BF16)
        qhat, _ = oracle.query_prep(q, signs, dtype)
        ids = oracle.rank_centroids(qhat, dtype)
        sc = refforms.centroid_scores(torch.from_numpy(qhat).to(tdt)).float()
        for b in range(16):
            assert sorted(ids[b].tolist()) == list(range(256))  # a permutation
            s = sc[b][torch.from_numpy(ids[b])]
            assert (s[:-1] >= s[1:]).all()  # descending by the library's scores
            # antipodal symmetry of the sign codebook: rank r and 255-r are complements
            assert np.array_equal(ids[b] ^ 255, ids[b][::-1]) or dtype == oracle.BF16
        if dtype == oracle.BF16:
            # bf16 sums of 8 bf16 terms are exact in fp32, so ties are real ties:
            # equal to a stable descending argsort (ties -> smaller id first)
            ref = torch.argsort(sc, dim=-1, descending=True, stable=True).numpy()
            assert np.array_equal(ids, ref)


def _collision_recipe(bs, kv_heads, B, K, kv_len, seed=42):
    """Seeded input recipe of collision_fused/collision_test.py:16-53."""
    torch.manual_seed(seed)
    ids = torch.stack([torch.stack([torch.stack([torch.randperm(K) for _ in range(B)])
                                    for _ in range(kv_heads)]) for _ in range(bs)]).to(torch.int64)
    counts = torch.randint(1, max(2, kv_len // 2), (bs, kv_heads, B, K), dtype=torch.int32)
    codebook = torch.randint(0, K, (bs, kv_heads, B, kv_len), dtype=torch.int32)
    return ids, counts, codebook


@pytest.mark.parametrize("kv_len,ratio,tiers", [(2048, 0.2, None), (777, 0.5, None), (1500, 0.3, [1.0])])
def test_collision_vote_matches_reference_form(oracle, kv_len, ratio, tiers):
    tier_ratios = list(oracle.TIER_RATIOS) if tiers is None else tiers
    ids, counts, codebook = _collision_recipe(1, 4, 16, 256, kv_len)
    ref = refforms.update_cache_cnt_overall(ids, counts, codebook, tier_ratios, kv_len, ratio)
    tc = oracle.tier_counts(kv_len, ratio, tier_ratios)
    for h in range(4):
        lut = oracle.tier_lut(ids[0, h].numpy(), counts[0, h].numpy(), tc)
        cnt = oracle.collision_count(codebook[0, h].numpy().T.astype(np.uint8), lut)
        assert np.array_equal(cnt, ref[0, h].numpy())
        assert cnt.min() >= 0 and cnt.max() <= len(tc) * 16


def test_collision_vote_brute_force_tiny(oracle):
    """O(N*B*K) loop form of collision_fused/collision.cu:126-139,204-228."""
    rng = np.random.default_rng(4)
    n, tiers = 97, [3, 9, 20, 40, 70, 120]
    ids = np.stack([rng.permutation(256) for _ in range(16)])
    counts = rng.integers(0, 5, size=(16, 256)).astype(np.int32)
    codes = rng.integers(0, 256, size=(n, 16)).astype(np.uint8)
    lut = oracle.tier_lut(ids, counts, tiers)
    cnt = oracle.collision_count(codes, lut)
    for i in range(n):
        c = 0
        for b in range(16):
            prefix = 0
            for r in range(256):
                cl = ids[b, r]
                if cl == codes[i, b]:
                    c += sum(1 for t in tiers if prefix < t)
                prefix += counts[b, cl]
        assert c == cnt[i]
    # top-ranked cluster always carries full weight; weights are monotone along the ranking
    for b in range(16):
        assert lut[b, ids[b, 0]] == 6
        wr = lut[b, ids[b]]
        assert (wr[:-1] >= wr[1:]).all()


def test_tier_counts_known_values(oracle):
    assert oracle.tier_counts(8192, 0.3) == [123, 369, 738, 1229, 1844, 2458]
    assert oracle.tier_counts(32768, 0.2) == [328, 984, 1967, 3277, 4916, 6554]
    assert oracle.tier_counts(131072, 0.2) == [1311, 3933, 7865, 13108, 19661, 26215]


def test_select_candidates_is_topk_with_index_tiebreak(oracle):
    rng = np.random.default_rng(8)
    for n, k in [(5000, 250), (1000, 1000), (300, 1), (4096, 4095), (64, 10)]:
        cnt = rng.integers(0, 97, size=n).astype(np.int32)
        out, theta = oracle.select_candidates(cnt, k)
        if n == k:
            assert np.array_equal(out, np.arange(n))  # radix_topk.cu:154-159 identity
            continue
        order = np.lexsort((np.arange(n), -cnt))[:k]  # (count desc, index asc)
        assert set(out.tolist()) == set(order.tolist())
        # value multiset equals torch.topk's (topk/__init__.py:206-234)
        tv = torch.topk(torch.from_numpy(cnt), k).values.numpy()
        assert np.array_equal(np.sort(cnt[out]), np.sort(tv))
        # documented order: strictly-above-threshold ascending, then threshold ties ascending
        gt = out[cnt[out] > theta]
        eq = out[cnt[out] == theta]
        assert np.array_equal(out, np.concatenate([gt, eq]))
        assert (np.diff(gt) > 0).all() and (np.diff(eq) > 0).all()
    cnt = np.full(100, 7, np.int32)  # all equal: first k indices
    assert np.array_equal(oracle.select_candidates(cnt, 13)[0], np.arange(13))


def test_rerank_matches_reference_form_and_dequantised_dot(oracle, signs):
    keys = oracle.synth_keys(3000, seed=5, bf16=True)
    codes, nib, w = oracle.encode(keys, signs, oracle.BF16)
    q = oracle.synth_queries(keys, 4, seed=1, bf16=True)
    qhat, qn = oracle.query_prep(q, signs, oracle.BF16)
    cand = np.random.default_rng(0).permutation(3000)[:700].astype(np.int64)
    th, ce = oracle.mag_constants()
    s = oracle.rerank(cand, nib, w, qhat, qn)
    # (1) the reference's torch expression in fp32
    _, nib_r, w_r = oracle.to_reference_layout(codes, nib, w)
    ref = refforms.rerank_scores(torch.from_numpy(cand), torch.from_numpy(nib_r), torch.from_numpy(w_r),
                                 torch.from_numpy(qhat).view(16, 8), torch.tensor(qn), torch.from_numpy(ce))
    np.testing.assert_allclose(s, ref.numpy(), rtol=1e-5, atol=1e-5 * np.abs(ref.numpy()).max())
    # (2) brute force: dequantise each key (sum_b w_b * v_b) and take a float64 dot
    lo, hi = nib & 0x0F, nib >> 4
    v4 = np.stack([lo, hi], axis=-1).reshape(-1, 16, 8)
    val = np.where(v4 & 8, 1.0, -1.0) * ce[v4 & 7].astype(np.float64)
    deq = (val * w[:, :, None].astype(np.float64)).reshape(-1, 128)
    bf = (deq[cand] @ qhat.astype(np.float64)) * qn
    np.testing.assert_allclose(s, bf, rtol=1e-5, atol=1e-5 * np.abs(bf).max())
    # (3) the estimator tracks the true inner product <q_mean, k>
    true = keys[cand].astype(np.float64) @ q.mean(axis=0).astype(np.float64)
    assert np.corrcoef(true, s)[0, 1] > 0.97


def test_topk_f32_total_order(oracle):
    rng = np.random.default_rng(3)
    scores = rng.standard_normal(5000).astype(np.float32)
    scores[::7] = scores[3]  # many exact ties
    ids = rng.permutation(100000)[:5000].astype(np.int64)
    out_ids, out_pos = oracle.topk_f32(scores, ids, 300)
    order = np.lexsort((ids, -scores.astype(np.float64)))[:300]
    assert np.array_equal(out_pos, order) and np.array_equal(out_ids, ids[order])
    tv = torch.topk(torch.from_numpy(scores), 300).values.numpy()
    assert np.array_equal(scores[out_pos], tv)  # same values, same (sorted) order as torch.topk
    assert np.array_equal(oracle.topk_f32(scores, None, 5000)[1], np.lexsort((np.arange(5000), -scores.astype(np.float64))))


def test_gather_rows_is_index_select(oracle):
    rng = np.random.default_rng(1)
    src = rng.integers(0, 65535, size=(500, 128)).astype(np.uint16)  # bf16 payload as raw bits
    idx = rng.integers(0, 500, size=77)
    assert np.array_equal(oracle.gather_rows(src, idx), src[idx])


def test_expf_accuracy(oracle):
    x = np.concatenate([np.linspace(-87, 0, 20001), np.linspace(0, 88, 5001), [-100.0, -87.5]]).astype(np.float32)
    y = oracle.expf(x)
    ref = np.exp(x.astype(np.float64))
    ok = x >= -87
    rel = np.abs(y[ok] - ref[ok]) / ref[ok]
    assert rel.max() < 3e-7  # ~2.5 ulp
    assert (y[~ok] == 0).all() and oracle.expf(np.float32([0.0]))[0] == 1.0


def _adaptive_recipe(kv_heads, sl_len, cand_len, seed, head_dim=128):
    """Seeded input recipe of adaptive_k_fused/adaptive_topk.py:178-249 on CPU."""
    torch.manual_seed(seed)
    q = torch.randn(kv_heads, head_dim).to(torch.bfloat16) * 0.1
    slk = torch.randn(kv_heads, sl_len, head_dim).to(torch.bfloat16) * 0.1
    sl_vnorm = torch.rand(kv_heads, sl_len) + 0.5
    base = math.sqrt(head_dim)
    cs = torch.randn(kv_heads, cand_len) * (0.3 * base)
    rng = torch.Generator().manual_seed(seed)
    heavy = torch.randint(16, 1025, (kv_heads,), generator=rng).tolist()
    for h in range(kv_heads):
        cs[h, :heavy[h]] += torch.rand(heavy[h]) * 5.0 * base + 3.0 * base
    cs = cs.to(torch.bfloat16)
    ci = torch.stack([torch.randperm(cand_len) for _ in range(kv_heads)])
    cv = torch.rand(kv_heads, cand_len) + 0.5
    scale = 1.0 / base
    logits_sl = torch.einsum("hd,hkd->hk", q.float(), slk.float()) * scale
    return logits_sl, sl_vnorm, cs.float() * scale, ci, cv


@pytest.mark.parametrize("cfg", [dict(kv_heads=8, sl_len=320, cand_len=12500, cap=2048, thr=0.95, seed=42),
                                 dict(kv_heads=8, sl_len=832, cand_len=5000, cap=2048, thr=0.95, seed=7),
                                 dict(kv_heads=8, sl_len=576, cand_len=8000, cap=2048, thr=0.85, seed=123),
                                 dict(kv_heads=4, sl_len=320, cand_len=1500, cap=2048, thr=0.95, seed=99)])
def test_adaptive_topk_matches_reference_form(oracle, cfg):
    """Acceptance rule of adaptive_topk.py:433-461: k exact, first-k index sets equal."""
    lsl, slv, lc, ci, cv = _adaptive_recipe(cfg["kv_heads"], cfg["sl_len"], cfg["cand_len"], cfg["seed"])
    ks = []
    for h in range(cfg["kv_heads"]):
        k_ref, idx_ref, ben = refforms.adaptive_topk(lsl[h], slv[h], lc[h], ci[h], cv[h], cfg["thr"], cfg["cap"])
        k_out = min(cfg["cap"], cfg["cand_len"])
        k, idx = oracle.adaptive_topk(lsl[h].numpy(), slv[h].numpy(), lc[h].numpy(), cv[h].numpy(), ci[h].numpy(),
                                      cfg["thr"], k_out)
        assert abs(k - k_ref) <= 1  # exp() differs by ulps between libm and the fixed-sequence exp
        kk = min(k, k_ref)
        assert set(idx[:kk].tolist()) == set(idx_ref[:kk].tolist())
        ks.append((k, k_ref))
        # minimality of k by brute force in float64
        b = np.sort(ben.numpy().astype(np.float64))[::-1]
        slb = float((torch.exp(lsl[h] - max(lsl[h].max(), lc[h].max())).double() * slv[h].double()).sum())
        tot = slb + b.sum()
        if k < k_out:
            assert slb + b[:k + 1].sum() >= cfg["thr"] * tot * (1 - 1e-5)
            assert k <= 2 or slb + b[:k - 2].sum() < cfg["thr"] * tot * (1 + 1e-5)
    assert sum(1 for a, b in ks if a == b) >= len(ks) - 1


@pytest.mark.parametrize("rate,thr", [(0.5, 0.9), (0.25, 0.75), (1.0, 0.99), (0.1, 0.6), (0.5, 0.5)])
def test_adaptive_topk_forced_k_equals_reference_form_exactly(oracle, rate, thr):
    """Benefits in a geometric ladder (logit of the j-th best candidate = -rate * j, unit value norms): the mass
    reached after k candidates is known in closed form and sits far from the threshold on both sides of the answer,
    so neither exp()'s last ulp nor the summation order can move k.  k and the whole ordered index prefix must equal
    the reference form (adaptive_topk.py:282-311) exactly, with and without dense tokens in the mix."""
    n, cap = 3000, 256
    g = np.random.default_rng(int(rate * 1000) + int(thr * 100))
    for dense_share in (0.0, 0.3):
        ladder = (-rate * np.arange(n)).astype(np.float32)
        perm = g.permutation(n)
        logits = np.empty(n, np.float32)
        logits[perm] = ladder                                   # candidate position perm[j] holds the j-th best
        ids = g.permutation(10 ** 6)[:n].astype(np.int64)
        vn = np.ones(n, np.float32)
        q = math.exp(-rate)
        cand_mass = 1.0 / (1.0 - q)                             # sum of the ladder's benefits (joint max = 0)
        # dense tokens: two of them, each with logit -20 and a value norm that makes their mass the wanted share
        slb = dense_share * cand_mass / (1.0 - dense_share)
        lsl = np.full(2, -20.0, np.float32)
        slv = np.full(2, slb / 2.0 / math.exp(-20.0), np.float32)
        total = slb + cand_mass
        reached = [slb + (1.0 - q ** k) / (1.0 - q) for k in range(0, cap + 1)]
        k_true = next(k for k in range(1, cap + 1) if reached[k] >= thr * total)
        # far from the boundary on both sides (relative margin >> fp32 round-off of a few thousand terms)
        assert reached[k_true] > thr * total * (1 + 1e-3) and reached[k_true - 1] < thr * total * (1 - 1e-3)
        k, idx = oracle.adaptive_topk(lsl, slv, logits, vn, ids, thr, cap)
        k_ref, idx_ref, _ = refforms.adaptive_topk(torch.from_numpy(lsl), torch.from_numpy(slv), torch.from_numpy(logits),
                                                   torch.from_numpy(ids), torch.from_numpy(vn), thr, cap)
        assert k == k_ref == k_true
        # float32 exp(-rate * j) underflows to ties far down the ladder: compare the prefix that is strictly ordered
        strict = int(min(cap, 80.0 / rate))
        assert np.array_equal(idx[:strict], idx_ref.numpy()[:strict]) and np.array_equal(idx[:strict], ids[perm[:strict]])


def test_adaptive_topk_edge_cases(oracle):
    # total <= 0 -> k = 1 ; never reached -> k_out
    z = np.zeros(10, np.float32)
    k, _ = oracle.adaptive_topk(z[:3], z[:3], z, z, np.arange(10), 0.95, 5)
    assert k == 1
    lsl = np.zeros(1, np.float32)
    k, idx = oracle.adaptive_topk(lsl, np.ones(1, np.float32), np.zeros(100, np.float32), np.ones(100, np.float32),
                                  np.arange(100)[::-1].copy(), 0.95, 10)
    assert k == 10 and np.array_equal(idx, np.arange(100)[::-1][:10])  # ties: candidate position ascending


def test_dense_logits_and_value_norm_match_torch_forms(oracle):
    """The two numpy restatements that feed adaptive-k (reference polar_cache_adaptivek_varlen.py:1418-1419, :1731,
    :1179) against the torch expressions the reference evaluates and against float64: exact up to the last rounding
    (one bf16 step in the bf16 chain, 1e-6 relative in fp32), and invariant facts a slip would break."""
    g = torch.Generator().manual_seed(17)
    G, n = 4, 300
    for dtype, tdt, rtol in ((oracle.BF16, torch.bfloat16, 2.0 ** -7), (oracle.F32, torch.float32, 2e-6)):
        q = torch.randn(G, 128, generator=g).to(tdt)
        k = (torch.randn(n, 128, generator=g) * 2).to(tdt)
        v = (torch.randn(n, 128, generator=g) * torch.rand(n, 1, generator=g) * 3).to(tdt)
        scale = 1.0 / math.sqrt(128)
        got = oracle.dense_logits(q.float().numpy(), k.float().numpy(), scale, dtype)
        ref = (torch.einsum("d,kd->k", q.mean(dim=0), k).to(torch.float32) * scale).numpy()
        f64 = (k.double() @ q.double().mean(dim=0)).numpy() * scale
        assert np.allclose(got, ref, rtol=rtol, atol=rtol * np.abs(f64).max())
        assert np.allclose(got, f64, rtol=rtol, atol=rtol * np.abs(f64).max())
        vn = oracle.value_norm(v.float().numpy(), dtype)
        vref = torch.linalg.vector_norm(v, dim=-1).float().numpy()
        assert np.allclose(vn, vref, rtol=rtol)
        assert np.allclose(vn, np.linalg.norm(v.double().numpy(), axis=1), rtol=rtol)
        # a query group of four identical heads is that head (4a / 4 is exact); one-hot rows pick out single dimensions
        same = oracle.dense_logits(np.repeat(q[:1].float().numpy(), 4, axis=0), k.float().numpy(), 1.0, dtype)
        assert np.array_equal(same, oracle.dense_logits(q[:1].float().numpy(), k.float().numpy(), 1.0, dtype))
        eye = np.eye(128, dtype=np.float32) * 3.0
        assert np.array_equal(oracle.dense_logits(q[:1].float().numpy(), eye, 1.0, dtype),
                              oracle.bf16_round(q[0].float().numpy() * 3.0) if dtype == oracle.BF16 else q[0].numpy() * 3.0)
        assert np.array_equal(oracle.value_norm(eye, dtype), np.full(128, 3.0, np.float32))


def test_retrieve_row_composes_the_stages(oracle, signs):
    n, C, K = 4096, 512, 128
    keys = oracle.synth_keys(n, seed=0)
    codes, nib, w = oracle.encode(keys, signs, oracle.F32)
    cc = oracle.count_cluster_keys(codes)
    q = oracle.synth_queries(keys, 4, seed=0)
    tiers = oracle.tier_counts(n, 0.5)
    out = oracle.retrieve_row(q, signs, oracle.F32, codes, nib, w, cc, tiers, C, K)
    qhat, qn = oracle.query_prep(q, signs, oracle.F32)
    lut = oracle.tier_lut(oracle.rank_centroids(qhat, oracle.F32), cc, tiers)
    cand, _ = oracle.select_candidates(oracle.collision_count(codes, lut), C)
    ids, _ = oracle.topk_f32(oracle.rerank(cand, nib, w, qhat, qn), cand, K)
    assert np.array_equal(out, ids)
    # retrieval quality: most of the true top-K inner products are recovered
    true = np.argsort(-(keys @ q.mean(axis=0)))[:K]
    assert len(set(true.tolist()) & set(out.tolist())) > 0.5 * K   # chance level would be K * K / n = 4


def test_attention_matches_torch_sdpa_and_closed_forms(oracle):
    """pkv_o_attention against the library routine (fp32 scaled_dot_product_attention, GQA group 4) and
    two closed forms: identical keys give the mean of the values; one dominant key gives its value row."""
    import torch
    import torch.nn.functional as F

    O = oracle
    g = torch.Generator().manual_seed(5)
    G, S = 4, 777
    q = torch.randn(G, 128, generator=g)
    k = torch.randn(S, 128, generator=g)
    v = torch.randn(S, 128, generator=g)
    ref = F.scaled_dot_product_attention(q.view(1, G, 1, 128), k.view(1, 1, S, 128).expand(1, G, S, 128),
                                         v.view(1, 1, S, 128).expand(1, G, S, 128)).view(G, 128)
    got = O.attention(q.numpy(), k.numpy(), v.numpy())
    np.testing.assert_allclose(got, ref.numpy(), rtol=0, atol=2e-6)
    # a non-default scale
    ref2 = F.scaled_dot_product_attention(q.view(1, G, 1, 128), k.view(1, 1, S, 128).expand(1, G, S, 128),
                                          v.view(1, 1, S, 128).expand(1, G, S, 128), scale=0.3).view(G, 128)
    np.testing.assert_allclose(O.attention(q.numpy(), k.numpy(), v.numpy(), 0.3), ref2.numpy(), rtol=0, atol=2e-6)
    # identical keys: uniform weights
    same = np.tile(k[:1].numpy(), (S, 1))
    np.testing.assert_allclose(O.attention(q.numpy(), same, v.numpy()), np.tile(v.numpy().mean(0), (G, 1)), atol=1e-6)
    # one key aligned with the query and far larger than the rest
    kk = 0.01 * k.numpy()
    kk[123] = 50.0 * q[2].numpy()
    out = O.attention(q[2:3].numpy(), kk, v.numpy())
    np.testing.assert_allclose(out[0], v[123].numpy(), atol=1e-5)


@pytest.mark.parametrize("dtype", [0, 1])  # oracle.F32, oracle.BF16
def test_torch_cpu_baseline_selects_the_oracles_keys_up_to_ties(oracle, dtype):
    """oracle/torch_baseline.py (the batched torch form timed as the CPU baseline) against the C oracle: the two break
    ties differently (torch.topk / argsort vs the fixed rule) and the torch rerank rounds in the tensor dtype, so the
    final id sets agree on all but a few boundary keys."""
    import torch

    import workloads as W
    from oracle import torch_baseline as TB

    w = W.make_workload("tb", 2, 2, 4, 6000, 600, 128, dtype, 0.3, seed0=1)
    tdt = torch.bfloat16 if dtype == oracle.BF16 else torch.float32
    q = torch.from_numpy(w.queries).to(tdt).view(w.bs, 1, w.H * w.G, 128)
    cb = torch.from_numpy(w.codes.reshape(w.bs, w.H, w.N, 16)).permute(0, 1, 3, 2).contiguous()
    k4 = torch.from_numpy(w.nib.reshape(w.bs, w.H, w.N, 16, 4)).permute(0, 1, 3, 2, 4).contiguous()
    kw = torch.from_numpy(w.weight.reshape(w.bs, w.H, w.N, 16)).to(torch.bfloat16).permute(0, 1, 3, 2).contiguous()
    cc = torch.from_numpy(w.cluster_counts.reshape(w.bs, w.H, 16, 256))
    keys = torch.from_numpy(w.keys.reshape(w.bs, w.H, w.N, 128))
    ids, gk, gv = TB.retrieve_layer(q, torch.from_numpy(w.signs), cb, k4, kw, cc, w.tiers, w.C, w.K, keys, keys)
    assert ids.shape == (w.bs, w.H, w.K) and torch.equal(gk, gv)
    same = 0
    for r in range(w.R):
        b, h = divmod(r, w.H)
        same += len(np.intersect1d(ids[b, h].numpy(), W.oracle_stages(w, r)["final"]))
        assert torch.equal(gk[b, h], keys[b, h][ids[b, h]])
    assert same >= 0.95 * w.R * w.K
