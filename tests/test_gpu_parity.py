"""GPU parity tests: every HIP entry point, called through the C ABI, against the
CPU oracle on identical seeded inputs.

Bar: bit-exact for codes, nibbles, weights (bf16 bits), vote counts, candidate
lists and final top-k indices; rerank scores within 1e-5 relative of the oracle
(they are in fact evaluated in the same order, so equality is also asserted).
"""
import math

import numpy as np
import pytest
import torch

import workloads as W
from oracle import pkv_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from pariskv_amd import ops as _ops

    return _ops


@pytest.fixture(scope="module")
def wl_cfg1():
    return W.cfg1()


@pytest.fixture(scope="module")
def wl_cfg2():
    return W.cfg2()


@pytest.fixture(scope="module")
def wl_small_bf16():
    # ragged length (not a multiple of any tile), 2 sequences
    return W.make_workload("small", 2, 2, 4, 5000 + 37, 333, 100, O.BF16, 0.5, seed0=5)


def _say(msg):
    print(msg, flush=True)


# ------------------------------------------------------------------- encode


@pytest.mark.parametrize("dtype", [O.F32, O.BF16])
@pytest.mark.parametrize("layout", ["keymajor", "reference"])
def test_encode_append_bit_exact(ops, dtype, layout):
    _say(f"encode dtype={dtype} layout={layout}")
    bs, H, S = 2, 3, 1000 + 13
    tdt = torch.bfloat16 if dtype == O.BF16 else torch.float32
    signs = O.srht_signs(42)
    keys = np.stack([O.synth_keys(S, 100 + r, bf16=dtype == O.BF16) for r in range(bs * H)]).reshape(bs, H, S, 128)
    keys[0, 0, 5] = 0.0  # a zero key must not produce NaNs
    tk = torch.from_numpy(keys).to(tdt).to(DEV)
    if layout == "keymajor":
        _, _, _, cb, k4, kw = ops.alloc_keymajor(bs, H, S, DEV)
    else:
        cb = torch.zeros(bs, H, 16, S, dtype=torch.uint8, device=DEV)
        k4 = torch.zeros(bs, H, 16, S, 4, dtype=torch.uint8, device=DEV)
        kw = torch.zeros(bs, H, 16, S, dtype=torch.bfloat16, device=DEV)
    cc = torch.zeros(bs, H, 16, 256, dtype=torch.int32, device=DEV)
    ops.encode_append(tk, torch.from_numpy(signs).to(DEV), cb, k4, kw, cc)
    ops.encode_append(tk[:, :, :100], torch.from_numpy(signs).to(DEV), cb[..., :100], k4[:, :, :, :100], kw[..., :100], cc)
    torch.cuda.synchronize()
    for r in range(bs * H):
        b, h = divmod(r, H)
        codes, nib, w = O.encode(keys[b, h], signs, dtype)
        assert np.array_equal(cb[b, h].cpu().numpy().T, codes)
        assert np.array_equal(k4[b, h].cpu().numpy().transpose(1, 0, 2), nib)
        assert np.array_equal(kw[b, h].float().cpu().numpy().T, w)
        ref_cc = O.count_cluster_keys(codes)
        ref_cc = O.count_cluster_keys(codes[:100], ref_cc)  # += semantics
        assert np.array_equal(cc[b, h].cpu().numpy(), ref_cc)
    # count_cluster_keys on its own
    cc2 = torch.zeros_like(cc)
    ops.count_cluster_keys(cb, cc2)
    ops.count_cluster_keys(cb[..., :100], cc2)
    assert torch.equal(cc2, cc)


@pytest.mark.parametrize("dtype", [O.BF16, O.F32])
@pytest.mark.parametrize("S", [1, 15, 16, 17, 255, 256, 257, 300])
def test_encode_ragged_block_stays_inside_its_keys(ops, S, dtype):
    """The lanes past the end of a ragged block repeat its last key's stores: nothing beyond key S - 1 may change, and
    the cluster sizes count every key once."""
    _say(f"encode ragged S={S} dtype={dtype}")
    cap = S + 40
    signs = O.srht_signs(42)
    keys = O.synth_keys(S, 31 + S, bf16=dtype == O.BF16).reshape(1, 1, S, 128)
    codes_km, nib_km, w_km, cb, k4, kw = ops.alloc_keymajor(1, 2, cap, DEV)
    rec = nib_km.as_strided((1, 2, cap, 128), nib_km.stride(), nib_km.storage_offset())  # the whole 128-byte records
    codes_km.fill_(0xAB)
    rec.fill_(0xAB)
    cc = torch.zeros(1, 2, 16, 256, dtype=torch.int32, device=DEV)
    tk = torch.from_numpy(keys).to(torch.bfloat16 if dtype == O.BF16 else torch.float32).to(DEV)
    ops.encode_append(tk, torch.from_numpy(signs).to(DEV), cb[:, 1:, :, :S], k4[:, 1:, :, :S], kw[:, 1:, :, :S], cc[:, 1:])
    torch.cuda.synchronize()
    codes, nib, w = O.encode(keys[0, 0], signs, dtype)
    assert np.array_equal(cb[0, 1, :, :S].cpu().numpy().T, codes)
    assert np.array_equal(k4[0, 1, :, :S].cpu().numpy().transpose(1, 0, 2), nib)
    assert np.array_equal(kw[0, 1, :, :S].float().cpu().numpy().T, w)
    assert np.array_equal(cc[0, 1].cpu().numpy(), O.count_cluster_keys(codes)) and int(cc[0, 0].abs().sum()) == 0
    # untouched: head 0, the keys from S on of head 1, and bytes 96..127 of every record (the value-norm slot)
    assert bool((codes_km[0, 0] == 0xAB).all()) and bool((codes_km[0, 1, S:] == 0xAB).all())
    assert bool((rec[0, 0] == 0xAB).all()) and bool((rec[0, 1, S:] == 0xAB).all()) and bool((rec[0, 1, :, 96:] == 0xAB).all())


def _adversarial_keys(n, seed, bf16=True):
    """Keys that stress every rounding decision of the encoder: magnitudes from 2^-30 to 2^30, outlier dims,
    exact zeros and components far below the norm, powers of two, one-hot and constant vectors, tiny norms."""
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((n, 128)).astype(np.float32)
    kind = np.arange(n) % 16
    k *= np.exp2(rng.integers(-30, 31, size=(n, 1))).astype(np.float32) * (kind[:, None] < 6) + (kind[:, None] >= 6)
    k[kind == 6] *= np.where(rng.random((int((kind == 6).sum()), 128)) < 0.05, 30.0, 1.0).astype(np.float32)   # outlier dims
    k[kind == 7] *= (rng.random((int((kind == 7).sum()), 128)) < 0.5)                                          # half zeros
    k[kind == 8] *= np.where(rng.random((int((kind == 8).sum()), 128)) < 0.1, 1e-30, 1.0).astype(np.float32)   # far below the norm
    k[kind == 9] = np.exp2(rng.integers(-8, 9, size=(int((kind == 9).sum()), 128))) * rng.choice([-1.0, 1.0], size=(int((kind == 9).sum()), 128))
    oh = np.where(kind == 10)[0]
    k[oh] = 0.0
    k[oh, rng.integers(0, 128, size=oh.size)] = rng.standard_normal(oh.size).astype(np.float32) + 3.0          # one-hot
    k[kind == 11] = (rng.standard_normal((int((kind == 11).sum()), 1)) * np.ones((1, 128))).astype(np.float32)  # constant
    k[kind == 12] *= 1e-9                                                                                      # norm below the 1e-8 clamp
    k[kind == 13] = np.round(k[kind == 13] * 4.0) / 4.0                                                        # many exact ties and zeros
    k[kind == 14] *= 3e-8                                                                                      # norm just above the clamp
    k = k.astype(np.float32)
    return O.bf16_round(k) if bf16 else k


def _adversarial_bf16_keys(n, seed):
    return _adversarial_keys(n, seed, True)


def test_encode_bf16_bit_exact_on_adversarial_keys(ops):
    """The bf16 encoder replaces divisions by reciprocals where that provably gives the same bf16 result and falls
    back to correctly rounded arithmetic per wave elsewhere; both routes must equal the oracle bit for bit."""
    H, S = 4, 16384 + 5
    signs = O.srht_signs(42)
    keys = np.stack([_adversarial_bf16_keys(S, 700 + h) for h in range(H)]).reshape(1, H, S, 128)
    _say(f"encode adversarial bf16 keys {keys.shape}")
    tk = torch.from_numpy(keys).to(torch.bfloat16).to(DEV)
    _, _, _, cb, k4, kw = ops.alloc_keymajor(1, H, S, DEV)
    cc = torch.zeros(1, H, 16, 256, dtype=torch.int32, device=DEV)
    ops.encode_append(tk, torch.from_numpy(signs).to(DEV), cb, k4, kw, cc)
    torch.cuda.synchronize()
    for h in range(H):
        codes, nib, w = O.encode(keys[0, h], signs, O.BF16)
        bad = np.where((cb[0, h].cpu().numpy().T != codes).any(axis=1))[0]
        assert bad.size == 0, f"codes differ at keys {bad[:8]} (kinds {bad[:8] % 16})"
        bad = np.where((k4[0, h].cpu().numpy().transpose(1, 0, 2) != nib).any(axis=(1, 2)))[0]
        assert bad.size == 0, f"4-bit codes differ at keys {bad[:8]} (kinds {bad[:8] % 16})"
        got_w = kw[0, h].float().cpu().numpy().T
        bad = np.where((got_w.view(np.uint32) != w.astype(np.float32).view(np.uint32)).any(axis=1))[0]
        assert bad.size == 0, f"weights differ at keys {bad[:8]} (kinds {bad[:8] % 16})"
        assert np.array_equal(cc[0, h].cpu().numpy(), O.count_cluster_keys(codes))


def test_encode_f32_bit_exact_on_adversarial_keys(ops):
    """The fp32 encoder shares one refined reciprocal among the quotients of a denominator and leaves out the range
    scaling of divisions and roots inside a checked range, falling back to the plain correctly rounded operations per
    wave elsewhere; both routes must equal the oracle bit for bit."""
    H, S = 4, 16384 + 5
    signs = O.srht_signs(42)
    keys = np.stack([_adversarial_keys(S, 900 + h, bf16=False) for h in range(H)]).reshape(1, H, S, 128)
    keys[0, 1] *= np.float32(2.0) ** np.random.default_rng(3).integers(-70, 50, size=(S, 1)).astype(np.float32)  # beyond the checked range too
    _say(f"encode adversarial fp32 keys {keys.shape}")
    tk = torch.from_numpy(keys).to(DEV)
    _, _, _, cb, k4, kw = ops.alloc_keymajor(1, H, S, DEV)
    cc = torch.zeros(1, H, 16, 256, dtype=torch.int32, device=DEV)
    ops.encode_append(tk, torch.from_numpy(signs).to(DEV), cb, k4, kw, cc)
    cb2 = torch.zeros(1, H, 16, S, dtype=torch.uint8, device=DEV)
    ops.encode_append(tk, torch.from_numpy(signs).to(DEV), cb2, None, None, None)  # codes only: the other kernel form
    torch.cuda.synchronize()
    for h in range(H):
        codes, nib, w = O.encode(keys[0, h], signs, O.F32)
        bad = np.where((cb[0, h].cpu().numpy().T != codes).any(axis=1))[0]
        assert bad.size == 0, f"codes differ at keys {bad[:8]} (kinds {bad[:8] % 16})"
        bad = np.where((cb2[0, h].cpu().numpy().T != codes).any(axis=1))[0]
        assert bad.size == 0, f"codes of the codes-only form differ at keys {bad[:8]} (kinds {bad[:8] % 16})"
        bad = np.where((k4[0, h].cpu().numpy().transpose(1, 0, 2) != nib).any(axis=(1, 2)))[0]
        assert bad.size == 0, f"4-bit codes differ at keys {bad[:8]} (kinds {bad[:8] % 16})"
        got_w = kw[0, h].float().cpu().numpy().T
        bad = np.where((got_w.view(np.uint32) != w.astype(np.float32).view(np.uint32)).any(axis=1))[0]
        assert bad.size == 0, f"weights differ at keys {bad[:8]} (kinds {bad[:8] % 16})"
        assert np.array_equal(cc[0, h].cpu().numpy(), O.count_cluster_keys(codes))


def test_encode_without_rabitq_outputs(ops):
    S = 300
    signs = O.srht_signs(42)
    keys = O.synth_keys(S, 9)
    cb = torch.zeros(1, 1, 16, S, dtype=torch.uint8, device=DEV)
    ops.encode_append(torch.from_numpy(keys).view(1, 1, S, 128).to(DEV), torch.from_numpy(signs).to(DEV), cb, None, None, None)
    assert np.array_equal(cb[0, 0].cpu().numpy().T, O.encode(keys, signs, O.F32)[0])


# --------------------------------------------------------------- query side


@pytest.mark.parametrize("wl_name", ["wl_cfg1", "wl_small_bf16"])
def test_query_prep_lut_bit_exact(ops, request, wl_name):
    w = request.getfixturevalue(wl_name)
    _say(f"query_prep_lut {w.name}")
    d = W.to_device(w, DEV, torch)
    qhat, qnorm, lut, ids = ops.query_prep_lut(d["queries"], w.H, d["signs"], d["cluster_counts"], w.tiers, want_sorted_ids=True)
    torch.cuda.synchronize()
    for r in range(w.R):
        st = W.oracle_stages(w, r)
        b, h = divmod(r, w.H)
        assert np.array_equal(qhat[b, h].cpu().numpy().view(np.uint32), st["qhat"].view(np.uint32))
        assert np.float32(qnorm[b, h].item()) == np.float32(st["qnorm"])
        assert np.array_equal(ids[b, h].cpu().numpy(), st["sorted_ids"])
        assert np.array_equal(lut[b, h].cpu().numpy(), st["lut"])


def test_query_prep_single_tier_and_group1(ops, wl_cfg1):
    w = wl_cfg1
    d = W.to_device(w, DEV, torch)
    q1 = d["queries"].view(w.bs, w.H, w.G, 128)[:, :, 0].contiguous()  # group size 1
    qhat, qnorm, lut, ids = ops.query_prep_lut(q1.view(w.bs, w.H, 128), w.H, d["signs"], d["cluster_counts"], [500], True)
    torch.cuda.synchronize()
    for r in range(w.R):
        qh, qn = O.query_prep(w.queries[0, r * w.G:r * w.G + 1], w.signs, w.dtype)
        lut_ref = O.tier_lut(O.rank_centroids(qh, w.dtype), w.cluster_counts[r], [500])
        assert np.array_equal(lut[0, r].cpu().numpy(), lut_ref) and lut_ref.max() == 1


def _collision_recipe(bs, kv_heads, kv_len, seed=42):
    """Input recipe of the reference's collision self-test (collision_fused/collision_test.py:16-53)."""
    torch.manual_seed(seed)
    ids = torch.stack([torch.stack([torch.stack([torch.randperm(256) for _ in range(16)])
                                    for _ in range(kv_heads)]) for _ in range(bs)]).to(torch.int64)
    counts = torch.randint(1, max(2, kv_len // 2), (bs, kv_heads, 16, 256), dtype=torch.int32)
    codebook = torch.randint(0, 256, (bs, kv_heads, 16, kv_len), dtype=torch.int32).to(torch.uint8)
    return ids, counts, codebook


@pytest.mark.parametrize("kv_len,ratio,ntier", [(2048, 0.2, 6), (4999, 0.5, 6), (2048, 0.3, 1), (70001, 0.2, 6)])
@pytest.mark.parametrize("layout", ["reference", "keymajor"])
def test_update_cache_cnt_interface(ops, kv_len, ratio, ntier, layout):
    from pariskv_amd.cache_hub.collision_fused import update_cache_cnt_cuda_interface

    _say(f"update_cache_cnt kv_len={kv_len} ntier={ntier} layout={layout}")
    bs, H = 2, 3
    ids, counts, codebook = _collision_recipe(bs, H, kv_len)
    ratios = list(O.TIER_RATIOS) if ntier == 6 else [1.0]
    tiers = O.tier_counts(kv_len, ratio, ratios)
    cb = codebook.to(DEV)
    if layout == "keymajor":
        cb = cb.permute(0, 1, 3, 2).contiguous().permute(0, 1, 3, 2)  # same logical tensor, key-major memory
    cnt = update_cache_cnt_cuda_interface(ids.to(DEV), counts.to(DEV), cb, tiers)
    torch.cuda.synchronize()
    assert cnt.dtype == torch.int32 and tuple(cnt.shape) == (bs, H, kv_len)
    for b in range(bs):
        for h in range(H):
            lut = O.tier_lut(ids[b, h].numpy(), counts[b, h].numpy(), tiers)
            ref = O.collision_count(np.ascontiguousarray(codebook[b, h].numpy().T), lut)
            assert np.array_equal(cnt[b, h].cpu().numpy(), ref)


def test_update_cache_cnt_sliced_views(ops):
    """The cache passes slices [.., start:end] of larger tensors (polar_cache.py:1051-1055)."""
    from pariskv_amd.cache_hub.collision_fused import update_cache_cnt_cuda_interface

    bs, H, cap, s, e = 1, 2, 3000, 129, 2777
    ids, counts, codebook = _collision_recipe(bs, H, cap)
    tiers = O.tier_counts(e - s, 0.5)
    for layout in ("reference", "keymajor"):
        cb = codebook.to(DEV)
        if layout == "keymajor":
            cb = cb.permute(0, 1, 3, 2).contiguous().permute(0, 1, 3, 2)
        cnt = update_cache_cnt_cuda_interface(ids.to(DEV), counts.to(DEV), cb[:, :, :, s:e], tiers)
        for h in range(H):
            lut = O.tier_lut(ids[0, h].numpy(), counts[0, h].numpy(), tiers)
            ref = O.collision_count(np.ascontiguousarray(codebook[0, h, :, s:e].numpy().T), lut)
            assert np.array_equal(cnt[0, h].cpu().numpy(), ref)


@pytest.mark.parametrize("layout", ["reference", "keymajor"])
def test_collision_scan_histograms(ops, layout):
    """Stand-alone scan from a ready table: u8 counts plus the per-chunk and per-row suffix histograms."""
    bs, H, N = 2, 2, 9001
    ids, counts, codebook = _collision_recipe(bs, H, N)
    tiers = O.tier_counts(N, 0.3)
    lut = np.stack([np.stack([O.tier_lut(ids[b, h].numpy(), counts[b, h].numpy(), tiers) for h in range(H)])
                    for b in range(bs)])
    cb = codebook.to(DEV)
    if layout == "keymajor":
        cb = cb.permute(0, 1, 3, 2).contiguous().permute(0, 1, 3, 2)
    cnt, (row_suf, chunk_suf), chunk = ops.collision_scan(cb, torch.from_numpy(lut).to(DEV), torch.uint8, want_hist=True)
    torch.cuda.synchronize()
    n_chunks = (N + chunk - 1) // chunk
    for b in range(bs):
        for h in range(H):
            r = b * H + h
            ref = O.collision_count(np.ascontiguousarray(codebook[b, h].numpy().T), lut[b, h])
            assert np.array_equal(cnt[b, h].cpu().numpy(), ref.astype(np.uint8))
            suf = lambda x: np.cumsum(np.bincount(x, minlength=128)[::-1])[::-1]
            assert np.array_equal(row_suf[r].cpu().numpy(), suf(ref))
            got = chunk_suf[r].cpu().numpy().astype(np.int64) & 0xFFFF
            for c in range(n_chunks):
                assert np.array_equal(got[c], suf(ref[c * chunk:(c + 1) * chunk]))


def test_update_cache_cnt_legacy(ops):
    from pariskv_amd.cache_hub.collision.collision import update_cache_cnt_cuda

    bs, H, N = 1, 4, 3001
    torch.manual_seed(42)  # recipe of collision/collision.py:11-26
    ids = torch.stack([torch.stack([torch.stack([torch.randperm(256) for _ in range(16)]) for _ in range(H)])
                       for _ in range(bs)]).to(torch.int32)
    topk_cnt = torch.randint(1, 256, (bs, H, 16), dtype=torch.int32)
    codebook = torch.randint(0, 256, (bs, H, 16, N), dtype=torch.int32)
    cnt = update_cache_cnt_cuda(ids.to(DEV), topk_cnt.to(DEV), codebook.to(DEV)).cpu()
    # membership form of collision/collision.py:29-45
    for h in range(H):
        ref = np.zeros(N, np.int32)
        for b in range(16):
            sel = set(ids[0, h, b, :int(topk_cnt[0, h, b])].tolist())
            ref += np.isin(codebook[0, h, b].numpy(), list(sel)).astype(np.int32)
        assert np.array_equal(cnt[0, h].numpy(), ref)


def test_interface_errors(ops):
    from pariskv_amd.cache_hub.collision_fused import update_cache_cnt_cuda_interface
    from pariskv_amd.cache_hub.topk import load_radix_topk_ext

    ids, counts, codebook = _collision_recipe(1, 1, 512)
    with pytest.raises(RuntimeError, match="uint8"):
        update_cache_cnt_cuda_interface(ids.to(DEV), counts.to(DEV), codebook.to(torch.int32).to(DEV), [10])
    with pytest.raises(RuntimeError, match="int64"):
        update_cache_cnt_cuda_interface(ids.to(torch.int32).to(DEV), counts.to(DEV), codebook.to(DEV), [10])
    with pytest.raises(RuntimeError, match="tier_num"):
        update_cache_cnt_cuda_interface(ids.to(DEV), counts.to(DEV), codebook.to(DEV), [])
    ext = load_radix_topk_ext()
    x = torch.zeros(2, 100, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="exceed"):
        ext.bucket_topk(x, 101)
    with pytest.raises(RuntimeError, match="positive"):
        ext.radix_topk(x.float(), 0)
    with pytest.raises(RuntimeError, match="3D"):
        ext.radix_topk_3d(x, 5)


# --------------------------------------------------------------- selections


@pytest.mark.parametrize("rows,L,k", [(8, 8192, 1024), (3, 5037, 333), (2, 2048, 2048), (4, 100000, 5000), (1, 300, 1),
                                      (2, 4096, 4095)])
def test_bucket_and_radix_topk_on_counts(ops, rows, L, k):
    from pariskv_amd.cache_hub.topk import load_radix_topk_ext

    _say(f"bucket_topk rows={rows} L={L} k={k}")
    ext = load_radix_topk_ext()
    rng = np.random.default_rng(L + k)
    x = rng.binomial(96, 0.1, size=(rows, L)).astype(np.int32)
    tx = torch.from_numpy(x).to(DEV)
    out_b = ext.bucket_topk(tx, k).cpu().numpy()
    out_r = ext.radix_topk_3d(tx.view(1, rows, L), k).cpu().numpy()[0]  # hot call of polar_cache.py:1241
    assert out_b.dtype == np.int64
    for r in range(rows):
        ref, _ = O.select_candidates(x[r], k)
        assert np.array_equal(out_b[r], ref)
        assert np.array_equal(out_r[r], ref)
        tv = torch.topk(torch.from_numpy(x[r]), k).values.numpy()  # the reference's own check: same value multiset
        assert np.array_equal(np.sort(x[r][out_b[r]]), np.sort(tv))


def test_bucket_topk_all_equal_and_clamp(ops):
    x = torch.full((2, 3000), 7, dtype=torch.int32, device=DEV)
    assert torch.equal(ops.bucket_topk(x, 50).cpu(), torch.arange(50).expand(2, 50))
    y = torch.tensor([[500, -3, 4, 127, 128, 0, 9, 9]], dtype=torch.int32, device=DEV)
    assert ops.bucket_topk(y, 3).cpu().tolist() == [[0, 3, 4]]  # values clamp to [0,127]: 500,127,128 tie at 127


@pytest.mark.parametrize("rows,L,k", [(32, 4096, 1024), (8, 1024, 256), (3, 777, 100), (2, 8192, 8192), (4, 20000, 2048),
                                      (2, 105000, 2048), (1, 9000, 1), (5, 13107, 1024), (2, 16384, 8192), (3, 16385, 100)])
def test_topk_f32_exact(ops, rows, L, k):
    _say(f"topk_f32 rows={rows} L={L} k={k}")
    rng = np.random.default_rng(L * 7 + k)
    x = rng.standard_normal((rows, L)).astype(np.float32)
    x[:, ::5] = np.round(x[:, ::5], 1)  # exact ties
    ids = np.stack([rng.permutation(4 * L)[:L] for _ in range(rows)]).astype(np.int64)
    tx, tid = torch.from_numpy(x).to(DEV), torch.from_numpy(ids).to(DEV)
    out, vals = ops.topk_f32(tx, k, tid, want_values=True)
    out_pos = ops.topk_f32(tx, k)
    torch.cuda.synchronize()
    for r in range(rows):
        ref_ids, ref_pos = O.topk_f32(x[r], ids[r], k)
        assert np.array_equal(out[r].cpu().numpy(), ref_ids)
        assert np.array_equal(vals[r].cpu().numpy(), x[r][ref_pos])
        assert np.array_equal(out_pos[r].cpu().numpy(), O.topk_f32(x[r], None, k)[1])
    tv = torch.topk(tx, k, dim=-1).values  # same values, same order as torch.topk
    assert torch.equal(vals, tv)


def test_topk_f32_one_workgroup_score_distributions(ops):
    """Rows that one workgroup selects from (at most 8192 scores, k at most half of them) on score distributions
    that steer the kernel through each of its routes: evenly spread scores (bins of the row's own range, counting
    sort), a crowded winner bin (same bins, bitonic sort), a crowded threshold bin, a constant row, an outlier that
    stretches the range, infinities (radix select), exact ties decided by the ids, padded rows and k = 1."""
    rng = np.random.default_rng(2024)
    cases = []
    cases.append(("gaussian", rng.standard_normal((4, 4096)).astype(np.float32) * 20 + 30, 1024))
    x = rng.standard_normal((3, 4096)).astype(np.float32)
    x[:, 100:400] = np.float32(5.0)                                   # 300 winners in one bin
    cases.append(("crowded winner bin", x, 1024))
    x = rng.standard_normal((3, 4096)).astype(np.float32)
    x[:, :2000] = np.float32(0.5) + rng.integers(0, 3, (3, 2000)).astype(np.float32) * np.float32(2.0 ** -22)
    cases.append(("crowded threshold bin", x, 1500))
    cases.append(("constant", np.full((2, 4096), -3.5, np.float32), 700))
    x = rng.standard_normal((2, 4096)).astype(np.float32)
    x[0, 17], x[1, 4000] = 1e6, -1e6
    cases.append(("outlier", x, 1024))
    x = (rng.standard_normal((2, 4096)) * 100).astype(np.float32)
    x[0, 5], x[0, 77], x[1, 4095] = np.inf, -np.inf, np.inf
    cases.append(("infinities", x, 1000))
    cases.append(("ties by id", np.round(rng.standard_normal((3, 4096)) * 16).astype(np.float32) / 16, 1024))
    cases.append(("negative scores", -np.abs(rng.standard_normal((2, 4096))).astype(np.float32) - 1, 1024))
    cases.append(("padded row", rng.standard_normal((5, 3000)).astype(np.float32), 1))
    cases.append(("padded row, k=1500", rng.standard_normal((2, 3001)).astype(np.float32), 1500))
    cases.append(("2 keys per thread", rng.standard_normal((2, 2048)).astype(np.float32), 1024))
    cases.append(("8 keys per thread", rng.standard_normal((2, 8192)).astype(np.float32) ** 3, 4096))
    cases.append(("subnormal range", (rng.integers(0, 50, (2, 4096)).astype(np.float32) * np.float32(1e-45)), 512))
    for name, x, k in cases:
        _say(f"topk_f32 one workgroup: {name} {x.shape} k={k}")
        rows, L = x.shape
        ids = np.stack([rng.permutation(3 * L)[:L] for _ in range(rows)]).astype(np.int64)
        out, vals = ops.topk_f32(torch.from_numpy(x).to(DEV), k, torch.from_numpy(ids).to(DEV), want_values=True)
        torch.cuda.synchronize()
        for r in range(rows):
            ref_ids, ref_pos = O.topk_f32(x[r], ids[r], k)
            assert np.array_equal(out[r].cpu().numpy(), ref_ids), name
            assert np.array_equal(vals[r].cpu().numpy().view(np.uint32), x[r][ref_pos].view(np.uint32)), name


def test_topk_f32_wide_rows_edge_cases(ops):
    """Rows wider than one workgroup sorts (more than 8192 keys): the multi-workgroup histogram / compaction
    path with a threshold bin that holds the whole row (constant scores: every key ties, ids decide), one that
    holds more than 8192 keys, k = 8192, len = 8193, and mixed signs with infinities."""
    rng = np.random.default_rng(99)
    cases = []
    L = 30000
    cases.append(("constant", np.full((2, L), 1.25, np.float32), 700))
    x = rng.standard_normal((3, L)).astype(np.float32)
    x[:, : L // 2] = np.float32(0.75) + rng.integers(0, 4, (3, L // 2)).astype(np.float32) * np.float32(2.0 ** -20)
    cases.append(("crowded threshold bin", x, 9000 // 2))
    # the same with a list short enough for the one-binning selection + sort of the finish kernel, which must hand a
    # threshold bin this crowded (15 000 keys in four values) to the two-step path
    x2 = rng.standard_normal((3, L)).astype(np.float32)
    x2[:, : L // 2] = np.float32(2.5) + rng.integers(0, 4, (3, L // 2)).astype(np.float32) * np.float32(2.0 ** -20)
    cases.append(("crowded threshold bin, short list", x2, 1500))
    cases.append(("k=8192", rng.standard_normal((2, 70000)).astype(np.float32), 8192))
    cases.append(("len=8193", rng.standard_normal((5, 8193)).astype(np.float32), 100))
    y = (rng.standard_normal((2, 20001)) * 1e3).astype(np.float32)
    y[0, 5], y[0, 77], y[1, 20000] = np.inf, -np.inf, np.inf
    y[:, 100:4000] = -np.abs(y[:, 100:4000])
    cases.append(("signs and infinities", y, 3000))
    # scores that share their exponent: bins of fixed key bits would put the whole row into a few bins; the bins of
    # the row's own range keep the threshold bin small
    cases.append(("one binade", (rng.standard_normal((3, 52429)) * 2 + 100).astype(np.float32), 2048))
    cases.append(("narrow range", (rng.standard_normal((2, 20000)) * 1e-3 + 1.5).astype(np.float32), 1000))
    z = (rng.standard_normal((2, 30000)) * 5).astype(np.float32)
    z[0, 123] = 1e30                                   # an outlier stretches the range: everything else in one bin
    cases.append(("outlier", z, 512))
    # more slices than a row has range slots of its own: the control block is cleared by a launch and the slices'
    # ranges meet in two atomic words
    cases.append(("eighteen slices", rng.standard_normal((2, 140000)).astype(np.float32), 1500))
    for name, x, k in cases:
        _say(f"topk_f32 wide: {name} {x.shape} k={k}")
        rows, L = x.shape
        ids = np.stack([rng.permutation(3 * L)[:L] for _ in range(rows)]).astype(np.int64)
        out, vals = ops.topk_f32(torch.from_numpy(x).to(DEV), k, torch.from_numpy(ids).to(DEV), want_values=True)
        torch.cuda.synchronize()
        for r in range(rows):
            ref_ids, ref_pos = O.topk_f32(x[r], ids[r], k)
            assert np.array_equal(out[r].cpu().numpy(), ref_ids), name
            assert np.array_equal(vals[r].cpu().numpy(), x[r][ref_pos]), name
    with pytest.raises(RuntimeError, match="k up to"):
        ops.topk_f32(torch.zeros(1, 20000, device=DEV), 8193)


def test_radix_topk_float_api(ops):
    from pariskv_amd.cache_hub.topk import radix_topk, fast_topk, fast_topk_with_ratio

    g = torch.Generator().manual_seed(0)
    x = torch.rand(4, 3000, generator=g) * 96
    out = radix_topk(x.to(DEV), 64).cpu()
    assert torch.equal(torch.gather(x, 1, out), torch.topk(x, 64).values)
    xi = (x * 1).to(torch.int32)
    assert fast_topk(xi.to(DEV), 64).shape == (4, 64)
    assert fast_topk_with_ratio(xi.to(DEV).view(2, 2, 3000), 0.05).shape == (2, 2, 150)


# ------------------------------------------------------------------- rerank


@pytest.mark.parametrize("layout", ["keymajor", "reference"])
def test_partial_rerank_parity(ops, wl_small_bf16, layout):
    from pariskv_amd.cache_hub.rerank.rerank import partial_rerank_cuda

    w = wl_small_bf16
    _say(f"rerank layout={layout}")
    d = W.to_device(w, DEV, torch)
    k4 = d["nib_km"].view(w.bs, w.H, w.N, 16, 4).permute(0, 1, 3, 2, 4)
    kw = d["w_km"].permute(0, 1, 3, 2)
    if layout == "reference":
        k4, kw = k4.contiguous(), kw.contiguous()
    rng = np.random.default_rng(1)
    cand = np.stack([rng.permutation(w.N)[:w.C] for _ in range(w.R)]).astype(np.int64).reshape(w.bs, w.H, w.C)
    stages = [W.oracle_stages(w, r) for r in range(w.R)]
    q_blocks = torch.from_numpy(np.stack([s["qhat"] for s in stages])).view(w.bs, w.H, 16, 8).to(torch.bfloat16).to(DEV)
    q_norm = torch.tensor([s["qnorm"] for s in stages]).view(w.bs, w.H, 1).to(torch.bfloat16).to(DEV)
    centers = torch.tensor(ops.MAG_CENTERS, dtype=torch.bfloat16, device=DEV)
    scores, v4b = partial_rerank_cuda(torch.from_numpy(cand).to(DEV), k4, kw, q_blocks, q_norm, centers, 16, 8)
    torch.cuda.synchronize()
    assert scores.dtype == torch.float32 and tuple(v4b.shape) == (w.bs, w.H, 16, w.C, 8)
    th, ce = O.mag_constants()
    for r in range(w.R):
        b, h = divmod(r, w.H)
        ref = O.rerank(cand[b, h], w.nib[r], w.weight[r], stages[r]["qhat"], stages[r]["qnorm"])
        got = scores[b, h].cpu().numpy()
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5 * np.abs(ref).max())  # the stated tolerance
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))                 # and in fact identical
        # unpacked values (reference's second output): +-centers by nibble
        nibs = w.nib[r][cand[b, h]]  # [C,16,4]
        v = np.stack([nibs & 0x0F, nibs >> 4], axis=-1).reshape(w.C, 16, 8)
        ref_v = np.where(v & 8, 1.0, -1.0).astype(np.float32) * ce[v & 7]
        assert np.array_equal(v4b[b, h].float().cpu().numpy(), ref_v.transpose(1, 0, 2))


def test_rerank_out_of_range_candidate_is_masked(ops, wl_small_bf16):
    w = wl_small_bf16
    d = W.to_device(w, DEV, torch)
    k4 = d["nib_km"].view(w.bs, w.H, w.N, 16, 4).permute(0, 1, 3, 2, 4)
    kw = d["w_km"].permute(0, 1, 3, 2)
    cand = torch.tensor([0, w.N - 1, w.N, -1, 5], dtype=torch.int64, device=DEV).expand(w.bs, w.H, 5).contiguous()
    qhat = torch.zeros(w.bs, w.H, 128, device=DEV)
    scores, _ = ops.rerank4(cand, k4, kw, qhat, torch.ones(w.bs, w.H, device=DEV), ops.mag_centers(DEV))
    s = scores[0, 0].cpu()
    assert torch.isinf(s[2]) and torch.isinf(s[3]) and s[0] == 0 and s[1] == 0 and s[4] == 0


# ------------------------------------------------------------------ gathers


def test_h2d_gather_kv_matches_index_select(ops):
    from pariskv_amd.cache_hub.gather_trans import h2d_gather_kv

    bs, heads, kv_len, topk, max_topk = 2, 8, 32 * 1024, 100, 160  # shape of trans_h2d.py:108-120
    g = torch.Generator().manual_seed(0)
    src_k = torch.randn(bs, heads, kv_len, 128, generator=g).to(torch.bfloat16).pin_memory()
    src_v = torch.randn(bs, heads, kv_len, 128, generator=g).to(torch.bfloat16).pin_memory()
    idx = torch.randint(0, kv_len, (bs, heads, topk), generator=g)
    dst_k = torch.zeros(bs, heads, max_topk, 128, dtype=torch.bfloat16, device=DEV)
    dst_v = torch.zeros_like(dst_k)
    h2d_gather_kv(src_k, src_v, idx.to(DEV), dst_k, dst_v)
    torch.cuda.synchronize()
    ek = torch.gather(src_k, 2, idx.unsqueeze(-1).expand(-1, -1, -1, 128))
    ev = torch.gather(src_v, 2, idx.unsqueeze(-1).expand(-1, -1, -1, 128))
    assert torch.equal(dst_k[:, :, :topk].cpu().view(torch.int16), ek.view(torch.int16))
    assert torch.equal(dst_v[:, :, :topk].cpu().view(torch.int16), ev.view(torch.int16))
    assert not dst_k[:, :, topk:].any()  # rows beyond topk untouched
    # oracle gather on one row
    ref = O.gather_rows(src_k[1, 3].view(torch.int16).numpy(), idx[1, 3].numpy())
    assert np.array_equal(dst_k[1, 3, :topk].cpu().view(torch.int16).numpy(), ref)
    with pytest.raises(AssertionError):
        h2d_gather_kv(src_k.clone(), src_v, idx.to(DEV), dst_k, dst_v)  # unpinned source


def test_gather_hbm_with_offset_and_bounds(ops):
    bs, H, n, k = 1, 2, 500, 40
    g = torch.Generator().manual_seed(1)
    sk = torch.randn(bs, H, n, 128, generator=g).to(torch.bfloat16).to(DEV)
    sv = torch.randn(bs, H, n, 128, generator=g).to(torch.bfloat16).to(DEV)
    idx = torch.randint(0, n - 20, (bs, H, k), generator=g)
    idx[0, 0, 0] = n  # out of range after the offset -> zero row, no fault
    dk = torch.ones(bs, H, 64, 128, dtype=torch.bfloat16, device=DEV)
    dv = torch.ones_like(dk)
    ops.gather_hbm(sk, sv, idx.to(DEV), dk, dv, idx_offset=20, dst_row0=8)
    torch.cuda.synchronize()
    exp = torch.gather(sk.cpu(), 2, (idx + 20).clamp(max=n - 1).unsqueeze(-1).expand(-1, -1, -1, 128))
    exp[0, 0, 0] = 0
    assert torch.equal(dk[:, :, 8:8 + k].cpu(), exp) and (dk[:, :, :8] == 1).all() and (dk[:, :, 8 + k:] == 1).all()


def test_gather_uva_packed_layout(ops):
    """Ragged gather contract of polar_cache_adaptivek_varlen.py:1573-1644."""
    bs, H, n, sl_end = 2, 2, 1000, 6
    V = bs * H
    g = torch.Generator().manual_seed(2)
    ks = torch.tensor([5, 0, 17, 9])
    src_k = torch.randn(bs, H, n, 128, generator=g).to(torch.bfloat16).pin_memory()
    src_v = torch.randn(bs, H, n, 128, generator=g).to(torch.bfloat16).pin_memory()
    idx_packed = torch.randint(0, n, (int(ks.sum()),), generator=g)
    cu_topk = torch.zeros(V + 1, dtype=torch.int32)
    cu_topk[1:] = torch.cumsum(ks, 0)
    cu_k = torch.zeros(V + 1, dtype=torch.int32)
    cu_k[1:] = torch.cumsum(ks + sl_end, 0)
    total = int(cu_k[-1])
    kp = torch.zeros(total, 128, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros_like(kp)
    ops.gather_uva_packed(src_k, src_v, kp, vp, idx_packed.to(DEV), cu_topk.to(DEV), cu_k.to(DEV), sl_end, int(ks.max()))
    torch.cuda.synchronize()
    exp_k = torch.zeros(total, 128, dtype=torch.bfloat16)
    exp_v = torch.zeros_like(exp_k)
    for v in range(V):
        b, h = divmod(v, H)
        for s in range(int(ks[v])):
            src = int(idx_packed[int(cu_topk[v]) + s])
            exp_k[int(cu_k[v]) + sl_end + s] = src_k[b, h, src]
            exp_v[int(cu_k[v]) + sl_end + s] = src_v[b, h, src]
    assert torch.equal(kp.cpu(), exp_k) and torch.equal(vp.cpu(), exp_v)


# ------------------------------------------------------- fused decode step


def _run_fused(ops, w, gather_host=False):
    d = W.to_device(w, DEV, torch)
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.C, w.K)
    scores = torch.empty(w.bs, w.H, w.K, dtype=torch.float32, device=DEV)
    out = plan.run(d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], 0,
                   w.N, w.tiers, w.C, w.K, out_scores=scores)
    torch.cuda.synchronize()
    return plan, out, scores


def _any_order_model(scores, ids, k):
    """The order in which the one-workgroup top-k writes its k winners when the final sort is left out, restated:
    512 even bins of [row min, row max] (bin = min(511, floor((x - lo) * (512 / (hi - lo)))), fp32 operations); the
    threshold bin b* is the one in which the k-th largest score lies; the winners of the bins above b* come first,
    ordered by the wave that loaded them (element i is loaded by thread i % 1024 as its (i // 1024)-th element), then
    by element, then by lane; the winners inside b* follow in descending (score, smaller id first) order.  None
    where the kernel takes another route (more than 256 scores in b*, or no positive finite range)."""
    x = scores.astype(np.float32)
    lo, hi = x.min(), x.max()
    rng = np.float32(hi - lo)
    if not (np.isfinite(rng) and rng > 0):
        return None
    scale = np.float32(512.0) / rng
    t = ((x - lo) * scale).astype(np.float32)
    b = np.minimum(511, t.astype(np.int64))
    hist = np.bincount(b, minlength=512)
    above = np.cumsum(hist[::-1])[::-1] - hist          # scores in the bins above b
    bstar = int(np.max(np.nonzero((above < k) & (above + hist >= k))[0]))
    if hist[bstar] > 256:
        return None
    need = k - int(above[bstar])
    i = np.arange(len(x))
    tid, e = i % 1024, i // 1024
    first = np.nonzero(b > bstar)[0]
    first = first[np.lexsort((tid[first] % 64, e[first], tid[first] // 64))]
    inside = np.nonzero(b == bstar)[0]
    inside = inside[np.lexsort((ids[inside], -x[inside].astype(np.float64)))][:need]
    return np.concatenate([ids[first], ids[inside]])


@pytest.mark.parametrize("wl_name", ["wl_cfg1", "wl_cfg2", "wl_small_bf16"])
def test_retrieve_any_order_is_the_same_set_in_a_fixed_order(ops, request, wl_name):
    """any_order leaves the final sort out: the k ids are the sorted mode's ids exactly (as a set, scores attached
    to the right ids), they come in the documented order of their candidate-list positions (restated by
    _any_order_model), and two runs agree bit for bit."""
    w = request.getfixturevalue(wl_name)
    _say(f"retrieve any_order {w.name}")
    d = W.to_device(w, DEV, torch)
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.C, w.K)
    args = (d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], 0, w.N, w.tiers,
            w.C, w.K)
    s_sorted = torch.empty(w.bs, w.H, w.K, dtype=torch.float32, device=DEV)
    s_any = torch.empty_like(s_sorted)
    ids_sorted = plan.run(*args, out_scores=s_sorted).clone()
    ids_any = plan.run(*args, out_scores=s_any, any_order=True).clone()
    cand = plan.view("cand", w.N, w.C, w.K, torch.int64).view(w.R, w.C).cpu().numpy()
    ids_again = plan.run(*args, any_order=True)
    torch.cuda.synchronize()
    assert torch.equal(ids_any, ids_again)
    a, b_ = ids_sorted.view(w.R, w.K).cpu().numpy(), ids_any.view(w.R, w.K).cpu().numpy()
    sa, sb = s_sorted.view(w.R, w.K).cpu().numpy(), s_any.view(w.R, w.K).cpu().numpy()
    for r in range(w.R):
        assert np.array_equal(np.sort(a[r]), np.sort(b_[r]))
        assert dict(zip(a[r].tolist(), sa[r].tolist())) == dict(zip(b_[r].tolist(), sb[r].tolist()))
        if 2048 <= w.C <= 8192 and 4 * w.K <= w.C:
            # the select kernel without its sort: the documented order, restated from the candidate list and its scores
            sc_all = plan.view("scores", w.N, w.C, w.K, torch.float32).view(w.R, w.C)[r].cpu().numpy()
            want = _any_order_model(sc_all, cand[r], w.K)
            if want is not None:
                assert np.array_equal(b_[r], want), f"any-order ids of row {r} are not in the documented order"
        else:                                         # other shapes keep the descending-score order
            assert np.array_equal(a[r], b_[r])


@pytest.mark.parametrize("wl_name", ["wl_cfg1", "wl_cfg2", "wl_small_bf16"])
def test_retrieve_fused_matches_oracle(ops, request, wl_name):
    w = request.getfixturevalue(wl_name)
    _say(f"retrieve {w.name}: R={w.R} N={w.N} C={w.C} K={w.K}")
    plan, out, scores = _run_fused(ops, w)
    cnt_stride = (w.N + 15) // 16 * 16
    cnt = plan.view("cnt_u8", w.N, w.C, w.K, torch.uint8).view(w.R, cnt_stride)[:, :w.N].cpu().numpy()
    cand = plan.view("cand", w.N, w.C, w.K, torch.int64).view(w.R, w.C).cpu().numpy()
    sc = plan.view("scores", w.N, w.C, w.K, torch.float32).view(w.R, w.C).cpu().numpy()
    suf = plan.view("chunk_suffix_hist", w.N, w.C, w.K, torch.int16).view(w.R, -1, 128).cpu().numpy().astype(np.int64) & 0xFFFF
    row_suf = plan.view("row_suffix_hist", w.N, w.C, w.K, torch.int32).view(w.R, 128).cpu().numpy().astype(np.int64)
    for r in range(w.R):
        b, h = divmod(r, w.H)
        st = W.oracle_stages(w, r)
        assert np.array_equal(cnt[r], st["cnt"].astype(np.uint8)), f"vote counts differ in row {r}"
        ref_suf = np.cumsum(np.bincount(st["cnt"], minlength=128)[::-1])[::-1]  # keys with count >= t
        assert np.array_equal(suf[r].sum(axis=0), ref_suf) and np.array_equal(row_suf[r], ref_suf), f"histogram row {r}"
        assert np.array_equal(cand[r], st["cand"]), f"candidate list differs in row {r}"
        np.testing.assert_allclose(sc[r], st["scores"], rtol=1e-5, atol=1e-5 * np.abs(st["scores"]).max())
        assert np.array_equal(out[b, h].cpu().numpy(), st["final"]), f"final top-k differs in row {r}"
        assert np.array_equal(scores[b, h].cpu().numpy(), st["final_scores"])
        # whole-row oracle entry point agrees as well
        q = w.queries[b, h * w.G:(h + 1) * w.G]
        whole = O.retrieve_row(q, w.signs, w.dtype, w.codes[r], w.nib[r], w.weight[r], w.cluster_counts[r], w.tiers, w.C, w.K)
        assert np.array_equal(out[b, h].cpu().numpy(), whole)


@pytest.mark.parametrize("wl_name", ["wl_cfg1", "wl_cfg2", "wl_small_bf16"])
def test_one_launch_plan_equals_three_launches(ops, request, wl_name):
    """pkv_retrieve_args.launch_plan = PKV_PLAN_ONE_LAUNCH (query prep, scan and select + rerank as one launch whose
    workgroups hand the vote table and the histogram over) against the three launches: every intermediate and every
    output bit for bit, and against the oracle; with the flag area full of garbage before the first launch, three
    launches back to back on one workspace, no workgroup giving up a wait."""
    from pariskv_amd import _lib

    w = request.getfixturevalue(wl_name)
    _say(f"one-launch plan {w.name}: R={w.R} N={w.N} C={w.C} K={w.K}")
    d = W.to_device(w, DEV, torch)
    args = (d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], 0, w.N, w.tiers,
            w.C, w.K)
    names = (("qhat", torch.float32), ("qnorm", torch.float32), ("lut", torch.uint8), ("chunk_suffix_hist", torch.int16),
             ("row_suffix_hist", torch.int32), ("cand", torch.int64), ("scores", torch.float32))
    cnt_stride = (w.N + 15) // 16 * 16
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.C, w.K)
    ref_sc = torch.empty(w.bs, w.H, w.K, dtype=torch.float32, device=DEV)
    ref_ids = plan.run(*args, out_scores=ref_sc).clone()
    ref = {n: plan.view(n, w.N, w.C, w.K, dt).clone() for n, dt in names}
    ref_cnt = plan.view("cnt_u8", w.N, w.C, w.K, torch.uint8).view(w.R, cnt_stride)[:, :w.N].clone()
    plan.launch_plan = _lib.PLAN_ONE_LAUNCH
    plan.ws.fill_(0xA5)
    for rep in range(3):
        plan.skip_vote_counts = rep == 2
        if rep == 2:
            plan.view("cnt_u8", w.N, w.C, w.K, torch.uint8).zero_()
        sc = torch.empty_like(ref_sc)
        ids = plan.run(*args, out_scores=sc)
        torch.cuda.synchronize()
        assert int(plan.view("handover_status", w.N, w.C, w.K, torch.int32)[0]) == 0
        assert torch.equal(ids, ref_ids) and torch.equal(sc, ref_sc)
        for n, dt in names:
            assert torch.equal(plan.view(n, w.N, w.C, w.K, dt), ref[n]), f"{n} differs in launch {rep}"
        cnt = plan.view("cnt_u8", w.N, w.C, w.K, torch.uint8).view(w.R, cnt_stride)[:, :w.N]
        if rep == 2:
            assert not bool(cnt.any())  # the counts stayed on chip
        else:
            assert torch.equal(cnt, ref_cnt)
    for r in range(w.R):
        b, h = divmod(r, w.H)
        assert np.array_equal(ids[b, h].cpu().numpy(), W.oracle_stages(w, r)["final"])


def test_retrieve_large_rows_strided_pieces(ops):
    """Rows long enough for 8192-key chunks (8 rows x 600 000 keys): the collision scan and the select + rerank then
    work on four pieces per chunk spread over the row.  Keys with a drifting mean (candidates bunch in bands) and a
    ragged last chunk; candidate list, scores and final ids of three rows against the oracle, all rows against the
    one-launch plan (whole chunks)."""
    from pariskv_amd import _lib

    bs, H, G, N, C, K = 1, 8, 4, 600_000, 30_000, 512
    _say(f"strided pieces: N={N} C={C} K={K}")
    assert ops.pick_chunk_keys(bs * H, N) == 8192
    g = torch.Generator(device=DEV).manual_seed(11)
    keys = torch.randn(bs, H, N, 128, generator=g, device=DEV)
    keys[..., [7, 31, 64, 101]] *= 10.0
    ang = torch.arange(N, device=DEV, dtype=torch.float32) * (5.0 / 1000.0) * (math.pi / 180.0)
    keys[..., 0] += 2.0 * torch.cos(ang)
    keys[..., 1] += 2.0 * torch.sin(ang)
    keys = keys.to(torch.bfloat16)
    q = (keys[:, :, -2048:].float().mean(dim=2, keepdim=True) + 0.5 * torch.randn(bs, H, G, 128, generator=g, device=DEV))
    q = q.to(torch.bfloat16).view(bs, 1, H * G, 128).contiguous()
    signs, centers = ops.srht_signs(DEV), ops.mag_centers(DEV)
    codes_km, nib_km, w_km, cb, k4, kw = ops.alloc_keymajor(bs, H, N, DEV)
    cc = torch.zeros(bs, H, 16, 256, dtype=torch.int32, device=DEV)
    ops.encode_append(keys, signs, cb, k4, kw, cc)
    tiers = O.tier_counts(N, 0.2)
    plan = ops.RetrievePlan(bs, H, G, N, DEV, N, C, K)
    args = (q, signs, centers, cc, codes_km, nib_km, w_km, 0, N, tiers, C, K)
    sc = torch.empty(bs, H, K, device=DEV)
    ids = plan.run(*args, out_scores=sc).clone()
    cand = plan.view("cand", N, C, K, torch.int64).view(H, C).clone()
    csc = plan.view("scores", N, C, K, torch.float32).view(H, C).clone()
    per_chunk = torch.bincount(cand[0] // 8192, minlength=(N + 8191) // 8192)
    assert int(per_chunk.max()) > 1.5 * C / per_chunk.numel()  # the data does bunch
    plan.launch_plan = _lib.PLAN_ONE_LAUNCH
    ids1 = plan.run(*args)
    torch.cuda.synchronize()
    assert int(plan.view("handover_status", N, C, K, torch.int32)[0]) == 0
    assert torch.equal(ids, ids1)
    assert torch.equal(plan.view("cand", N, C, K, torch.int64).view(H, C), cand)
    assert torch.equal(plan.view("scores", N, C, K, torch.float32).view(H, C), csc)
    sg = signs.cpu().numpy()
    for r in (0, 4, 7):
        qh, qn = O.query_prep(q.view(bs, H, G, 128)[0, r].float().cpu().numpy(), sg, O.BF16)
        lut = O.tier_lut(O.rank_centroids(qh, O.BF16), cc[0, r].cpu().numpy(), tiers)
        cand_ref, _ = O.select_candidates(O.collision_count(codes_km[0, r].cpu().numpy(), lut), C)
        assert np.array_equal(cand[r].cpu().numpy(), cand_ref), f"candidate list of row {r}"
        sc_ref = O.rerank(cand_ref, nib_km[0, r].cpu().numpy().reshape(N, 16, 4), w_km[0, r].float().cpu().numpy(), qh, qn)
        np.testing.assert_allclose(csc[r].cpu().numpy(), sc_ref, rtol=1e-5, atol=1e-5 * np.abs(sc_ref).max())
        final, _ = O.topk_f32(sc_ref, cand_ref, K)
        assert np.array_equal(ids[0, r].cpu().numpy(), final), f"final ids of row {r}"


def test_retrieve_subrange_and_candidates_equal_keys(ops, wl_small_bf16):
    """Retrieval zone = [key0, key0+n) of a larger capacity; and C == N (identity candidates)."""
    w = wl_small_bf16
    d = W.to_device(w, DEV, torch)
    key0, n = 64, 2000
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.N, 64)
    tiers = O.tier_counts(n, 0.5)
    out = plan.run(d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], key0,
                   n, tiers, 200, 64)
    out_all = plan.run(d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"],
                       key0, n, tiers, n, 64)
    torch.cuda.synchronize()
    for r in range(w.R):
        b, h = divmod(r, w.H)
        q = w.queries[b, h * w.G:(h + 1) * w.G]
        sl = slice(key0, key0 + n)
        ref = O.retrieve_row(q, w.signs, w.dtype, w.codes[r][sl], w.nib[r][sl], w.weight[r][sl], w.cluster_counts[r], tiers, 200, 64)
        assert np.array_equal(out[b, h].cpu().numpy(), ref)
        qhat, qn = O.query_prep(q, w.signs, w.dtype)
        s_all = O.rerank(np.arange(n), w.nib[r][sl], w.weight[r][sl], qhat, qn)
        assert np.array_equal(out_all[b, h].cpu().numpy(), O.topk_f32(s_all, None, 64)[0])


def test_retrieve_with_uva_gather(ops, wl_small_bf16):
    w = wl_small_bf16
    d = W.to_device(w, DEV, torch)
    kcpu = torch.from_numpy(w.keys.reshape(w.bs, w.H, w.N, 128)).to(torch.bfloat16).pin_memory()
    vcpu = torch.from_numpy(w.values.reshape(w.bs, w.H, w.N, 128)).to(torch.bfloat16).pin_memory()
    dk = torch.zeros(w.bs, w.H, w.K + 3, 128, dtype=torch.bfloat16, device=DEV)
    dv = torch.zeros_like(dk)
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.C, w.K)
    out = plan.run(d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], 0,
                   w.N, w.tiers, w.C, w.K,
                   gather=dict(src_k=kcpu, src_v=vcpu, from_host=True, dst_k=dk, dst_v=dv, dst_row0=3))
    torch.cuda.synchronize()
    idx = out.cpu().unsqueeze(-1).expand(-1, -1, -1, 128)
    assert torch.equal(dk[:, :, 3:].cpu(), torch.gather(kcpu, 2, idx))
    assert torch.equal(dv[:, :, 3:].cpu(), torch.gather(vcpu, 2, idx))
    for r in range(w.R):
        b, h = divmod(r, w.H)
        assert np.array_equal(out[b, h].cpu().numpy(), W.oracle_stages(w, r)["final"])


def test_retrieve_argument_errors(ops, wl_small_bf16):
    w = wl_small_bf16
    d = W.to_device(w, DEV, torch)
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.C, w.K)
    args = (d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"])
    with pytest.raises(RuntimeError):
        plan.run(*args, 0, w.N, w.tiers, w.C, w.C + 1)        # k > n_cand
    with pytest.raises(RuntimeError):
        plan.run(*args, 10, w.N, w.tiers, w.C, w.K)           # zone exceeds capacity
    with pytest.raises(RuntimeError):
        plan.run(*args, 0, w.N, w.tiers, w.N + 1, w.K)        # n_cand > n_keys


# ------------------------------------------------ full-size property checks


@pytest.mark.parametrize("N,R,C,K", [(131072, 32, 4096, 1024)])
def test_full_size_properties(ops, N, R, C, K):
    """BASELINE config 3 at full size on GPU-generated inputs (batch 4, an independent seed per sequence, K/V in
    pinned host memory): size-independent properties of the whole step, the UVA gather of all 32 x 1024 selected rows
    bit for bit against torch.gather on the pinned tensors, and 8 rows spread over the four sequences against the
    oracle (GPU-encoded index copied back to the host; the encode of those rows against the oracle's too).  Both
    launch plans."""
    from pariskv_amd import _lib

    _say(f"full-size N={N} R={R} C={C} K={K}")
    bs, H, G = 4, 8, 4
    signs = ops.srht_signs(DEV)
    codes_km, nib_km, w_km, cb, k4, kw = ops.alloc_keymajor(bs, H, N, DEV)
    cc = torch.zeros(bs, H, 16, 256, dtype=torch.int32, device=DEV)
    q = torch.empty(bs, 1, H * G, 128, dtype=torch.bfloat16, device=DEV)
    keys = torch.empty(bs, H, N, 128, dtype=torch.bfloat16, device=DEV)
    kcpu = torch.empty(bs, H, N, 128, dtype=torch.bfloat16, pin_memory=True)
    vcpu = torch.empty(bs, H, N, 128, dtype=torch.bfloat16, pin_memory=True)
    for b in range(bs):
        g = torch.Generator(device=DEV).manual_seed(1000 * 3 + b)  # one seed per sequence
        kf = torch.randn(1, H, N, 128, generator=g, device=DEV, dtype=torch.float32)
        kf[..., [7, 31, 64, 101]] *= 10
        keys[b] = kf[0].to(torch.bfloat16)
        q[b, 0] = (kf.mean(dim=2, keepdim=True) + 0.5 * torch.randn(1, H, G, 128, generator=g, device=DEV)).view(H * G, 128).to(torch.bfloat16)
        ops.encode_append(keys[b:b + 1], signs, cb[b:b + 1], k4[b:b + 1], kw[b:b + 1], cc[b:b + 1])
        kcpu[b].copy_(keys[b])
        vcpu[b].copy_(torch.randn(H, N, 128, generator=g, device=DEV).to(torch.bfloat16))
        del kf
    assert int(cc.sum()) == R * N * 16 and bool((cc.sum(dim=-1) == N).all())  # every key lands in one cluster per subspace
    tiers = O.tier_counts(N, 0.2)
    plan = ops.RetrievePlan(bs, H, G, N, DEV, N, C, K)
    sc = torch.empty(bs, H, K, device=DEV)
    dk = torch.zeros(bs, H, K, 128, dtype=torch.bfloat16, device=DEV)
    dv = torch.zeros_like(dk)
    gather = dict(src_k=kcpu, src_v=vcpu, from_host=True, dst_k=dk, dst_v=dv)
    out1 = plan.run(q, signs, ops.mag_centers(DEV), cc, codes_km, nib_km, w_km, 0, N, tiers, C, K, out_scores=sc, gather=gather).clone()
    cand = plan.view("cand", N, C, K, torch.int64).view(R, C).clone()
    cnt = plan.view("cnt_u8", N, C, K, torch.uint8).view(R, N).clone()
    out2 = plan.run(q, signs, ops.mag_centers(DEV), cc, codes_km, nib_km, w_km, 0, N, tiers, C, K)
    plan.launch_plan = _lib.PLAN_ONE_LAUNCH
    out3 = plan.run(q, signs, ops.mag_centers(DEV), cc, codes_km, nib_km, w_km, 0, N, tiers, C, K).clone()
    out4 = plan.run(q, signs, ops.mag_centers(DEV), cc, codes_km, nib_km, w_km, 0, N, tiers, C, K)
    torch.cuda.synchronize()
    assert int(plan.view("handover_status", N, C, K, torch.int32)[0]) == 0
    assert torch.equal(out1, out2) and torch.equal(out1, out3) and torch.equal(out1, out4)  # deterministic, both plans
    assert torch.equal(plan.view("cand", N, C, K, torch.int64).view(R, C), cand)
    # the gather of every selected row out of pinned host memory
    idx = out1.cpu().unsqueeze(-1).expand(-1, -1, -1, 128)
    assert torch.equal(dk.cpu(), torch.gather(kcpu, 2, idx)) and torch.equal(dv.cpu(), torch.gather(vcpu, 2, idx))
    assert bool((sc[..., :-1] >= sc[..., 1:]).all())                 # descending scores
    assert bool((out1 >= 0).all()) and bool((out1 < N).all())
    srt = out1.sort(dim=-1).values
    assert bool((srt[..., 1:] != srt[..., :-1]).all())               # no duplicates
    # candidates: distinct, and every non-candidate has a count <= every candidate's
    cs = cand.sort(dim=-1).values
    assert bool((cs[:, 1:] != cs[:, :-1]).all())
    cand_cnt = torch.gather(cnt, 1, cand)
    mask = torch.ones_like(cnt, dtype=torch.bool).scatter_(1, cand, False)
    rest_max = torch.where(mask, cnt, torch.zeros_like(cnt)).max(dim=1).values
    assert bool((cand_cnt.min(dim=1).values >= rest_max).all())
    # final ids are a subset of the candidates
    assert bool(torch.isin(out1.view(R, K), cand).all())
    # rows of every sequence against the oracle, using the GPU-encoded index
    sg = signs.cpu().numpy()
    for r in (0, 5, 10, 13, 19, 22, 28, 31):
        b, h = divmod(r, H)
        ref = O.retrieve_row(q.view(bs, H, G, 128)[b, h].float().cpu().numpy(), sg, O.BF16,
                             codes_km[b, h].cpu().numpy(), nib_km[b, h].cpu().numpy().reshape(N, 16, 4),
                             w_km[b, h].float().cpu().numpy(), cc[b, h].cpu().numpy(), tiers, C, K)
        assert np.array_equal(out1[b, h].cpu().numpy(), ref), f"row {r}"
    for r in (0, 13, 31):  # and the GPU encode of these rows equals the oracle's encode
        b, h = divmod(r, H)
        codes, nib, wt = O.encode(keys[b, h].float().cpu().numpy(), sg, O.BF16)
        assert np.array_equal(codes_km[b, h].cpu().numpy(), codes)
        assert np.array_equal(nib_km[b, h].cpu().numpy().reshape(N, 16, 4), nib)
        assert np.array_equal(w_km[b, h].float().cpu().numpy(), wt)


# --------------------------------------------------------------- adaptive-k


def _adaptive_recipe(bs, kv_heads, sl_len, cand_len, seed, head_dim=128):
    """Seeded input recipe of the reference's adaptive-k self-test (adaptive_topk.py:178-249), on the CPU."""
    torch.manual_seed(seed)
    q = (torch.randn(bs, kv_heads, head_dim) * 0.1).to(torch.bfloat16)
    slk = (torch.randn(bs, kv_heads, sl_len, head_dim) * 0.1).to(torch.bfloat16)
    sl_vnorm = torch.rand(bs, kv_heads, sl_len) + 0.5
    base = math.sqrt(head_dim)
    cs = torch.randn(bs, kv_heads, cand_len) * (0.3 * base)
    rng = torch.Generator().manual_seed(seed)
    heavy = torch.randint(16, 1025, (bs, kv_heads), generator=rng).tolist()
    for b in range(bs):
        for h in range(kv_heads):
            n = min(heavy[b][h], cand_len)
            cs[b, h, :n] += torch.rand(n) * 5.0 * base + 3.0 * base
    ci = torch.stack([torch.stack([torch.randperm(cand_len) for _ in range(kv_heads)]) for _ in range(bs)])
    cv = torch.rand(bs, kv_heads, cand_len) + 0.5
    return q, slk, sl_vnorm, cs.to(torch.bfloat16), ci, cv, 1.0 / base


@pytest.mark.parametrize("cfg", [dict(bs=1, kv_heads=8, sl_len=320, cand_len=12500, topk_cap=2048, threshold=0.95, seed=42),
                                 dict(bs=1, kv_heads=8, sl_len=832, cand_len=5000, topk_cap=2048, threshold=0.95, seed=7),
                                 dict(bs=2, kv_heads=8, sl_len=576, cand_len=8000, topk_cap=2048, threshold=0.85, seed=123),
                                 dict(bs=1, kv_heads=16, sl_len=320, cand_len=15000, topk_cap=2048, threshold=0.95, seed=99),
                                 dict(bs=1, kv_heads=2, sl_len=64, cand_len=700, topk_cap=2048, threshold=0.95, seed=5),
                                 dict(bs=1, kv_heads=2, sl_len=320, cand_len=104858, topk_cap=2048, threshold=0.95, seed=6)])
def test_adaptive_topk_matches_oracle(ops, cfg):
    """The reference's four seeded shapes (adaptive_topk.py:492-497) + a short and a 1M-context-sized one.
    Its acceptance rule is `k exact, first-k index sets equal`; with the fixed tie rule the whole list is compared."""
    from pariskv_amd.cache_hub.adaptive_k_fused import adaptive_topk_cuda

    _say(f"adaptive_topk {cfg}")
    q, slk, slv, cs, ci, cv, scale = _adaptive_recipe(cfg["bs"], cfg["kv_heads"], cfg["sl_len"], cfg["cand_len"], cfg["seed"])
    ak, ids = adaptive_topk_cuda(q.to(DEV), slk.to(DEV), slv.to(DEV), cs.to(DEV), ci.to(DEV), cv.to(DEV), scale,
                                 cfg["threshold"], cfg["topk_cap"])
    torch.cuda.synchronize()
    k_out = min(cfg["topk_cap"], cfg["cand_len"])
    assert tuple(ids.shape) == (cfg["bs"], cfg["kv_heads"], k_out) and ak.dtype == torch.int64
    # same dense logits expression as the call under test, evaluated by torch on the GPU
    sl_logits = (torch.einsum("bhd,bhkd->bhk", q.to(DEV), slk.to(DEV)).to(torch.float32) * scale).cpu().numpy()
    for b in range(cfg["bs"]):
        for h in range(cfg["kv_heads"]):
            lc = (cs[b, h].float() * np.float32(scale)).numpy()
            k_ref, ids_ref = O.adaptive_topk(sl_logits[b, h], slv[b, h].numpy(), lc, cv[b, h].numpy(), ci[b, h].numpy(),
                                             cfg["threshold"], k_out)
            assert int(ak[b, h]) == k_ref, (b, h, int(ak[b, h]), k_ref)
            assert np.array_equal(ids[b, h].cpu().numpy(), ids_ref)
    assert int(ak.min()) >= 1 and int(ak.max()) <= k_out


def test_adaptive_topk_value_norm_gather_and_edges(ops):
    """v2 form: bf16 scores scaled in the kernel, ||v|| gathered at cand_idx + sink (varlen call site :1741-1753);
    plus total <= 0 -> 1 and never reached -> k_out."""
    bs, H, sl, Cn, cap, sink = 1, 3, 100, 3000, 5000, 64
    q, slk, slv, cs, ci, cv, scale = _adaptive_recipe(bs, H, sl, Cn, 11)
    vn = torch.rand(bs, H, cap) + 0.5
    sl_logits = (torch.einsum("bhd,bhkd->bhk", q, slk).float() * scale)
    ak, ids = ops.adaptive_topk(sl_logits.to(DEV), slv.to(DEV), cs.to(DEV), scale, ci.to(DEV), 0.9, 1024,
                                value_norm=vn.to(DEV), vn_offset=sink)
    for h in range(H):
        cvn = vn[0, h][ci[0, h] + sink]
        k_ref, ids_ref = O.adaptive_topk(sl_logits[0, h].numpy(), slv[0, h].numpy(), (cs[0, h].float() * np.float32(scale)).numpy(),
                                         cvn.numpy(), ci[0, h].numpy(), 0.9, 1024)
        assert int(ak[0, h]) == k_ref and np.array_equal(ids[0, h].cpu().numpy(), ids_ref)
    z = torch.zeros(1, 1, 50, device=DEV)
    ak, _ = ops.adaptive_topk(z[..., :5], z[..., :5], z, 1.0, torch.arange(50, device=DEV).view(1, 1, 50), 0.95, 10, cand_vnorm=z)
    assert int(ak) == 1
    one = torch.ones(1, 1, 50, device=DEV)
    ak, ids = ops.adaptive_topk(z[..., :1], one[..., :1], z, 1.0, torch.arange(50, device=DEV).flip(0).view(1, 1, 50).contiguous(),
                                0.95, 10, cand_vnorm=one)
    assert int(ak) == 10 and ids[0, 0].cpu().tolist() == list(range(49, 39, -1))


@pytest.mark.parametrize("sl,Cn,k_out,thr,mode", [(9000, 3000, 3000, 0.97, "cv"),       # dense sum over two slices, k_out == n_cand
                                                  (0, 20000, 4096, 0.5, "cv"),          # no dense tokens, wide path, early k
                                                  (300, 40000, 8192, 0.999, "gather"),  # wide path, largest k_out, norm gather
                                                  (300, 8192, 1000, 0.6, "gather"),     # widest one-workgroup row
                                                  (300, 8193, 1000, 0.6, "gather"),     # narrowest multi-workgroup row
                                                  (50, 30000, 500, 0.9, "ties")])       # quantised benefits: crowded bins
def test_adaptive_topk_shapes_and_orders(ops, sl, Cn, k_out, thr, mode):
    """Adaptive-k against the CPU checker on shapes that exercise each summation / selection branch: k exact,
    ids identical (both follow the same fixed orders)."""
    _say(f"adaptive_topk sl={sl} C={Cn} k_out={k_out} thr={thr} {mode}")
    g = torch.Generator().manual_seed(sl * 31 + Cn)
    H, cap, off = 3, 50000, 17
    sc = torch.randn(1, H, Cn, generator=g) * 6 + 4
    if mode == "ties":
        sc = torch.round(sc)
    sll = torch.randn(1, H, sl, generator=g) * 2 + 6
    slv = torch.rand(1, H, sl, generator=g) + 0.5
    ci = torch.stack([torch.randperm(cap - off, generator=g)[:Cn] for _ in range(H)]).view(1, H, Cn)
    scale = 0.25
    if mode == "gather":
        vn = torch.rand(1, H, cap, generator=g) + 0.5
        ak, ids = ops.adaptive_topk(sll.to(DEV), slv.to(DEV), sc.to(DEV), scale, ci.to(DEV), thr, k_out,
                                    value_norm=vn.to(DEV), vn_offset=off)
        cv = torch.stack([vn[0, h][ci[0, h] + off] for h in range(H)]).view(1, H, Cn)
    else:
        cv = torch.rand(1, H, Cn, generator=g) + 0.5 if mode == "cv" else torch.ones(1, H, Cn)
        ak, ids = ops.adaptive_topk(sll.to(DEV), slv.to(DEV), sc.to(DEV), scale, ci.to(DEV), thr, k_out, cand_vnorm=cv.to(DEV))
    torch.cuda.synchronize()
    ks = []
    for h in range(H):
        k_ref, ids_ref = O.adaptive_topk(sll[0, h].numpy(), slv[0, h].numpy(), (sc[0, h] * np.float32(scale)).numpy(),
                                         cv[0, h].numpy(), ci[0, h].numpy(), thr, k_out)
        assert int(ak[0, h]) == k_ref
        assert np.array_equal(ids[0, h].cpu().numpy(), ids_ref)
        ks.append(k_ref)
    if thr <= 0.6:
        assert max(ks) < k_out  # the threshold is reached inside the list in these cases


def test_adaptive_topk_config4_rows_land_at_different_k(ops):
    """BASELINE config 4's adaptive-k shape (8 rows x ceil(0.05 * 2^20) candidates, list 2048, mass 0.95, clamp
    [256, 2048], value norms gathered from a 2^20-entry table) on scores whose mass is spread differently per row:
    benefits decay like exp(-rank / tau_r), so the 0.95 mass is reached near 3 tau_r and every row stops at its own
    k strictly inside the clamp.  k and the whole id list against the CPU checker."""
    H, N, sink, sl = 8, 1 << 20, 64, 64 + 512
    Cn, k_out, thr, k_min, k_max = int(math.ceil(N * 0.05)), 2048, 0.95, 256, 2048
    taus = [110.0, 170.0, 240.0, 320.0, 400.0, 480.0, 560.0, 630.0]
    g = torch.Generator().manual_seed(44)
    scale = 1.0 / math.sqrt(128)
    sc = torch.empty(1, H, Cn)
    ci = torch.empty(1, H, Cn, dtype=torch.int64)
    for h in range(H):
        rank = torch.randperm(Cn, generator=g).float()                          # rank of candidate i in its row
        sc[0, h] = (-(rank / taus[h]) + 0.3 * torch.rand(Cn, generator=g)) / scale
        ci[0, h] = torch.sort(torch.randperm(N, generator=g)[:Cn]).values       # sorted positions, as the select emits them
    sll = torch.randn(1, H, sl, generator=g) * 0.5 - 6.0                          # the dense tokens hold a small share of the mass
    slv = torch.rand(1, H, sl, generator=g) + 0.5
    vn = torch.rand(1, H, N + sink, generator=g) * 0.2 + 0.9
    _say(f"adaptive-k config 4 shape: {H} rows x {Cn} candidates")
    ak, ids, rk = ops.adaptive_topk(sll.to(DEV), slv.to(DEV), sc.to(DEV), scale, ci.to(DEV), thr, k_out,
                                    value_norm=vn.to(DEV), vn_offset=sink, k_min=k_min, k_max=k_max, row_keys_base=sl)
    torch.cuda.synchronize()
    rk = rk.view(-1)
    ks = []
    for h in range(H):
        cvn = vn[0, h][ci[0, h] + sink]
        k_ref, ids_ref = O.adaptive_topk(sll[0, h].numpy(), slv[0, h].numpy(), (sc[0, h] * np.float32(scale)).numpy(),
                                         cvn.numpy(), ci[0, h].numpy(), thr, k_out)
        assert k_min < k_ref < k_max, (h, k_ref)
        assert int(ak[0, h]) == k_ref and int(rk[h]) == sl + k_ref
        assert np.array_equal(ids[0, h].cpu().numpy(), ids_ref)
        ks.append(k_ref)
    assert len(set(ks)) == H and ks == sorted(ks), ks
    _say(f"adaptive k per row: {ks}")


def test_adaptive_topk_wide_zero_mass(ops):
    """total <= 0 on the multi-workgroup path: k = 1 (adaptive_topk.py:304-306); ids still ordered by position."""
    Cn = 10000
    z = torch.zeros(1, 2, Cn, device=DEV)
    ci = torch.arange(Cn, device=DEV).flip(0).expand(1, 2, Cn).contiguous()
    ak, ids = ops.adaptive_topk(z[..., :7], z[..., :7], z, 1.0, ci, 0.95, 300, cand_vnorm=z)
    assert ak.flatten().tolist() == [1, 1]
    assert ids[0, 1].cpu().tolist() == list(range(Cn - 1, Cn - 301, -1))


# ---------------------------------- BASELINE config 4: 1M keys, adaptive-k, packed gather


def test_million_key_adaptive_pipeline(ops):
    """Llama-3-8B head shape, batch 1, 1M cached keys per head with a slowly drifting key mean (0.5 degrees per 1K
    tokens), bucket top-k over 1M vote counts, rerank of all candidates, adaptive-k (k clamped to [256, 2048], mass
    0.95), packed UVA gather.  Every stage of two sampled rows is compared with the oracle; the rest by properties."""
    from pariskv_amd.cache_hub.topk import load_radix_topk_ext

    _say("cfg4: N=2^20")
    bs, H, G, N = 1, 8, 4, 1 << 20
    sink, sl = 64, 64 + 512
    Cn = int(math.ceil(N * 0.05))
    cap_k, min_k, thr = 2048, 256, 0.95
    g = torch.Generator(device=DEV).manual_seed(4)
    keys = torch.randn(bs, H, N, 128, generator=g, device=DEV)
    keys[..., [7, 31, 64, 101]] *= 10.0
    ang = torch.arange(N, device=DEV, dtype=torch.float32) * (0.5 / 1000.0) * (math.pi / 180.0)
    keys[..., 0] += 3.0 * torch.cos(ang)
    keys[..., 1] += 3.0 * torch.sin(ang)
    keys = keys.to(torch.bfloat16)
    q = (keys[:, :, -4096:].float().mean(dim=2, keepdim=True) + 0.5 * torch.randn(bs, H, G, 128, generator=g, device=DEV))
    q = q.to(torch.bfloat16).view(bs, 1, H * G, 128).contiguous()
    signs = ops.srht_signs(DEV)
    codes_km, nib_km, w_km, cb, k4, kw = ops.alloc_keymajor(bs, H, N, DEV)
    cc = torch.zeros(bs, H, 16, 256, dtype=torch.int32, device=DEV)
    ops.encode_append(keys, signs, cb, k4, kw, cc)
    tiers = O.tier_counts(N, 0.2)
    assert tiers == [10486, 31458, 62915, 104858, 157287, 209716]
    qhat, qnorm, lut, _ = ops.query_prep_lut(q, H, signs, cc, tiers)
    cnt, _, _ = ops.collision_scan(cb, lut, out_dtype=torch.int32)
    cand = load_radix_topk_ext().radix_topk_3d(cnt, Cn)          # "radix top-k over 1M scores" (polar_cache.py:1241)
    scores, _ = ops.rerank4(cand, k4, kw, qhat, qnorm, ops.mag_centers(DEV))
    # dense side of adaptive-k: logits and value norms of sink + local tokens, ||v|| of every cached token
    sl_logits = torch.randn(bs, H, sl, generator=g, device=DEV) * 0.5
    sl_vnorm = torch.rand(bs, H, sl, generator=g, device=DEV) + 0.5
    value_norm = torch.rand(bs, H, N + sink, generator=g, device=DEV) + 0.5
    scale = 1.0 / math.sqrt(128)
    k_out = min(cap_k, Cn)
    ak, ids = ops.adaptive_topk(sl_logits, sl_vnorm, scores, scale, cand, thr, k_out, value_norm=value_norm, vn_offset=sink)
    ak = ak.clamp(min=max(1, min_k), max=max(1, cap_k))           # polar_cache_adaptivek_varlen.py:1759
    torch.cuda.synchronize()
    sg = signs.cpu().numpy()
    for r in (1, 6):
        codes = codes_km[0, r].cpu().numpy()
        ec, en, ew = O.encode(keys[0, r].float().cpu().numpy(), sg, O.BF16)
        assert np.array_equal(codes, ec) and np.array_equal(nib_km[0, r].cpu().numpy().reshape(N, 16, 4), en)
        assert np.array_equal(w_km[0, r].float().cpu().numpy(), ew)
        assert np.array_equal(cc[0, r].cpu().numpy(), O.count_cluster_keys(ec))
        qh, qn = O.query_prep(q.view(bs, H, G, 128)[0, r].float().cpu().numpy(), sg, O.BF16)
        lut_ref = O.tier_lut(O.rank_centroids(qh, O.BF16), cc[0, r].cpu().numpy(), tiers)
        cnt_ref = O.collision_count(ec, lut_ref)
        assert np.array_equal(cnt[0, r].cpu().numpy(), cnt_ref)
        cand_ref, _ = O.select_candidates(cnt_ref, Cn)
        assert np.array_equal(cand[0, r].cpu().numpy(), cand_ref)
        sc_ref = O.rerank(cand_ref, en, ew, qh, qn)
        got = scores[0, r].cpu().numpy()
        np.testing.assert_allclose(got, sc_ref, rtol=1e-5, atol=1e-5 * np.abs(sc_ref).max())
        vn = value_norm[0, r].cpu().numpy()[cand_ref + sink]
        k_ref, ids_ref = O.adaptive_topk(sl_logits[0, r].cpu().numpy(), sl_vnorm[0, r].cpu().numpy(), got * np.float32(scale), vn,
                                         cand_ref, thr, k_out)
        assert int(ak[0, r]) == min(max(k_ref, min_k), cap_k)
        assert np.array_equal(ids[0, r].cpu().numpy(), ids_ref)
    assert int(ak.min()) >= min_k and int(ak.max()) <= cap_k
    # pack the per-head prefixes (polar_cache_adaptivek_varlen.py:1817-1832) and gather them raggedly out of host memory
    V = bs * H
    mask = torch.arange(k_out, device=DEV).unsqueeze(0) < ak.view(V, 1)
    packed = ids.view(V, k_out)[mask].contiguous()
    cu_topk = torch.zeros(V + 1, dtype=torch.int32, device=DEV)
    cu_topk[1:] = torch.cumsum(ak.view(V), 0)
    cu_k = torch.zeros(V + 1, dtype=torch.int32, device=DEV)
    cu_k[1:] = torch.cumsum(ak.view(V) + sl, 0)
    total = int(cu_k[-1])
    kcpu = torch.empty(bs, H, N, 128, dtype=torch.bfloat16, pin_memory=True)
    vcpu = torch.empty(bs, H, N, 128, dtype=torch.bfloat16, pin_memory=True)
    kcpu.copy_(keys)
    vcpu.copy_(-keys)
    kp = torch.zeros(total, 128, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros_like(kp)
    ops.gather_uva_packed(kcpu, vcpu, kp, vp, packed, cu_topk, cu_k, sl, int(ak.max()))
    torch.cuda.synchronize()
    for v in range(V):
        n = int(ak.view(V)[v])
        sel = ids.view(V, k_out)[v, :n]
        base = int(cu_k[v]) + sl
        assert torch.equal(kp[base:base + n], keys[0, v][sel]) and torch.equal(vp[base:base + n], -keys[0, v][sel])
        assert not kp[int(cu_k[v]):base].any()   # the sink/local slots are the caller's to fill


# ------------------------------------------------------- decode attention


@pytest.mark.parametrize("dtype,group,lens", [
    (torch.bfloat16, 4, (64, 1024, 512)),          # sink | gathered top-k | local window
    (torch.bfloat16, 4, (64, 300, 1000, 37)),      # four ragged segments
    (torch.bfloat16, 1, (5,)),                     # fewer keys than one workgroup step
    (torch.bfloat16, 8, (2000,)),
    (torch.float32, 2, (129, 64)),
    (torch.bfloat16, 7, (64, 500)),                # 28 query / 4 KV heads
])
def test_decode_attention_segments_vs_oracle(ops, dtype, group, lens):
    """softmax(q k^T / sqrt(128)) v over row segments read in place, against the double-precision
    CPU oracle on the same (bf16-exact) inputs.  Tolerance 2e-2 absolute in bf16, 1e-4 in fp32."""
    bs, H = 2, 3
    _say(f"decode attention dtype={dtype} G={group} segments={lens}")
    g = torch.Generator(device=DEV).manual_seed(11)
    q = (torch.randn(bs, 1, H * group, 128, generator=g, device=DEV) * 1.5).to(dtype)
    segs, ks, vs = [], [], []
    for i, n in enumerate(lens):
        cap = n + 17 + i
        row0 = 3 + i
        k = torch.randn(bs, H, cap, 128, generator=g, device=DEV).to(dtype)
        v = torch.randn(bs, H, cap, 128, generator=g, device=DEV).to(dtype)
        if i == 1:  # a sliced parent tensor: batch/head strides larger than rows * 128
            big_k = torch.randn(bs, H + 1, cap + 5, 128, generator=g, device=DEV).to(dtype)
            big_v = torch.randn(bs, H + 1, cap + 5, 128, generator=g, device=DEV).to(dtype)
            k, v = big_k[:, :H, :cap], big_v[:, :H, :cap]
        segs.append((k, v, row0, n))
        ks.append(k[:, :, row0:row0 + n])
        vs.append(v[:, :, row0:row0 + n])
    att = ops.DecodeAttention(bs, H, group, sum(lens), DEV)
    out = att.run(q, segs)
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == dtype
    kc = torch.cat(ks, dim=2).float().cpu().numpy()
    vc = torch.cat(vs, dim=2).float().cpu().numpy()
    qc = q.float().cpu().numpy().reshape(bs, H, group, 128)
    got = out.float().cpu().numpy().reshape(bs, H, group, 128)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    for b in range(bs):
        for h in range(H):
            ref = O.attention(qc[b, h], kc[b, h], vc[b, h])
            assert np.abs(got[b, h] - ref).max() <= tol, (b, h, np.abs(got[b, h] - ref).max())


@pytest.mark.parametrize("dtype,group,K", [(torch.bfloat16, 4, 300), (torch.bfloat16, 8, 77), (torch.bfloat16, 1, 1500),
                                           (torch.float32, 4, 130), (torch.float32, 7, 64)])
def test_decode_attention_indexed_segment_equals_gathered(ops, dtype, group, K):
    """A segment given as an index list (rows row0 + idx[b,h,j], read in place) against the same rows gathered into a
    buffer first (reference polar_cache.py:1089-1095 + 1097-1105): the two outputs are identical, and both match the
    CPU oracle.  Sink and local segments surround the indexed one, as in the no-offload decode step; a ragged
    row_keys case and out-of-range indices (clamped, no fault) are included."""
    bs, H, cap, sink, tail0, tail = 2, 3, 2500, 5, 2300, 140
    _say(f"indexed attention dtype={dtype} G={group} K={K}")
    g = torch.Generator(device=DEV).manual_seed(21)
    q = (torch.randn(bs, 1, H * group, 128, generator=g, device=DEV) * 1.5).to(dtype)
    kk = torch.randn(bs, H, cap, 128, generator=g, device=DEV).to(dtype)
    vv = torch.randn(bs, H, cap, 128, generator=g, device=DEV).to(dtype)
    idx = torch.stack([torch.randperm(tail0 - sink, generator=g, device=DEV)[:K + 9] for _ in range(bs * H)]).view(bs, H, K + 9)
    gk = torch.empty(bs, H, K, 128, dtype=dtype, device=DEV)
    gv = torch.empty_like(gk)
    ops.gather_hbm(kk, vv, idx[:, :, :K].contiguous(), gk, gv, idx_offset=sink)
    att = ops.DecodeAttention(bs, H, group, sink + K + tail, DEV)
    for row_keys in (None, torch.tensor([[sink + K + tail, sink + 3, sink + K], [40 if K > 40 else K, sink + K + 1, 1]],
                                        dtype=torch.int32, device=DEV)):
        a = att.run(q, [(kk, vv, 0, sink), (kk, vv, sink, K, idx), (kk, vv, tail0, tail)], row_keys=row_keys).clone()
        b_ = att.run(q, [(kk, vv, 0, sink), (gk, gv, 0, K), (kk, vv, tail0, tail)], row_keys=row_keys).clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b_)
    kc = torch.cat([kk[:, :, :sink], gk, kk[:, :, tail0:tail0 + tail]], dim=2).float().cpu().numpy()
    vc = torch.cat([vv[:, :, :sink], gv, vv[:, :, tail0:tail0 + tail]], dim=2).float().cpu().numpy()
    full = att.run(q, [(kk, vv, 0, sink), (kk, vv, sink, K, idx), (kk, vv, tail0, tail)])
    got = full.float().cpu().numpy().reshape(bs, H, group, 128)
    qc = q.float().cpu().numpy().reshape(bs, H, group, 128)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    for b in range(bs):
        for h in range(H):
            assert np.abs(got[b, h] - O.attention(qc[b, h], kc[b, h], vc[b, h])).max() <= tol
    wild = idx.clone()
    wild[:, :, ::7] = 10 ** 9          # far outside the tensor: clamped to its last row, must not fault
    wild[:, :, 3::11] = -5
    out = att.run(q, [(kk, vv, sink, K, wild)])
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out.float()).all())
    with pytest.raises(RuntimeError, match="segment indices"):
        att.run(q, [(kk, vv, sink, K, idx.to(torch.int32))])


def test_decode_attention_argument_errors(ops):
    att = ops.DecodeAttention(1, 2, 4, 64, DEV)
    q = torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(1, 2, 64, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="out of range"):
        att.run(q, [(k, k, 10, 60)])
    with pytest.raises(RuntimeError, match="share a dtype"):
        att.run(q, [(k.float(), k.float(), 0, 8)])
    with pytest.raises(RuntimeError, match="no keys"):
        att.run(q, [(k, k, 0, 0)])
    bad = ops.DecodeAttention(1, 2, 9, 64, DEV)
    with pytest.raises(RuntimeError, match="group must be"):
        bad.run(torch.zeros(1, 1, 18, 128, dtype=torch.bfloat16, device=DEV), [(k, k, 0, 8)])


# --------------------------------------------------- randomised small shapes


def test_retrieve_random_shapes_vs_oracle(ops):
    """Whole retrieval on 16 seeded shapes (ragged key counts, group sizes 1-7, candidate counts from 1 to
    every key, k from 1 to the candidate count, both dtype chains): final indices bit-exact against the oracle."""
    rng = np.random.default_rng(2024)
    shapes = [(1, 1, 1, 50, 1, 1), (1, 2, 7, 333, 333, 17), (2, 1, 3, 4097, 4096, 4096), (1, 1, 4, 8193, 5000, 1),
              (1, 2, 4, 30000, 12000, 3000), (1, 1, 2, 20000, 20000, 8192)]   # candidate rows wider than one workgroup sorts
    while len(shapes) < 16:
        N = int(rng.integers(60, 20000))
        C = int(rng.integers(1, N + 1))
        shapes.append((int(rng.integers(1, 3)), int(rng.integers(1, 3)), int(rng.integers(1, 8)), N, C,
                       int(rng.integers(1, C + 1))))
    for i, (bs, H, G, N, C, K) in enumerate(shapes):
        dtype = O.BF16 if i % 3 else O.F32
        _say(f"random shape {i}: bs={bs} H={H} G={G} N={N} C={C} K={K} dtype={dtype}")
        w = W.make_workload(f"rand{i}", bs, H, G, N, C, K, dtype, float(rng.choice([0.2, 0.3, 0.5])), seed0=100 + i,
                            with_values=False)
        plan, out, scores = _run_fused(ops, w)
        for r in range(w.R):
            b, h = divmod(r, w.H)
            ref = O.retrieve_row(w.queries[b, h * G:(h + 1) * G], w.signs, w.dtype, w.codes[r], w.nib[r], w.weight[r],
                                 w.cluster_counts[r], w.tiers, C, K)
            assert np.array_equal(out[b, h].cpu().numpy(), ref), f"shape {i} row {r}"
            s = scores[b, h].cpu().numpy()
            assert np.all(s[:-1] >= s[1:])


def test_decode_step_single_call_equals_separate_calls(ops, wl_small_bf16):
    """pkv_decode_step (retrieve + gather + attention from one host call) against the three separate entry points."""
    w = wl_small_bf16
    d = W.to_device(w, DEV, torch)
    g = torch.Generator(device=DEV).manual_seed(3)
    src_k = torch.randn(w.bs, w.H, w.N, 128, generator=g, device=DEV).to(torch.bfloat16)
    src_v = torch.randn(w.bs, w.H, w.N, 128, generator=g, device=DEV).to(torch.bfloat16)
    dense_k = torch.randn(w.bs, w.H, 40, 128, generator=g, device=DEV).to(torch.bfloat16)
    dense_v = torch.randn(w.bs, w.H, 40, 128, generator=g, device=DEV).to(torch.bfloat16)
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.C, w.K)
    att = ops.DecodeAttention(w.bs, w.H, w.G, 40 + w.K, DEV)
    outs = []
    for fused in (False, True):
        dst_k = torch.zeros(w.bs, w.H, w.K, 128, dtype=torch.bfloat16, device=DEV)
        dst_v = torch.zeros_like(dst_k)
        gather = dict(src_k=src_k, src_v=src_v, from_host=False, dst_k=dst_k, dst_v=dst_v)
        segs = [(dense_k, dense_v, 0, 8), (dst_k, dst_v, 0, w.K), (dense_k, dense_v, 8, 32)]
        args = (d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], 0, w.N,
                w.tiers, w.C, w.K)
        if fused:
            ids = plan.run(*args, gather=gather, attention=(att, segs, None))
            out = plan.attn_out
        else:
            ids = plan.run(*args, gather=gather)
            out = att.run(d["queries"], segs)
        torch.cuda.synchronize()
        outs.append((ids.clone(), out.clone(), dst_k.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][2], outs[1][2])
    assert torch.equal(outs[0][1], outs[1][1]) and outs[1][1].shape == d["queries"].shape
    # and the attention agrees with the oracle on the gathered rows of one (b, h)
    b, h = 1, 0
    sel = outs[1][0][b, h].cpu()
    kk = torch.cat([dense_k[b, h, :8].cpu(), src_k[b, h].cpu()[sel], dense_k[b, h, 8:40].cpu()]).float().numpy()
    vv = torch.cat([dense_v[b, h, :8].cpu(), src_v[b, h].cpu()[sel], dense_v[b, h, 8:40].cpu()]).float().numpy()
    qq = d["queries"][b, 0, h * w.G:(h + 1) * w.G].float().cpu().numpy()
    got = outs[1][1][b, 0, h * w.G:(h + 1) * w.G].float().cpu().numpy()
    assert np.abs(got - O.attention(qq, kk, vv)).max() <= 2e-2


def test_decode_step_replays_from_a_captured_graph(ops, wl_small_bf16):
    """The launch sequence allocates nothing, synchronises nothing and records no memset: it can be captured into
    a graph once and replayed.  Three replays with different queries and eager work in between, each checked
    against the eager result of the same inputs."""
    w = wl_small_bf16
    d = W.to_device(w, DEV, torch)
    g = torch.Generator(device=DEV).manual_seed(4)
    src_k = torch.randn(w.bs, w.H, w.N, 128, generator=g, device=DEV).to(torch.bfloat16)
    src_v = torch.randn(w.bs, w.H, w.N, 128, generator=g, device=DEV).to(torch.bfloat16)
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, w.C, w.K)
    att = ops.DecodeAttention(w.bs, w.H, w.G, w.K, DEV)
    dst_k = torch.zeros(w.bs, w.H, w.K, 128, dtype=torch.bfloat16, device=DEV)
    dst_v = torch.zeros_like(dst_k)
    gather = dict(src_k=src_k, src_v=src_v, from_host=False, dst_k=dst_k, dst_v=dst_v)
    q_static = d["queries"].clone()
    ids_static = torch.zeros(w.bs, w.H, w.K, dtype=torch.int64, device=DEV)
    out_static = torch.zeros_like(q_static)

    def step():
        plan.run(q_static, d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], 0, w.N,
                 w.tiers, w.C, w.K, out_ids=ids_static, gather=gather, attention=(att, [(dst_k, dst_v, 0, w.K)], out_static))

    step()  # warm-up outside the capture (module load, workspace sizing)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for rep in range(3):
        q_new = (d["queries"].float() + 0.3 * torch.randn(d["queries"].shape, generator=g, device=DEV)).to(torch.bfloat16)
        q_static.copy_(q_new)
        ids_static.zero_(), out_static.zero_(), dst_k.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got_ids, got_out = ids_static.clone(), out_static.clone()
        scratch = torch.randn(1 << 20, device=DEV).sum().item()  # unrelated eager work between replays
        ids_static.zero_(), out_static.zero_()
        step()
        torch.cuda.synchronize()
        assert torch.equal(got_ids, ids_static), f"replay {rep}: indices differ from the eager run"
        assert torch.equal(got_out, out_static), f"replay {rep}: attention differs from the eager run"
        assert scratch == scratch


def test_rerank_rabitq_fused_helper(ops, wl_small_bf16):
    """rerank_rabitq_fused (reference rerank.py:266-293): coarse filter + rerank + final top-k from the vote counts."""
    from pariskv_amd.cache_hub.rerank.rerank import rerank_rabitq_fused

    w = wl_small_bf16
    d = W.to_device(w, DEV, torch)
    codes_km, nib_km, w_km = d["codes_km"], d["nib_km"], d["w_km"]
    k4 = nib_km.view(w.bs, w.H, w.N, 16, 4).permute(0, 1, 3, 2, 4)   # reference-shaped views of key-major memory
    kw = w_km.permute(0, 1, 3, 2)
    cb = codes_km.permute(0, 1, 3, 2)
    qhat, qnorm, lut, _ = ops.query_prep_lut(d["queries"], w.H, d["signs"], d["cluster_counts"], w.tiers)
    cnt, _, _ = ops.collision_scan(cb, lut, out_dtype=torch.int32)
    ratio, final_k = 0.05, 40
    ids, scores, v4b = rerank_rabitq_fused(cnt, k4, kw, qhat.view(w.bs, w.H, 16, 8), qnorm.view(w.bs, w.H, 1),
                                           ops.mag_centers(DEV), ratio, final_k, 16, 8)
    torch.cuda.synchronize()
    n_cand = int(math.ceil(w.N * ratio))
    assert ids.shape == (w.bs, w.H, final_k) and scores.shape == (w.bs, w.H, n_cand)
    for r in range(w.R):
        b, h = divmod(r, w.H)
        st = W.oracle_stages(w, r)
        cand, _ = O.select_candidates(st["cnt"], n_cand)
        sc = O.rerank(cand, w.nib[r], w.weight[r], st["qhat"], st["qnorm"])
        final, _ = O.topk_f32(sc, cand, final_k)
        assert np.array_equal(ids[b, h].cpu().numpy(), final)
    # candidate set not larger than final_topk: the coarse indices come back, nothing is scored
    ids2, s2, v2 = rerank_rabitq_fused(cnt, k4, kw, qhat.view(w.bs, w.H, 16, 8), qnorm.view(w.bs, w.H, 1),
                                       ops.mag_centers(DEV), 0.001, 40, 16, 8)
    assert s2 is None and v2 is None and ids2.shape[2] == int(math.ceil(w.N * 0.001))


def test_srht_signs_equal_the_device_generator_draw(ops):
    """The reference draws the SRHT diagonal from torch's device generator (polar_cache.py:57-63); the host
    restatement used here must give the same vector, for the shipped seed and others, and leave the generators alone."""
    cpu_state, dev_state = torch.get_rng_state(), torch.cuda.get_rng_state(0)
    for seed in (42, 0, 7, 123456789012):
        before = torch.get_rng_state(), torch.cuda.get_rng_state(0)
        mine = ops.srht_signs(DEV, seed)
        assert torch.equal(torch.get_rng_state(), before[0]) and torch.equal(torch.cuda.get_rng_state(0), before[1])
        torch.manual_seed(seed)
        ref = torch.randint(0, 2, (128,), device=DEV, dtype=torch.bfloat16) * 2 - 1   # the reference's expression
        assert torch.equal(mine, ref.float())
        assert np.array_equal(O.srht_signs(seed), mine.cpu().numpy())
    torch.set_rng_state(cpu_state)
    torch.cuda.set_rng_state(dev_state, 0)


def test_gather_uva_ragged_moves_only_each_rows_prefix(ops):
    """pkv_gather_uva_ragged: row (b, h) fetches its first row_counts[b, h] selected rows; the rest of dst is untouched;
    counts 0 and K included."""
    g = torch.Generator().manual_seed(8)
    bs, H, N, K, D = 2, 3, 500, 40, 128
    sk = torch.randn(bs, H, N, D, generator=g).to(torch.bfloat16).pin_memory()
    sv = torch.randn(bs, H, N, D, generator=g).to(torch.bfloat16).pin_memory()
    idx = torch.stack([torch.randperm(N, generator=g)[:K] for _ in range(bs * H)]).view(bs, H, K)
    counts = torch.tensor([[0, K, 7], [1, 39, 20]], dtype=torch.int64)
    dk = torch.full((bs, H, K + 5, D), 3.0, dtype=torch.bfloat16, device=DEV)
    dv = torch.full((bs, H, K + 5, D), 5.0, dtype=torch.bfloat16, device=DEV)
    want_k, want_v = dk.cpu().clone(), dv.cpu().clone()
    ops.gather_uva_ragged(sk, sv, idx.to(DEV), counts.to(DEV), dk, dv, dst_row0=2)
    torch.cuda.synchronize()
    for b in range(bs):
        for h in range(H):
            c = int(counts[b, h])
            want_k[b, h, 2:2 + c] = sk[b, h][idx[b, h, :c]]
            want_v[b, h, 2:2 + c] = sv[b, h][idx[b, h, :c]]
    assert torch.equal(dk.cpu(), want_k) and torch.equal(dv.cpu(), want_v)


def test_append_kv_equals_indexed_assignment(ops):
    """pkv_append_kv against the two indexed assignments it replaces (reference polar_cache.py:848-856), with
    contiguous and strided new rows and a strided (sliced-batch) store."""
    g = torch.Generator().manual_seed(5)
    bs, H, cap, D = 3, 4, 37, 128
    for dtype in (torch.bfloat16, torch.float32):
        kg = torch.randn(bs + 1, H, cap, D, generator=g).to(dtype).to(DEV)
        vg = torch.randn(bs + 1, H, cap, D, generator=g).to(dtype).to(DEV)
        dk, dv = kg[1:], vg[1:]
        fused = torch.randn(bs, 1, 3 * H, D, generator=g).to(dtype).to(DEV)   # rows of a fused projection: strided heads
        for k1, v1 in ((fused[:, :, :H], fused[:, :, 2 * H:]),
                       (fused[:, :, H:2 * H].contiguous(), fused[:, :, :H].contiguous())):
            for slot in (0, 17, cap - 1):
                wk, wv = dk.clone(), dv.clone()
                wk[:, :, slot, :] = k1[:, 0]
                wv[:, :, slot, :] = v1[:, 0]
                ops.append_kv(k1, v1, dk, dv, slot)
                torch.cuda.synchronize()
                assert torch.equal(dk, wk) and torch.equal(dv, wv)
        with pytest.raises(RuntimeError, match="slot"):
            ops.append_kv(fused[:, :, :H], fused[:, :, H:2 * H], dk, dv, cap)
    with pytest.raises(RuntimeError):
        ops.append_kv(fused[:, :, :H], fused[:, :, H:2 * H + 1], dk, dv, 0)


def test_append_kv_value_norm(ops):
    """The value norm written by pkv_append_kv (adaptive-k bookkeeping, reference polar_cache_adaptivek_varlen.py:1179):
    bit-equal to the oracle's fixed-order restatement, within one step of the dtype of torch's vector_norm; the other
    slots of the norm table stay untouched."""
    g = torch.Generator().manual_seed(8)
    bs, H, cap, D = 3, 4, 21, 128
    for dtype, odt, rtol in ((torch.bfloat16, O.BF16, 2.0 ** -7), (torch.float32, O.F32, 2e-6)):
        dk = torch.zeros(bs, H, cap, D, dtype=dtype, device=DEV)
        dv = torch.zeros_like(dk)
        table = torch.full((bs + 1, H, cap + 3), -1.0, device=DEV)
        vn = table[1:]                                         # a batch slice: strided rows
        fused = (torch.randn(bs, 1, 3 * H, D, generator=g) * torch.rand(bs, 1, 3 * H, 1, generator=g) * 4).to(dtype).to(DEV)
        for slot, (k1, v1) in ((5, (fused[:, :, :H], fused[:, :, 2 * H:])), (cap - 1, (fused[:, :, H:2 * H], fused[:, :, :H]))):
            ops.append_kv(k1, v1, dk, dv, slot, vnorm=vn)
            torch.cuda.synchronize()
            assert torch.equal(dv[:, :, slot], v1[:, 0]) and torch.equal(dk[:, :, slot], k1[:, 0])
            want = O.value_norm(v1[:, 0].float().cpu().numpy().reshape(-1, D), odt).reshape(bs, H)
            assert np.array_equal(vn[:, :, slot].cpu().numpy(), want)
            ref = torch.linalg.vector_norm(v1[:, 0], dim=-1).float()
            assert torch.allclose(vn[:, :, slot], ref, rtol=rtol, atol=0)
        untouched = torch.ones(cap + 3, dtype=torch.bool)
        untouched[[5, cap - 1]] = False
        assert (vn[:, :, untouched] == -1).all() and (table[0] == -1).all()
    with pytest.raises(RuntimeError, match="vnorm"):
        ops.append_kv(fused[:, :, :H], fused[:, :, H:2 * H], dk, dv, 0, vnorm=vn[:, :, :0])


@pytest.mark.parametrize("bs,H,G,rows,n", [(1, 8, 4, 700, 700), (2, 2, 7, 100, 33), (3, 1, 1, 17, 17), (1, 4, 12, 2000, 1999)])
def test_dense_logits_match_oracle(ops, bs, H, G, rows, n):
    """pkv_dense_logits (reference polar_cache_adaptivek_varlen.py:1418-1419 + :1731): bit-equal to the oracle's
    fixed-order restatement in both rounding chains, and within one bf16 step / 2e-6 of the torch expressions; rows
    beyond n and the padding of a longer output row are not written."""
    g = torch.Generator().manual_seed(bs * 100 + G)
    scale = 1.0 / math.sqrt(128)
    for dtype, odt, rtol in ((torch.bfloat16, O.BF16, 2.0 ** -7), (torch.float32, O.F32, 2e-6)):
        q = torch.randn(bs, 1, H * G, 128, generator=g).to(dtype).to(DEV)
        store = (torch.randn(bs + 1, H, rows, 128, generator=g) * 1.5).to(dtype).to(DEV)
        k = store[1:]                                           # strided batch
        out = torch.full((bs, H, rows + 5), 7.0, device=DEV)
        got = ops.dense_logits(q, k, n, scale, out=out)
        torch.cuda.synchronize()
        assert got.data_ptr() == out.data_ptr() and (out[:, :, n:] == 7.0).all()
        qc, kc = q.float().cpu().numpy().reshape(bs, H, G, 128), k.float().cpu().numpy()
        for b in range(bs):
            for h in range(H):
                want = O.dense_logits(qc[b, h], kc[b, h, :n], scale, odt)
                assert np.array_equal(out[b, h, :n].cpu().numpy(), want), (b, h)
        ref = torch.einsum("bhd,bhkd->bhk", q[:, 0].view(bs, H, G, 128).mean(dim=2), k[:, :, :n]).to(torch.float32) * scale
        assert torch.allclose(out[:, :, :n], ref, rtol=rtol, atol=rtol * float(ref.abs().max()))
        fresh = ops.dense_logits(q, k, n, scale)
        assert fresh.shape == (bs, H, n) and torch.equal(fresh, out[:, :, :n])
    with pytest.raises(RuntimeError):
        ops.dense_logits(q, k, rows + 1, scale)


def test_adaptive_topk_clamp_and_row_keys(ops):
    """The clamp of k (reference polar_cache_adaptivek_varlen.py:1759) and the per-row key count folded into the
    adaptive-k kernels, on the one-workgroup and the multi-workgroup path: equal to clamping the unclamped result."""
    for Cn, k_out in ((3000, 800), (20000, 800)):
        bs, H, sl = 2, 3, 200
        q, slk, slv, cs, ci, cv, scale = _adaptive_recipe(bs, H, sl, Cn, 23)
        sl_logits = (torch.einsum("bhd,bhkd->bhk", q, slk).float() * scale).to(DEV)
        args = (sl_logits, slv.to(DEV), cs.to(DEV), scale, ci.to(DEV))
        for thr in (0.3, 0.9, 0.9999):
            ak0, ids0 = ops.adaptive_topk(*args, thr, k_out, cand_vnorm=cv.to(DEV))
            ak1, ids1, rk = ops.adaptive_topk(*args, thr, k_out, cand_vnorm=cv.to(DEV), k_min=100, k_max=500, row_keys_base=sl + 7)
            assert torch.equal(ids0, ids1)
            assert torch.equal(ak1, ak0.clamp(min=100, max=500))
            assert rk.dtype == torch.int32 and torch.equal(rk.long(), ak1 + sl + 7)
        assert len({int(v) for v in ak0.flatten()} | {int(v) for v in ak1.flatten()}) > 1
    with pytest.raises(RuntimeError, match="clamp"):
        ops.adaptive_topk(*args, 0.9, k_out, cand_vnorm=cv.to(DEV), k_min=600, k_max=500)


def test_uniform_k_is_the_row_maximum(ops):
    """pkv_uniform_k: max over all rows, broadcast, plus the attention's key count (the reference reads
    adaptive_k.max().item() on the host, polar_cache_atten_value_indices_adaptive_k.py:1585)."""
    g = torch.Generator().manual_seed(2)
    for shape in ((1, 1), (2, 3), (8, 8), (40, 64)):   # up to 2560 rows: more than one pass of the 1024 threads
        ak = torch.randint(1, 5000, shape, generator=g).to(DEV)
        uk, rk = ops.uniform_k(ak, row_keys_base=77)
        assert uk.shape == ak.shape and (uk == ak.max()).all()
        assert rk.dtype == torch.int32 and (rk == int(ak.max()) + 77).all()
        assert torch.equal(ops.uniform_k(ak), uk)


@pytest.mark.parametrize("engine", ["kernel", "dma", "dma-one-command"])
def test_offload_rows_equals_sliced_copy(ops, engine):
    """pkv_offload_rows / pkv_offload_rows_dma against the sliced copy_ it replaces (reference polar_cache.py:457-471, :778-799): rows read in
    place from the model's [bs,seq,h,d] layout and from a partly filled staging buffer, into a batch slice of the pinned
    store; rows outside the written window stay untouched."""
    kw = {"kernel": {}, "dma": {"dma": True}, "dma-one-command": {"dma": True, "dma_flags": ops.OFFLOAD_ONE_COMMAND}}[engine]
    g = torch.Generator().manual_seed(3)
    bs, H, cap, D = 3, 4, 50, 128
    kc = torch.randn(bs + 1, H, cap, D, generator=g).to(torch.bfloat16).pin_memory()
    vc = torch.randn(bs + 1, H, cap, D, generator=g).to(torch.bfloat16).pin_memory()
    want_k, want_v = kc.clone(), vc.clone()
    model_k = torch.randn(bs, 40, H, D, generator=g).to(torch.bfloat16).to(DEV)    # [bs, seq, h, d]
    model_v = torch.randn(bs, 40, H, D, generator=g).to(torch.bfloat16).to(DEV)
    src_k, src_v = model_k[:, 5:33].permute(0, 2, 1, 3), model_v[:, 5:33].permute(0, 2, 1, 3)
    ops.offload_rows(src_k, src_v, kc[1:], vc[1:], 7, **kw)
    want_k[1:, :, 7:35] = src_k.cpu()
    want_v[1:, :, 7:35] = src_v.cpu()
    stage_k = torch.randn(bs, H, 16, D, generator=g).to(torch.bfloat16).to(DEV)   # staging buffer, first 9 rows valid
    stage_v = torch.randn(bs, H, 16, D, generator=g).to(torch.bfloat16).to(DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    ops.offload_rows(stage_k[:, :, :9], stage_v[:, :, :9], kc[:bs], vc[:bs], cap - 9, stream=side, **kw)
    want_k[:bs, :, cap - 9:] = stage_k[:, :, :9].cpu()
    want_v[:bs, :, cap - 9:] = stage_v[:, :, :9].cpu()
    torch.cuda.synchronize()
    assert torch.equal(kc, want_k) and torch.equal(vc, want_v)
    with pytest.raises(RuntimeError, match="outside the host store"):
        ops.offload_rows(stage_k, stage_v, kc[:bs], vc[:bs], cap - 9, **kw)
    with pytest.raises(RuntimeError):
        ops.offload_rows(stage_k, stage_v, kc[:bs].clone(), vc[:bs], 0, **kw)   # not pinned
