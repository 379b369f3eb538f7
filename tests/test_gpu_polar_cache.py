"""End-to-end tests of the polar_cache drop-in on the GPU: prefill, decode appends with index
refreshes and host offload, retrieval and attention, for several layers.

Checked per step: (1) the retrieved index set equals the CPU oracle's on the cache's own index
(exact; the cache leaves the final sort out, the order is checked in test_gpu_parity.py); (2) the attention output equals an fp32 torch softmax attention over
sink ++ selected ++ dense tail taken from the test's own record of every K/V it fed
(bf16 tolerance 2e-2 abs)."""
import math

import numpy as np
import pytest
import torch

from oracle import pkv_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _make_cache(offload, bs, Hkv, Hq, layers, S, max_new, sink, local, interval, final_topk, thr=100, **kw):
    from pariskv_amd.cache_hub.polar_cache import polar_cache

    return polar_cache(valid_start=[0] * bs, layer_num=layers, batch_size=bs, max_length=S + max_new,
                       num_key_value_heads=Hkv, num_heads=Hq, head_dim=128, dtype=torch.bfloat16,
                       layer_mapping={i: DEV for i in range(layers)}, max_new_length=max_new, sink_size=sink,
                       local_size=local, core=1, nprobe=1, cache_unit_size=1, cache_cluster_num=1, num_gpus=1, model_size=7,
                       final_topk=final_topk, dynamic_update_interval=interval, full_attention_threshold=thr,
                       enable_offload=offload, **kw)


def _ref_attention(q, K, V, G):
    """fp32 softmax(q k^T / sqrt(D)) v.  q [Hq,D], K/V [Hkv,S,D] -> [Hq,D]."""
    Hq, D = q.shape
    out = torch.empty(Hq, D)
    for hq in range(Hq):
        h = hq // G
        s = (K[h].float() @ q[hq].float()) / math.sqrt(D)
        out[hq] = torch.softmax(s, dim=0) @ V[h].float()
    return out


def _synth_kv(gen, bs, S, Hkv):
    k = torch.randn(bs, S, Hkv, 128, generator=gen)
    k[..., [7, 31, 64, 101]] *= 10.0
    v = torch.randn(bs, S, Hkv, 128, generator=gen)
    return k.to(torch.bfloat16), v.to(torch.bfloat16)


# 16 rows: selected rows attended in place; "mixed": a host budget that holds one layer, the other stays in HBM
@pytest.mark.parametrize("offload,bs,Hkv", [(True, 2, 2), ("kernel", 2, 2), (False, 2, 2), (False, 4, 4), ("mixed", 2, 2), ("mixed", 4, 4)])
def test_decode_loop_matches_oracle_and_dense_reference(offload, bs, Hkv):
    from pariskv_amd.attn_hub import polar_decode_attn

    print(f"polar_cache decode loop offload={offload} bs={bs} Hkv={Hkv}", flush=True)
    extra = {}
    if offload == "kernel":    # the host offload through the shader kernel instead of the copy engines
        offload, extra = True, {"offload_engine": "kernel"}
    Hq, layers, S, steps = 4 * Hkv, 2, 3000, 70
    sink, local, I, topk = 4, 64, 32, 200
    G = Hq // Hkv
    if offload == "mixed":
        layer_bytes = 2 * bs * Hkv * (S + steps + 10 - sink - local) * 128 * 2
        cache = _make_cache(True, bs, Hkv, Hq, layers, S, steps + 10, sink, local, I, topk,
                            host_kv_budget_bytes=layer_bytes + layer_bytes // 2)
        assert cache._layer_offload == [True, False]
        assert cache.kv_placement["host_layers"] == 1 and cache.kv_placement["hbm_layers"] == 1
        assert cache.kv_placement["host_pinned_bytes"] == layer_bytes
        assert cache.unified_keys_cpu[1] is None and cache.unified_keys_gpu[1].shape[2] == S + steps + 10
    else:
        cache = _make_cache(offload, bs, Hkv, Hq, layers, S, steps + 10, sink, local, I, topk, **extra)
        assert cache._layer_offload == [bool(offload)] * layers
    gen = torch.Generator().manual_seed(0)
    hist_k = [None] * layers
    hist_v = [None] * layers
    for l in range(layers):
        k, v = _synth_kv(gen, bs, S, Hkv)
        hist_k[l], hist_v[l] = k, v
        ko, vo = cache.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), l, 0)
        assert ko.shape == k.shape
    assert cache.current_seq_len == [S] * layers and cache.context == S
    signs = O.srht_signs(42)
    checked = 0
    for step in range(steps):
        for l in range(layers):
            k1, v1 = _synth_kv(gen, bs, 1, Hkv)
            q = (hist_k[l].float().mean(dim=1).repeat_interleave(G, dim=1) + 0.5 * torch.randn(bs, Hq, 128, generator=gen))
            q = q.to(torch.bfloat16).view(bs, 1, Hq, 128)
            hist_k[l] = torch.cat([hist_k[l], k1], dim=1)
            hist_v[l] = torch.cat([hist_v[l], v1], dim=1)
            assert cache.decode_update_kv_cache(k1.to(DEV), v1.to(DEV), l) == (None, None)
            out = polar_decode_attn(q.to(DEV), None, None, l, cache)
            assert out.shape == (bs, 1, Hq, 128)
            if step % 9 != 0 and step not in (I - 1, I, 2 * I - 1, 2 * I):
                continue
            torch.cuda.synchronize()
            total = S + step + 1
            z = cache._zones[l]
            assert z.seq_len == total
            n_keys, n_cand, kk, tiers = cache.retrieval_shape(l)
            assert n_keys == z.encoded == (S - sink - local) + I * ((step + 1) // I)
            got_ids = cache.last_topk_indices.cpu().numpy()
            codes = cache._codes_km[l].cpu().numpy()
            nib = cache._nib_km[l].cpu().numpy()
            w = cache._w_km[l].float().cpu().numpy()
            cc = cache.cluster_key_counts_gpu[l].cpu().numpy()
            for b in range(bs):
                for h in range(Hkv):
                    sl = slice(sink, sink + n_keys)
                    # the cache's index over the retrieval zone equals the oracle's encoding of the true keys
                    if step == 0:
                        ec, en, ew = O.encode(hist_k[l][b, sink:sink + n_keys, h].float().numpy(), signs, O.BF16)
                        assert np.array_equal(codes[b, h][sl], ec) and np.array_equal(nib[b, h][sl].reshape(-1, 16, 4), en)
                        assert np.array_equal(w[b, h][sl], ew)
                        assert np.array_equal(cc[b, h], O.count_cluster_keys(ec))
                    ref_ids = O.retrieve_row(q[b, 0, h * G:(h + 1) * G].float().numpy(), signs, O.BF16, codes[b, h][sl],
                                             nib[b, h][sl].reshape(-1, 16, 4), w[b, h][sl], cc[b, h], tiers, n_cand, kk)
                    # the cache asks for the selected set in any fixed order (no final sort): compare as sets
                    assert np.array_equal(np.sort(got_ids[b, h]), np.sort(ref_ids)), f"step {step} layer {l} row {(b, h)}"
                # fp32 reference attention over sink ++ selected ++ dense tail
                K = hist_k[l][b].permute(1, 0, 2)  # [Hkv, total, D]
                V = hist_v[l][b].permute(1, 0, 2)
                ref = torch.empty(Hq, 128)
                for h in range(Hkv):
                    sel = torch.cat([torch.arange(sink), torch.from_numpy(got_ids[b, h]) + sink,
                                     torch.arange(sink + n_keys, total)])
                    assert len(sel) == sink + kk + (total - sink - n_keys)
                    ref[h * G:(h + 1) * G] = _ref_attention(q[b, 0, h * G:(h + 1) * G], K[h:h + 1, sel], V[h:h + 1, sel], G=G * 10)
                err = (out[b, 0].float().cpu() - ref).abs().max().item()
                assert err < 2e-2, f"attention differs by {err} at step {step} layer {l}"
            checked += 1
    assert checked >= 10
    assert cache.context == S + steps


@pytest.mark.parametrize("offload", [True, False])
def test_short_sequences_use_dense_attention(offload):
    """Below the retrieval threshold the cache attends to every token (polar_cache.py:1033-1045), whether the
    tokens sit in the GPU window or already in the (host) retrieval zone; and a prompt shorter than
    sink+local fills the dense rows first."""
    bs, Hkv, Hq, S, steps = 1, 2, 4, 300, 40
    G = Hq // Hkv
    for S in (300, 20):
        cache = _make_cache(offload, bs, Hkv, Hq, 1, S, steps + 5, 4, 32, 16, 50, thr=2000)
        gen = torch.Generator().manual_seed(1)
        k, v = _synth_kv(gen, bs, S, Hkv)
        cache.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), 0, 0)
        for step in range(steps):
            k1, v1 = _synth_kv(gen, bs, 1, Hkv)
            k, v = torch.cat([k, k1], 1), torch.cat([v, v1], 1)
            q = torch.randn(bs, 1, Hq, 128, generator=gen).to(torch.bfloat16)
            cache.decode_update_kv_cache(k1.to(DEV), v1.to(DEV), 0)
            out = cache.compute(q.to(DEV), 0)
            ref = _ref_attention(q[0, 0], k[0].permute(1, 0, 2), v[0].permute(1, 0, 2), G)
            err = (out[0, 0].float().cpu() - ref).abs().max().item()
            assert err < 2e-2, (S, step, err)
        cache._zones[0].check()


def test_single_sample_prefill_and_constructor_errors():
    from pariskv_amd.cache_hub.polar_cache import polar_cache

    bs, Hkv, Hq, S = 3, 2, 4, 600
    cache = _make_cache(True, bs, Hkv, Hq, 1, S, 8, 4, 32, 16, 40)
    gen = torch.Generator().manual_seed(2)
    ks = []
    for b in range(bs):  # one sample at a time (reference _prefill_single_sample)
        k, v = _synth_kv(gen, 1, S, Hkv)
        ks.append(k)
        cache.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), 0, b)
    torch.cuda.synchronize()
    signs = O.srht_signs(42)
    n = S - 36
    for b in range(bs):
        ec, _, _ = O.encode(ks[b][0, 4:4 + n, 1].float().numpy(), signs, O.BF16)
        assert np.array_equal(cache._codes_km[0][b, 1, 4:4 + n].cpu().numpy(), ec)
        assert torch.equal(cache.unified_keys_cpu[0][b, :, :n], ks[b][0, 4:4 + n].permute(1, 0, 2))
    assert cache.context == S and cache.codebook_gpu[0].shape == (bs, Hkv, 16, S + 8)
    with pytest.raises(ValueError):
        _make_cache(True, 1, 2, 4, 1, 100, 8, 4, 32, 16, 40, codebook_path="/nonexistent.json")
    with pytest.raises(ValueError):
        polar_cache([0], 1, 1, 100, 2, 4, 64, torch.bfloat16, {0: DEV}, 8, 4, 32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_adaptive_k_cache_decode_loop(dtype):
    """Adaptive-k variant (reference polar_cache_adaptivek_varlen.py): value-norm caches follow the K/V slots
    through prefill, decode writes and index refreshes; per-row k and the selected set equal the CPU oracle's on
    the cache's own index; attention equals an fp32 softmax over sink ++ each row's own selection ++ dense tail.
    In bfloat16 (the reference's dtype) and in float32 (the fp32 chains of every kernel on the step)."""
    from pariskv_amd.cache_hub.polar_cache_adaptivek_varlen import polar_cache as adaptive_cache

    odt, step_tol = (O.BF16, 2.0 ** -7) if dtype == torch.bfloat16 else (O.F32, 2e-6)
    bs, Hkv, Hq, layers, S, steps = 2, 2, 8, 2, 3000, 40
    sink, local, I = 4, 64, 16
    G = Hq // Hkv
    thr = 0.6
    cache = adaptive_cache(valid_start=[0] * bs, layer_num=layers, batch_size=bs, max_length=S + steps + 10,
                           num_key_value_heads=Hkv, num_heads=Hq, head_dim=128, dtype=dtype,
                           layer_mapping={i: DEV for i in range(layers)}, max_new_length=steps + 10, sink_size=sink,
                           local_size=local, core=1, nprobe=1, cache_unit_size=1, cache_cluster_num=1, num_gpus=1,
                           model_size=7, final_topk=100, dynamic_update_interval=I, full_attention_threshold=100,
                           enable_offload=True, adaptive_topk_threshold=thr)
    cache._HARDCODED_MAX_K, cache._HARDCODED_MIN_K = 300, 20   # what ADAPTIVE_TOPK_MAX_K / _MIN_K would set
    with pytest.raises(AssertionError):
        adaptive_cache([0], 1, 1, 100, 2, 4, 128, torch.bfloat16, {0: DEV}, 8, 4, 32, enable_offload=False)
    gen = torch.Generator().manual_seed(3)
    hist_k, hist_v = [None] * layers, [None] * layers

    def synth(n):  # values of the cache dtype (fp32: not representable in bf16)
        k, v = _synth_kv(gen, bs, n, Hkv)
        if dtype == torch.float32:
            k, v = k.float() * (1 + 1e-3 * torch.rand(k.shape, generator=gen)), v.float() * (1 + 1e-3 * torch.rand(v.shape, generator=gen))
        return k, v

    for l in range(layers):
        k, v = synth(S)
        v = v * (0.25 + 2.0 * torch.rand(bs, S, Hkv, 1, generator=gen)).to(dtype)  # uneven value norms
        hist_k[l], hist_v[l] = k, v
        cache.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), l, 0)
    signs = O.srht_signs(42)
    scale = 1.0 / math.sqrt(128)
    seen_k = set()
    for step in range(steps):
        for l in range(layers):
            k1, v1 = synth(1)
            # queries near a handful of recent keys make the attention mass concentrate, so k varies by row
            q = (hist_k[l][:, -3:].float().mean(dim=1).repeat_interleave(G, dim=1) * 0.3
                 + 0.5 * torch.randn(bs, Hq, 128, generator=gen)).to(dtype).view(bs, 1, Hq, 128)
            hist_k[l] = torch.cat([hist_k[l], k1], dim=1)
            hist_v[l] = torch.cat([hist_v[l], v1], dim=1)
            cache.decode_update_kv_cache(k1.to(DEV), v1.to(DEV), l)
            out = cache.compute(q.to(DEV), l)
            if step % 7 != 0 and step not in (I - 1, I, 2 * I - 1):
                continue
            torch.cuda.synchronize()
            total = S + step + 1
            z = cache._zones[l]
            n_keys, n_cand, _, tiers = cache.retrieval_shape(l)
            assert n_keys == z.encoded and z.seq_len == total
            sl_end = z.gpu_prefix_rows
            # value norms: retrieval zone by absolute position, dense rows by GPU slot
            vn_ref = torch.linalg.vector_norm(hist_v[l], dim=-1).float().permute(0, 2, 1)      # [bs, H, total]
            assert torch.allclose(cache.value_norm_gpu[l][:, :, sink:sink + n_keys].cpu(), vn_ref[:, :, sink:sink + n_keys],
                                  rtol=step_tol, atol=0)
            if dtype == torch.bfloat16:  # rows encoded at prefill: torch's own norm
                assert torch.equal(cache.value_norm_gpu[l][:, :, sink:S - local].cpu(), vn_ref[:, :, sink:S - local])
            dense_pos = torch.cat([torch.arange(sink), torch.arange(sink + n_keys, total)])
            assert sl_end == len(dense_pos)
            # dense rows written at decode time carry the append kernel's norm: torch's within one bf16 step (bit
            # parity of that kernel with the oracle's restatement is a test of its own)
            assert torch.allclose(cache._sl_vnorm_cache[l][:, :, :sl_end].cpu(), vn_ref[:, :, dense_pos], rtol=step_tol, atol=0)
            codes = cache._codes_km[l].cpu().numpy()
            nib = cache._nib_km[l].cpu().numpy()
            w = cache._w_km[l].float().cpu().numpy()
            cc = cache.cluster_key_counts_gpu[l].cpu().numpy()
            ak = cache.last_adaptive_k.cpu().numpy()
            dense_keys = cache.unified_keys_gpu[l][:, :, :sl_end].float().cpu().numpy()
            sl_vnorm = cache._sl_vnorm_cache[l][:, :, :sl_end].cpu().numpy()
            for b in range(bs):
                K = hist_k[l][b].permute(1, 0, 2)
                V = hist_v[l][b].permute(1, 0, 2)
                ref = torch.empty(Hq, 128)
                for h in range(Hkv):
                    zone = slice(sink, sink + n_keys)
                    qh, qn = O.query_prep(q[b, 0, h * G:(h + 1) * G].float().numpy(), signs, odt)
                    lut = O.tier_lut(O.rank_centroids(qh, odt), cc[b, h], tiers)
                    cand_ref, _ = O.select_candidates(O.collision_count(codes[b, h][zone], lut), n_cand)
                    sc = O.rerank(cand_ref, nib[b, h][zone].reshape(-1, 16, 4), w[b, h][zone], qh, qn)
                    vn = cache.value_norm_gpu[l][b, h].cpu().numpy()[cand_ref + sink]
                    cap_k = min(cache._HARDCODED_MAX_K, n_cand)
                    sl_logits = O.dense_logits(q[b, 0, h * G:(h + 1) * G].float().numpy(), dense_keys[b, h], scale, odt)
                    k_ref, ids_ref = O.adaptive_topk(sl_logits, sl_vnorm[b, h], sc * np.float32(scale), vn, cand_ref,
                                                     thr, cap_k)
                    k_ref = min(max(k_ref, min(cache._HARDCODED_MIN_K, cap_k)), cap_k)
                    assert int(ak[b, h]) == k_ref, f"step {step} layer {l} row {(b, h)}: k {ak[b, h]} vs {k_ref}"
                    seen_k.add(k_ref)
                    sel = torch.cat([torch.arange(sink), torch.from_numpy(ids_ref[:k_ref]) + sink,
                                     torch.arange(sink + n_keys, total)])
                    ref[h * G:(h + 1) * G] = _ref_attention(q[b, 0, h * G:(h + 1) * G], K[h:h + 1, sel], V[h:h + 1, sel], G=G * 10)
                err = (out[b, 0].float().cpu() - ref).abs().max().item()
                assert err < 2e-2, f"attention differs by {err} at step {step} layer {l}"
            if step == 35:
                # the reference's own method form (:1684-1832) from the same operands: same k, ids packed row by row
                qd = q.to(DEV)
                cand, scores = cache._plan.run_candidates(qd, cache._srht_signs, cache._mag_centers, cache.cluster_key_counts_gpu[l],
                                                          cache._codes_km[l], cache._nib_km[l], cache._w_km[l], sink, n_keys,
                                                          tiers, n_cand)
                qv = qd[:, 0].view(bs, Hkv, G, 128).float()
                q_avg = qv[:, :, 0]
                for gi in range(1, G):  # the group mean with the heads added in order (fp32 sums are order-dependent)
                    q_avg = q_avg + qv[:, :, gi]
                k_form, packed, global_k = cache._compute_adaptive_topk(
                    (q_avg / G).to(dtype), cache.unified_keys_gpu[l][:, :, :sl_end],
                    cache._sl_vnorm_cache[l][:, :, :sl_end], scores, cand, l, thr)
                assert np.array_equal(k_form.cpu().numpy(), ak) and global_k == int(ak.max())
                cap_k = min(cache._HARDCODED_MAX_K, n_cand)
                ids_step = cache._topk_ids[:bs * Hkv * cap_k].view(bs * Hkv, cap_k).cpu()
                want = torch.cat([ids_step[r, :int(ak.reshape(-1)[r])] for r in range(bs * Hkv)])
                assert torch.equal(packed.cpu(), want)
    assert len(seen_k) >= 3, f"k should vary across rows and steps, saw {sorted(seen_k)}"


def test_adaptive_k_cache_with_more_than_8192_candidates():
    """The fused adaptive step where a row has more candidates than one workgroup holds (multi-workgroup adaptive-k
    kernels, value norms handed over by the rerank): 170 K-token prompt, 8.5 K candidates per row; k and the selected
    set against the CPU oracle on the cache's own index."""
    from pariskv_amd.cache_hub.polar_cache_adaptivek_varlen import polar_cache as adaptive_cache

    bs, Hkv, Hq, S, steps = 1, 2, 8, 170_000, 3
    sink, local, thr = 4, 64, 0.7
    G = Hq // Hkv
    cache = adaptive_cache(valid_start=[0] * bs, layer_num=1, batch_size=bs, max_length=S + steps + 10,
                           num_key_value_heads=Hkv, num_heads=Hq, head_dim=128, dtype=torch.bfloat16, layer_mapping={0: DEV},
                           max_new_length=steps + 10, sink_size=sink, local_size=local, core=1, nprobe=1, cache_unit_size=1,
                           cache_cluster_num=1, num_gpus=1, model_size=7, final_topk=100, dynamic_update_interval=16,
                           full_attention_threshold=100, enable_offload=True, adaptive_topk_threshold=thr)
    gen = torch.Generator().manual_seed(11)
    hk, hv = _synth_kv(gen, bs, S, Hkv)
    hv = hv * (0.25 + 2.0 * torch.rand(bs, S, Hkv, 1, generator=gen)).to(torch.bfloat16)
    cache.prefill_update_kv_cache(None, hk.to(DEV), hv.to(DEV), 0, 0)
    signs = O.srht_signs(42)
    scale = 1.0 / math.sqrt(128)
    for step in range(steps):
        k1, v1 = _synth_kv(gen, bs, 1, Hkv)
        q = (hk[:, -3:].float().mean(dim=1).repeat_interleave(G, dim=1) * 0.3
             + 0.5 * torch.randn(bs, Hq, 128, generator=gen)).to(torch.bfloat16).view(bs, 1, Hq, 128)
        hk, hv = torch.cat([hk, k1], dim=1), torch.cat([hv, v1], dim=1)
        cache.decode_update_kv_cache(k1.to(DEV), v1.to(DEV), 0)
        out = cache.compute(q.to(DEV), 0)
    torch.cuda.synchronize()
    total = S + steps
    z = cache._zones[0]
    n_keys, n_cand, _, tiers = cache.retrieval_shape(0)
    assert n_cand > 8192 and n_keys == z.encoded
    sl_end = z.gpu_prefix_rows
    dense_keys = cache.unified_keys_gpu[0][:, :, :sl_end].float().cpu().numpy()
    sl_vnorm = cache._sl_vnorm_cache[0][:, :, :sl_end].cpu().numpy()
    value_norm = cache.value_norm_gpu[0].cpu().numpy()
    codes, nib = cache._codes_km[0].cpu().numpy(), cache._nib_km[0].cpu().numpy()
    w, cc = cache._w_km[0].float().cpu().numpy(), cache.cluster_key_counts_gpu[0].cpu().numpy()
    ak = cache.last_adaptive_k.cpu().numpy()
    cap_k = min(cache._HARDCODED_MAX_K, n_cand)
    ids_gpu = cache._topk_ids[:bs * Hkv * cap_k].view(bs, Hkv, cap_k).cpu().numpy()
    K, V = hk[0].permute(1, 0, 2), hv[0].permute(1, 0, 2)
    ref = torch.empty(Hq, 128)
    for h in range(Hkv):
        zone = slice(sink, sink + n_keys)
        qh, qn = O.query_prep(q[0, 0, h * G:(h + 1) * G].float().numpy(), signs, O.BF16)
        lut = O.tier_lut(O.rank_centroids(qh, O.BF16), cc[0, h], tiers)
        cand_ref, _ = O.select_candidates(O.collision_count(codes[0, h][zone], lut), n_cand)
        sc = O.rerank(cand_ref, nib[0, h][zone].reshape(-1, 16, 4), w[0, h][zone], qh, qn)
        sl_logits = O.dense_logits(q[0, 0, h * G:(h + 1) * G].float().numpy(), dense_keys[0, h], scale, O.BF16)
        k_ref, ids_ref = O.adaptive_topk(sl_logits, sl_vnorm[0, h], sc * np.float32(scale), value_norm[0, h][cand_ref + sink],
                                         cand_ref, thr, cap_k)
        k_ref = min(max(k_ref, min(cache._HARDCODED_MIN_K, cap_k)), cap_k)
        assert int(ak[0, h]) == k_ref and np.array_equal(ids_gpu[0, h], ids_ref), (h, int(ak[0, h]), k_ref)
        sel = torch.cat([torch.arange(sink), torch.from_numpy(ids_ref[:k_ref]) + sink, torch.arange(sink + n_keys, total)])
        ref[h * G:(h + 1) * G] = _ref_attention(q[0, 0, h * G:(h + 1) * G], K[h:h + 1, sel], V[h:h + 1, sel], G=G * 10)
    assert (out[0, 0].float().cpu() - ref).abs().max().item() < 2e-2


@pytest.mark.parametrize("offload", [True, False])
def test_dense_adaptive_k_cache_decode_loop(offload):
    """Dense-form adaptive-k variant (reference polar_cache_atten_value_indices_adaptive_k.py), both storage modes:
    per-row k (capped by adaptive_topk_max_k, no lower clamp) equals the CPU oracle's on the cache's own index, and the
    attention equals an fp32 softmax over sink ++ the first max-over-rows(k) ids of each row's benefit order ++ dense
    tail, which is the set the reference attends to (:1462-1499, :1585-1589)."""
    from pariskv_amd.cache_hub.polar_cache_atten_value_indices_adaptive_k import polar_cache as dense_adaptive_cache

    bs, Hkv, Hq, S, steps = 2, 2, 8, 3000, 40
    sink, local, I, thr, max_k = 4, 64, 16, 0.6, 250
    G = Hq // Hkv
    cache = dense_adaptive_cache(valid_start=[0] * bs, layer_num=1, batch_size=bs, max_length=S + steps + 10,
                                 num_key_value_heads=Hkv, num_heads=Hq, head_dim=128, dtype=torch.bfloat16,
                                 layer_mapping={0: DEV}, max_new_length=steps + 10, sink_size=sink, local_size=local, core=1,
                                 nprobe=1, cache_unit_size=1, cache_cluster_num=1, num_gpus=1, model_size=7, final_topk=100,
                                 dynamic_update_interval=I, full_attention_threshold=100, enable_offload=offload,
                                 adaptive_topk_threshold=thr, adaptive_topk_max_k=max_k)
    gen = torch.Generator().manual_seed(5)
    hk, hv = _synth_kv(gen, bs, S, Hkv)
    hv = hv * (0.25 + 2.0 * torch.rand(bs, S, Hkv, 1, generator=gen)).to(torch.bfloat16)
    cache.prefill_update_kv_cache(None, hk.to(DEV), hv.to(DEV), 0, 0)
    signs = O.srht_signs(42)
    scale = 1.0 / math.sqrt(128)
    seen_k, uneven = set(), False
    for step in range(steps):
        k1, v1 = _synth_kv(gen, bs, 1, Hkv)
        q = (hk[:, -3:].float().mean(dim=1).repeat_interleave(G, dim=1) * 0.3
             + 0.5 * torch.randn(bs, Hq, 128, generator=gen)).to(torch.bfloat16).view(bs, 1, Hq, 128)
        hk, hv = torch.cat([hk, k1], dim=1), torch.cat([hv, v1], dim=1)
        cache.decode_update_kv_cache(k1.to(DEV), v1.to(DEV), 0)
        out = cache.compute(q.to(DEV), 0)
        if step % 6 != 0 and step not in (I - 1, I, 2 * I - 1):
            continue
        torch.cuda.synchronize()
        total = S + step + 1
        z = cache._zones[0]
        n_keys, n_cand, _, tiers = cache.retrieval_shape(0)
        assert n_keys == z.encoded and z.seq_len == total
        dense_pos = torch.cat([torch.arange(sink), torch.arange(sink + n_keys, total)])
        vn_ref = torch.linalg.vector_norm(hv, dim=-1).float().permute(0, 2, 1)
        norms = cache._sl_vnorm_cache[0].cpu()
        sl_vnorm = (norms[:, :, :len(dense_pos)] if offload else norms[:, :, dense_pos]).numpy()
        assert np.allclose(sl_vnorm, vn_ref[:, :, dense_pos].numpy(), rtol=2.0 ** -7, atol=0)
        value_norm = cache.value_norm_gpu[0].cpu().numpy()
        assert np.allclose(value_norm[:, :, sink:sink + n_keys], vn_ref[:, :, sink:sink + n_keys].numpy(), rtol=2.0 ** -7, atol=0)
        codes, nib = cache._codes_km[0].cpu().numpy(), cache._nib_km[0].cpu().numpy()
        w, cc = cache._w_km[0].float().cpu().numpy(), cache.cluster_key_counts_gpu[0].cpu().numpy()
        ak = cache.last_adaptive_k.cpu().numpy()
        cap_k = min(max_k, n_cand)
        ids_ref = np.zeros((bs, Hkv, cap_k), np.int64)
        for b in range(bs):
            for h in range(Hkv):
                zone = slice(sink, sink + n_keys)
                qh, qn = O.query_prep(q[b, 0, h * G:(h + 1) * G].float().numpy(), signs, O.BF16)
                lut = O.tier_lut(O.rank_centroids(qh, O.BF16), cc[b, h], tiers)
                cand_ref, _ = O.select_candidates(O.collision_count(codes[b, h][zone], lut), n_cand)
                sc = O.rerank(cand_ref, nib[b, h][zone].reshape(-1, 16, 4), w[b, h][zone], qh, qn)
                sl_logits = O.dense_logits(q[b, 0, h * G:(h + 1) * G].float().numpy(), hk[b, dense_pos, h].float().numpy(),
                                           scale, O.BF16)
                k_ref, ids_ref[b, h] = O.adaptive_topk(sl_logits, sl_vnorm[b, h], sc * np.float32(scale),
                                                       value_norm[b, h][cand_ref + sink], cand_ref, thr, cap_k)
                assert int(ak[b, h]) == k_ref, f"step {step} row {(b, h)}: k {ak[b, h]} vs {k_ref}"
                seen_k.add(k_ref)
        global_k = int(ak.max())
        uneven = uneven or int(ak.min()) < global_k
        for b in range(bs):
            K, V = hk[b].permute(1, 0, 2), hv[b].permute(1, 0, 2)
            ref = torch.empty(Hq, 128)
            for h in range(Hkv):
                sel = torch.cat([torch.arange(sink), torch.from_numpy(ids_ref[b, h, :global_k]) + sink,
                                 torch.arange(sink + n_keys, total)])
                ref[h * G:(h + 1) * G] = _ref_attention(q[b, 0, h * G:(h + 1) * G], K[h:h + 1, sel], V[h:h + 1, sel], G=G * 10)
            err = (out[b, 0].float().cpu() - ref).abs().max().item()
            assert err < 2e-2, f"attention differs by {err} at step {step}"
        if step == 36:  # the reference's method form (:1508-1589)
            qd = q.to(DEV)
            cand, scores = cache._plan.run_candidates(qd, cache._srht_signs, cache._mag_centers, cache.cluster_key_counts_gpu[0],
                                                      cache._codes_km[0], cache._nib_km[0], cache._w_km[0], sink, n_keys,
                                                      tiers, n_cand)
            dense_k = torch.from_numpy(np.stack([[hk[b, dense_pos, h].float().numpy() for h in range(Hkv)]
                                                 for b in range(bs)])).to(torch.bfloat16).to(DEV)
            k_form, idx_form, gk = cache._compute_adaptive_topk(
                qd[:, 0].view(bs, Hkv, G, 128).float().mean(dim=2).to(torch.bfloat16), dense_k,
                torch.from_numpy(sl_vnorm).to(DEV), scores, cand, 0, thr)
            assert np.array_equal(k_form.cpu().numpy(), ak) and gk == global_k
            assert np.array_equal(idx_form.cpu().numpy(), ids_ref[:, :, :global_k])
    assert len(seen_k) >= 3 and uneven, f"k should vary across rows and steps, saw {sorted(seen_k)}"


def test_reference_multibatch_smoke_shape():
    """The reference's own integration smoke (tests/test_multibatch_smoke.py:23-117): batch 8 in lockstep, 28 layers,
    4 KV heads x GQA 8, prefill 20480, 50 decode steps, sink 128 / local 256, refresh every 128 tokens, offload on,
    integer device ids in layer_mapping, the shipped codebook file -- same constructor call minus the two keywords
    that the reference class itself no longer accepts.  Beyond "does not crash": outputs are finite and, at the last
    step, one layer's retrieved indices equal the CPU oracle's on the cache's own index."""
    import os

    from pariskv_amd.cache_hub.polar_cache import polar_cache

    print("reference multibatch smoke shape", flush=True)
    bs, layers, Hkv, Hq, D, S, steps = 8, 28, 4, 32, 128, 20480, 50
    max_new = steps + 100
    codebook = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "codebook_d128_m8_Kr1_Kw256_rabitq_sign.json")
    cache = polar_cache(valid_start=[0] * bs, layer_num=layers, batch_size=bs, max_length=S + max_new,
                        num_key_value_heads=Hkv, num_heads=Hq, head_dim=D, dtype=torch.bfloat16,
                        layer_mapping={i: 0 for i in range(layers)}, max_new_length=max_new, sink_size=128, local_size=256,
                        core=1, nprobe=1, cache_unit_size=1, cache_cluster_num=1, num_gpus=1, model_size=7,
                        codebook_path=codebook, final_topk=100, dynamic_update_interval=128, enable_offload=True)
    g = torch.Generator(device=DEV).manual_seed(0)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device=DEV, dtype=torch.bfloat16)
    for l in range(layers):
        k_out, v_out = cache.prefill_update_kv_cache(rnd(bs, 8, Hkv * 8, D), rnd(bs, S, Hkv, D), rnd(bs, S, Hkv, D), l, batch_idx=0)
        assert k_out.shape == (bs, S, Hkv, D) and v_out.shape == (bs, S, Hkv, D)
    assert cache.current_seq_len[0] == S
    probe = layers - 3
    for step in range(steps):
        for l in range(layers):
            q = rnd(bs, 1, Hq, D)
            cache.decode_update_kv_cache(rnd(bs, 1, Hkv, D), rnd(bs, 1, Hkv, D), l)
            out = cache.compute(q, l)
            if step == steps - 1 and l == probe:
                q_probe, ids_probe = q.clone(), cache.last_topk_indices.clone()
        if step % 10 == 0 or step == steps - 1:
            assert out.shape == (bs, 1, Hq, D) and bool(torch.isfinite(out.float()).all())
    torch.cuda.synchronize()
    assert cache.current_seq_len == [S + steps] * layers and cache.context == S + steps
    n_keys, n_cand, kk, tiers = cache.retrieval_shape(probe)
    assert kk == 100 and n_keys == S - 128 - 256          # 50 tokens: no refresh yet (interval 128)
    signs = O.srht_signs(42)
    G = Hq // Hkv
    for b, h in ((0, 0), (5, 3)):
        zone = slice(128, 128 + n_keys)
        codes = cache._codes_km[probe][b, h, zone].cpu().numpy()
        nib = cache._nib_km[probe][b, h, zone].cpu().numpy().reshape(-1, 16, 4)
        w = cache._w_km[probe][b, h, zone].float().cpu().numpy()
        cc = cache.cluster_key_counts_gpu[probe][b, h].cpu().numpy()
        ref = O.retrieve_row(q_probe[b, 0, h * G:(h + 1) * G].float().cpu().numpy(), signs, O.BF16, codes, nib, w, cc, tiers,
                             n_cand, kk)
        assert np.array_equal(np.sort(ids_probe[b, h].cpu().numpy()), np.sort(ref))   # the cache needs the set, not the order


@pytest.mark.parametrize("offload", [True, False])
def test_prefill_per_sample_and_valid_start_equal_lockstep(offload):
    """The two prefill entry forms of the reference (polar_cache.py:379-387): one call per sample (bsz == 1, with
    batch_idx) and one lockstep call for the whole batch, the latter also with a non-zero valid_start that skips
    left padding.  All three caches must hold the same index, the same K/V rows and give the same first decode step."""
    bs, Hkv, Hq, S, pad = 3, 2, 8, 2600, 7
    sink, local, I, topk = 4, 64, 32, 100
    gen = torch.Generator().manual_seed(12)
    k, v = _synth_kv(gen, bs, S, Hkv)
    kd, vd = k.to(DEV), v.to(DEV)
    lock = _make_cache(offload, bs, Hkv, Hq, 1, S, 20, sink, local, I, topk)
    lock.prefill_update_kv_cache(None, kd, vd, 0, 0)
    single = _make_cache(offload, bs, Hkv, Hq, 1, S, 20, sink, local, I, topk)
    for b in range(bs):
        ko, vo = single.prefill_update_kv_cache(None, kd[b:b + 1], vd[b:b + 1], 0, b)
        assert ko.shape == (1, S, Hkv, 128) and torch.equal(vo, vd[b:b + 1])
    from pariskv_amd.cache_hub.polar_cache import polar_cache
    padded = polar_cache(valid_start=[pad] * bs, layer_num=1, batch_size=bs, max_length=S + pad + 20, num_key_value_heads=Hkv,
                         num_heads=Hq, head_dim=128, dtype=torch.bfloat16, layer_mapping={0: DEV}, max_new_length=20,
                         sink_size=sink, local_size=local, core=1, nprobe=1, cache_unit_size=1, cache_cluster_num=1, num_gpus=1,
                         model_size=7, final_topk=topk, dynamic_update_interval=I, full_attention_threshold=100,
                         enable_offload=offload)
    junk_k, junk_v = _synth_kv(gen, bs, pad, Hkv)
    ko, vo = padded.prefill_update_kv_cache(None, torch.cat([junk_k.to(DEV), kd], dim=1), torch.cat([junk_v.to(DEV), vd], dim=1), 0, 0)
    assert torch.equal(ko, kd) and torch.equal(vo, vd)                       # the states from valid_start on
    assert padded.prefill_update_kv_cache(None, torch.cat([junk_k.to(DEV), kd], dim=1), torch.cat([junk_v.to(DEV), vd], dim=1),
                                          0, 1)[0].shape == (bs, S, Hkv, 128)  # batch_idx != 0: slices only
    torch.cuda.synchronize()
    k1, v1 = _synth_kv(gen, bs, 1, Hkv)
    q = (k.float().mean(dim=1).repeat_interleave(Hq // Hkv, dim=1) + 0.5 * torch.randn(bs, Hq, 128, generator=gen))
    q = q.to(torch.bfloat16).view(bs, 1, Hq, 128).to(DEV)
    outs = []
    for c in (lock, single, padded):
        assert c.current_seq_len == [S] and c.context == S
        c.decode_update_kv_cache(k1.to(DEV), v1.to(DEV), 0)
        outs.append((c.compute(q, 0).clone(), c.last_topk_indices.clone()))
    torch.cuda.synchronize()
    for c in (single, padded):
        assert torch.equal(c.cluster_key_counts_gpu[0], lock.cluster_key_counts_gpu[0])
        for name in ("_codes_km", "_nib_km", "_w_km", "unified_keys_gpu", "unified_values_gpu"):
            a, b_ = getattr(c, name)[0], getattr(lock, name)[0]
            rows = min(a.shape[2], b_.shape[2])     # the padded cache was sized for a longer prompt
            assert torch.equal(a[:, :, :rows], b_[:, :, :rows]), name
        if offload:
            n = lock.cpu_valid_end[0]
            assert c.cpu_valid_end[0] == n
            assert torch.equal(c.unified_keys_cpu[0][:, :, :n], lock.unified_keys_cpu[0][:, :, :n])
            assert torch.equal(c.unified_values_cpu[0][:, :, :n], lock.unified_values_cpu[0][:, :, :n])
    for out, ids in outs[1:]:
        assert torch.equal(ids, outs[0][1]) and torch.equal(out, outs[0][0])


def test_model_decode_glue_matches_dense_model():
    """The decode glue (reference model_hub/LLM.py:157-198 + qwen.py ops) on a small random Qwen3-shaped model: with a
    prompt short enough that the cache attends to every token, each decode step must equal a plain fp32 restatement of
    the same decoder that keeps its own K/V history (RMSNorm, per-head q/k norm, rotary embedding, GQA attention,
    SiLU-gated MLP), to bf16 tolerance; then a long prompt runs the retrieval path for a few steps."""
    import torch.nn.functional as F

    from pariskv_amd.model_hub import QwenConfig, QwenModel

    cfg = QwenConfig(hidden_size=256, num_layers=2, num_heads=8, num_key_value_heads=2, head_dim=128, intermediate_size=512,
                     vocab_size=1000)
    bs, S, steps = 2, 40, 6
    cache = _make_cache(True, bs, cfg.num_key_value_heads, cfg.num_heads, cfg.num_layers, S, steps + 4, 4, 64, 32, 100, thr=2000)
    gen = torch.Generator().manual_seed(4)
    hk, hv = [], []
    for l in range(cfg.num_layers):
        k, v = _synth_kv(gen, bs, S, cfg.num_key_value_heads)
        k = (k.float() * 0.1).to(torch.bfloat16)
        hk.append(k.float()), hv.append(v.float())
        cache.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), l, 0)
    model = QwenModel(cfg, cache, device=DEV, max_positions=S + steps + 8, seed=1)
    f = lambda t: t.float().cpu()

    def rms(x, w, eps):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w

    def ref_step(ids, pos, hidden):
        x = f(model.embed_tokens)[ids]                                   # [bs, 1, h]
        for l, ly in enumerate(model.layers):
            hidden.append(x)
            y = rms(x, f(ly.input_layernorm_weight), cfg.rms_norm_eps)
            qkv = y @ f(ly.wqkv).T
            q, k, v = qkv.split([cfg.num_heads * 128, cfg.num_key_value_heads * 128, cfg.num_key_value_heads * 128], dim=-1)
            q = rms(q.view(bs, 1, cfg.num_heads, 128), f(ly.q_norm_weight), cfg.rms_norm_eps)
            k = rms(k.view(bs, 1, cfg.num_key_value_heads, 128), f(ly.k_norm_weight), cfg.rms_norm_eps)
            c, s = f(model.cos_cache)[pos][None, None, None, :], f(model.sin_cache)[pos][None, None, None, :]
            rot = lambda t: torch.cat((t[..., :64] * c - t[..., 64:] * s, t[..., 64:] * c + t[..., :64] * s), dim=-1)
            q, k = rot(q), rot(k)
            hk[l] = torch.cat([hk[l], k], dim=1)
            hv[l] = torch.cat([hv[l], v.view(bs, 1, cfg.num_key_value_heads, 128)], dim=1)
            G = cfg.num_heads // cfg.num_key_value_heads
            kk, vv = hk[l].repeat_interleave(G, dim=2), hv[l].repeat_interleave(G, dim=2)     # [bs, T, Hq, D]
            att = F.scaled_dot_product_attention(q.transpose(1, 2), kk.transpose(1, 2), vv.transpose(1, 2))   # [bs,Hq,1,D]
            x = x + att.transpose(1, 2).reshape(bs, 1, -1) @ f(ly.wo).T
            hidden.append(x)
            y = rms(x, f(ly.post_attention_layernorm_weight), cfg.rms_norm_eps)
            gu = y @ f(ly.gate_up_proj).T
            x = x + (F.silu(gu[..., :cfg.intermediate_size]) * gu[..., cfg.intermediate_size:]) @ f(ly.down_proj).T
        return rms(x, f(model.norm_weight), cfg.rms_norm_eps) @ f(model.lm_head).T

    # the residual stream at both points of every layer (entering it, and after its attention): the fused decode path
    # materialises exactly these sums in ops.add_rmsnorm, which is wrapped here to record them
    from pariskv_amd import ops as _ops

    seen = []
    real_add_rmsnorm = _ops.add_rmsnorm

    def recording_add_rmsnorm(x, residual, weight, eps, want_sum=True):
        out_sum, out_norm = real_add_rmsnorm(x, residual, weight, eps, want_sum)
        if want_sum:
            seen.append(out_sum.float().cpu())
        return out_sum, out_norm

    ids = torch.randint(0, cfg.vocab_size, (bs, 1), generator=gen)
    _ops.add_rmsnorm = recording_add_rmsnorm
    try:
        for step in range(steps):
            seen.clear()
            logits = model.decode_forward(ids.to(DEV))
            want = []
            ref = ref_step(ids, S + step, want)
            assert logits.shape == (bs, 1, cfg.vocab_size) and logits.dtype == torch.float32
            assert len(seen) == len(want) == 2 * cfg.num_layers
            # per element, in units of the tensor's rms: a bf16 residual stream carries 2^-9 relative rounding per
            # value and per bf16 GEMM operand, accumulated over at most 2 layers; a wrong head, a swapped
            # rotary half or a missing norm weight moves whole blocks of elements by O(1) rms
            for i, (got, exp) in enumerate(zip(seen, want)):
                err = ((got - exp).abs().max() / exp.pow(2).mean().sqrt()).item()
                assert err < 0.03, f"step {step}: hidden state {i} differs by {err:.4f} rms"
            err = ((logits.cpu() - ref).abs().max() / ref.pow(2).mean().sqrt()).item()
            assert err < 0.04, f"step {step}: logits differ by {err:.4f} rms"
            ids = ref.argmax(dim=-1)
    finally:
        _ops.add_rmsnorm = real_add_rmsnorm
    assert cache.context == S + steps
    # long prompt: the same glue over the retrieval path (offload, index refresh inside the run)
    S2 = 3000
    cache2 = _make_cache(True, bs, cfg.num_key_value_heads, cfg.num_heads, cfg.num_layers, S2, 50, 4, 64, 32, 100)
    for l in range(cfg.num_layers):
        k, v = _synth_kv(gen, bs, S2, cfg.num_key_value_heads)
        cache2.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), l, 0)
    model2 = QwenModel(cfg, cache2, device=DEV, max_positions=S2 + 64, seed=1)
    ids = torch.randint(0, cfg.vocab_size, (bs, 1), generator=gen).to(DEV)
    for step in range(40):
        logits = model2.decode_forward(ids)
        ids = logits.argmax(dim=-1)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(logits).all()) and cache2.context == S2 + 40 and cache2._zones[0].encoded > S2 - 68


def test_qk_norm_rope_matches_torch_ops():
    """pkv_qk_norm_rope against the reference's op sequence (qwen.py:327-340 head_rmsnorm of q and k, :434-498 rotary
    embedding) evaluated in fp32 on the same bf16 inputs: within one bf16 rounding of the result; with and without
    norm weights; q/k read from a fused projection output with a padded row stride."""
    from pariskv_amd import ops

    g = torch.Generator(device=DEV).manual_seed(2)
    bs, Hq, Hkv, D = 3, 32, 8, 128
    width = (Hq + 2 * Hkv) * D
    buf = torch.randn(bs, 1, width + 64, generator=g, device=DEV).to(torch.bfloat16)
    qkv = buf[..., :width]                                   # row stride larger than the row
    qw = (1 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
    kw = (1 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
    ang = torch.rand(D // 2, generator=g, device=DEV) * 6.28
    cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
    eps = 1e-6

    def ref(x, heads, w):
        x = x.float().reshape(bs, 1, heads, D)
        if w is not None:
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        c, s = cos.float(), sin.float()
        return torch.cat((x[..., :64] * c - x[..., 64:] * s, x[..., 64:] * c + x[..., :64] * s), dim=-1)

    for weights in ((qw, kw), (None, None)):
        q, k = ops.qk_norm_rope(qkv, Hq, Hkv, weights[0], weights[1], eps, cos, sin)
        torch.cuda.synchronize()
        assert q.shape == (bs, 1, Hq, D) and k.shape == (bs, 1, Hkv, D)
        for got, want in ((q, ref(qkv[..., :Hq * D], Hq, weights[0])), (k, ref(qkv[..., Hq * D:(Hq + Hkv) * D], Hkv, weights[1]))):
            err = (got.float() - want).abs()
            assert bool((err <= want.abs() * 2 ** -7 + 1e-6).all()), float(err.max())
    with pytest.raises(RuntimeError, match="go together"):
        ops.qk_norm_rope(qkv, Hq, Hkv, qw, None, eps, cos, sin)


def test_qk_norm_rope_with_the_vote_table_in_the_same_launch():
    """pkv_qk_norm_rope_table: q / k bit for bit as pkv_qk_norm_rope writes them, and in the bound step's workspace the
    rotated query, its norm and the vote table exactly as the query-prep launch computes them from that q; the
    decode step launched with table_ready then returns the attention output and the ids of the ordinary step.  Run
    through the cache class (offload and no-offload) on its own bound step, as the model glue does."""
    from pariskv_amd import ops
    from pariskv_amd.cache_hub.polar_cache import polar_cache

    bs, Hq, Hkv, D, S = 2, 8, 2, 128, 3000
    g = torch.Generator(device=DEV).manual_seed(9)
    for offload in (True, False):
        cache = _make_cache(offload, bs, Hkv, Hq, 1, S, 64, 4, 64, 16, 100)
        k, v = _synth_kv(torch.Generator().manual_seed(1), bs, S, Hkv)
        cache.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), 0, 0)
        width = (Hq + 2 * Hkv) * D
        qw = (1 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
        kw = (1 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
        ang = torch.rand(D // 2, generator=g, device=DEV) * 6.28
        cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
        assert cache.query_table_target(0) is None           # nothing bound before the first retrieval
        used = 0
        for step in range(20):                                # crosses an index refresh (interval 16)
            qkv = torch.randn(bs, 1, width, generator=g, device=DEV).to(torch.bfloat16)
            target = cache.query_table_target(0)
            q0, k0 = ops.qk_norm_rope(qkv, Hq, Hkv, qw, kw, 1e-6, cos, sin)
            q1, k1 = ops.qk_norm_rope(qkv, Hq, Hkv, qw, kw, 1e-6, cos, sin, table_for=target)
            assert torch.equal(q0, q1) and torch.equal(k0, k1)
            vv = qkv[..., (Hq + Hkv) * D:].reshape(bs, 1, Hkv, D)
            if target is not None:
                used += 1
                n_keys, n_cand, topk, tiers = cache.retrieval_shape(0)
                plan = cache._plan
                tab = {n: plan.view(n, n_keys, n_cand, topk, dt).clone() for n, dt in
                       (("qhat", torch.float32), ("qnorm", torch.float32), ("lut", torch.uint8))}
                assert not bool(plan.view("row_suffix_hist", n_keys, n_cand, topk, torch.int32).any())
                qhat, qnorm, lut, _ = ops.query_prep_lut(q1, Hkv, cache._srht_signs, cache.cluster_key_counts_gpu[0], tiers)
                assert torch.equal(tab["qhat"].view(-1), qhat.reshape(-1)) and torch.equal(tab["qnorm"].view(-1), qnorm.reshape(-1))
                assert torch.equal(tab["lut"].view(-1), lut.reshape(-1))
            cache.decode_update_kv_cache(k1, vv, 0)
            assert target is None or target.a.table_ready == 1
            out1 = cache.compute(q1, 0)
            ids1 = cache.last_topk_indices.clone() if getattr(cache, "last_topk_indices", None) is not None else None
            assert target is None or target.a.table_ready == 0
            out0 = cache.compute(q0, 0)                       # the same step again, its own query-prep launch this time
            torch.cuda.synchronize()
            assert torch.equal(out0, out1), f"step {step}: attention output differs with the table from the q/k launch"
            if ids1 is not None:
                assert torch.equal(ids1, cache.last_topk_indices)
        assert used >= 15, used


def test_qk_norm_rope_writes_the_tokens_rows_into_the_cache():
    """ops.qk_norm_rope(append=...) + decode_update_kv_cache(appended=True) against the ordinary append, two caches
    side by side over 40 tokens and two index refreshes (offload and no-offload): the dense K/V tensors, the zone
    counters, the attention outputs and the selected ids stay identical; an adaptive-k cache declines the fused form."""
    from pariskv_amd import ops
    from pariskv_amd.cache_hub.polar_cache import polar_cache
    from pariskv_amd.cache_hub.polar_cache_adaptivek_varlen import polar_cache as adaptive_cache

    bs, Hq, Hkv, D, S = 2, 8, 2, 128, 3000
    g = torch.Generator(device=DEV).manual_seed(11)
    for offload in (True, False):
        a = _make_cache(offload, bs, Hkv, Hq, 1, S, 64, 4, 64, 16, 100)
        b = _make_cache(offload, bs, Hkv, Hq, 1, S, 64, 4, 64, 16, 100)
        k, v = _synth_kv(torch.Generator().manual_seed(1), bs, S, Hkv)
        for c in (a, b):
            c.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), 0, 0)
        width = (Hq + 2 * Hkv) * D
        qw = (1 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
        kw = (1 + 0.1 * torch.randn(D, generator=g, device=DEV)).to(torch.bfloat16)
        ang = torch.rand(D // 2, generator=g, device=DEV) * 6.28
        cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
        fused = 0
        for step in range(40):
            qkv = torch.randn(bs, 1, width, generator=g, device=DEV).to(torch.bfloat16)
            vv = qkv[..., (Hq + Hkv) * D:].reshape(bs, 1, Hkv, D)
            # cache a: the glue's way; cache b: separate launches
            target = a.query_table_target(0)
            rows = a.fused_append_target(0) if target is not None else None
            qa, ka = ops.qk_norm_rope(qkv, Hq, Hkv, qw, kw, 1e-6, cos, sin, table_for=target, append=rows)
            if rows is not None:
                fused += 1
                assert rows[2] == b._zones[0].append_slot()
                a.decode_update_kv_cache(ka, vv, 0, appended=True)
            else:
                a.decode_update_kv_cache(ka, vv, 0)
            qb, kb = ops.qk_norm_rope(qkv, Hq, Hkv, qw, kw, 1e-6, cos, sin)
            b.decode_update_kv_cache(kb, vv, 0)
            out_a, out_b = a.compute(qa, 0), b.compute(qb, 0)
            torch.cuda.synchronize()
            assert torch.equal(a.unified_keys_gpu[0], b.unified_keys_gpu[0]), f"step {step}: key rows differ"
            assert torch.equal(a.unified_values_gpu[0], b.unified_values_gpu[0]), f"step {step}: value rows differ"
            assert torch.equal(out_a, out_b), f"step {step}: attention output differs"
            assert a._zones[0].seq_len == b._zones[0].seq_len and a.current_seq_len == b.current_seq_len
            if getattr(a, "last_topk_indices", None) is not None and b.last_topk_indices is not None:
                assert torch.equal(a.last_topk_indices, b.last_topk_indices)
        assert fused >= 30, fused
    # bad slot / shapes are refused, and the adaptive-k cache (its append also writes value norms) opts out
    with pytest.raises(Exception):
        ops.qk_norm_rope(qkv, Hq, Hkv, qw, kw, 1e-6, cos, sin, table_for=a.query_table_target(0),
                         append=(a.unified_keys_gpu[0], a.unified_values_gpu[0], a.unified_keys_gpu[0].shape[2]))
    with pytest.raises(Exception):
        ops.qk_norm_rope(qkv, Hq, Hkv, qw, kw, 1e-6, cos, sin, append=(a.unified_keys_gpu[0], a.unified_values_gpu[0], 0))
    assert adaptive_cache.fused_append_target is polar_cache.fused_append_target
    assert adaptive_cache._append is not polar_cache._append   # which is what makes fused_append_target return None there


def test_add_rmsnorm_and_silu_mul_match_torch_ops():
    """The two fused element-wise kernels of the decode glue against the torch op sequences they replace (bf16 add then
    F.rms_norm; F.silu then multiply), element for element up to one bf16 rounding."""
    import torch.nn.functional as F

    from pariskv_amd import ops

    g = torch.Generator(device=DEV).manual_seed(6)
    for rows, width in ((8, 4096), (3, 256), (1, 16384), (5, 1000)):
        x = torch.randn(rows, 1, width, generator=g, device=DEV).to(torch.bfloat16)
        r = torch.randn(rows, 1, width, generator=g, device=DEV).to(torch.bfloat16)
        w = (1 + 0.2 * torch.randn(width, generator=g, device=DEV)).to(torch.bfloat16)
        s, n = ops.add_rmsnorm(x, r, w, 1e-6)
        want_s = x + r
        assert torch.equal(s, want_s)
        want_n = F.rms_norm(want_s.float(), (width,), w.float(), 1e-6)
        assert bool(((n.float() - want_n).abs() <= want_n.abs() * 2 ** -7 + 1e-6).all())
        s2, n2 = ops.add_rmsnorm(x, None, w, 1e-6)
        assert s2 is x and bool(((n2.float() - F.rms_norm(x.float(), (width,), w.float(), 1e-6)).abs()
                                 <= n2.float().abs() * 2 ** -7 + 1e-6).all())
    gu = (torch.randn(8, 1, 2 * 12288, generator=g, device=DEV) * 3).to(torch.bfloat16)
    got = ops.silu_mul(gu)
    want = F.silu(gu[..., :12288].float()) * gu[..., 12288:].float()
    assert got.shape == (8, 1, 12288)
    assert bool(((got.float() - want).abs() <= want.abs() * 2 ** -6 + 1e-6).all())


@pytest.mark.parametrize("offload", [True, False])
def test_fp32_cache_decode_steps(offload):
    """The cache class with dtype float32 (BASELINE config 1's dtype): fp32 K/V rows (512-byte rows through append,
    offload and gather), the fp32 encoder / query chains and the fp32 attention kernel.  Index set equal to the
    oracle's fp32 chain on the cache's own index, attention within 1e-3 of an fp32 softmax over the same rows."""
    from pariskv_amd.cache_hub.polar_cache import polar_cache

    bs, Hkv, Hq, S, steps = 2, 2, 8, 2500, 40
    sink, local, I, topk = 4, 64, 32, 150
    G = Hq // Hkv
    cache = polar_cache(valid_start=[0] * bs, layer_num=1, batch_size=bs, max_length=S + steps + 8, num_key_value_heads=Hkv,
                        num_heads=Hq, head_dim=128, dtype=torch.float32, layer_mapping={0: DEV}, max_new_length=steps + 8,
                        sink_size=sink, local_size=local, core=1, nprobe=1, cache_unit_size=1, cache_cluster_num=1, num_gpus=1,
                        model_size=7, final_topk=topk, dynamic_update_interval=I, full_attention_threshold=100,
                        enable_offload=offload)
    gen = torch.Generator().manual_seed(9)
    k = torch.randn(bs, S, Hkv, 128, generator=gen)
    k[..., [7, 31, 64, 101]] *= 10.0
    v = torch.randn(bs, S, Hkv, 128, generator=gen)
    cache.prefill_update_kv_cache(None, k.to(DEV), v.to(DEV), 0, 0)
    signs = O.srht_signs(42)
    hk, hv = k, v
    for step in range(steps):
        k1, v1 = torch.randn(bs, 1, Hkv, 128, generator=gen), torch.randn(bs, 1, Hkv, 128, generator=gen)
        q = (hk.mean(dim=1).repeat_interleave(G, dim=1) + 0.5 * torch.randn(bs, Hq, 128, generator=gen)).view(bs, 1, Hq, 128)
        hk, hv = torch.cat([hk, k1], dim=1), torch.cat([hv, v1], dim=1)
        cache.decode_update_kv_cache(k1.to(DEV), v1.to(DEV), 0)
        out = cache.compute(q.to(DEV), 0)
        if step not in (0, I - 1, I, steps - 1):
            continue
        torch.cuda.synchronize()
        assert out.dtype == torch.float32
        total = S + step + 1
        n_keys, n_cand, kk, tiers = cache.retrieval_shape(0)
        ids = cache.last_topk_indices.cpu().numpy()
        for b in range(bs):
            ref = torch.empty(Hq, 128)
            for h in range(Hkv):
                zone = slice(sink, sink + n_keys)
                codes = cache._codes_km[0][b, h, zone].cpu().numpy()
                nib = cache._nib_km[0][b, h, zone].cpu().numpy().reshape(-1, 16, 4)
                w = cache._w_km[0][b, h, zone].float().cpu().numpy()
                if step == 0:
                    ec, en, ew = O.encode(hk[b, sink:sink + n_keys, h].numpy(), signs, O.F32)
                    assert np.array_equal(codes, ec) and np.array_equal(nib, en) and np.array_equal(w, ew)
                want = O.retrieve_row(q[b, 0, h * G:(h + 1) * G].numpy(), signs, O.F32, codes, nib, w,
                                      cache.cluster_key_counts_gpu[0][b, h].cpu().numpy(), tiers, n_cand, kk)
                assert np.array_equal(np.sort(ids[b, h]), np.sort(want)), (step, b, h)
                sel = torch.cat([torch.arange(sink), torch.from_numpy(ids[b, h]) + sink, torch.arange(sink + n_keys, total)])
                ref[h * G:(h + 1) * G] = _ref_attention(q[b, 0, h * G:(h + 1) * G], hk[b].permute(1, 0, 2)[h:h + 1, sel],
                                                        hv[b].permute(1, 0, 2)[h:h + 1, sel], G=G * 10)
            err = (out[b, 0].cpu() - ref).abs().max().item()
            assert err < 1e-3, f"step {step}: attention differs by {err}"
