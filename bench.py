#!/usr/bin/env python3
"""Benchmark of the retrieval hot path on one MI355X.

A "step" is one layer's retrieval for one decode step: query prep + vote table ->
collision scan -> candidate select -> 4-bit rerank -> exact top-k -> UVA gather
of the selected K/V rows out of pinned host memory.  The workload is
BASELINE.json's config 3 (the one the metric is quoted on): batch 4 x 8 KV heads
(32 q heads, head_dim 128), 131072 cached keys per head, 4096 candidates, top-k
1024, bf16, full-precision KV in pinned host memory.

Steps rotate over LAYERS distinct layer indexes (448 MiB each) so that no
layer's codes are still in the 256 MB last-level cache when it is scanned again,
as in a real decode step, which walks all layers of the model.

Prints ONE JSON line: metric/value/unit, the per-stage times (`stages_us`, with both launch plans of the on-GPU
stages), the roofline of the dominant kernel (collision scan, timed by its own dispatch timestamps), the
single-thread CPU baseline, and three more objects measured the same way on their own data: `cfg2` and `cfg4`
(the retrieval at BASELINE configs 2 and 4, each with its algorithmic bytes, HBM fraction and oracle check) and `cfg5`
(decode tokens/s of the model loop).  `--no-cfg2 / --no-cfg4 / --no-cfg5 / --no-cpu-baseline` leave legs out; `--only
scan | copy | decode-loop | model-decode` runs one leg alone (for profiling).
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E
TIER_RATIOS = (0.05, 0.15, 0.30, 0.50, 0.75, 1.0)

# HBM bytes moved by one collision-scan launch at this workload, from the two
# rocprofv3 --pmc runs summarised in profiles/ (None until measured).
SCAN_TRAFFIC_BYTES = 72834000
SCAN_TRAFFIC_SOURCE = "profiles/scan_cfg3_hbm_traffic.md"
SCAN_KERNEL = "pkv_scan_keymajor_kernel"


def model_decode(torch, dev, L, bs, S, T, K, warmup, offload, host_budget):
    """BASELINE config 5: T decode tokens of a random-initialised Qwen3-8B-shaped decoder (L layers) at batch bs over a
    synthetic S-token prompt held by polar_cache (sink 64, local 512, update buffer 1024, final_topk K); returns
    decode tokens/s and where the K/V store was placed.  host_budget: bytes of pinned host memory the cache may use for
    the offloaded K/V (None: all of it); layers beyond the budget keep their K/V in HBM."""
    from pariskv_amd.cache_hub.polar_cache import polar_cache
    from pariskv_amd.model_hub import QwenConfig, QwenModel

    cfg = QwenConfig(num_layers=L)
    H, D = cfg.num_key_value_heads, cfg.head_dim
    cache = polar_cache(valid_start=[0] * bs, layer_num=L, batch_size=bs, max_length=S + T + 8,
                        num_key_value_heads=H, num_heads=cfg.num_heads, head_dim=D,
                        dtype=torch.bfloat16, layer_mapping={i: dev for i in range(L)}, max_new_length=T + 8,
                        sink_size=64, local_size=512, core=1, nprobe=1, cache_unit_size=1, cache_cluster_num=1,
                        num_gpus=1, model_size=8, final_topk=K, dynamic_update_interval=1024,
                        full_attention_threshold=2000, enable_offload=offload,
                        host_kv_budget_bytes=host_budget if offload else None)
    g = torch.Generator(device=dev).manual_seed(0)
    t0 = time.perf_counter()
    # the prompt's K/V are synthetic (the prompt is not run through the model): keys ~ N(mean_t, 1) with four
    # outlier channels and a mean that rotates by 0.5 degrees per 1K tokens in the (0, 1) plane; values ~ N(0, 1)
    ang = torch.arange(S, device=dev, dtype=torch.float32) * (0.5 / 1000.0) * (math.pi / 180.0)
    for l in range(L):
        k = torch.randn(bs, S, H, D, generator=g, device=dev, dtype=torch.bfloat16)
        k[..., 0] += ang.cos().to(torch.bfloat16)[None, :, None]
        k[..., 1] += ang.sin().to(torch.bfloat16)[None, :, None]
        k[..., [7, 31, 64, 101]] *= 10.0
        v = torch.randn(bs, S, H, D, generator=g, device=dev, dtype=torch.bfloat16)
        cache.prefill_update_kv_cache(None, k, v, l, 0)
        del k, v
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    model = QwenModel(cfg, cache, device=dev, max_positions=S + T + 8)
    ids = torch.randint(0, cfg.vocab_size, (bs, 1), generator=g, device=dev)
    for _ in range(warmup):
        ids = model.decode_forward(ids).argmax(dim=-1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(T - warmup):
        ids = model.decode_forward(ids).argmax(dim=-1)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    n_tok = T - warmup
    pl = cache.kv_placement
    return {"model": "Qwen3-8B shape, random init, bf16", "layers": L, "batch": bs, "prompt": S, "generated": T,
            "timed_tokens": n_tok, "offload": bool(offload), "final_topk": K,
            "placement": {"host_layers": pl["host_layers"], "hbm_layers": pl["hbm_layers"],
                          "host_pinned_GiB": round(pl["host_pinned_bytes"] / 2**30, 2),
                          "hbm_kv_GiB": round(pl["hbm_kv_bytes"] / 2**30, 2),
                          "host_budget_GiB": None if host_budget is None else round(host_budget / 2**30, 2)},
            "cache_fill_s": round(t_prefill, 2), "ms_per_token": round(dt * 1e3 / n_tok, 3),
            "decode_tokens_per_s": round(bs * n_tok / dt, 1), "us_per_layer": round(dt * 1e6 / n_tok / L, 1)}


def decode_loop(torch, dev, L, bs, S, T, K, adaptive=False, offload=True, k_range=(256, 2048), threshold=0.95,
                key_drift=0.0, H=8, G=4, D=128):
    """The cache class itself in a loop, no model around it: L layers, S prompt tokens of synthetic K/V (keys ~ N(0,1)
    with four outlier channels, optionally a mean of norm 2 turning by ``key_drift`` degrees per 1K tokens), T decode
    tokens (append + retrieval + gather + attention per layer; index refresh and host offload every 1024 tokens).
    Returns (figures, cache, queries of the last step)."""
    from pariskv_amd.attn_hub import polar_decode_attn
    if adaptive:
        from pariskv_amd.cache_hub.polar_cache_adaptivek_varlen import polar_cache
    else:
        from pariskv_amd.cache_hub.polar_cache import polar_cache

    extra = {}
    if adaptive:  # the class takes its caps from the environment, like the reference
        os.environ["ADAPTIVE_TOPK_MIN_K"], os.environ["ADAPTIVE_TOPK_MAX_K"] = (str(v) for v in k_range)
        extra["adaptive_topk_threshold"] = threshold
    cache = polar_cache(valid_start=[0] * bs, layer_num=L, batch_size=bs, max_length=S + T + 8, num_key_value_heads=H,
                        num_heads=H * G, head_dim=D, dtype=torch.bfloat16, layer_mapping={i: dev for i in range(L)},
                        max_new_length=T + 8, sink_size=64, local_size=512, core=1, nprobe=1, cache_unit_size=1,
                        cache_cluster_num=1, num_gpus=1, model_size=8, final_topk=K, dynamic_update_interval=1024,
                        full_attention_threshold=2000, enable_offload=offload, **extra)
    g = torch.Generator(device=dev).manual_seed(0)
    t0 = time.perf_counter()
    for l in range(L):
        k = torch.randn(bs, S, H, D, generator=g, device=dev, dtype=torch.bfloat16)
        k[..., [7, 31, 64, 101]] *= 10.0
        if key_drift:  # key mean of norm 2 turning in the plane of dims (0, 1)
            ang = torch.arange(S, device=dev, dtype=torch.float32) * (key_drift * math.pi / 180.0 / 1000.0)
            k[..., 0] += (2.0 * torch.cos(ang)).to(torch.bfloat16)[None, :, None]
            k[..., 1] += (2.0 * torch.sin(ang)).to(torch.bfloat16)[None, :, None]
        v = torch.randn(bs, S, H, D, generator=g, device=dev, dtype=torch.bfloat16)
        cache.prefill_update_kv_cache(None, k, v, l, 0)
        kmean = k[:, -1024:].float().mean(dim=1)  # [bs, H, D]
        del k, v
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    k1 = torch.randn(T, bs, 1, H, D, generator=g, device=dev, dtype=torch.bfloat16)
    v1 = torch.randn(T, bs, 1, H, D, generator=g, device=dev, dtype=torch.bfloat16)
    # queries = mean of the recent keys of the head + N(0, 0.5), one per query head
    q = (kmean.repeat_interleave(G, dim=1) + 0.5 * torch.randn(bs, H * G, D, generator=g, device=dev)
         ).to(torch.bfloat16).view(bs, 1, H * G, D)
    torch.cuda.synchronize()
    tok_us, issue = [], []
    for t in range(T):
        a = time.perf_counter()
        for l in range(L):
            cache.decode_update_kv_cache(k1[t], v1[t], l)
            polar_decode_attn(q, None, None, l, cache)
        b = time.perf_counter()
        torch.cuda.synchronize()
        tok_us.append((time.perf_counter() - a) * 1e6)
        issue.append((b - a) * 1e6)
    skip = min(8, T // 2)
    body = sorted(tok_us[skip:])
    res = {"cache": "adaptive-k" if adaptive else "fixed-k", "key_drift_deg_per_1k": key_drift, "offload": bool(offload),
           "layers": L, "batch": bs, "prompt": S, "generated": T, "final_topk": K, "prefill_s": round(t_prefill, 2),
           "us_per_layer_step_median": round(body[len(body) // 2] / L, 1),
           "us_per_layer_step_mean": round(sum(tok_us[skip:]) / len(tok_us[skip:]) / L, 1),
           "us_per_layer_step_worst_token": round(body[-1] / L, 1),
           "host_issue_us_per_layer_step": round(sorted(issue[skip:])[len(issue[skip:]) // 2] / L, 1),
           "index_refreshes": T // 1024}
    if adaptive:
        ak = cache.last_adaptive_k.flatten().tolist()
        res["adaptive"] = {"k_range": list(k_range), "threshold": threshold, "k_of_last_step": [min(ak), max(ak)]}
    return res, cache, q


def build_index_layers(torch, ops, dev, bs, H, G, N, L, signs, seed0=0, D=128):
    """L layers of synthetic keys (~N(0,1), four outlier channels x10, independent seed per sequence and layer) encoded
    on the GPU into the key-major index, with one query per query head = key mean + N(0, 0.5).  Returns the list of
    layers and the bf16 keys / values of layer 0 (for the callers that keep full-precision K/V)."""
    layers, k0, v0 = [], None, None
    for l in range(L):
        codes_km, nib_km, w_km, cb, k4, kw = ops.alloc_keymajor(bs, H, N, dev)
        cc = torch.zeros(bs, H, 16, 256, dtype=torch.int32, device=dev)
        q = torch.empty(bs, 1, H * G, D, dtype=torch.bfloat16, device=dev)
        if l == 0:
            k0 = torch.empty(bs, H, N, D, dtype=torch.bfloat16, device=dev)
            v0 = torch.empty(bs, H, N, D, dtype=torch.bfloat16, device=dev)
        for b in range(bs):
            g = torch.Generator(device=dev).manual_seed(seed0 + 1000 * l + b)
            keys = torch.randn(1, H, N, D, generator=g, device=dev, dtype=torch.float32)
            keys[..., [7, 31, 64, 101]] *= 10.0
            kb = keys.to(torch.bfloat16)
            qq = keys.mean(dim=2, keepdim=True) + 0.5 * torch.randn(1, H, G, D, generator=g, device=dev)
            q[b, 0] = qq.view(H * G, D).to(torch.bfloat16)
            ops.encode_append(kb, signs, cb[b:b + 1], k4[b:b + 1], kw[b:b + 1], cc[b:b + 1])
            if l == 0:
                k0[b].copy_(kb[0])
                v0[b].copy_(torch.randn(H, N, D, generator=g, device=dev).to(torch.bfloat16))
            del keys, kb
        layers.append(dict(codes=codes_km, nib=nib_km, w=w_km, cc=cc, q=q))
    return layers, k0, v0


def timed_us(torch, fn, n):
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(n):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1000.0 / n  # us per call


def oracle_rows_equal(torch, O, layer, signs, out_ids, rows, bs, H, G, N, tiers, Cn, K, D=128):
    """out_ids [bs,H,K] of one layer against O.retrieve_row on the GPU-encoded index, for the given rows."""
    import numpy as np

    sg = signs.cpu().numpy()
    ok = True
    for r in rows:
        b, h = divmod(r, H)
        ref = O.retrieve_row(layer["q"].view(bs, H, G, D)[b, h].float().cpu().numpy(), sg, O.BF16,
                             layer["codes"][b, h].cpu().numpy(), layer["nib"][b, h][:, :64].cpu().numpy().reshape(N, 16, 4),
                             layer["w"][b, h].float().cpu().numpy(), layer["cc"][b, h].cpu().numpy(), tiers, Cn, K)
        ok = ok and bool(np.array_equal(out_ids.view(bs * H, K)[r].cpu().numpy(), ref))
    return ok


def cfg2_leg(torch, ops, _lib, dev, steps, warmup):
    """BASELINE config 2: batch 1, 32 q / 8 KV heads, 32K keys per head, 2048 candidates, top-512, K/V in HBM: the
    retrieval with the gather of the selected rows out of HBM, as one host call per step."""
    from oracle import pkv_oracle as O

    bs, H, G, N, Cn, K, L = 1, 8, 4, 32768, 2048, 512, 8
    R = bs * H
    signs, centers = ops.srht_signs(dev), ops.mag_centers(dev)
    tiers = [int(math.ceil(N * 0.2 * r)) for r in TIER_RATIOS]
    layers, kd, vd = build_index_layers(torch, ops, dev, bs, H, G, N, L, signs, seed0=20000)
    dst_k = torch.empty(bs, H, K, 128, dtype=torch.bfloat16, device=dev)
    dst_v = torch.empty_like(dst_k)
    out_ids = torch.empty(bs, H, K, dtype=torch.int64, device=dev)
    plan = ops.RetrievePlan(bs, H, G, N, dev, N, Cn, K)
    plan.skip_vote_counts = True
    gather = dict(src_k=kd, src_v=vd, from_host=False, dst_k=dst_k, dst_v=dst_v)

    def step(i, with_gather=True):
        ly = layers[i % L]
        plan.run(ly["q"], signs, centers, ly["cc"], ly["codes"], ly["nib"], ly["w"], 0, N, tiers, Cn, K, out_ids=out_ids,
                 gather=gather if with_gather else None)

    for i in range(warmup):
        step(i)
    us_full = timed_us(torch, step, steps)
    us_nogather = timed_us(torch, lambda i: step(i, False), steps)
    plan.launch_plan = _lib.PLAN_ONE_LAUNCH
    step(0)
    us_full_one = timed_us(torch, step, steps)
    plan.launch_plan = _lib.PLAN_SEPARATE
    step(0)
    torch.cuda.synchronize()
    idx = out_ids.unsqueeze(-1).expand(-1, -1, -1, 128)
    gather_ok = bool(torch.equal(dst_k, torch.gather(kd, 2, idx)) and torch.equal(dst_v, torch.gather(vd, 2, idx)))
    O.build()
    parity = oracle_rows_equal(torch, O, layers[0], signs, out_ids, (0, 3, 5, 7), bs, H, G, N, tiers, Cn, K)
    a_hbm = R * (16 * N + 96 * Cn + 8 * K + 512 * K + 512 * K)  # codes + records + ids + rows read + rows written
    return {"workload": f"BASELINE config 2: batch {bs} x {H} KV heads (GQA {G}), {N} keys/head, collision -> {Cn} "
                        f"candidates, 4-bit rerank -> top-{K}, K/V in HBM (gather of the selected rows out of HBM "
                        f"included), {L} rotating layers",
            "rows": R, "on_gpu_stages_us": round(us_full, 2), "on_gpu_stages_without_the_gather_us": round(us_nogather, 2),
            "on_gpu_stages_one_launch_plan_us": round(us_full_one, 2),
            "algorithmic_bytes_hbm_per_step": a_hbm,
            "hbm_fraction_on_gpu_stages": round(a_hbm / (us_full * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "parity_vs_oracle_rows_checked": 4, "parity_vs_oracle": bool(parity), "gathered_rows_equal_torch_gather": gather_ok}


def cfg4_leg(torch, ops, _lib, dev):
    """BASELINE config 4: batch 1, 32 q / 8 KV heads, 2^20 keys per head whose mean turns by 0.5 degrees per 1K tokens,
    adaptive-k (k in [256, 2048] by benefit mass 0.95): the layer step through the adaptive cache class (one host call
    = pkv_adaptive_decode_step: candidates, dense logits, adaptive k, ragged UVA gather, attention), and beside it the
    fixed-k retrieval of the same index (query prep, scan, select + rerank, top-2048 of the 52429 candidates) as the
    on-GPU figure."""
    import numpy as np

    from oracle import pkv_oracle as O

    bs, H, G, S, L, T = 1, 8, 4, 1 << 20, 2, 40
    res, cache, q = decode_loop(torch, dev, L, bs, S, T, 100, adaptive=True, offload=True, k_range=(256, 2048),
                                threshold=0.95, key_drift=0.5)
    torch.cuda.synchronize()
    l = L - 1
    n_keys, n_cand, _, tiers = cache.retrieval_shape(l)
    sink = cache.sink_size
    # the step's own outputs for this layer are still in place (it ran last): k per row and the ids in benefit order
    ak = cache.last_adaptive_k.cpu().numpy()
    cap_k, k_min, _ = cache._caps(n_cand)
    ids_gpu = cache._topk_ids[:bs * H * cap_k].view(bs * H, cap_k).cpu().numpy()
    z = cache._zones[l]
    sl_end = z.gpu_prefix_rows
    O.build()
    signs = O.srht_signs(42)
    scale = 1.0 / math.sqrt(128)
    ok = True
    for r in (0, 2, 5, 7):
        b, h = divmod(r, H)
        zone = slice(sink, sink + n_keys)
        qrow = q[b, 0, h * G:(h + 1) * G].float().cpu().numpy()
        qh, qn = O.query_prep(qrow, signs, O.BF16)
        lut = O.tier_lut(O.rank_centroids(qh, O.BF16), cache.cluster_key_counts_gpu[l][b, h].cpu().numpy(), tiers)
        cand_ref, _ = O.select_candidates(O.collision_count(cache._codes_km[l][b, h][zone].cpu().numpy(), lut), n_cand)
        sc = O.rerank(cand_ref, cache._nib_km[l][b, h][zone][:, :64].cpu().numpy().reshape(-1, 16, 4),
                      cache._w_km[l][b, h][zone].float().cpu().numpy(), qh, qn)
        vn = cache.value_norm_gpu[l][b, h].cpu().numpy()[cand_ref + sink]
        sl_logits = O.dense_logits(qrow, cache.unified_keys_gpu[l][b, h, :sl_end].float().cpu().numpy(), scale, O.BF16)
        k_ref, ids_ref = O.adaptive_topk(sl_logits, cache._sl_vnorm_cache[l][b, h, :sl_end].cpu().numpy(),
                                         sc * np.float32(scale), vn, cand_ref, 0.95, cap_k)
        k_ref = min(max(k_ref, k_min), cap_k)
        ok = ok and int(ak[b, h]) == k_ref and bool(np.array_equal(ids_gpu[r, :k_ref], ids_ref[:k_ref]))
    # the fixed-k retrieval over the same index: on-GPU stages only, one host call per step
    K = 2048
    plan = ops.RetrievePlan(bs, H, G, cache._codes_km[0].shape[2], dev, n_keys, n_cand, K)
    plan.skip_vote_counts = True
    out_ids = torch.empty(bs, H, K, dtype=torch.int64, device=dev)

    def step(i):
        ll = i % L
        plan.run(q, cache._srht_signs, cache._mag_centers, cache.cluster_key_counts_gpu[ll], cache._codes_km[ll],
                 cache._nib_km[ll], cache._w_km[ll], sink, n_keys, tiers, n_cand, K, out_ids=out_ids)

    for i in range(4):
        step(i)
    us_gpu = timed_us(torch, step, 24)
    plan.launch_plan = _lib.PLAN_ONE_LAUNCH
    step(0)
    us_gpu_one = timed_us(torch, step, 24)
    R = bs * H
    a_hbm = R * (16 * n_keys + 96 * n_cand + 8 * K)
    k_sum = int(ak.sum())
    return {"workload": f"BASELINE config 4: batch {bs} x {H} KV heads (GQA {G}), {S} prompt tokens per head, key mean "
                        f"turning 0.5 degrees per 1K tokens, {n_keys} indexed keys, {n_cand} candidates, adaptive k in "
                        f"[256, 2048] at mass 0.95, K/V in pinned host memory, {L} layers",
            "rows": R, "adaptive_layer_step": res,
            "pcie_bytes_last_step": k_sum * 512, "k_of_last_step_sum_over_rows": k_sum,
            "fixed_k_retrieval_on_gpu_stages_us": round(us_gpu, 2),
            "fixed_k_retrieval_one_launch_plan_us": round(us_gpu_one, 2),
            "fixed_k_retrieval": f"query prep, scan, select + rerank, top-{K} of {n_cand} candidates; no gather",
            "algorithmic_bytes_hbm_per_step": a_hbm,
            "hbm_fraction_on_gpu_stages": round(a_hbm / (us_gpu * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "parity_vs_oracle_rows_checked": 4, "parity_vs_oracle": bool(ok),
            "parity_checked": "adaptive k and the first k ids of the last step, layer " + str(l)}


def encoder_leg(torch, ops, dev, shapes=((8, 8, 65536, "bf16"), (1, 8, 131072, "bf16"), (1, 8, 131072, "f32")), reps=10):
    """The index build of a prefill or refresh (`pkv_encode_append`: keys -> codes, 4-bit records, weights, cluster
    sizes) on synthetic keys, per shape (batch, kv heads, keys per head, key dtype): microseconds per 2^20 key-heads
    and the rate over the bytes a key-head must move (bf16 keys: 256 read + 112 written = 368; fp32 keys: 512 + 112
    = 624)."""
    signs = ops.srht_signs(dev)
    out = []
    for bs, H, N, dt in shapes:
        g = torch.Generator(device=dev).manual_seed(5)
        keys = torch.randn(bs, H, N, 128, generator=g, device=dev)
        keys[..., [7, 31, 64, 101]] *= 10.0
        kb = keys.to(torch.bfloat16) if dt == "bf16" else keys
        nbytes = 368 if dt == "bf16" else 624
        del keys
        _, _, _, cb, k4, kw = ops.alloc_keymajor(bs, H, N, dev)
        cc = torch.zeros(bs, H, 16, 256, dtype=torch.int32, device=dev)
        for _ in range(max(3, (48 << 20) // (bs * H * N))):  # ~6 ms of the same launch first: the shader clock settles
            ops.encode_append(kb, signs, cb, k4, kw, cc)
        us = timed_us(torch, lambda i: ops.encode_append(kb, signs, cb, k4, kw, cc), reps)
        kh = bs * H * N
        out.append({"batch": bs, "kv_heads": H, "keys_per_head": N, "key_dtype": dt, "us_per_launch": round(us, 1),
                    "us_per_2^20_key_heads": round(us / kh * 2**20, 1),
                    f"GBps_over_{nbytes}B_per_key_head": round(kh * nbytes / us / 1e3, 1),
                    "hbm_fraction": round(kh * nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)})
        del kb, cb, k4, kw, cc
    return {"kernel": "pkv_encode_kernel", "bound": "between vector issue (about 225 instructions per key and 16-lane group for bf16 keys, 345 for fp32 keys) and the memory system",
            "shapes": out}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=8, help="distinct layer indexes rotated through")
    ap.add_argument("--context", type=int, default=131072)
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--candidates", type=int, default=4096)
    ap.add_argument("--topk", type=int, default=1024)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", choices=["scan", "copy", "adaptive", "topk", "decode-loop", "model-decode", "encode"],
                    default=None,
                    help="profiling aid: launch only the collision scan, the calibration copy, the adaptive-k stage "
                         "(--candidates scores per row, dense prefix 1600, value norms gathered from a --context table, "
                         "list length --topk) or the exact top-k (--topk of --candidates N(30,20) scores per row) "
                         "--steps times; decode-loop: the polar_cache class itself, --layers layers, "
                         "--context prompt tokens, --steps generated tokens (append + retrieval + gather + attention per "
                         "layer, index refresh and host offload every 1024 tokens); model-decode: the same loop inside a "
                         "random-initialised Qwen3-8B-shaped decoder (config 5: --layers 36 --batch 8 --context 65536 "
                         "--topk 100 --steps 256), end-to-end decode tokens/s; encode: the index build "
                         "(pkv_encode_append) at two shapes")
    ap.add_argument("--no-offload", action="store_true", help="decode-loop: keep K/V in HBM (config 2's mode)")
    ap.add_argument("--host-kv-budget-gib", type=float, default=56.0,
                    help="model-decode / the default run's cfg5 leg: pinned host memory the cache may use for offloaded "
                         "K/V; layers beyond it keep their K/V in HBM (0: no limit, every layer offloads)")
    ap.add_argument("--no-cfg5", action="store_true", help="default run: leave out the config-5 decode leg")
    ap.add_argument("--no-cfg2", action="store_true", help="default run: leave out the config-2 leg (32K keys, K/V in HBM)")
    ap.add_argument("--no-cfg4", action="store_true", help="default run: leave out the config-4 leg (1M keys, adaptive k)")
    ap.add_argument("--adaptive", action="store_true", help="decode-loop: the adaptive-k cache class (config 4's mode)")
    ap.add_argument("--adaptive-k-range", type=int, nargs=2, default=[256, 2048], metavar=("MIN", "MAX"),
                    help="decode-loop --adaptive: clamp of k (config 4: 256 2048; the reference's built-in caps: 100 800)")
    ap.add_argument("--adaptive-threshold", type=float, default=0.95, help="decode-loop --adaptive: mass threshold")
    ap.add_argument("--key-drift", type=float, default=0.0,
                    help="decode-loop: rotate the key mean by this many degrees per 1K tokens (config 4: 0.5)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (rows would shard across GPUs by (batch, kv-head))",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from pariskv_amd import _lib, ops

    dev = "cuda:0"
    torch.cuda.set_device(0)
    bs, H, G, D = args.batch, 8, 4, 128
    N, Cn, K, L = args.context, args.candidates, args.topk, args.layers
    R = bs * H
    lib = _lib.lib()

    if args.only == "model-decode":
        print(json.dumps({"only": "model-decode",
                          **model_decode(torch, dev, L, bs, N, args.steps, K, args.warmup, not args.no_offload,
                                         None if args.host_kv_budget_gib <= 0 else int(args.host_kv_budget_gib * 2**30))}))
        return

    if args.only == "encode":
        print(json.dumps({"only": "encode", **encoder_leg(torch, ops, dev, reps=max(4, args.steps // 4))}))
        return

    if args.only == "decode-loop":
        res, _, _ = decode_loop(torch, dev, L, bs, N, args.steps, K, adaptive=args.adaptive, offload=not args.no_offload,
                                k_range=args.adaptive_k_range, threshold=args.adaptive_threshold, key_drift=args.key_drift)
        print(json.dumps({"only": "decode-loop", **res}))
        return

    if args.only == "adaptive":
        g = torch.Generator(device=dev).manual_seed(0)
        scores = torch.randn(bs, H, Cn, generator=g, device=dev) * 20 + 30
        cand = torch.stack([torch.randperm(N, generator=g, device=dev)[:Cn].sort().values for _ in range(R)]).view(bs, H, Cn)
        vnorm = torch.rand(bs, H, N, generator=g, device=dev) + 0.5
        sl_logits = torch.randn(bs, H, 1600, generator=g, device=dev) * 2
        sl_vnorm = torch.rand(bs, H, 1600, generator=g, device=dev) + 0.5
        for _ in range(args.warmup + args.steps):
            ak, _ = ops.adaptive_topk(sl_logits, sl_vnorm, scores, 1.0 / math.sqrt(D), cand, 0.95, K, value_norm=vnorm)
        torch.cuda.synchronize()
        print(json.dumps({"only": "adaptive", "launches": args.warmup + args.steps, "rows": R, "candidates": Cn,
                          "list": K, "adaptive_k_row0": int(ak.flatten()[0])}))
        return

    if args.only == "topk":
        g = torch.Generator(device=dev).manual_seed(0)
        scores = torch.randn(R, Cn, generator=g, device=dev) * 20 + 30
        for _ in range(args.warmup + args.steps):
            ids = ops.topk_f32(scores, K)
        torch.cuda.synchronize()
        print(json.dumps({"only": "topk", "launches": args.warmup + args.steps, "rows": R, "scores_per_row": Cn, "k": K,
                          "values_equal_torch_topk": bool(torch.equal(torch.gather(scores, 1, ids),
                                                                      torch.topk(scores, K, dim=-1).values))}))
        return

    # ---------------------------------------------------------------- inputs
    signs = ops.srht_signs(dev)
    centers = ops.mag_centers(dev)
    tiers = [int(math.ceil(N * 0.2 * r)) for r in TIER_RATIOS]  # collision_ratio 0.2 for >= 30K keys
    layers = []
    kcpu = torch.empty(bs, H, N, D, dtype=torch.bfloat16, pin_memory=True)
    vcpu = torch.empty(bs, H, N, D, dtype=torch.bfloat16, pin_memory=True)
    for l in range(L):
        codes_km, nib_km, w_km, cb, k4, kw = ops.alloc_keymajor(bs, H, N, dev)
        cc = torch.zeros(bs, H, 16, 256, dtype=torch.int32, device=dev)
        q = torch.empty(bs, 1, H * G, D, dtype=torch.bfloat16, device=dev)
        for b in range(bs):  # independent seed per sequence (and per layer)
            g = torch.Generator(device=dev).manual_seed(1000 * l + b)
            keys = torch.randn(1, H, N, D, generator=g, device=dev, dtype=torch.float32)
            keys[..., [7, 31, 64, 101]] *= 10.0  # four fixed outlier channels
            kb = keys.to(torch.bfloat16)
            qq = keys.mean(dim=2, keepdim=True) + 0.5 * torch.randn(1, H, G, D, generator=g, device=dev)
            q[b, 0] = qq.view(H * G, D).to(torch.bfloat16)
            ops.encode_append(kb, signs, cb[b:b + 1], k4[b:b + 1], kw[b:b + 1], cc[b:b + 1])
            if l == 0:
                kcpu[b].copy_(kb[0])
                vcpu[b].copy_(torch.randn(H, N, D, generator=g, device=dev).to(torch.bfloat16))
            del keys, kb
        layers.append(dict(codes=codes_km, nib=nib_km, w=w_km, cc=cc, q=q))
    dst_k = torch.empty(bs, H, K, D, dtype=torch.bfloat16, device=dev)
    dst_v = torch.empty_like(dst_k)
    out_ids = torch.empty(bs, H, K, dtype=torch.int64, device=dev)
    plan = ops.RetrievePlan(bs, H, G, N, dev, N, Cn, K)
    plan.skip_vote_counts = True  # nothing here looks at the per-key vote counts
    gather = dict(src_k=kcpu, src_v=vcpu, from_host=True, dst_k=dst_k, dst_v=dst_v)
    torch.cuda.synchronize()

    def step(i, with_gather=True):
        ly = layers[i % L]
        plan.run(ly["q"], signs, centers, ly["cc"], ly["codes"], ly["nib"], ly["w"], 0, N, tiers, Cn, K, out_ids=out_ids,
                 gather=gather if with_gather else None)

    def timed(fn, n):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1000.0 / n  # us per call

    # ------------------------------------------------ profiling-only modes
    chunk = ops.pick_chunk_keys(R, N)
    n_chunks = (N + chunk - 1) // chunk
    cnt_stride = (N + 15) // 16 * 16
    cnt_ws = torch.empty(R, cnt_stride, dtype=torch.uint8, device=dev)
    hist_ws = torch.empty(R, n_chunks, 128, dtype=torch.int16, device=dev)
    rowsuf_ws = torch.zeros(R, 128, dtype=torch.int32, device=dev)
    luts = []
    for ly in layers:
        _, _, lut, _ = ops.query_prep_lut(ly["q"], H, signs, ly["cc"], tiers)
        luts.append(lut)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def scan_only(i):
        ly = layers[i % L]
        _lib.check(lib.pkv_collision_scan(ly["codes"].data_ptr(), H * N * 16, N * 16, 16, 1, bs, H, N,
                                          luts[i % L].data_ptr(), cnt_ws.data_ptr(), None, rowsuf_ws.data_ptr(),
                                          hist_ws.data_ptr(), chunk, stream))

    if args.only == "scan":
        for i in range(args.warmup + args.steps):
            scan_only(i)
        torch.cuda.synchronize()
        print(json.dumps({"only": "scan", "launches": args.warmup + args.steps, "bytes_per_launch": R * N * 17}))
        return
    if args.only == "copy":
        nbytes = R * N * 16
        a = layers[0]["codes"]
        b2 = torch.empty_like(a)
        for i in range(args.warmup + args.steps):
            _lib.check(lib.pkv_copy_bytes(layers[i % L]["codes"].data_ptr(), b2.data_ptr(), nbytes, stream))
        torch.cuda.synchronize()
        print(json.dumps({"only": "copy", "launches": args.warmup + args.steps, "read_bytes": nbytes, "write_bytes": nbytes}))
        return

    # ------------------------------------------------------------- timing
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t_wall0 = time.perf_counter()
    us_step = timed(step, args.steps)                       # full retrieval incl. UVA gather  (the metric)
    t_wall = time.perf_counter() - t_wall0
    us_gpu = timed(lambda i: step(i, False), args.steps)    # on-GPU stages only
    plan.launch_plan = _lib.PLAN_ONE_LAUNCH                 # the same with query prep, scan, select + rerank as one launch
    step(0, False)
    us_gpu_one = timed(lambda i: step(i, False), args.steps)
    one_launch_status = int(plan.view("handover_status", N, Cn, K, torch.int32)[0])
    plan.launch_plan = _lib.PLAN_SEPARATE
    step(0, False)

    def step_any_order(i):  # what polar_cache.compute asks for: the same k ids as a set, final sort left out
        ly = layers[i % L]
        plan.run(ly["q"], signs, centers, ly["cc"], ly["codes"], ly["nib"], ly["w"], 0, N, tiers, Cn, K, out_ids=out_ids,
                 any_order=True)

    step_any_order(0)
    us_gpu_any = timed(step_any_order, args.steps)

    def gather_only(i):
        ops.gather_uva(kcpu, vcpu, out_ids, dst_k, dst_v)

    step(0)
    us_gather = timed(gather_only, max(8, args.steps // 4))

    # the attention that consumes the gathered rows (reported beside the metric, not part of it):
    # sink 64 + local 512 dense rows in HBM plus the K gathered rows, GQA 4, one query token
    dense_k = torch.randn(bs, H, 576, D, device=dev).to(torch.bfloat16)
    dense_v = torch.randn(bs, H, 576, D, device=dev).to(torch.bfloat16)
    att = ops.DecodeAttention(bs, H, G, 576 + K, dev)
    att_out = torch.empty(bs, 1, H * G, D, dtype=torch.bfloat16, device=dev)
    att_segs = [(dense_k, dense_v, 0, 64), (dst_k, dst_v, 0, K), (dense_k, dense_v, 64, 512)]
    att_args = [att.c_args(ly["q"], att_segs, out=att_out)[0] for ly in layers]   # validated once: the loop below
    att_q = [C.c_void_p(ly["q"].data_ptr()) for ly in layers]                      # must not be bound by host time

    def attention_only(i):
        a = att_args[i % L]
        lib.pkv_decode_attention(att_q[i % L], _lib.DTYPE_BF16, bs, H, G, a.segments, a.n_segments, None, a.scale, a.out,
                                 a.ws, a.ws_bytes, stream)

    att.run(layers[0]["q"], att_segs, out=att_out)  # checked call first
    us_attn = timed(attention_only, args.steps)

    def step_with_attention(i):  # retrieval + gather + attention from one host call
        ly = layers[i % L]
        plan.run(ly["q"], signs, centers, ly["cc"], ly["codes"], ly["nib"], ly["w"], 0, N, tiers, Cn, K, out_ids=out_ids,
                 gather=gather, attention=(att, att_segs, att_out))

    step_with_attention(0)
    us_step_attn = timed(step_with_attention, args.steps)

    # the same on-GPU stages recorded once into a HIP graph and replayed (a caller that captures its decode step;
    # reported beside the metric): the launches then follow each other without the host in between
    us_gpu_graph = None
    try:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            for i in range(L):
                step(i, False)
            graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for i in range(args.steps):
                    step(i, False)
        torch.cuda.synchronize()
        graph.replay()
        us_gpu_graph = timed(lambda i: graph.replay(), 4) / args.steps
        del graph
    except Exception as exc:  # a build of torch without graph capture: the figure is left out
        print(f"bench.py: graph replay not measured ({exc})", file=sys.stderr)

    # dominant kernel: the collision scan, timed by its own begin/end timestamps
    kus = C.c_float()
    scan_us = []
    for i in range(args.warmup + args.steps):
        ly = layers[i % L]
        _lib.check(lib.pkv_collision_scan_timed(ly["codes"].data_ptr(), H * N * 16, N * 16, 16, 1, bs, H, N,
                                                luts[i % L].data_ptr(), cnt_ws.data_ptr(), cnt_stride,
                                                rowsuf_ws.data_ptr(), hist_ws.data_ptr(), chunk, C.byref(kus), stream))
        if i >= args.warmup:
            scan_us.append(kus.value)
    scan_avg_us = sum(scan_us) / len(scan_us)
    scan_bytes = R * N * 16                           # algorithmic bytes of one launch: 16 B of sign codes per key
    scan_bytes_with_counts = R * N * (16 + 1)         # ... plus the 1 B vote count it writes (an intermediate)
    achieved = scan_bytes / (scan_avg_us * 1e-6) / 1e9

    # PCIe yardstick beside the gather: one plain pinned-host -> device copy of the gather's byte count
    # (hipMemcpyAsync through the copy engines), same timing method
    pin_src = torch.empty(R * 512 * K, dtype=torch.uint8, pin_memory=True)
    pin_dst = torch.empty(R * 512 * K, dtype=torch.uint8, device=dev)
    pin_dst.copy_(pin_src, non_blocking=True)
    us_memcpy = timed(lambda i: pin_dst.copy_(pin_src, non_blocking=True), max(8, args.steps // 4))

    # yardstick beside the published peak: a read-only kernel with the scan's access pattern over the same arrays
    sink = torch.zeros(64, dtype=torch.int32, device=dev)
    code_bytes = R * N * 16

    def read_only(i):
        lib.pkv_read_bytes(layers[i % L]["codes"].data_ptr(), code_bytes, sink.data_ptr(), stream)

    read_only(0)
    read_gbps = code_bytes / (timed(read_only, args.steps) * 1e-6) / 1e9

    a_hbm = R * (16 * N + 96 * Cn + 8 * K + 512 * K)  # algorithmic HBM bytes of the whole pipeline, gathered rows written included
    a_hbm_timed = R * (16 * N + 96 * Cn + 8 * K)      # ... of the launches `on_gpu_stages` times (no gather: no rows written)
    a_pcie = R * 512 * K
    default_shape = (bs, N, Cn, K) == (4, 131072, 4096, 1024)
    shape_name = "BASELINE config 3" if default_shape else "config 3's pipeline at another shape"

    result = {
        "metric": "retrieval us/layer/decode-step at 128K ctx; achieved HBM GB/s vs peak",
        "value": round(us_step, 2),
        "unit": "us/layer/decode-step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_step / 1000.0, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8 votes / f32 rerank (bf16 keys)",
        "data": "synthetic",
        "config": {"workload": f"{shape_name}: batch {bs} x {H} KV heads (GQA {G}), head_dim {D}, {N} keys/head, "
                               f"collision -> {Cn} candidates, 4-bit rerank -> top-{K}, KV in pinned host memory "
                               f"(UVA gather), {L} rotating layers",
                   "rows": R, "keys_per_row": N, "candidates": Cn, "topk": K, "collision_ratio": 0.2},
        "stages_us": {"full_retrieval_with_uva_gather": round(us_step, 2), "on_gpu_stages": round(us_gpu, 2),
                      "on_gpu_stages_one_launch_plan": round(us_gpu_one, 2),
                      "on_gpu_stages_ids_in_any_order": round(us_gpu_any, 2),
                      "on_gpu_stages_replayed_from_a_hip_graph": None if us_gpu_graph is None else round(us_gpu_graph, 2),
                      "uva_gather_alone": round(us_gather, 2),
                      "decode_attention_over_gathered_set": round(us_attn, 2),
                      "full_step_plus_attention_one_host_call": round(us_step_attn, 2)},
        "hbm_fraction_on_gpu_stages": round(a_hbm / (us_gpu * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "hbm_fraction_on_gpu_stages_counting_only_bytes_the_timed_launches_move": round(
            a_hbm_timed / (us_gpu * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "algorithmic_bytes": {"hbm_per_step": a_hbm, "hbm_per_step_without_the_gathered_rows": a_hbm_timed,
                              "pcie_per_step": a_pcie},
        "streaming_read_GBps_same_arrays": round(read_gbps, 1),
        "pcie_GBps_gather": round(a_pcie / (us_gather * 1e-6) / 1e9, 2),
        "pcie_GBps_plain_memcpy_same_bytes": round(a_pcie / (us_memcpy * 1e-6) / 1e9, 2),
        "roofline": {"kernel": SCAN_KERNEL, "bound": "hbm", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": SCAN_TRAFFIC_BYTES if default_shape else None,
                     "traffic_source": ("constant from " + SCAN_TRAFFIC_SOURCE + " (rocprofv3 --pmc FETCH_SIZE / "
                                        "WRITE_SIZE of this command), not measured in this run") if default_shape
                                       else "not measured at this shape",
                     "bytes_per_launch": scan_bytes, "bytes_per_key": 16,
                     "avg_launch_us": round(scan_avg_us, 2),
                     "avg_launch_us_source": "begin/end timestamps of each dispatch (hipExtLaunchKernelGGL events); "
                                             "the rocprofv3 --kernel-trace average in profiles/ is the cross-check",
                     "GBps_counting_the_1B_vote_count_written": round(
                         scan_bytes_with_counts / (scan_avg_us * 1e-6) / 1e9, 1)},
        "wall_s_timed_region": round(t_wall, 4),
        "one_launch_plan_handover_status": one_launch_status,
    }

    if args.no_cpu_baseline:  # still check a few rows of the benchmarked GPU path against the oracle
        import numpy as np

        from oracle import pkv_oracle as O

        O.build()
        ly, sg = layers[0], signs.cpu().numpy()
        step(0)
        torch.cuda.synchronize()
        ok = True
        for r in (0, 1, R // 2, R - 1):
            b, h = divmod(r, H)
            ref = O.retrieve_row(ly["q"].view(bs, H, G, D)[b, h].float().cpu().numpy(), sg, O.BF16,
                                 ly["codes"][b, h].cpu().numpy(), ly["nib"][b, h].cpu().numpy().reshape(N, 16, 4),
                                 ly["w"][b, h].float().cpu().numpy(), ly["cc"][b, h].cpu().numpy(), tiers, Cn, K)
            ok = ok and np.array_equal(out_ids.view(R, K)[r].cpu().numpy(), ref)
        result["parity_vs_oracle_on_bench_workload"] = bool(ok)
        result["parity_rows_checked"] = 4

    # ------------------------------------------------------- CPU baseline
    if not args.no_cpu_baseline:
        import numpy as np

        from oracle import pkv_oracle as O  # the checker, timed here as the reported CPU baseline only

        O.build()
        ly = layers[0]
        rows = list(range(R))
        host = []
        for r in rows:
            b, h = divmod(r, H)
            host.append(dict(
                q=ly["q"].view(bs, H, G, D)[b, h].float().cpu().numpy(),
                codes=ly["codes"][b, h].cpu().numpy(), nib=ly["nib"][b, h].cpu().numpy().reshape(N, 16, 4),
                w=ly["w"][b, h].float().cpu().numpy(), cc=ly["cc"][b, h].cpu().numpy(),
                k=kcpu[b, h].view(torch.int16).numpy(), v=vcpu[b, h].view(torch.int16).numpy()))
        sg = signs.cpu().numpy()

        def cpu_layer_step():
            outs = []
            for hst in host:
                ids = O.retrieve_row(hst["q"], sg, O.BF16, hst["codes"], hst["nib"], hst["w"], hst["cc"], tiers, Cn, K)
                O.gather_rows(hst["k"], ids)
                O.gather_rows(hst["v"], ids)
                outs.append(ids)
            return outs

        ref_ids = cpu_layer_step()  # warm-up, and a parity check of the benchmarked GPU path on the real workload
        step(0)
        torch.cuda.synchronize()
        gpu_ids = out_ids.view(R, K).cpu().numpy()
        parity = all(np.array_equal(gpu_ids[r], ref_ids[r]) for r in rows)
        times = []
        t_end = time.perf_counter() + 25.0
        while len(times) < 20 and (time.perf_counter() < t_end or len(times) < 3):
            t0 = time.perf_counter()
            cpu_layer_step()
            times.append(time.perf_counter() - t0)
        times.sort()
        med = times[len(times) // 2]
        # the same math as batched torch ops on the host (the form the reference's own torch code has), at the default
        # intra-op thread count and at one thread (the reference pins torch.set_num_threads(1), polar_cache.py:320-326)
        from oracle import torch_baseline as TB

        tb = dict(q=ly["q"].cpu(), signs=signs.cpu(), cb=ly["codes"].permute(0, 1, 3, 2).contiguous().cpu(),
                  k4=ly["nib"].view(bs, H, N, 16, 4).permute(0, 1, 3, 2, 4).contiguous().cpu(),
                  kw=ly["w"].permute(0, 1, 3, 2).contiguous().cpu(), cc=ly["cc"].cpu())

        def torch_layer_step():
            return TB.retrieve_layer(tb["q"], tb["signs"], tb["cb"], tb["k4"], tb["kw"], tb["cc"], tiers, Cn, K, kcpu, vcpu)[0]

        def time_torch(n_threads, budget_s):
            torch.set_num_threads(n_threads)
            ids = torch_layer_step()  # warm-up
            ts = []
            t_end = time.perf_counter() + budget_s
            while len(ts) < 20 and (time.perf_counter() < t_end or len(ts) < 3):
                t0 = time.perf_counter()
                torch_layer_step()
                ts.append(time.perf_counter() - t0)
            ts.sort()
            return ts[len(ts) // 2], len(ts), ids

        default_threads = torch.get_num_threads()
        t_def, n_def, tids = time_torch(default_threads, 10.0)
        t_one, n_one, _ = time_torch(1, 12.0)
        torch.set_num_threads(default_threads)
        overlap = sum(len(np.intersect1d(tids.view(R, K)[r].numpy(), ref_ids[r])) for r in rows) / float(R * K)
        # the gather alone by the reference's own host code (cache_hub/gather/gather_cpu.cpp, built into oracle/_ref)
        from oracle import build_ref

        ref_gather = None
        ref_mod = build_ref.load()
        if ref_mod is not None:
            gids = torch.from_numpy(np.stack(ref_ids)).view(bs, H, K)
            gk, gv = torch.empty(bs, H, K, D, dtype=kcpu.dtype), torch.empty(bs, H, K, D, dtype=kcpu.dtype)

            def ref_gather_step():
                ref_mod.gather_kv_out_cpu(kcpu, gids, gk)
                ref_mod.gather_kv_out_cpu(vcpu, gids, gv)

            ref_gather = {"kind": "reference", "bytes": 2 * R * K * D * 2}
            for name, nt in (("default_threads", default_threads), ("one_thread", 1)):
                torch.set_num_threads(nt)
                ref_gather_step()
                ts = []
                for _ in range(20):
                    t0 = time.perf_counter()
                    ref_gather_step()
                    ts.append(time.perf_counter() - t0)
                ts.sort()
                ref_gather[name] = {"value_us": round(ts[10] * 1e6, 1), "threads": nt}
            torch.set_num_threads(default_threads)
            step(0)  # the GPU's rows of the same layer and ids, gathered over PCIe
            torch.cuda.synchronize()
            ref_gather["rows_equal_the_uva_gather"] = bool(
                parity and torch.equal(gk.view(torch.int16), dst_k.cpu().view(torch.int16)) and
                torch.equal(gv.view(torch.int16), dst_v.cpu().view(torch.int16)))
        result["cpu_baseline"] = {"value": round(med * 1e6, 1), "unit": "us/layer/decode-step", "cores": 1, "kind": "port",
                                  "sample": f"all {R} rows of one layer at the full workload (C oracle, single thread, "
                                            f"host gather included), median of {len(times)} repetitions",
                                  "host_cpus": os.cpu_count(),
                                  "host_gather_alone_by_the_reference_build": ref_gather,
                                  "torch_cpu_default_threads": {"value": round(t_def * 1e6, 1), "threads": default_threads,
                                                                "repetitions": n_def},
                                  "torch_cpu_one_thread": {"value": round(t_one * 1e6, 1), "threads": 1,
                                                           "repetitions": n_one},
                                  "torch_cpu_sample": f"the same {R} rows as batched torch ops on the reference's "
                                                      f"subspace-major tensors, in the form of the reference's torch "
                                                      f"fallback code (oracle/torch_baseline.py; a timing yardstick, "
                                                      f"not a parity target: its ties and bf16 matmul are torch's), "
                                                      f"host gather included, median; final ids overlap with the C "
                                                      f"oracle's: {overlap:.4f}"}
        result["parity_vs_oracle_on_bench_workload"] = bool(parity)

    # ------------------- the other configs' shapes (objects beside the headline; a failure costs only its own object)
    del layers, luts, kcpu, vcpu, dst_k, dst_v, cnt_ws, hist_ws, plan, gather
    if not args.no_cpu_baseline:
        del host, tb
    import gc

    gc.collect()
    torch.cuda.empty_cache()

    def leg(name, fn):
        try:
            result[name] = fn()
        except Exception as e:  # e.g. an allocation the box cannot satisfy
            result[name] = {"error": f"{type(e).__name__}: {e}"[:400]}
        gc.collect()
        torch.cuda.empty_cache()

    leg("encoder", lambda: encoder_leg(torch, ops, dev))
    if not args.no_cfg2:
        leg("cfg2", lambda: cfg2_leg(torch, ops, _lib, dev, args.steps, args.warmup))
    if not args.no_cfg4:
        leg("cfg4", lambda: cfg4_leg(torch, ops, _lib, dev))
    # config 5: end-to-end decode tokens/s
    if not args.no_cfg5:
        def cfg5():
            r = model_decode(torch, dev, 36, 8, 65536, 256, 100, 8, True, int(args.host_kv_budget_gib * 2**30)
                             if args.host_kv_budget_gib > 0 else None)
            pl = r["placement"]
            r["headline"] = (f"decode_tokens_per_s with {pl['host_layers']} of 36 layers' K/V offloaded to pinned host "
                             f"memory and {pl['hbm_layers']} resident in HBM (the box pins at most ~65 GiB; the "
                             f"reference's enable_offload would put all 36 on the host)")
            if pl["hbm_layers"] > 0:
                # the same loop with every layer offloaded, at as many layers as the host budget holds: its time per
                # layer is what a 36-layer all-offload run would show on a box that can pin the whole store
                gc.collect()
                torch.cuda.empty_cache()
                n_l = pl["host_layers"] - pl["host_layers"] % 4
                a = model_decode(torch, dev, n_l, 8, 65536, 136, 100, 8, True, None)
                r["every_layer_offloaded"] = {"layers": n_l, "us_per_layer": a["us_per_layer"],
                                              "ms_per_token": a["ms_per_token"],
                                              "decode_tokens_per_s_at_that_many_layers": a["decode_tokens_per_s"],
                                              "host_pinned_GiB": a["placement"]["host_pinned_GiB"],
                                              "hbm_layers": a["placement"]["hbm_layers"]}
            # and with no offload at all: 72 GiB of K/V beside 22 GB of index and 16 GB of weights fit the 288 GB of HBM
            gc.collect()
            torch.cuda.empty_cache()
            try:
                h = model_decode(torch, dev, 36, 8, 65536, 136, 100, 8, False, None)
                r["kv_resident_in_hbm"] = {"decode_tokens_per_s": h["decode_tokens_per_s"], "ms_per_token": h["ms_per_token"],
                                           "us_per_layer": h["us_per_layer"], "hbm_kv_GiB": h["placement"]["hbm_kv_GiB"]}
            except Exception as e:
                r["kv_resident_in_hbm"] = {"error": f"{type(e).__name__}: {e}"[:300]}
            return r

        leg("cfg5", cfg5)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
