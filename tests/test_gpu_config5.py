"""BASELINE config 5 at its stated size: random-initialised Qwen3-8B decode (36 layers, 32/8 heads, head_dim 128, bf16),
batch 8, 64K prompt, sink 64 + local 512 + update buffer 1024, K/V placement split between pinned host memory and HBM.

The host of a GPU box pins less than the 72 GiB this config's K/V store needs, so the cache is given a host budget and
keeps the remaining layers' K/V resident in HBM (the reference's one global ``enable_offload`` switch,
cache_hub/polar_cache.py:213-237, cannot run the config there).  Checked: the placement split, finite logits on every
step, the zone counters of every layer after the index refresh that the run crosses, and, for one host-resident and
one HBM-resident layer, the retrieved id set of sampled (batch, kv-head) rows against the CPU oracle evaluated on the
cache's own index.
"""
import math

import numpy as np
import pytest
import torch

from oracle import pkv_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

HOST_BUDGET = 40 << 30   # bytes of pinned host memory the cache may use; the other layers stay in HBM


def test_config5_full_size_decode_with_split_placement():
    from pariskv_amd.cache_hub.polar_cache import polar_cache
    from pariskv_amd.model_hub import QwenConfig, QwenModel

    L, bs, S, T = 36, 8, 65536, 1032     # 1032 decode tokens: the update buffer (1024) fills once and is refreshed
    sink, local, interval, topk = 64, 512, 1024, 100
    cfg = QwenConfig(num_layers=L)
    H, G, D = cfg.num_key_value_heads, cfg.num_heads // cfg.num_key_value_heads, cfg.head_dim
    print(f"config 5: {L} layers x batch {bs} x {S} prompt tokens, host budget {HOST_BUDGET >> 30} GiB", flush=True)
    cache = polar_cache(valid_start=[0] * bs, layer_num=L, batch_size=bs, max_length=S + T + 8, num_key_value_heads=H,
                        num_heads=cfg.num_heads, head_dim=D, dtype=torch.bfloat16, layer_mapping={i: DEV for i in range(L)},
                        max_new_length=T + 8, sink_size=sink, local_size=local, core=1, nprobe=1, cache_unit_size=1,
                        cache_cluster_num=1, num_gpus=1, model_size=8, final_topk=topk, dynamic_update_interval=interval,
                        full_attention_threshold=2000, enable_offload=True, host_kv_budget_bytes=HOST_BUDGET)
    pl = cache.kv_placement
    layer_bytes = 2 * bs * H * (S + T + 8 - sink - local) * D * 2
    assert pl["host_layers"] + pl["hbm_layers"] == L
    assert 1 <= pl["host_layers"] <= HOST_BUDGET // layer_bytes and pl["hbm_layers"] >= 1
    assert pl["host_pinned_bytes"] == pl["host_layers"] * layer_bytes <= HOST_BUDGET
    assert cache._layer_offload == [True] * pl["host_layers"] + [False] * pl["hbm_layers"]
    print(f"placement: {pl}", flush=True)

    g = torch.Generator(device=DEV).manual_seed(0)
    ang = torch.arange(S, device=DEV, dtype=torch.float32) * (0.5 / 1000.0) * (math.pi / 180.0)   # drifting key mean
    for l in range(L):
        k = torch.randn(bs, S, H, D, generator=g, device=DEV, dtype=torch.bfloat16)
        k[..., 0] += ang.cos().to(torch.bfloat16)[None, :, None]
        k[..., 1] += ang.sin().to(torch.bfloat16)[None, :, None]
        k[..., [7, 31, 64, 101]] *= 10.0
        v = torch.randn(bs, S, H, D, generator=g, device=DEV, dtype=torch.bfloat16)
        cache.prefill_update_kv_cache(None, k, v, l, 0)
        del k, v
    torch.cuda.synchronize()
    assert cache.context == S
    model = QwenModel(cfg, cache, device=DEV, max_positions=S + T + 8)

    # record the queries and the selected ids of one host-resident and one HBM-resident layer on chosen steps
    probe_layers = (pl["host_layers"] - 1, L - 1)
    assert cache._layer_offload[probe_layers[0]] and not cache._layer_offload[probe_layers[1]]
    probes, armed = {}, [False]
    inner = cache.compute

    def spy(queries, layer_idx):
        out = inner(queries, layer_idx)
        if armed[0] and layer_idx in probe_layers:
            probes[layer_idx] = (queries.clone(), cache.last_topk_indices.clone(), cache.retrieval_shape(layer_idx))
        return out

    cache.compute = spy
    appended = {l: [] for l in probe_layers}    # the decode tokens' keys of the probe layers, as the model produced them
    inner_update = cache.decode_update_kv_cache

    def spy_update(key_states, value_states, layer_idx, **kw):   # kw: appended=True where the glue wrote the rows itself
        if layer_idx in appended:
            appended[layer_idx].append(key_states.clone())
        return inner_update(key_states, value_states, layer_idx, **kw)

    cache.decode_update_kv_cache = spy_update
    ids = torch.randint(0, cfg.vocab_size, (bs, 1), generator=g, device=DEV)
    finite = torch.ones((), dtype=torch.bool, device=DEV)
    checked_steps = (5, T - 1)           # one before and one after the refresh at token 1024
    signs = O.srht_signs(42)
    for t in range(T):
        armed[0] = t in checked_steps
        logits = model.decode_forward(ids)
        finite &= torch.isfinite(logits).all()
        ids = logits.argmax(dim=-1)
        if not armed[0]:
            continue
        torch.cuda.synchronize()
        assert logits.shape == (bs, 1, cfg.vocab_size) and bool(finite), f"non-finite logits by token {t}"
        for l in probe_layers:
            q, got, (n_keys, n_cand, kk, tiers) = probes[l]
            refreshed = (t + 1) // interval
            assert n_keys == S - sink - local + interval * refreshed and kk == topk
            for b, h in ((0, 0), (bs - 1, H - 1)):
                sl = slice(sink, sink + n_keys)
                ref = O.retrieve_row(q[b, 0, h * G:(h + 1) * G].float().cpu().numpy(), signs, O.BF16,
                                     cache._codes_km[l][b, h, sl].cpu().numpy(),
                                     cache._nib_km[l][b, h, sl].cpu().numpy().reshape(-1, 16, 4),
                                     cache._w_km[l][b, h, sl].float().cpu().numpy(),
                                     cache.cluster_key_counts_gpu[l][b, h].cpu().numpy(), tiers, n_cand, kk)
                assert np.array_equal(np.sort(got[b, h].cpu().numpy()), np.sort(ref)), f"token {t} layer {l} row {(b, h)}"
    torch.cuda.synchronize()
    assert bool(finite)
    # zone counters after the refresh: every layer moved 1024 tokens into its retrieval zone, 8 are in the buffer
    assert cache.context == S + T
    for l in range(L):
        z = cache._zones[l]
        z.check()
        assert z.seq_len == S + T == cache.current_seq_len[l]
        assert z.encoded == S - sink - local + interval and z.buffered == T - interval
        assert z.dense_tail_len == local + z.buffered
        if cache._layer_offload[l]:
            assert cache.cpu_valid_end[l] == z.encoded
    # where the decode tokens' keys ended up.  Host-resident layer: the refresh moved the oldest 1024 tokens of
    # local ++ buffer (512 prompt tokens, then decode tokens 0..511) to host rows [n0, n0 + 1024); decode tokens
    # 512..1023 became the local window (GPU rows sink ..) and 1024.. sit in the update buffer.  HBM-resident layer:
    # every token at its absolute position.
    l_host, l_hbm = probe_layers
    n0 = S - sink - local
    new_host = torch.cat(appended[l_host], dim=1).permute(0, 2, 1, 3)    # [bs, H, T, D]
    new_hbm = torch.cat(appended[l_hbm], dim=1).permute(0, 2, 1, 3)
    half = interval - local
    assert torch.equal(cache.unified_keys_cpu[l_host][:, :, n0 + local:n0 + interval], new_host[:, :, :half].cpu())
    assert torch.equal(cache.unified_keys_gpu[l_host][:, :, sink:sink + local], new_host[:, :, half:interval])
    assert torch.equal(cache.unified_keys_gpu[l_host][:, :, sink + local:sink + local + T - interval], new_host[:, :, interval:])
    assert torch.equal(cache.unified_keys_gpu[l_hbm][:, :, S:S + T], new_hbm)
