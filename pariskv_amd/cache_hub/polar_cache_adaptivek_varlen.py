"""Adaptive-k variant of the retrieval cache (reference: ``cache_hub/polar_cache_adaptivek_varlen.py``).

Every decode step the number of retrieved tokens is chosen per (batch, kv-head) row: candidates are ranked by
``exp(logit) * ||v||`` and the smallest k whose mass, together with the dense sink/local tokens, reaches
``adaptive_topk_threshold`` of the total is kept (clamped to [min_k, max_k]).  Only ``sum(k)`` K/V rows cross PCIe.

What differs from :class:`polar_cache`:

* two value-norm caches, kept in step with the key/value slots (reference ``:450-483``, ``:1075-1078``,
  ``:1130-1133``, ``:1179``): ``_sl_vnorm_cache [bs,H,gpu_rows]`` for the dense GPU rows and ``value_norm_gpu
  [bs,H,capacity]`` by absolute position for the retrieval zone;
* ``compute`` stops the retrieval after the rerank (all candidates with their scores), runs the adaptive-k
  kernel, gathers each row's own k rows over UVA and attends over ``[sink | local | buffer]`` plus those rows.  The
  reference packs indices and K/V per row for ``flash_attn_varlen_func`` and reads the largest k back to the host
  (``:1597-1670``); here the gathered rows land in a dense ``[bs,H,max_k,128]`` buffer, the gather and the attention
  kernel take the per-row count from device memory, the sink/local rows are attended in place, and the step has no
  host synchronisation.

Offload mode only, like the reference (``:222-226``).
"""
from __future__ import annotations

import math
import os

import torch

from .. import ops, ranges
from .polar_cache import polar_cache as _polar_cache_base


class polar_cache(_polar_cache_base):
    def __init__(self, valid_start, layer_num, batch_size, max_length, num_key_value_heads, num_heads, head_dim, dtype,
                 layer_mapping, max_new_length, sink_size, local_size, core=0, nprobe=0, cache_unit_size=0,
                 cache_cluster_num=0, num_gpus=1, model_size=0, codebook_path=None, collision_ratio: float = 0.3,
                 candidate_ratio: float = 0.05, final_topk: int = 100, dynamic_update_interval: int = 512,
                 full_attention_threshold: int = 2000, enable_offload: bool = True, enable_recall: bool = False,
                 adaptive_topk_threshold: float = 0.85, adaptive_topk_min_k: int = 50,
                 adaptive_topk_max_k_ratio: float = 0.1) -> None:
        assert enable_offload, "the adaptive-k variant only supports enable_offload=True"  # reference :222-226
        # the two ratios are stored like the reference does (:218-219) but, as there, the per-step ratios come from
        # the retrieval length (_get_adaptive_ratios)
        super().__init__(valid_start, layer_num, batch_size, max_length, num_key_value_heads, num_heads, head_dim, dtype,
                         layer_mapping, max_new_length, sink_size, local_size, core, nprobe, cache_unit_size,
                         cache_cluster_num, num_gpus, model_size, codebook_path=codebook_path, final_topk=final_topk,
                         dynamic_update_interval=dynamic_update_interval, full_attention_threshold=full_attention_threshold,
                         enable_offload=True)
        self.collision_ratio = collision_ratio
        self.candidate_ratio = candidate_ratio
        self.enable_recall = enable_recall
        self.adaptive_topk_threshold = adaptive_topk_threshold
        self.adaptive_topk_min_k = max(0, int(adaptive_topk_min_k)) if adaptive_topk_min_k is not None else 0
        r = float(adaptive_topk_max_k_ratio) if adaptive_topk_max_k_ratio is not None else 0.0
        self.adaptive_topk_max_k_ratio = min(1.0, max(0.0, r))
        # the caps the reference actually applies (:255-257): environment overrides with the same names
        self._HARDCODED_MAX_K = int(os.environ.get("ADAPTIVE_TOPK_MAX_K", "800"))
        self._HARDCODED_MIN_K = int(os.environ.get("ADAPTIVE_TOPK_MIN_K", "100"))
        self._init_adaptive_state(self._HARDCODED_MAX_K, uniform_k=False)

    def _init_adaptive_state(self, buffer_cap: int, uniform_k: bool) -> None:
        """Value-norm caches, the gathered-row buffer of ``buffer_cap`` rows and the operands of the fused step that
        all layers share.  ``uniform_k``: every row gathers and attends to max(adaptive_k) ids (the dense form of
        polar_cache_atten_value_indices_adaptive_k.py) instead of its own k."""
        self._adaptive_topk_buffer_cap = buffer_cap
        self._attn_scale = 1.0 / math.sqrt(self.head_dim)
        layer_num = len(self._zones)
        dev, bs, H = self.device, self.batch_size, self.kv_head
        self._sl_vnorm_cache = [torch.zeros((bs, H, self.gpu_kv_capacity), dtype=torch.float32, device=dev)
                                for _ in range(layer_num)]
        # value norm by absolute position: the spare fp32 word of each key's rerank record, so that a candidate's
        # norm is in the HBM line the rerank fetches anyway (the reference keeps a separate [bs,H,cap] tensor)
        self.value_norm_gpu = [ops.record_value_norm_view(self._nib_km[l]) for l in range(layer_num)]
        cap = max(1, buffer_cap)
        self._dense_logits = torch.empty((bs, H, self.gpu_kv_capacity), dtype=torch.float32, device=dev)
        self._adaptive_k = torch.zeros((bs, H), dtype=torch.int64, device=dev)
        self._uniform_k = torch.zeros((bs, H), dtype=torch.int64, device=dev) if uniform_k else None
        self._topk_ids = torch.zeros((bs * H * cap,), dtype=torch.int64, device=dev)
        self._row_keys = torch.zeros((bs, H), dtype=torch.int32, device=dev)
        self._adk_ws = None
        self._adaptive_bound = [None] * layer_num  # per layer: (n_keys, ops.BoundAdaptiveStep, topk_cap)
        self.last_adaptive_k = None  # [bs, H] int64 of the most recent retrieval step
        if self.enable_offload:
            self._topk_k = torch.zeros((bs, H, cap, self.head_dim), dtype=self.dtype, device=dev)
            self._topk_v = torch.zeros((bs, H, cap, self.head_dim), dtype=self.dtype, device=dev)

    # ------------------------------------------------------------ ratios
    def _get_adaptive_ratios(self, retrieval_len):
        """(candidate_ratio, collision_ratio) by retrieval-zone length (reference :2107-2128)."""
        if retrieval_len < 5000:
            return 0.5, 0.5
        if retrieval_len < 10000:
            return 0.25, 0.3
        if retrieval_len < 30000:
            return 0.2, 0.25
        return 0.05, 0.2

    # ------------------------------------------------ value-norm bookkeeping
    def _vnorm(self, values):
        """||v||_2 per token as the reference computes it: in the tensor's dtype, then widened (:680, :756, :1179)."""
        return torch.linalg.vector_norm(values.to(self.dtype), dim=-1).to(torch.float32)

    def _on_prefill(self, layer_idx, b0, b1, values_bhsd, retrieval, local_len):
        S0 = self.sink_size
        sl = self._sl_vnorm_cache[layer_idx]
        if retrieval == 0:  # short prompt: all tokens are dense GPU rows (:680)
            sl[b0:b1, :, :local_len] = self._vnorm(values_bhsd[:, :, :local_len])
            return
        r_end = S0 + retrieval
        sl[b0:b1, :, :S0] = self._vnorm(values_bhsd[:, :, :S0])                              # :704
        sl[b0:b1, :, S0:S0 + local_len] = self._vnorm(values_bhsd[:, :, r_end:r_end + local_len])  # :706
        self.value_norm_gpu[layer_idx][b0:b1, :, S0:r_end] = self._vnorm(values_bhsd[:, :, S0:r_end])  # :753-756

    def _append(self, layer_idx, slot, key_states, value_states):
        """K/V rows and the value norm of the new token (:1179) in one launch."""
        ops.append_kv(key_states, value_states, self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx], slot,
                      vnorm=self._sl_vnorm_cache[layer_idx])

    def _on_refresh(self, layer_idx, r):
        S0, n, L = self.sink_size, r.n_new, self.local_size
        sl = self._sl_vnorm_cache[layer_idx]
        self.value_norm_gpu[layer_idx][:, :, r.encode_abs0:r.encode_abs0 + n] = sl[:, :, S0:S0 + n]  # :1075-1078
        sl[:, :, S0:S0 + L] = sl[:, :, S0 + n:S0 + n + L].clone()                                 # :1130-1133

    # ---------------------------------------------------------------- compute
    def _pack_indices(self, dense_indices, adaptive_k, topk_cap):
        """Dense [bs,H,cap] indices -> packed [sum(k)] in (b, h) row-major order (reference :1817-1832)."""
        V = adaptive_k.numel()
        mask = torch.arange(topk_cap, device=dense_indices.device).unsqueeze(0) < adaptive_k.view(V, 1)
        return dense_indices.contiguous().view(V, topk_cap)[mask]

    def _caps(self, cand_len):
        """(topk_cap, k_min, k_max) for a candidate list of ``cand_len`` (reference :1703-1712, :1759)."""
        effective_max_k = min(self._HARDCODED_MAX_K, cand_len)
        effective_min_k = min(self._HARDCODED_MIN_K, effective_max_k)
        return effective_max_k, max(1, effective_min_k), max(1, effective_max_k)

    def _adaptive_topk_device(self, query_avg, sink_local_keys, sl_vnorm, all_cand_scores, all_cand_indices, layer_idx,
                              threshold):
        """Per-row k and the candidate ids in benefit order, all on the GPU (reference :1684-1759).
        Returns (adaptive_k [bs,H] int64 after the clamp, topk_ids [bs,H,topk_cap] int64, topk_cap)."""
        topk_cap, k_min, k_max = self._caps(all_cand_scores.shape[-1])
        # logits of the dense tokens (:1731); a [bs,H,D] mean query is a query group of one head
        logits_sl = ops.dense_logits(query_avg.contiguous(), sink_local_keys, sink_local_keys.shape[2], self._attn_scale)
        adaptive_k, topk_ids = ops.adaptive_topk(logits_sl, sl_vnorm, all_cand_scores, self._attn_scale, all_cand_indices,
                                                 float(threshold), topk_cap, value_norm=self.value_norm_gpu[layer_idx],
                                                 vn_offset=self.sink_size, k_min=k_min, k_max=k_max)   # clamp: :1759
        return adaptive_k, topk_ids, topk_cap

    def _compute_adaptive_topk(self, query_avg, sink_local_keys, sl_vnorm, all_cand_scores, all_cand_indices, layer_idx,
                               threshold):
        """The reference's return form (:1684-1832): (adaptive_k [bs,H] int64, indices_packed [sum(k)] int64,
        global_k int).  Reads k back to the host; :meth:`compute` does not go through here."""
        adaptive_k, topk_ids, topk_cap = self._adaptive_topk_device(query_avg, sink_local_keys, sl_vnorm, all_cand_scores,
                                                                    all_cand_indices, layer_idx, threshold)
        global_k = int(adaptive_k.max().item())
        return adaptive_k, self._pack_indices(topk_ids, adaptive_k, topk_cap), global_k

    def _bound_step_of(self, layer_idx):
        return self._adaptive_bound[layer_idx]

    def compute(self, queries, layer_idx):
        """Decode attention for one token: [bs,1,Hq,D] -> [bs,1,Hq,D] (reference :1391-1677)."""
        z = self._zones[layer_idx]
        total = z.seq_len
        n_keys = self.cpu_valid_end[layer_idx]
        min_total = max(self.FULL_ATTENTION_THRESHOLD, self.sink_size + self.local_size + self.final_topk * 2)
        if total < min_total or n_keys <= 0:
            return super().compute(queries, layer_idx)  # dense branch
        q = queries if queries.is_contiguous() else queries.contiguous()
        step = self._adaptive_bound[layer_idx]
        if step is None or step[0] != n_keys:
            step = self._bind_adaptive_step(layer_idx, q, n_keys)
        _, bound, _ = step
        # what moves with every token: the dense rows (sink + local + update buffer) grow by one
        sl_end = z.gpu_prefix_rows
        bound.ad.dense_rows = sl_end
        bound.ad.row_keys_base = sl_end
        bound.segs[0].n_rows = sl_end
        self._wait_offload(layer_idx)
        self.last_adaptive_k = self._adaptive_k
        # One host call: candidates + rerank scores -> logits of the dense rows -> adaptive k -> ragged UVA gather (row
        # (b, h) receives its own k rows at the head of its slice of the dense buffer) -> attention.  The reference
        # packs the indices and reads the largest k back to the host to size its launch (:1597-1644); the gather and
        # the attention take the per-row count from device memory instead, so the step never waits for the GPU.
        # The range covers the reference's "collision_based_topk_batch", "adaptive_k0_pre", "adaptive_k1_qk_logits",
        # "adaptive_k2_cuda_kernel", "pack_sink_local", "h2d_gather_kv_packed" and "compute_attention_varlen" (:1483-1771).
        if ranges.enabled:
            with ranges.span("collision_topk+adaptive_k+gather+attention_varlen"):
                return bound.launch(q)
        return bound.launch(q)

    def _bind_adaptive_step(self, layer_idx, q, n_keys):
        """Argument blocks of this layer's step, valid until the next index refresh changes ``n_keys``."""
        z = self._zones[layer_idx]
        n_keys, n_cand, _, tiers = self.retrieval_shape(layer_idx)
        topk_cap, k_min, k_max = self._caps(n_cand)
        kg, vg = self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx]
        sl_end = z.gpu_prefix_rows
        need = ops.adaptive_topk_ws_bytes(self.batch_groups, n_cand, topk_cap)
        if self._adk_ws is None or self._adk_ws.numel() < need:
            self._adk_ws = torch.empty(need, dtype=torch.uint8, device=self.device)
        adaptive = dict(dense_k=kg, dense_rows=sl_end, dense_vnorm=self._sl_vnorm_cache[layer_idx],
                        dense_logits=self._dense_logits, scale=self._attn_scale, value_norm=self.value_norm_gpu[layer_idx],
                        vn_offset=self.sink_size, record_word_offset=ops.RECORD_VALUE_NORM_OFFSET, threshold=self.adaptive_topk_threshold, k_out=topk_cap, k_min=k_min,
                        k_max=k_max, adaptive_k=self._adaptive_k, topk_ids=self._topk_ids, row_keys=self._row_keys,
                        row_keys_base=sl_end, uniform_k=self._uniform_k, ws=self._adk_ws, src_k=self.unified_keys_cpu[layer_idx],
                        src_v=self.unified_values_cpu[layer_idx], dst_k=self._topk_k, dst_v=self._topk_v)
        segments = [(kg, vg, 0, sl_end), (self._topk_k, self._topk_v, 0, topk_cap)]
        bound = self._plan.bind_adaptive(q, self._srht_signs, self._mag_centers, self.cluster_key_counts_gpu[layer_idx],
                                         self._codes_km[layer_idx], self._nib_km[layer_idx], self._w_km[layer_idx],
                                         self.sink_size, n_keys, tiers, n_cand, adaptive, self._attention, segments)
        step = (n_keys, bound, topk_cap)
        self._adaptive_bound[layer_idx] = step
        return step
