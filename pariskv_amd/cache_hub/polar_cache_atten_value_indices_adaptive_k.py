"""Dense-form adaptive-k variant of the retrieval cache (reference:
``cache_hub/polar_cache_atten_value_indices_adaptive_k.py``).

Like :mod:`polar_cache_adaptivek_varlen`, every decode step ranks the candidates of each (batch, kv-head) row by
``exp(logit) * ||v||`` and finds the smallest k whose mass, together with the dense sink/local tokens, reaches
``adaptive_topk_threshold`` of the total.  What differs (reference ``:1298-1589``):

* k is capped by ``adaptive_topk_max_k`` (default 2048, also the size of the gathered-row buffer) and has no lower
  clamp (``:1564-1577``);
* the attended set is dense: every row keeps ``global_k = max over rows of k`` ids of its own benefit order
  (``:1585-1589``, ``:1462-1499``), so rows with a small k still attend to the next-best candidates of their list.
  The reference reads ``global_k`` back to the host to size its tensors; here a one-workgroup kernel broadcasts the
  maximum on the device and the gather and the attention take it from there, so the step has no host synchronisation;
* both storage modes are supported: with ``enable_offload=False`` the K/V rows and the value norms live at their
  absolute positions on the GPU (``:377-381``, ``:1086``, ``:967``) and the selected rows are attended in place through
  the index list.
"""
from __future__ import annotations

import torch

from .. import ops
from .polar_cache import polar_cache as _polar_cache_base
from .polar_cache_adaptivek_varlen import polar_cache as _adaptive_base


class polar_cache(_adaptive_base):
    def __init__(self, valid_start, layer_num, batch_size, max_length, num_key_value_heads, num_heads, head_dim, dtype,
                 layer_mapping, max_new_length, sink_size, local_size, core=0, nprobe=0, cache_unit_size=0,
                 cache_cluster_num=0, num_gpus=1, model_size=0, codebook_path=None, collision_ratio: float = 0.3,
                 candidate_ratio: float = 0.05, final_topk: int = 100, dynamic_update_interval: int = 512,
                 full_attention_threshold: int = 2000, enable_offload: bool = True, enable_recall: bool = False,
                 adaptive_topk_threshold: float = 0.9, adaptive_topk_max_k: int = 2048) -> None:
        # the two ratios are stored (:197-198); the per-step ratios come from the retrieval length (:1825-1845)
        _polar_cache_base.__init__(self, valid_start, layer_num, batch_size, max_length, num_key_value_heads, num_heads,
                                   head_dim, dtype, layer_mapping, max_new_length, sink_size, local_size, core, nprobe,
                                   cache_unit_size, cache_cluster_num, num_gpus, model_size, codebook_path=codebook_path,
                                   final_topk=final_topk, dynamic_update_interval=dynamic_update_interval,
                                   full_attention_threshold=full_attention_threshold, enable_offload=enable_offload)
        self.collision_ratio = collision_ratio
        self.candidate_ratio = candidate_ratio
        self.enable_recall = enable_recall
        self.adaptive_topk_threshold = adaptive_topk_threshold
        self.adaptive_topk_max_k = int(adaptive_topk_max_k) if adaptive_topk_max_k is not None else final_topk  # :201
        self._init_adaptive_state(self.adaptive_topk_max_k, uniform_k=True)

    def _caps(self, cand_len):
        """(topk_cap, k_min, k_max): k in [1, min(adaptive_topk_max_k, cand_len)] (:1564, :1574-1582)."""
        cap = max(1, min(self.adaptive_topk_max_k, cand_len))
        return cap, 1, cap

    # ------------------------------------------------ value-norm bookkeeping
    def _on_prefill(self, layer_idx, b0, b1, values_bhsd, retrieval, local_len):
        if self.enable_offload:
            return super()._on_prefill(layer_idx, b0, b1, values_bhsd, retrieval, local_len)
        # every token at its absolute position (:611-614); the retrieval zone's norms also by position (:634-637)
        S0, n = self.sink_size, values_bhsd.shape[2]
        vn = self._vnorm(values_bhsd)
        self._sl_vnorm_cache[layer_idx][b0:b1, :, :n] = vn
        if retrieval > 0:
            self.value_norm_gpu[layer_idx][b0:b1, :, S0:S0 + retrieval] = vn[:, :, S0:S0 + retrieval]

    def _on_refresh(self, layer_idx, r):
        if self.enable_offload:
            return super()._on_refresh(layer_idx, r)
        a0, n = r.encode_abs0, r.n_new
        self.value_norm_gpu[layer_idx][:, :, a0:a0 + n] = self._sl_vnorm_cache[layer_idx][:, :, a0:a0 + n]  # :967

    # ---------------------------------------------------------------- compute
    def _compute_adaptive_topk(self, query_avg, sink_local_keys, sl_vnorm, all_cand_scores, all_cand_indices, layer_idx,
                               threshold: float = 0.9):
        """The reference's return form (:1508-1589): (adaptive_k [bs,H] int64, topk_indices [bs,H,global_k] int64 in
        descending benefit order, global_k int).  Reads k back to the host; :meth:`compute` does not go through here."""
        adaptive_k, topk_ids, _ = self._adaptive_topk_device(query_avg, sink_local_keys, sl_vnorm, all_cand_scores,
                                                             all_cand_indices, layer_idx, threshold)
        global_k = int(adaptive_k.max().item())
        return adaptive_k, topk_ids[:, :, :global_k].contiguous(), global_k

    def compute(self, queries, layer_idx):
        """Decode attention for one token: [bs,1,Hq,D] -> [bs,1,Hq,D] (reference :1298-1502)."""
        if self.enable_offload:
            return super().compute(queries, layer_idx)  # the fused step, with the broadcast of max k switched on
        z = self._zones[layer_idx]
        total, n_keys = z.seq_len, z.encoded
        min_total = max(self.FULL_ATTENTION_THRESHOLD, self.sink_size + self.local_size + self.final_topk * 2)
        if total < min_total or n_keys <= 0:
            return _polar_cache_base.compute(self, queries, layer_idx)  # dense branch
        q = queries if queries.is_contiguous() else queries.contiguous()
        bs, H, S0 = self.batch_size, self.kv_head, self.sink_size
        n_keys, n_cand, _, tiers = self.retrieval_shape(layer_idx)
        cand, scores = self._plan.run_candidates(q, self._srht_signs, self._mag_centers, self.cluster_key_counts_gpu[layer_idx],
                                                 self._codes_km[layer_idx], self._nib_km[layer_idx], self._w_km[layer_idx],
                                                 S0, n_keys, tiers, n_cand)
        kg, vg = self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx]
        local0, local_len = z.local_start, z.dense_tail_len
        sl = S0 + local_len
        # dense tokens = sink rows ++ local rows, where they lie (:1421-1434 index_selects copies of them)
        logits = self._dense_logits[:, :, :sl]
        ops.dense_logits(q, kg, S0, self._attn_scale, out=logits)
        if local_len > 0:
            ops.dense_logits(q, kg[:, :, local0:], local_len, self._attn_scale, out=logits[:, :, S0:])
        norms = self._sl_vnorm_cache[layer_idx]
        sl_vnorm = torch.cat([norms[:, :, :S0], norms[:, :, local0:local0 + local_len]], dim=2)
        topk_cap, k_min, k_max = self._caps(n_cand)
        adaptive_k, topk_ids = ops.adaptive_topk(logits, sl_vnorm, scores, self._attn_scale, cand,
                                                 float(self.adaptive_topk_threshold), topk_cap,
                                                 value_norm=self.value_norm_gpu[layer_idx], vn_offset=S0, k_min=k_min,
                                                 k_max=k_max)
        self.last_adaptive_k = adaptive_k
        _, row_keys = ops.uniform_k(adaptive_k, row_keys_base=sl)
        # the selected rows are read in place through the index list (the reference gathers copies, :1481-1488); they
        # come last so that the per-row key count cuts inside them
        segments = [(kg, vg, 0, S0), (kg, vg, local0, local_len), (kg, vg, S0, topk_cap, topk_ids)]
        return self._attention.run(q, [s for s in segments if s[3] > 0], row_keys=row_keys)
