"""PolarANN KV cache with collision retrieval + 4-bit rerank, on the HIP kernels.

Same constructor and methods as the reference's ``cache_hub/polar_cache.py``
(``polar_cache.__init__`` :103-128, ``prefill_update_kv_cache`` :379,
``decode_update_kv_cache`` :827, ``compute`` :1002, ``sync`` :1310) so it drops in
under ``attn_hub/polar_attn.py``.  What differs inside:

* metadata is stored key-major (``ops.alloc_keymajor``); ``codebook_gpu``,
  ``key_4bit_packed_gpu`` and ``key_block_weight_gpu`` are reference-shaped views of it;
* one decode step's retrieval is a single ``pkv_retrieve`` call (6 launches) that
  also gathers the selected K/V rows straight behind the dense prefix, so no
  ``torch.cat`` / ``torch.gather`` of K/V happens per step;
* zone counters are per layer (see ``zones.py``);
* the offload copy is ordered by stream events, not a host-blocking synchronize;
* K/V placement is per layer: with ``host_kv_budget_bytes`` the first layers keep their retrieval-zone K/V in pinned
  host memory up to that many bytes and the remaining layers keep theirs in HBM (the reference has one global
  ``enable_offload``, :213-237, and fails when the host cannot pin the whole store).
"""
from __future__ import annotations

import json
import math
import os
from typing import Optional

import torch

from .. import ops, ranges
from .cache import KV_Cache
from .zones import LayerZones

USE_RABITQ_RERANK = True
DEFAULT_SRHT_ROUNDS = 1


def _sign_codebook_ok(path: Optional[str], d: int):
    """Read the codebook config (polar_cache.py:152-160) and make sure it is the sign enumeration."""
    if path is None:
        return 8, 1, 256
    try:
        with open(path, "r") as f:
            cb = json.load(f)
        cfg = cb["config"]
        m, k_r, k_omega = cfg["m"], cfg["K_r"], cfg["K_omega"]
    except (FileNotFoundError, KeyError, json.JSONDecodeError) as e:
        raise ValueError(f"Cannot read codebook parameters: {e}")
    if cfg.get("d", d) != d or m != 8 or k_r != 1 or k_omega != 256:
        raise ValueError(f"Codebook parameter mismatch! only d=128, m=8, K_r=1, K_omega=256 is built; got {cfg}")
    signs = cb.get("angular_signs")
    if signs is not None:
        for c in (0, 1, 2, 77, 128, 255):
            if [1 if (c >> j) & 1 else -1 for j in range(8)] != [1 if v >= 0 else -1 for v in signs[c]]:
                raise ValueError("only the sign-enumeration codebook (centroid id = sign bit pattern) is supported")
    return m, k_r, k_omega


class polar_cache(KV_Cache):

    def __init__(self, valid_start, layer_num: int, batch_size: int, max_length: int, num_key_value_heads: int,
                 num_heads: int, head_dim: int, dtype: torch.dtype, layer_mapping: dict, max_new_length: int,
                 sink_size: int, local_size: int, core: int = 0, nprobe: int = 0, cache_unit_size: int = 0,
                 cache_cluster_num: int = 0, num_gpus: int = 1, model_size: int = 0,
                 codebook_path: Optional[str] = None, final_topk: int = 100, dynamic_update_interval: int = 512,
                 full_attention_threshold: int = 2000, enable_offload: bool = True,
                 collision_ratio: Optional[float] = None, candidate_ratio: Optional[float] = None,
                 host_kv_budget_bytes=None, offload_engine: str = "dma") -> None:
        super().__init__(layer_num, batch_size, max_length, num_key_value_heads, num_heads, head_dim, dtype,
                         layer_mapping, num_gpus, model_size)
        if head_dim != ops.HEAD_DIM:
            raise ValueError("head_dim must be 128")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("dtype must be bfloat16 or float32")
        self.valid_start = valid_start
        self.sink_size = sink_size
        self.local_size = local_size
        self.steady_size = sink_size + local_size
        self.dynamic_update_interval = dynamic_update_interval if dynamic_update_interval is not None else local_size
        self.group_size = self.num_heads // self.kv_head
        self.batch_groups = self.batch_size * self.kv_head
        self.max_new_length = max_new_length
        self.input_length = self.max_length - max_new_length
        self.FULL_ATTENTION_THRESHOLD = full_attention_threshold
        self.current_seq_len = [0] * layer_num
        self.final_topk = final_topk
        self.enable_offload = enable_offload
        if offload_engine not in ("dma", "kernel"):
            raise ValueError("offload_engine must be 'dma' or 'kernel'")
        self._offload_dma = offload_engine == "dma"
        self._collision_ratio = collision_ratio
        self._candidate_ratio = candidate_ratio
        if codebook_path is not None and not os.path.isabs(codebook_path):
            codebook_path = os.path.abspath(codebook_path)
        self.codebook_path = codebook_path
        self.polar_m, self.polar_K_r, self.polar_K_omega = _sign_codebook_ok(codebook_path, head_dim)
        self.polar_B = head_dim // self.polar_m

        self.device = torch.device(list(layer_mapping.values())[0] if layer_mapping else "cuda:0")
        if self.device.type != "cuda":
            raise RuntimeError("GPU required")  # polar_cache.py:40-41
        dev, bs, H, D, I = self.device, batch_size, self.kv_head, head_dim, self.dynamic_update_interval
        self._srht_signs = ops.srht_signs(dev, seed=42)
        self._mag_centers = ops.mag_centers(dev)
        self.unified_kv_capacity = self.input_length + self.max_new_length

        # ---- K/V placement, per layer (the reference: one global switch, polar_cache.py:213-237) ----
        # A layer either offloads its retrieval zone to pinned host memory (GPU rows: [sink | local | update buffer |
        # gathered top-k (transient)]) or keeps every token at its absolute position in HBM.  With enable_offload and no
        # budget every layer offloads, as in the reference.  host_kv_budget_bytes = N: layers offload, in order, while
        # the pinned total stays within N bytes; "auto": until the host refuses to pin more.  The others stay in HBM.
        self.cpu_kv_capacity = max(1, self.unified_kv_capacity - sink_size - local_size)
        self.gpu_kv_capacity = sink_size + local_size + I if enable_offload else self.unified_kv_capacity
        layer_host_bytes = 2 * bs * H * self.cpu_kv_capacity * D * torch.empty((), dtype=dtype).element_size()
        self.unified_keys_cpu = [None] * layer_num if enable_offload else None
        self.unified_values_cpu = [None] * layer_num if enable_offload else None
        self.cpu_valid_end = [0] * layer_num if enable_offload else None
        self._layer_offload = [False] * layer_num
        self._offload_keys_buffer = [None] * layer_num
        self._offload_values_buffer = [None] * layer_num
        if enable_offload:
            self._copy_stream = torch.cuda.Stream(device=dev)
            self._copy_events = [torch.cuda.Event() for _ in range(layer_num)]
            self._offload_inflight = [False] * layer_num
            # prefill staging: two cache-owned [bsz,H,rows,D] K/V pairs used in turn, so that layer l's rows are being
            # copied out while layer l+1's are staged, and HBM holds two layers' worth of staging at most
            self._prefill_stage = [None, None]
            self._prefill_stage_event = [None, None]
            self._prefill_stage_next = 0
            budget = host_kv_budget_bytes
            if budget is not None and budget != "auto":
                budget = int(budget)
            pinned = 0
            for l in range(layer_num):
                if isinstance(budget, int) and pinned + layer_host_bytes > budget:
                    break
                try:
                    kc = ops.alloc_pinned((bs, H, self.cpu_kv_capacity, D), dtype)
                    vc = ops.alloc_pinned((bs, H, self.cpu_kv_capacity, D), dtype)
                except RuntimeError:
                    if budget is None:
                        raise  # the reference's behaviour: the whole store must fit
                    kc = vc = None
                    break
                self.unified_keys_cpu[l], self.unified_values_cpu[l] = kc, vc
                self._layer_offload[l] = True
                pinned += layer_host_bytes
                self._offload_keys_buffer[l] = torch.empty((bs, H, I, D), dtype=dtype, device=dev)
                self._offload_values_buffer[l] = torch.empty((bs, H, I, D), dtype=dtype, device=dev)
        self._gpu_rows = [(sink_size + local_size + I + final_topk) if off else self.unified_kv_capacity
                          for off in self._layer_offload]
        self.unified_keys_gpu = [torch.zeros((bs, H, r, D), dtype=dtype, device=dev) for r in self._gpu_rows]
        self.unified_values_gpu = [torch.zeros((bs, H, r, D), dtype=dtype, device=dev) for r in self._gpu_rows]
        self._zones = [LayerZones(sink_size, local_size, I, off) for off in self._layer_offload]
        n_host = sum(self._layer_offload)
        esz = torch.empty((), dtype=dtype).element_size()
        self.kv_placement = {
            "host_layers": n_host, "hbm_layers": layer_num - n_host,
            "host_pinned_bytes": n_host * layer_host_bytes,
            "hbm_kv_bytes": sum(2 * bs * H * r * D * esz for r in self._gpu_rows),
            "host_kv_budget_bytes": host_kv_budget_bytes,
        }

        # index metadata, addressed by absolute position (polar_cache.py:283-312)
        self.retrieval_zone_capacity = self.unified_kv_capacity
        cap = self.retrieval_zone_capacity
        self._codes_km, self._nib_km, self._w_km = [], [], []
        self.codebook_gpu, self.key_4bit_packed_gpu, self.key_block_weight_gpu = [], [], []
        for _ in range(layer_num):
            c, n, w, cb, k4, kw = ops.alloc_keymajor(bs, H, cap, dev)
            self._codes_km.append(c), self._nib_km.append(n), self._w_km.append(w)
            self.codebook_gpu.append(cb), self.key_4bit_packed_gpu.append(k4), self.key_block_weight_gpu.append(kw)
        self.cluster_key_counts_gpu = [torch.zeros((bs, H, self.polar_B, self.polar_K_omega), dtype=torch.int32, device=dev)
                                       for _ in range(layer_num)]
        self.context = 0
        self._hadamard_scale = 1.0 / math.sqrt(head_dim)
        max_keys = max(1, cap - sink_size)
        max_cand = max(1, math.ceil(max_keys * 0.5))
        self._plan = ops.RetrievePlan(bs, H, self.group_size, cap, dev, max_keys, max_cand, max(1, min(final_topk, max_cand)))
        self._plan.skip_vote_counts = True  # the cache never looks at the per-key vote counts of a step
        self._attn_k = self._attn_v = None  # no-offload mode with few rows: staging buffer of the selected rows
        self._bound = [None] * layer_num  # per layer: (n_keys, ops.BoundStep, topk, out_ids, index of the local segment)
        self._out_ids = torch.empty((bs, H, max(1, final_topk)), dtype=torch.int64, device=dev)
        self._attention = ops.DecodeAttention(bs, H, self.group_size, self.unified_kv_capacity, dev)
        self.last_topk_indices = None  # [bs, H, K] of the most recent retrieval (zone-relative), for inspection

    # ------------------------------------------------------------- helpers
    @property
    def _actual_retrieval_length(self):
        return self._zones[0].encoded

    def _vs(self, batch_idx=0) -> int:
        vs = self.valid_start
        if isinstance(vs, (list, tuple)) or hasattr(vs, "__len__"):
            return int(vs[batch_idx])
        return int(vs)

    def _get_adaptive_ratios(self, retrieval_len):
        """(candidate_ratio, collision_ratio) by retrieval-zone length (polar_cache.py:1113-1124)."""
        if retrieval_len < 5000:
            cand, coll = 0.5, 0.5
        elif retrieval_len < 10000:
            cand, coll = 0.25, 0.3
        elif retrieval_len < 30000:
            cand, coll = 0.2, 0.25
        else:
            cand, coll = 0.1, 0.2
        if self._candidate_ratio is not None:
            cand = self._candidate_ratio
        if self._collision_ratio is not None:
            coll = self._collision_ratio
        return cand, coll

    def _wait_offload(self, layer_idx: int) -> None:
        """Order the current stream after the layer's last host copy (GPU-side wait, no host block)."""
        if self._layer_offload[layer_idx] and self._offload_inflight[layer_idx]:
            torch.cuda.current_stream(self.device).wait_event(self._copy_events[layer_idx])
            self._offload_inflight[layer_idx] = False

    def _offload_rows(self, layer_idx: int, b0: int, b1: int, src_k: torch.Tensor, src_v: torch.Tensor, cpu_row0: int):
        """Async move of [b1-b0, H, n, D] GPU rows into the pinned host zone on the copy stream (polar_cache.py:457-471,
        778-799).  Default engine: one pitched copy-engine command per tensor (the source must then be a staging
        buffer: contiguous blocks per (b, h)); the model's kernels keep the compute units, and with them their speed,
        while it runs.  ``offload_engine="kernel"``: one kernel that writes through the host store's device mapping
        (any source strides; as fast alone, but it stalls the stores of every kernel that runs beside it).  A torch
        ``copy_`` into a slice of the pinned tensor would be a strided device-to-host copy, which torch stages
        through pageable memory and a blocking host loop (4-7 GB/s)."""
        ready = torch.cuda.Event()
        ready.record(torch.cuda.current_stream(self.device))
        self._copy_stream.wait_event(ready)
        ops.offload_rows(src_k, src_v, self.unified_keys_cpu[layer_idx][b0:b1], self.unified_values_cpu[layer_idx][b0:b1],
                         cpu_row0, stream=self._copy_stream, dma=self._offload_dma, dma_flags=ops.OFFLOAD_ONE_COMMAND)
        self._copy_events[layer_idx].record(self._copy_stream)
        src_k.record_stream(self._copy_stream)
        src_v.record_stream(self._copy_stream)
        self._offload_inflight[layer_idx] = True
        return self._copy_events[layer_idx]

    def _stage_prefill_rows(self, k: torch.Tensor, v: torch.Tensor):
        """Private contiguous copies of the [bsz,H,n,D] views k, v in one of the two staging pairs (the reference's
        ``.contiguous()`` copies, polar_cache.py:457-458): the caller may rewrite its tensors as soon as this call
        returns, and the copy engines get whole blocks.  Returns (slot, staged k, staged v)."""
        slot = self._prefill_stage_next
        self._prefill_stage_next ^= 1
        if self._prefill_stage_event[slot] is not None:   # the copy that last read this pair must be over
            torch.cuda.current_stream(self.device).wait_event(self._prefill_stage_event[slot])
        need = k.shape[0] * k.shape[1] * k.shape[2] * k.shape[3]
        pair = self._prefill_stage[slot]
        if pair is None or pair[0].numel() < need:
            self._prefill_stage[slot] = None
            pair = (torch.empty(need, dtype=self.dtype, device=self.device), torch.empty(need, dtype=self.dtype, device=self.device))
            self._prefill_stage[slot] = pair
        sk, sv = pair[0][:need].view(k.shape), pair[1][:need].view(v.shape)
        sk.copy_(k)
        sv.copy_(v)
        return slot, sk, sv

    def release_prefill_staging(self) -> None:
        """Free the prefill staging pairs (two layers' worth of retrieval-zone K/V in HBM) once prefill is over; they
        are allocated again on demand."""
        if self.enable_offload:
            self._copy_stream.synchronize()
            self._prefill_stage = [None, None]
            self._prefill_stage_event = [None, None]

    def _encode(self, layer_idx: int, keys_bhsd: torch.Tensor, b0: int, b1: int, abs0: int) -> None:
        """Encode keys [b1-b0, H, n, D] (any strides) into metadata positions [abs0, abs0+n) and add to the cluster sizes."""
        n = keys_bhsd.shape[2]
        if n == 0:
            return
        sl = slice(abs0, abs0 + n)
        ranges.push("batch_encode+cluster_count")  # the reference's prefill_step1_batch_encode / prefill_step3_cluster_count
        ops.encode_append(keys_bhsd, self._srht_signs, self.codebook_gpu[layer_idx][b0:b1, :, :, sl],
                          self.key_4bit_packed_gpu[layer_idx][b0:b1, :, :, sl], self.key_block_weight_gpu[layer_idx][b0:b1, :, :, sl],
                          self.cluster_key_counts_gpu[layer_idx][b0:b1])
        ranges.pop()

    # ------------------------------------------------------------- prefill
    def prefill_update_kv_cache(self, query_states, key_states, value_states, layer_idx, batch_idx):
        """key/value_states [bsz, S, Hkv, D].  bsz == 1: sample ``batch_idx``; bsz == batch_size: lockstep
        (uniform valid_start).  Returns the states from valid_start on, like the reference (:379-387, :504, :611)."""
        bsz, seq_len, _, _ = key_states.shape
        if bsz == 1:
            b0, vs = int(batch_idx), self._vs(batch_idx)
        else:
            assert bsz == self.batch_size, f"bsz({bsz}) must equal cache batch_size({self.batch_size}) for lockstep mode."
            vs = self._vs(0)
            if hasattr(self.valid_start, "__len__"):
                assert all(int(v) == vs for v in list(self.valid_start)[:bsz]), "lockstep multi-batch requires same valid_start"
            if batch_idx != 0:
                return key_states[:, vs:], value_states[:, vs:]
            b0 = 0
        b1 = b0 + bsz
        assert seq_len <= self.input_length
        z = self._zones[layer_idx]
        n_tok = seq_len - vs
        retrieval, local_len = z.prefill(n_tok)
        self.current_seq_len[layer_idx] = n_tok
        k = key_states[:, vs:].permute(0, 2, 1, 3)   # [bsz, H, n_tok, D] view of the model's layout
        v = value_states[:, vs:].permute(0, 2, 1, 3)
        kg, vg = self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx]
        last = (layer_idx == self.layer_num - 1) and (b1 == self.batch_size)
        if retrieval == 0:  # short prompt: everything stays dense on the GPU (:430-440)
            n = min(n_tok, self._gpu_rows[layer_idx])
            kg[b0:b1, :, :n] = k[:, :, :n].to(self.dtype)
            vg[b0:b1, :, :n] = v[:, :, :n].to(self.dtype)
            self._on_prefill(layer_idx, b0, b1, v, 0, n)
            if last:
                self.context += n
            return key_states[:, vs:], value_states[:, vs:]
        S0, r_end = self.sink_size, self.sink_size + retrieval
        if self._layer_offload[layer_idx]:
            kg[b0:b1, :, :S0] = k[:, :, :S0].to(self.dtype)
            vg[b0:b1, :, :S0] = v[:, :, :S0].to(self.dtype)
            kg[b0:b1, :, S0:S0 + local_len] = k[:, :, r_end:].to(self.dtype)
            vg[b0:b1, :, S0:S0 + local_len] = v[:, :, r_end:].to(self.dtype)
            self._wait_offload(layer_idx)
            slot, stage_k, stage_v = self._stage_prefill_rows(k[:, :, S0:r_end], v[:, :, S0:r_end])
            self._prefill_stage_event[slot] = self._offload_rows(layer_idx, b0, b1, stage_k, stage_v, 0)
            self.cpu_valid_end[layer_idx] = retrieval
            enc_src = stage_k
        else:
            kg[b0:b1, :, :n_tok] = k.to(self.dtype)
            vg[b0:b1, :, :n_tok] = v.to(self.dtype)
            enc_src = kg[b0:b1, :, S0:r_end]
        self.cluster_key_counts_gpu[layer_idx][b0:b1].zero_()  # prefill assigns, refresh accumulates (:493, :775)
        self._encode(layer_idx, enc_src, b0, b1, S0)
        self._on_prefill(layer_idx, b0, b1, v, retrieval, local_len)
        if last:
            self.context += n_tok
        return key_states[:, vs:], value_states[:, vs:]

    # -------------------------------------------------------------- decode
    def fused_append_target(self, layer_idx):
        """(dst_k, dst_v, slot) of the next decoded token of this layer, for a caller whose own launch writes the rows
        (``ops.qk_norm_rope(append=...)``) and then calls ``decode_update_kv_cache(..., appended=True)``; None where the
        append does more than the two slot writes (subclasses that keep value norms) or the dtype is not bf16."""
        if type(self)._append is not polar_cache._append or self.dtype != torch.bfloat16:
            return None
        return self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx], self._zones[layer_idx].append_slot()

    def decode_update_kv_cache(self, key_states, value_states, layer_idx, appended: bool = False):
        """Append one token ([bs,1,Hkv,D]); refresh the index when this layer's update buffer fills (:827-881).
        ``appended``: the rows are already at ``fused_append_target(layer_idx)`` (written on this stream)."""
        z = self._zones[layer_idx]
        if self.enable_offload and (self._prefill_stage[0] is not None or self._prefill_stage[1] is not None):
            self.release_prefill_staging()  # prefill is over: its staging pairs (two layers of K/V) go back to the allocator
        slot = z.append_slot()
        if not appended:
            if key_states.dtype != self.dtype or value_states.dtype != self.dtype:
                key_states, value_states = key_states.to(self.dtype), value_states.to(self.dtype)
            self._append(layer_idx, slot, key_states, value_states)
        refresh = z.appended()
        self.current_seq_len[layer_idx] = z.seq_len
        if layer_idx == 0:
            self.context += 1
        if refresh is not None:
            with ranges.span("update_polar_index"):  # the reference's (commented-out) range, polar_cache_adaptivek_varlen.py:1214
                self._update_polar_index(layer_idx, refresh)
        return None, None

    def _update_polar_index(self, layer_idx: int, r) -> None:
        """Move the oldest ``interval`` tokens of local ++ buffer into the retrieval zone (:743-821)."""
        kg, vg = self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx]
        n, S0 = r.n_new, self.sink_size
        bs = self.batch_size
        self._encode(layer_idx, kg[:, :, r.gpu_row0:r.gpu_row0 + n], 0, bs, r.encode_abs0)
        self._on_refresh(layer_idx, r)
        if not self._layer_offload[layer_idx]:
            return
        self._wait_offload(layer_idx)  # staging buffers are free again
        sk, sv = self._offload_keys_buffer[layer_idx][:, :, :n], self._offload_values_buffer[layer_idx][:, :, :n]
        sk.copy_(kg[:, :, S0:S0 + n])
        sv.copy_(vg[:, :, S0:S0 + n])
        self._offload_rows(layer_idx, 0, bs, sk, sv, r.cpu_row0)
        self.cpu_valid_end[layer_idx] = r.cpu_row0 + n
        # slide the window: rows [sink+n, sink+local+n) -> [sink, sink+local)
        L = self.local_size
        if n < L:
            kg[:, :, S0:S0 + L] = kg[:, :, S0 + n:S0 + n + L].clone()
            vg[:, :, S0:S0 + L] = vg[:, :, S0 + n:S0 + n + L].clone()
        else:
            kg[:, :, S0:S0 + L] = kg[:, :, S0 + n:S0 + n + L]
            vg[:, :, S0:S0 + L] = vg[:, :, S0 + n:S0 + n + L]

    # hooks for subclasses that keep more per-token state (value norms of the adaptive-k variant)
    def _on_prefill(self, layer_idx, b0, b1, values_bhsd, retrieval, local_len):
        pass

    def _append(self, layer_idx, slot, key_states, value_states):
        ops.append_kv(key_states, value_states, self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx], slot)

    def _on_refresh(self, layer_idx, r):
        pass

    # -------------------------------------------------------------- compute
    def get_region_indices(self, layer_idx, device=None):
        """Region summary (reference :645-684), from the per-layer counters."""
        z = self._zones[layer_idx]
        device = device or self.device
        sink_n = min(self.sink_size, z.seq_len)
        return {
            "sink_indices": torch.arange(0, sink_n, device=device, dtype=torch.long),
            "local_indices": torch.arange(z.local_start, z.seq_len, device=device, dtype=torch.long),
            "retrieval_start": self.sink_size,
            "retrieval_length": z.encoded,
            "total_len": z.seq_len,
            "local_len": z.dense_tail_len,
        }

    def _compute_local_start(self, layer_idx=0):
        return self._zones[layer_idx].local_start

    def _attend(self, queries, segments):
        """softmax(q k^T / sqrt(D)) v over the attended set (:1097-1105).  queries [bs,1,Hq,D]; segments: list of
        (k, v, row0, n_rows) runs of [bs,Hkv,rows,D] tensors, read in place by the HIP decode-attention kernel."""
        return self._attention.run(queries, [s for s in segments if s[3] > 0])

    def _full_kv(self, layer_idx):
        """Dense fallback: every stored token (reference _get_full_kv_for_attention :701-737)."""
        z = self._zones[layer_idx]
        kg, vg = self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx]
        if not self._layer_offload[layer_idx]:
            return kg[:, :, :z.seq_len], vg[:, :, :z.seq_len]
        n = z.gpu_prefix_rows
        if z.encoded == 0:
            return kg[:, :, :n], vg[:, :, :n]
        self._copy_stream.synchronize()  # the host reads below must see what the copy stream wrote (:707)
        self._offload_inflight[layer_idx] = False
        rk = self.unified_keys_cpu[layer_idx][:, :, :z.encoded].to(self.device, non_blocking=True)
        rv = self.unified_values_cpu[layer_idx][:, :, :z.encoded].to(self.device, non_blocking=True)
        return torch.cat([kg[:, :, :n], rk], dim=2), torch.cat([vg[:, :, :n], rv], dim=2)

    def retrieval_shape(self, layer_idx):
        """(n_keys, n_cand, k, tier_counts) the next retrieval of this layer will use."""
        z = self._zones[layer_idx]
        n_keys = self.cpu_valid_end[layer_idx] if self._layer_offload[layer_idx] else z.encoded
        cand_ratio, coll_ratio = self._get_adaptive_ratios(n_keys)
        n_cand = min(n_keys, max(1, int(math.ceil(n_keys * cand_ratio))))        # :1239-1240
        k = min(self.final_topk, n_cand)                                          # :1300
        tiers = [int(math.ceil(n_keys * coll_ratio * r)) for r in ops.TIER_RATIOS]  # :1221-1222
        return n_keys, n_cand, k, tiers

    def query_table_target(self, layer_idx):
        """The bound step whose retrieval the next ``compute`` of this layer will launch, for callers that build the
        retrieval's vote table in the launch that produces the queries (``ops.qk_norm_rope(table_for=...)``, called
        before ``decode_update_kv_cache``); None where that launch would not use it: no step bound yet for the
        current index, the coming token refreshes the index (cluster sizes and tier counts change), or the step
        will take the dense branch."""
        z = self._zones[layer_idx]
        step = self._bound_step_of(layer_idx)
        if step is None or self.dtype != torch.bfloat16:
            return None
        n_keys = self.cpu_valid_end[layer_idx] if self._layer_offload[layer_idx] else z.encoded
        if step[0] != n_keys or z.next_append_refreshes():
            return None
        min_total = max(self.FULL_ATTENTION_THRESHOLD, self.sink_size + self.local_size + self.final_topk * 2)
        return step[1] if z.seq_len + 1 >= min_total and n_keys > 0 else None

    def _bound_step_of(self, layer_idx):
        return self._bound[layer_idx]

    def compute(self, queries, layer_idx):
        """Decode attention for one token: [bs,1,Hq,D] -> [bs,1,Hq,D] (:1002-1107)."""
        z = self._zones[layer_idx]
        total = z.seq_len
        offload = self._layer_offload[layer_idx]
        n_keys = self.cpu_valid_end[layer_idx] if offload else z.encoded
        min_total = max(self.FULL_ATTENTION_THRESHOLD, self.sink_size + self.local_size + self.final_topk * 2)
        if total < min_total or n_keys <= 0:
            k, v = self._full_kv(layer_idx)
            if not (k.stride(3) == 1 and k.stride(2) == self.head_dim and v.stride() == k.stride()):
                k, v = k.contiguous(), v.contiguous()
            return self._attend(queries.contiguous(), [(k, v, 0, k.shape[2])])
        q = queries if queries.is_contiguous() else queries.contiguous()
        step = self._bound[layer_idx]
        if step is None or step[0] != n_keys:
            step = self._bind_step(layer_idx, q, n_keys)
        _, bound, topk, out_ids, local_seg = step
        # what moves with every token: where the gathered rows go / how long the dense tail is
        if offload:
            prefix = z.gpu_prefix_rows
            bound.a.dst_row0 = prefix
            bound.segs[0].n_rows = prefix + topk
        else:
            bound.segs[local_seg].row0 = z.local_start
            bound.segs[local_seg].n_rows = z.dense_tail_len
        self._wait_offload(layer_idx)
        self.last_topk_indices = out_ids  # the selected set; its order is fixed but not by score (the sort is left out)
        # retrieval, gather and attention from one host call: the range covers what the reference's
        # "collision_based_topk_batch", gather and attention ranges cover
        if ranges.enabled:
            with ranges.span("collision_topk+gather+attention"):
                return bound.launch(q)
        return bound.launch(q)

    def _bind_step(self, layer_idx, q, n_keys):
        """Build and validate the argument blocks of this layer's decode step; they stay valid until the next index
        refresh changes ``n_keys`` (every pointer in them belongs to a tensor this object keeps)."""
        z = self._zones[layer_idx]
        n_keys, n_cand, topk, tiers = self.retrieval_shape(layer_idx)
        kg, vg = self.unified_keys_gpu[layer_idx], self.unified_values_gpu[layer_idx]
        local_seg = 0
        offload = self._layer_offload[layer_idx]
        if offload:
            prefix = z.gpu_prefix_rows
            gather = dict(src_k=self.unified_keys_cpu[layer_idx], src_v=self.unified_values_cpu[layer_idx], from_host=True,
                          idx_offset=0, dst_k=kg, dst_v=vg, dst_row0=prefix)
            segments = [(kg, vg, 0, prefix + topk)]  # [sink | local + buffer | gathered top-k], one run
        out_ids = self._out_ids[:, :, :topk]
        if not out_ids.is_contiguous():
            out_ids = torch.empty((self.batch_size, self.kv_head, topk), dtype=torch.int64, device=self.device)
        if not offload:
            # The reference gathers sink ++ top-k ++ local rows into a new tensor (:1089-1095).  Sink and local window
            # are always attended in place here.  The selected rows are either a segment addressed through the index
            # list the retrieval just wrote (nothing is copied, one launch fewer) or gathered into a small buffer
            # first: with few (batch, kv-head) rows the extra dependent index load inside the attention kernel costs
            # more than the gather launch (65.2 vs 62.8 us per layer-step at 8 rows x 32K keys; 111.9 vs 113.2 us at
            # 32 rows x 128K keys).
            if self.batch_groups >= 16:
                gather = None
                selected = (kg, vg, self.sink_size, topk, out_ids)
            else:
                if self._attn_k is None or self._attn_k.shape[2] < topk:
                    shape = (self.batch_size, self.kv_head, max(topk, self.final_topk), self.head_dim)
                    self._attn_k = torch.zeros(shape, dtype=self.dtype, device=self.device)
                    self._attn_v = torch.zeros(shape, dtype=self.dtype, device=self.device)
                gather = dict(src_k=kg, src_v=vg, from_host=False, idx_offset=self.sink_size, dst_k=self._attn_k,
                              dst_v=self._attn_v, dst_row0=0)
                selected = (self._attn_k, self._attn_v, 0, topk)
            segments = [(kg, vg, 0, self.sink_size), selected, (kg, vg, z.local_start, z.dense_tail_len)]
            segments = [s for s in segments if s[3] > 0]
            local_seg = len(segments) - 1
        bound = self._plan.bind(q, self._srht_signs, self._mag_centers, self.cluster_key_counts_gpu[layer_idx],
                                self._codes_km[layer_idx], self._nib_km[layer_idx], self._w_km[layer_idx], self.sink_size,
                                n_keys, tiers, n_cand, topk, out_ids, gather, self._attention, segments, any_order=True)
        step = (n_keys, bound, topk, out_ids, local_seg)
        self._bound[layer_idx] = step
        return step

    def sync(self, layer_idx, batch_idx):
        """No-op, as in the reference (:1310-1312)."""
        pass
