"""Zone bookkeeping of the PolarANN cache: which token lives where, when the index is refreshed.

Restates the integer logic of the reference's ``cache_hub/polar_cache.py``
(``get_region_indices`` :645-684, ``_compute_local_start`` :686-699,
``decode_update_kv_cache`` :827-881, ``_update_polar_index`` :743-821) as a
per-layer state machine with no tensors, so it can be tested by brute force.

Token order of one sequence:  [ sink | retrieval zone | local window | update buffer ]

* sink:      the first ``sink`` tokens, always dense on the GPU.
* retrieval: encoded (codes / 4-bit / weights) and, in offload mode, stored in pinned host memory.
* local:     the most recent ``local`` tokens before the buffer, dense on the GPU.
* buffer:    up to ``interval`` newest tokens; when it fills, the oldest ``interval`` tokens of
             local ++ buffer move into the retrieval zone (encode + offload) and the window slides.

One deliberate difference from the reference: every layer keeps its own counters.  The reference
drives all layers from layer 0's counters (``:843,860-879``), so layers > 0 compute their buffer slot
from a counter layer 0 has already advanced and are refreshed before they have stored the step's
token; for layer 0 (the only layer whose bookkeeping is self-consistent there) both agree.
"""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class Refresh:
    """Work a full update buffer triggers."""
    n_new: int          # tokens moving into the retrieval zone
    encode_abs0: int    # absolute position (metadata index) of the first of them
    gpu_row0: int       # GPU row of the first of them (offload layout) / == encode_abs0 (no offload)
    cpu_row0: int       # host row they are offloaded to (offload only)


@dataclass
class LayerZones:
    sink: int
    local: int
    interval: int
    offload: bool
    seq_len: int = 0       # tokens stored for this layer (current_seq_len[layer])
    encoded: int = 0       # tokens in the retrieval zone (_actual_retrieval_length)
    buffered: int = 0      # tokens in the update buffer

    @property
    def steady(self) -> int:
        return self.sink + self.local

    # ---------------------------------------------------------------- prefill
    def prefill(self, n_tokens: int):
        """n_tokens = seq_len - valid_start.  Returns (retrieval_len, local_len) of the partition
        [sink | retrieval | local] (polar_cache.py:513-521)."""
        retrieval = max(0, n_tokens - self.local - self.sink)
        self.seq_len = n_tokens
        self.encoded = retrieval
        self.buffered = 0
        local_len = n_tokens - self.sink - retrieval if retrieval > 0 else max(0, n_tokens - self.sink)
        return retrieval, local_len

    # ----------------------------------------------------------------- decode
    def append_slot(self) -> int:
        """Row (offload: GPU buffer row; else absolute position) the next decoded token is written to."""
        if not self.offload:
            return self.seq_len
        if self.seq_len < self.steady:
            return self.seq_len                      # still filling [sink | local]
        return self.steady + self.buffered           # [sink | local | update buffer]

    def appended(self):
        """Account for one decoded token; returns a Refresh when the buffer just filled, else None."""
        in_buffer = self.seq_len >= self.steady
        self.seq_len += 1
        if not in_buffer:
            return None
        self.buffered += 1
        if self.buffered < self.interval:
            return None
        n = self.interval
        abs0 = self.sink + self.encoded
        r = Refresh(n_new=n, encode_abs0=abs0, gpu_row0=self.sink if self.offload else abs0, cpu_row0=self.encoded)
        self.encoded += n
        self.buffered = 0
        return r

    def next_append_refreshes(self) -> bool:
        """Whether the next ``appended()`` will return a Refresh (the token that fills the update buffer)."""
        return self.seq_len >= self.steady and self.buffered + 1 >= self.interval

    # ---------------------------------------------------------------- regions
    @property
    def retrieval_start(self) -> int:
        return self.sink

    @property
    def local_start(self) -> int:
        """Absolute position of the first dense token after the retrieval zone."""
        return min(self.seq_len, self.sink + self.encoded)

    @property
    def dense_tail_len(self) -> int:
        """Tokens after the retrieval zone (local window + buffer), all dense on the GPU."""
        return self.seq_len - self.local_start

    @property
    def gpu_prefix_rows(self) -> int:
        """Offload layout: rows [0, n) of the GPU buffer that hold sink ++ local ++ buffer."""
        return min(self.sink, self.seq_len) + self.dense_tail_len

    def check(self) -> None:
        assert 0 <= self.buffered < max(1, self.interval)
        assert self.seq_len == min(self.sink, self.seq_len) + self.encoded + self.dense_tail_len
        if self.encoded > 0:
            assert self.local <= self.dense_tail_len <= self.local + self.interval
