"""Zone bookkeeping (host logic, CPU only): brute-force simulation of where every token lives."""
import pytest

from pariskv_amd.cache_hub.zones import LayerZones


def simulate(sink, local, interval, offload, prefill, steps):
    """Track token ids through the GPU rows / host rows / retrieval zone exactly as polar_cache moves them."""
    z = LayerZones(sink, local, interval, offload)
    retrieval, local_len = z.prefill(prefill)
    gpu = {}        # row -> token id
    host = []       # host rows (offload) -> token id
    encoded = []    # absolute metadata positions -> token id
    if retrieval == 0:
        for t in range(prefill):
            gpu[t] = t
    elif offload:
        for t in range(sink):
            gpu[t] = t
        for i, t in enumerate(range(sink + retrieval, prefill)):
            gpu[sink + i] = t
        host = list(range(sink, sink + retrieval))
        encoded = list(range(sink, sink + retrieval))
    else:
        for t in range(prefill):
            gpu[t] = t
        encoded = list(range(sink, sink + retrieval))
    for step in range(steps):
        tok = prefill + step
        gpu[z.append_slot()] = tok
        predicted = z.next_append_refreshes()
        r = z.appended()
        assert predicted == (r is not None)
        if r is not None:
            moved = [gpu[r.gpu_row0 + i] for i in range(r.n_new)]
            assert r.encode_abs0 == sink + len(encoded)
            encoded += moved
            if offload:
                assert r.cpu_row0 == len(host)
                host += moved
                for i in range(local):  # slide
                    gpu[sink + i] = gpu[sink + r.n_new + i]
        z.check()
        total = tok + 1
        assert z.seq_len == total
        # the attended universe = sink ++ retrieval zone ++ dense tail must be every token exactly once, in order
        if offload:
            dense = [gpu[i] for i in range(z.gpu_prefix_rows)]
            sink_part, tail = dense[:min(sink, total)], dense[min(sink, total):]
            universe = sink_part + host + tail
            assert host == encoded
        else:
            universe = [gpu[i] for i in range(min(sink, total))] + encoded + [gpu[i] for i in range(z.local_start, total)]
        assert universe == list(range(total)), (step, universe[:10])
        # metadata position of retrieval token i is sink + i (absolute addressing)
        assert encoded == list(range(sink, sink + len(encoded)))
        assert z.encoded == len(encoded) and z.dense_tail_len == total - min(sink, total) - len(encoded)
    return z


@pytest.mark.parametrize("offload", [True, False])
@pytest.mark.parametrize("sink,local,interval,prefill", [(4, 16, 8, 100), (4, 16, 16, 100), (4, 8, 16, 64), (2, 16, 8, 10),
                                                          (4, 16, 8, 20), (4, 16, 8, 21), (0, 8, 4, 50), (128, 256, 128, 1000)])
def test_every_token_is_attended_exactly_once(offload, sink, local, interval, prefill):
    z = simulate(sink, local, interval, offload, prefill, steps=5 * interval + 3)
    assert z.encoded % interval == max(0, prefill - sink - local) % interval


def test_matches_reference_region_formula_for_layer0():
    """Reference get_region_indices (polar_cache.py:656-671) for a long prefill with S == input_length."""
    sink, local, I, S = 4, 512, 512, 20480
    z = LayerZones(sink, local, I, True)
    z.prefill(S)
    for t in range(1, 3 * I + 7):
        z.append_slot()
        z.appended()
        total = S + t
        ub = max(0, total - S) % I
        local_end = max(total - ub, sink)
        local_start = max(sink, local_end - local)
        assert z.local_start == local_start
        assert z.encoded == max(0, local_start - sink)
        assert z.dense_tail_len == total - local_start


def test_refresh_slots_match_reference_layer0():
    """Reference decode_update_kv_cache (:835-847): slot = steady + tokens_in_buffer % interval."""
    sink, local, I, S = 4, 16, 8, 100
    z = LayerZones(sink, local, I, True)
    z.prefill(S)
    counter = base = 0
    pending = False
    for t in range(40):
        expect = sink + local + (counter - base) % I
        assert z.append_slot() == expect
        r = z.appended()
        counter += 1
        if pending:
            base, pending = counter - 1, False
        buf = counter - base
        assert (r is not None) == (buf > 0 and buf % I == 0)
        if r is not None:
            pending = True


def test_ranges_are_no_ops_when_switched_off():
    """Range markers cost nothing and need no library unless PARISKV_RANGES=1 is set before the import."""
    import importlib
    import os

    os.environ.pop("PARISKV_RANGES", None)
    from pariskv_amd import ranges

    ranges = importlib.reload(ranges)
    assert ranges.enabled is False
    ranges.push("a")
    ranges.pop()
    with ranges.span("b"):
        pass
