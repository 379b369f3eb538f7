"""pkv_retrieve_noalloc (the entry point that allocates nothing) against pkv_retrieve, through the C ABI.

The two share their kernels; what differs is where the intermediates live: a fixed array inside the library instead
of the caller's workspace.  That array keeps the previous call's contents, so the check is made on two calls in a row,
the second on a smaller input, and every output (ids, scores, gathered K/V rows) must equal pkv_retrieve's bit for bit.
The oracle is consulted as well, so that the pair cannot agree on a wrong answer.
"""
import numpy as np
import pytest
import torch

import workloads as W
from oracle import pkv_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _both(ops, w, d, key0, n_keys, tiers, n_cand, k, any_order=False, host_gather=None):
    args = (d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], key0, n_keys,
            tiers, n_cand, k)
    plan = ops.RetrievePlan(w.bs, w.H, w.G, w.N, DEV, w.N, max(n_cand, 1), k)
    res = []
    for noalloc in (False, True):
        ids = torch.full((w.bs, w.H, k), -1, dtype=torch.int64, device=DEV)
        sc = torch.full((w.bs, w.H, k), float("nan"), dtype=torch.float32, device=DEV)
        gather = None
        if host_gather is not None:
            kcpu, vcpu = host_gather
            dk = torch.zeros(w.bs, w.H, k + 2, 128, dtype=torch.bfloat16, device=DEV)
            dv = torch.zeros_like(dk)
            gather = dict(src_k=kcpu, src_v=vcpu, from_host=True, dst_k=dk, dst_v=dv, dst_row0=2)
        if noalloc:
            ops.retrieve_noalloc(*args, ids, out_scores=sc, gather=gather, any_order=any_order)
        else:
            plan.run(*args, out_ids=ids, out_scores=sc, gather=gather, any_order=any_order)
        torch.cuda.synchronize()
        res.append((ids, sc, gather))
    (i0, s0, g0), (i1, s1, g1) = res
    assert torch.equal(i0, i1), "ids differ between pkv_retrieve and pkv_retrieve_noalloc"
    assert torch.equal(s0.view(torch.int32), s1.view(torch.int32)), "scores differ"
    if g0 is not None:
        assert torch.equal(g0["dst_k"], g1["dst_k"]) and torch.equal(g0["dst_v"], g1["dst_v"]), "gathered rows differ"
    return i1


def test_noalloc_equals_retrieve_on_two_calls_in_a_row():
    from pariskv_amd import _lib, ops

    print("no-alloc: cfg2-sized call, then a smaller ragged one", flush=True)
    assert _lib.lib().pkv_retrieve_noalloc_max_bytes() == 32 << 20
    assert _lib.lib().pkv_retrieve_noalloc_prepare() == 0  # the address look-up a caller does during set-up
    big = W.cfg2()                                                                    # 8 rows x 32768 keys, C 2048, K 512
    small = W.make_workload("small", 2, 2, 4, 5000 + 37, 333, 100, O.BF16, 0.5, seed0=5)  # 4 rows, ragged length
    db, ds = W.to_device(big, DEV, torch), W.to_device(small, DEV, torch)
    kcpu = torch.from_numpy(small.keys.reshape(small.bs, small.H, small.N, 128)).to(torch.bfloat16).pin_memory()
    vcpu = torch.from_numpy(small.values.reshape(small.bs, small.H, small.N, 128)).to(torch.bfloat16).pin_memory()

    ids_big = _both(ops, big, db, 0, big.N, big.tiers, big.C, big.K)
    ids_small = _both(ops, small, ds, 0, small.N, small.tiers, small.C, small.K, host_gather=(kcpu, vcpu))
    for w, ids in ((big, ids_big), (small, ids_small)):
        for r in range(w.R):
            b, h = divmod(r, w.H)
            assert np.array_equal(ids[b, h].cpu().numpy(), W.oracle_stages(w, r)["final"]), f"{w.name} row {r} vs the oracle"

    # again the larger shape after the smaller one, ids as a set; then a sub-range whose candidates are all its keys
    _both(ops, big, db, 0, big.N, big.tiers, big.C, big.K, any_order=True)
    _both(ops, small, ds, 64, 2000, O.tier_counts(2000, 0.5), 2000, 64)
    # a row wider than one workgroup sorts (multi-workgroup top-k: its control block must be cleared by the call itself)
    _both(ops, big, db, 0, big.N, big.tiers, 12000, 300)
    _both(ops, big, db, 0, big.N, big.tiers, 9000, 100)


def test_noalloc_rejects_what_it_cannot_hold():
    from pariskv_amd import _lib, ops

    print("no-alloc: limits", flush=True)
    lib = _lib.lib()
    w = W.make_workload("tiny", 1, 1, 4, 4096, 256, 64, O.BF16, 0.5, seed0=9)
    d = W.to_device(w, DEV, torch)
    ids = torch.empty(1, 1, 64, dtype=torch.int64, device=DEV)
    plan = ops.RetrievePlan(1, 1, 4, w.N, DEV, w.N, w.C, w.K)
    a = plan._fill(d["queries"], d["signs"], d["centers"], d["cluster_counts"], d["codes_km"], d["nib_km"], d["w_km"], 0, w.N,
                   w.tiers, w.C, w.K, ids, None, None, False)
    import ctypes as C
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    # too large for the fixed array: only the sizes are inspected before the refusal, nothing is launched
    a.bs, a.n_kv_heads, a.cap, a.n_keys, a.n_cand, a.k = 8, 8, 1 << 20, 1 << 20, 1 << 19, 1024
    assert lib.pkv_retrieve_ws_bytes(64, 1 << 20, 1 << 19, 1024) > lib.pkv_retrieve_noalloc_max_bytes()
    assert lib.pkv_retrieve_noalloc(C.byref(a), stream) == _lib.ENOMEM
    assert b"scratch" in lib.pkv_last_error()
    # candidates-only form is refused
    a.bs, a.n_kv_heads, a.cap, a.n_keys, a.n_cand, a.k = 1, 1, w.N, w.N, w.C, w.K
    a.out_ids = None
    assert lib.pkv_retrieve_noalloc(C.byref(a), stream) == _lib.EINVAL
    a.out_ids = ids.data_ptr()
    assert lib.pkv_retrieve_noalloc(C.byref(a), stream) == 0
    torch.cuda.synchronize()
    assert np.array_equal(ids[0, 0].cpu().numpy(), W.oracle_stages(w, 0)["final"])
