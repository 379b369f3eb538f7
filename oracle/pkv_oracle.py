"""ctypes/numpy front end of the CPU oracle (``libpkv_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py`` as the checker / timed CPU
baseline.  The product package never imports this module.

All arrays are numpy, key-major: ``codes [n,16] u8``, ``nib [n,16,4] u8``,
``weight [n,16] f32`` (bf16-representable values).  Helpers at the bottom
convert to the reference's subspace-major tensors
(``cache_hub/polar_cache.py:288-307``).
"""
from __future__ import annotations

import ctypes as C
import math
import os
import subprocess

import numpy as np

F32, BF16 = 0, 1
D, B, M, KW = 128, 16, 8, 256
TIER_RATIOS = (0.05, 0.15, 0.30, 0.50, 0.75, 1.0)  # polar_cache.py:1221

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libpkv_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (idempotent)."""
    src = os.path.join(_HERE, "pkv_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libpkv_oracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.pkv_o_bf16_round.restype = C.c_float
        _lib.pkv_o_bf16_round.argtypes = [C.c_float]
        _lib.pkv_o_expf.restype = C.c_float
        _lib.pkv_o_expf.argtypes = [C.c_float]
        _lib.pkv_o_select_candidates.restype = C.c_int
        _lib.pkv_o_adaptive_topk.restype = C.c_int64
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def bf16_round(x):
    """Round fp32 array to bfloat16 (RNE), returned as fp32 (numpy restatement)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) & 0xFFFF0000).astype(np.uint32)
    return r.view(np.float32).reshape(x.shape)


def mag_constants():
    th = np.zeros(7, np.float32)
    ce = np.zeros(8, np.float32)
    lib().pkv_o_mag_constants(_p(th), _p(ce))
    return th, ce


def fwht128(x):
    x = _f32(x).copy()
    flat = x.reshape(-1, D)
    for i in range(flat.shape[0]):
        row = np.ascontiguousarray(flat[i])
        lib().pkv_o_fwht128(_p(row))
        flat[i] = row
    return flat.reshape(x.shape)


def encode(keys, signs, dtype):
    """keys [n,128] -> (codes [n,16] u8, nib [n,16,4] u8, weight [n,16] f32)."""
    keys = _f32(keys).reshape(-1, D)
    n = keys.shape[0]
    codes = np.zeros((n, B), np.uint8)
    nib = np.zeros((n, B, 4), np.uint8)
    w = np.zeros((n, B), np.float32)
    lib().pkv_o_encode(_p(keys), C.c_int64(n), _p(_f32(signs)), C.c_int(dtype), _p(codes), _p(nib), _p(w))
    return codes, nib, w


def count_cluster_keys(codes, counts=None):
    codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1, B)
    if counts is None:
        counts = np.zeros((B, KW), np.int32)
    assert counts.dtype == np.int32 and counts.flags.c_contiguous
    lib().pkv_o_count_cluster_keys(_p(codes), C.c_int64(codes.shape[0]), _p(counts))
    return counts


def query_prep(q, signs, dtype):
    """q [G,128] -> (qhat [128] f32, qnorm float)."""
    q = _f32(q).reshape(-1, D)
    qhat = np.zeros(D, np.float32)
    qn = np.zeros(1, np.float32)
    lib().pkv_o_query_prep(_p(q), C.c_int(q.shape[0]), _p(_f32(signs)), C.c_int(dtype), _p(qhat), _p(qn))
    return qhat, float(qn[0])


def rank_centroids(qhat, dtype):
    ids = np.zeros((B, KW), np.int64)
    lib().pkv_o_rank_centroids(_p(_f32(qhat)), C.c_int(dtype), _p(ids))
    return ids


def tier_counts(kv_len: int, collision_ratio: float, ratios=TIER_RATIOS):
    """polar_cache.py:1221-1222, evaluated with Python doubles left to right."""
    return [int(math.ceil(kv_len * collision_ratio * r)) for r in ratios]


def tier_lut(sorted_ids, counts, tiers):
    sorted_ids = _i64(sorted_ids).reshape(-1, KW)
    counts = np.ascontiguousarray(counts, dtype=np.int32).reshape(-1, KW)
    n_sub = sorted_ids.shape[0]
    t = np.asarray(tiers, dtype=np.uint32)
    lut = np.zeros((n_sub, KW), np.uint8)
    lib().pkv_o_tier_lut(_p(sorted_ids), _p(counts), C.c_int(n_sub), _p(t), C.c_int(len(t)), _p(lut))
    return lut


def collision_count(codes, lut):
    """codes [n,n_sub] u8 (key-major), lut [n_sub,256] -> cnt [n] i32."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    n, n_sub = codes.shape
    lut = np.ascontiguousarray(lut, dtype=np.uint8)
    cnt = np.zeros(n, np.int32)
    lib().pkv_o_collision_count(_p(codes), C.c_int64(n), C.c_int64(n_sub), C.c_int64(1), C.c_int(n_sub), _p(lut), _p(cnt))
    return cnt


def select_candidates(cnt, k):
    cnt = np.ascontiguousarray(cnt, dtype=np.int32)
    out = np.zeros(k, np.int64)
    theta = lib().pkv_o_select_candidates(_p(cnt), C.c_int64(cnt.shape[0]), C.c_int64(k), _p(out))
    return out, theta


def rerank(cand, nib, weight, qhat, qnorm, centers=None):
    """nib [n,16,4] u8, weight [n,16] f32 (key-major) -> scores [len(cand)] f32."""
    cand = _i64(cand)
    nib = np.ascontiguousarray(nib, dtype=np.uint8)
    weight = _f32(weight)
    if centers is None:
        centers = mag_constants()[1]
    scores = np.zeros(cand.shape[0], np.float32)
    lib().pkv_o_rerank(_p(cand), C.c_int64(cand.shape[0]), _p(nib), C.c_int64(64), C.c_int64(4), _p(weight),
                       C.c_int64(16), C.c_int64(1), _p(_f32(qhat)), C.c_float(qnorm), _p(_f32(centers)), _p(scores))
    return scores


def topk_f32(scores, ids, k):
    scores = _f32(scores)
    n = scores.shape[0]
    ids_c = _i64(ids) if ids is not None else None
    out_ids = np.zeros(k, np.int64)
    out_pos = np.zeros(k, np.int64)
    lib().pkv_o_topk_f32(_p(scores), _p(ids_c), C.c_int64(n), C.c_int64(k), _p(out_ids), _p(out_pos))
    return out_ids, out_pos


def gather_rows(src, idx):
    src = np.ascontiguousarray(src)
    idx = _i64(idx)
    row_bytes = src.strides[0]
    dst = np.zeros((idx.shape[0],) + src.shape[1:], src.dtype)
    lib().pkv_o_gather_rows(_p(src), _p(idx), C.c_int64(idx.shape[0]), C.c_int64(row_bytes), _p(dst))
    return dst


def attention(q, k, v, scale=None):
    """q [G,128], k, v [S,128] -> [G,128] fp32 (softmax(q k^T * scale) v, double accumulation)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    if scale is None:
        scale = 1.0 / np.sqrt(128.0)
    out = np.empty_like(q)
    lib().pkv_o_attention(_p(q), C.c_int(q.shape[0]), _p(k), _p(v), C.c_int64(k.shape[0]), C.c_float(scale), _p(out))
    return out


def expf(x):
    x = _f32(x)
    out = np.empty_like(x)
    f = lib().pkv_o_expf
    flat_in, flat_out = x.reshape(-1), out.reshape(-1)
    for i in range(flat_in.shape[0]):
        flat_out[i] = f(C.c_float(float(flat_in[i])))
    return out


def adaptive_topk(sl_logits, sl_vnorm, cand_logits, cand_vnorm, cand_ids, threshold, k_out):
    sl_logits, sl_vnorm = _f32(sl_logits), _f32(sl_vnorm)
    cand_logits, cand_vnorm, cand_ids = _f32(cand_logits), _f32(cand_vnorm), _i64(cand_ids)
    out = np.zeros(k_out, np.int64)
    k = lib().pkv_o_adaptive_topk(_p(sl_logits), _p(sl_vnorm), C.c_int64(sl_logits.shape[0]), _p(cand_logits),
                                  _p(cand_vnorm), _p(cand_ids), C.c_int64(cand_logits.shape[0]),
                                  C.c_float(threshold), C.c_int64(k_out), _p(out))
    return int(k), out


def dense_logits(q, keys, scale, dtype):
    """Logits of the dense (sink / local / buffer) tokens of one KV head against the group-mean query
    (polar_cache_adaptivek_varlen.py:1418-1419 ``mean(dim=2)``, :1731 ``einsum(...).to(float32) * scale``), numpy.
    q [G,128], keys [n,128] (bf16-representable values for the bf16 chain).  The mean adds the heads in order and
    divides by G, like pkv_o_query_prep; the dot product is evaluated in one fixed order: dims in 16 groups of 8,
    each group left to right, the 16 group sums in a pairwise tree; mean and dot are rounded to the dtype."""
    q, keys = _f32(q), _f32(keys)
    rd = bf16_round if dtype == BF16 else (lambda x: x)
    acc = q[0].copy()
    for g in range(1, q.shape[0]):
        acc = acc + q[g]
    mean = rd(acc / np.float32(q.shape[0]))
    p = (keys * mean[None, :]).reshape(keys.shape[0], 16, 8)
    s = p[:, :, 0].copy()
    for j in range(1, 8):
        s = s + p[:, :, j]
    while s.shape[1] > 1:
        s = s[:, 0::2] + s[:, 1::2]
    return (rd(s[:, 0]) * np.float32(scale)).astype(np.float32)


def value_norm(v, dtype):
    """||v||_2 of rows [n,128] in the rows' dtype, widened to fp32 (polar_cache_adaptivek_varlen.py:1179
    ``torch.linalg.vector_norm(value_states, dim=-1).float()``), numpy: squares summed in a fixed order (bf16 rows:
    16 groups of 8 left to right; fp32 rows: 32 groups of 4; group sums in a pairwise tree), fp32 square root, rounded
    to the dtype."""
    v = _f32(v)
    per = 8 if dtype == BF16 else 4
    p = (v * v).reshape(v.shape[0], 128 // per, per)
    s = p[:, :, 0].copy()
    for j in range(1, per):
        s = s + p[:, :, j]
    while s.shape[1] > 1:
        s = s[:, 0::2] + s[:, 1::2]
    n = np.sqrt(s[:, 0], dtype=np.float32)
    return bf16_round(n) if dtype == BF16 else n


def retrieve_row(q, signs, dtype, codes, nib, weight, cluster_counts, tiers, n_cand, k):
    """Whole retrieval (query prep .. final top-k) for one (batch, kv-head) row."""
    q = _f32(q).reshape(-1, D)
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    nib = np.ascontiguousarray(nib, dtype=np.uint8)
    weight = _f32(weight)
    cc = np.ascontiguousarray(cluster_counts, dtype=np.int32)
    t = np.asarray(tiers, dtype=np.uint32)
    kk = min(k, n_cand)
    out = np.zeros(kk, np.int64)
    lib().pkv_o_retrieve_row(_p(q), C.c_int(q.shape[0]), _p(_f32(signs)), C.c_int(dtype), _p(codes), _p(nib),
                             _p(weight), _p(cc), C.c_int64(codes.shape[0]), _p(t), C.c_int(len(t)),
                             C.c_int64(n_cand), C.c_int64(k), _p(out))
    return out


# ------------------------------------------------------------------ fixtures


def philox4x32_10(ctr, key):
    """Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11), one block:
    ctr 4 x uint32, key 2 x uint32 -> 4 x uint32.  Pinned by the Random123 known-answer vectors."""
    c = [np.uint64(x) for x in ctr]
    k = [np.uint64(x) for x in key]
    m0, m1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    w0, w1, mask, s32 = np.uint64(0x9E3779B9), np.uint64(0xBB67AE85), np.uint64(0xFFFFFFFF), np.uint64(32)
    for _ in range(10):
        p0, p1 = m0 * c[0], m1 * c[2]
        c = [(p1 >> s32) ^ c[1] ^ k[0], p1 & mask, (p0 >> s32) ^ c[3] ^ k[1], p0 & mask]
        k = [(k[0] + w0) & mask, (k[1] + w1) & mask]
    return [int(x) for x in c]


def srht_signs(seed: int = 42):
    """SRHT diagonal D in {+-1}^128 (polar_cache.py:57-63: manual_seed(seed), then randint(0, 2, (128,)) * 2 - 1 on
    the GPU).  torch's device generator is Philox4x32-10 keyed by the seed; element i of the first draw after seeding
    is word 0 of the block with counter (0, 0, i, 0), reduced modulo the range."""
    bits = [philox4x32_10((0, 0, i, 0), (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))[0] % 2 for i in range(D)]
    return np.asarray([2.0 * b - 1.0 for b in bits], dtype=np.float32)


def synth_keys(n, seed, outliers=(7, 31, 64, 101), bf16=False, drift_deg_per_1k=0.0):
    """Synthetic keys ~N(0,1) with 4 fixed outlier channels x10; optional slow
    rotation of the key mean in the (0,1) plane."""
    import torch

    g = torch.Generator().manual_seed(seed)
    k = torch.randn(n, D, generator=g, dtype=torch.float32)
    k[:, list(outliers)] *= 10.0
    if drift_deg_per_1k:
        ang = torch.arange(n, dtype=torch.float32) * (drift_deg_per_1k / 1000.0) * (math.pi / 180.0)
        k[:, 0] += 3.0 * torch.cos(ang)
        k[:, 1] += 3.0 * torch.sin(ang)
    k = k.numpy()
    return bf16_round(k) if bf16 else k


def synth_queries(keys, G, seed, bf16=False):
    """queries = key mean + N(0, 0.5), one per q-head of the group."""
    import torch

    g = torch.Generator().manual_seed(seed + 1000003)
    q = torch.from_numpy(keys.mean(axis=0, dtype=np.float64).astype(np.float32)).unsqueeze(0) + 0.5 * torch.randn(
        G, D, generator=g, dtype=torch.float32)
    q = q.numpy()
    return bf16_round(q) if bf16 else q


def to_reference_layout(codes, nib, weight):
    """key-major -> reference tensors: codebook [16,n], key_4bit [16,n,4],
    block_weight [16,n] (per (b,h) row)."""
    return (np.ascontiguousarray(codes.T), np.ascontiguousarray(nib.transpose(1, 0, 2)),
            np.ascontiguousarray(weight.T))
