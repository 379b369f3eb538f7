"""Tensor-level wrappers over the C ABI: pointer/stride plumbing only.

Tensors use the reference's *logical* shapes (``cache_hub/polar_cache.py:288-312``):
``codebook [bs,H,B,N] u8``, ``key_4bit [bs,H,B,N,4] u8``, ``key_block_weight
[bs,H,B,N] bf16`` with arbitrary strides, so the same call accepts the
reference's subspace-major tensors and key-major storage exposed as permuted
views (see :func:`alloc_keymajor`).  PyTorch is used for device memory and
streams only; every computation happens in ``libpariskv_hip.so``.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import math

import torch

from . import _lib

B_SUB, M_SUB, K_CLUSTERS, HEAD_DIM = 16, 8, 256, 128
RERANK_RECORD_BYTES = 128  # one key's 64 nibble bytes + 16 bf16 weights, padded to an HBM line
RECORD_VALUE_NORM_OFFSET = 96  # spare bytes of the record: one fp32 word for the adaptive-k caches
TIER_RATIOS = (0.05, 0.15, 0.30, 0.50, 0.75, 1.0)  # cache_hub/polar_cache.py:1221
# cache_hub/polar_cache.py:188-193 rounded to bf16
MAG_THRESHOLDS = (0.08447265625, 0.169921875, 0.2578125, 0.349609375, 0.44921875, 0.55859375, 0.69140625)
MAG_CENTERS = (0.0419921875, 0.126953125, 0.212890625, 0.302734375, 0.396484375, 0.5, 0.6171875, 0.76171875)


def _p(t: Optional[torch.Tensor]):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _stream(t: torch.Tensor):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _dt(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _lib.DTYPE_F32
    if dtype == torch.bfloat16:
        return _lib.DTYPE_BF16
    raise RuntimeError(f"unsupported dtype {dtype}: float32 or bfloat16 expected")


def _need(cond: bool, msg: str):
    if not cond:
        raise RuntimeError(msg)


def _cuda(*ts):
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "tensor must be on the GPU")


def _philox4x32_10(ctr, key):
    """One block of the Philox4x32-10 counter-based generator (Salmon et al., SC'11): 4 x uint32 out."""
    m0, m1, w0, w1, mask = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
    c, k = list(ctr), list(key)
    for _ in range(10):
        p0, p1 = m0 * c[0], m1 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & mask, (p0 >> 32) ^ c[3] ^ k[1], p0 & mask]
        k = [(k[0] + w0) & mask, (k[1] + w1) & mask]
    return c


def srht_signs(device, seed: int = 42) -> torch.Tensor:
    """SRHT diagonal in {+-1}^128 as float32: the vector the reference draws with
    ``torch.manual_seed(seed); torch.randint(0, 2, (128,), device=gpu) * 2 - 1`` (``polar_cache.py:57-63``).

    torch's device generator is Philox4x32-10 with key = seed, subsequence = element index and offset 0 for the first
    draw after seeding, and ``randint`` keeps the first word modulo the range; this evaluates the same function on the
    host, so the vector needs no GPU, does not touch any generator state and is the same on every machine."""
    mask = 0xFFFFFFFF
    bits = [_philox4x32_10((0, 0, i, 0), (seed & mask, (seed >> 32) & mask))[0] % 2 for i in range(HEAD_DIM)]
    return torch.tensor([2.0 * b - 1.0 for b in bits], dtype=torch.float32, device=device)


def mag_centers(device) -> torch.Tensor:
    return torch.tensor(MAG_CENTERS, dtype=torch.float32, device=device)


def alloc_keymajor(bs: int, heads: int, cap: int, device):
    """Key-major storage + reference-shaped views.

    Returns ``(codes_km [bs,H,cap,16] u8, nib_km [bs,H,cap,64] u8, w_km [bs,H,cap,16] bf16,
    codebook [bs,H,16,cap], key_4bit [bs,H,16,cap,4], key_block_weight [bs,H,16,cap])``;
    the last three are permuted views of the first three.  The codes are one packed array (the collision scan
    streams them); a key's nibbles and weights share one 128-byte-aligned record (bytes 0-63 and 64-95): the
    rerank reads both for candidates scattered over the zone, HBM comes in 128-byte lines, and two packed arrays
    would cost two lines per candidate."""
    codes = torch.zeros(bs, heads, cap, B_SUB, dtype=torch.uint8, device=device)
    rec = torch.zeros(bs, heads, cap, RERANK_RECORD_BYTES, dtype=torch.uint8, device=device)
    _need(rec.data_ptr() % RERANK_RECORD_BYTES == 0, "allocator returned a buffer that is not 128-byte aligned")
    nib = rec[..., :B_SUB * 4]
    w = rec[..., B_SUB * 4:B_SUB * 4 + B_SUB * 2].view(torch.bfloat16)
    return (codes, nib, w, codes.permute(0, 1, 3, 2), nib.view(bs, heads, cap, B_SUB, 4).permute(0, 1, 3, 2, 4),
            w.permute(0, 1, 3, 2))


def record_value_norm_view(nib_km: torch.Tensor) -> torch.Tensor:
    """fp32 [bs,H,cap] view of the word at byte 96 of every key's record, given the record's nibble view from
    :func:`alloc_keymajor`.  The adaptive-k caches keep ``value_norm_gpu`` there: the fused select+rerank then
    passes a candidate's value norm through with the HBM line it reads anyway."""
    bs, H, cap, _ = nib_km.shape
    _need(nib_km.dtype == torch.uint8 and nib_km.stride(2) == RERANK_RECORD_BYTES and nib_km.stride(3) == 1,
          "expected the nibble view of 128-byte key records")
    rec = nib_km.as_strided((bs, H, cap, RERANK_RECORD_BYTES), nib_km.stride(), nib_km.storage_offset())
    return rec[..., RECORD_VALUE_NORM_OFFSET:RECORD_VALUE_NORM_OFFSET + 4].view(torch.float32).squeeze(-1)


# ------------------------------------------------------------------- append


def encode_append(keys: torch.Tensor, signs: torch.Tensor, codebook: torch.Tensor,
                  key_4bit: Optional[torch.Tensor], key_block_weight: Optional[torch.Tensor],
                  cluster_counts: Optional[torch.Tensor]) -> None:
    """keys [bs,H,S,128] -> writes codebook [bs,H,16,S], key_4bit [bs,H,16,S,4],
    key_block_weight [bs,H,16,S] (any strides) and ``cluster_counts += histogram``."""
    _cuda(keys, signs, codebook, key_4bit, key_block_weight, cluster_counts)
    bs, H, S, D = keys.shape
    _need(D == HEAD_DIM and keys.stride(3) == 1, "keys must be [bs,H,S,128] with a contiguous last dim")
    _need(signs.dtype == torch.float32 and signs.numel() == HEAD_DIM and signs.is_contiguous(), "signs: float32[128]")
    _need(codebook.dtype == torch.uint8 and tuple(codebook.shape) == (bs, H, B_SUB, S), "codebook must be u8 [bs,H,16,S]")
    ns = (0, 0, 0, 0)
    if key_4bit is not None:
        _need(key_4bit.dtype == torch.uint8 and tuple(key_4bit.shape) == (bs, H, B_SUB, S, 4) and
              key_4bit.stride(4) == 1, "key_4bit must be u8 [bs,H,16,S,4] with a contiguous last dim")
        ns = (key_4bit.stride(0), key_4bit.stride(1), key_4bit.stride(3), key_4bit.stride(2))
    ws = (0, 0, 0, 0)
    if key_block_weight is not None:
        _need(key_block_weight.dtype == torch.bfloat16 and tuple(key_block_weight.shape) == (bs, H, B_SUB, S),
              "key_block_weight must be bf16 [bs,H,16,S]")
        ws = (key_block_weight.stride(0), key_block_weight.stride(1), key_block_weight.stride(3),
              key_block_weight.stride(2))
    cc = (0, 0)
    if cluster_counts is not None:
        _need(cluster_counts.dtype == torch.int32 and tuple(cluster_counts.shape) == (bs, H, B_SUB, K_CLUSTERS) and
              cluster_counts.stride(3) == 1 and cluster_counts.stride(2) == K_CLUSTERS,
              "cluster_counts must be int32 [bs,H,16,256] with contiguous [16,256] blocks")
        cc = (cluster_counts.stride(0), cluster_counts.stride(1))
    _lib.check(_lib.lib().pkv_encode_append(
        _p(keys), _dt(keys.dtype), bs, H, S, keys.stride(0), keys.stride(1), keys.stride(2), _p(signs),
        _p(codebook), codebook.stride(0), codebook.stride(1), codebook.stride(3), codebook.stride(2),
        _p(key_4bit), *ns, _p(key_block_weight), *ws, _p(cluster_counts), *cc, _stream(keys)))


def count_cluster_keys(codebook: torch.Tensor, cluster_counts: torch.Tensor) -> None:
    """cluster_counts[bs,H,16,256] += per-subspace histogram of codebook [bs,H,16,N]."""
    _cuda(codebook, cluster_counts)
    bs, H, Bs, N = codebook.shape
    _need(codebook.dtype == torch.uint8 and Bs == B_SUB, "codebook must be u8 [bs,H,16,N]")
    _need(cluster_counts.dtype == torch.int32 and tuple(cluster_counts.shape) == (bs, H, B_SUB, K_CLUSTERS) and
          cluster_counts.stride(3) == 1 and cluster_counts.stride(2) == K_CLUSTERS, "cluster_counts: int32 [bs,H,16,256]")
    _lib.check(_lib.lib().pkv_count_cluster_keys(
        _p(codebook), codebook.stride(0), codebook.stride(1), codebook.stride(3), codebook.stride(2), bs, H, N,
        _p(cluster_counts), cluster_counts.stride(0), cluster_counts.stride(1), _stream(codebook)))


# --------------------------------------------------------------- query side


def _tiers(tier_counts: Sequence[int]):
    _need(1 <= len(tier_counts) <= _lib.MAX_TIERS, f"tier_num must be in [1,{_lib.MAX_TIERS}]")
    return (C.c_uint32 * len(tier_counts))(*[int(t) for t in tier_counts]), len(tier_counts)


def query_prep_lut(queries: torch.Tensor, n_kv_heads: int, signs: torch.Tensor, cluster_counts: torch.Tensor,
                   tier_counts: Sequence[int], want_sorted_ids: bool = False):
    """queries [bs,1,Hq,128] or [bs,Hq,128] -> (qhat [bs,H,128] f32, qnorm [bs,H] f32,
    lut [bs,H,16,256] u8, sorted_ids [bs,H,16,256] i64 or None)."""
    _cuda(queries, signs, cluster_counts)
    q = queries.reshape(queries.shape[0], -1, HEAD_DIM) if queries.dim() == 4 else queries
    _need(q.is_contiguous() and q.shape[-1] == HEAD_DIM, "queries must be contiguous [bs,(1,)Hq,128]")
    bs, Hq, _ = q.shape
    _need(Hq % n_kv_heads == 0, "num_heads must be a multiple of num_key_value_heads")
    group = Hq // n_kv_heads
    _need(cluster_counts.dtype == torch.int32 and tuple(cluster_counts.shape) == (bs, n_kv_heads, B_SUB, K_CLUSTERS)
          and cluster_counts.stride(3) == 1 and cluster_counts.stride(2) == K_CLUSTERS,
          "cluster_counts must be int32 [bs,H,16,256]")
    dev = q.device
    qhat = torch.empty(bs, n_kv_heads, HEAD_DIM, dtype=torch.float32, device=dev)
    qnorm = torch.empty(bs, n_kv_heads, dtype=torch.float32, device=dev)
    lut = torch.empty(bs, n_kv_heads, B_SUB, K_CLUSTERS, dtype=torch.uint8, device=dev)
    sorted_ids = torch.empty(bs, n_kv_heads, B_SUB, K_CLUSTERS, dtype=torch.int64, device=dev) if want_sorted_ids else None
    tc, nt = _tiers(tier_counts)
    _lib.check(_lib.lib().pkv_query_prep_lut(
        _p(q), _dt(q.dtype), bs, n_kv_heads, group, _p(signs), _p(cluster_counts), cluster_counts.stride(0),
        cluster_counts.stride(1), tc, nt, _p(qhat), _p(qnorm), _p(lut), _p(sorted_ids), _stream(q)))
    return qhat, qnorm, lut, sorted_ids


def update_cache_cnt(sorted_cluster_ids: torch.Tensor, cluster_key_counts: torch.Tensor, codebook: torch.Tensor,
                     tier_counts: Sequence[int]) -> torch.Tensor:
    """Tiered collision vote from a caller-supplied ranking -> int32 [bs,H,N]."""
    _cuda(sorted_cluster_ids, cluster_key_counts, codebook)
    _need(codebook.dtype == torch.uint8, "code_book must be uint8 tensor")
    _need(sorted_cluster_ids.dtype == torch.int64, "sorted_cluster_ids must be int64 tensor")
    _need(cluster_key_counts.dtype == torch.int32, "cluster_key_counts must be int32 tensor")
    _need(sorted_cluster_ids.dim() == 4 and codebook.dim() == 4 and cluster_key_counts.dim() == 4, "4-D tensors expected")
    bs, H, Bs, K = sorted_cluster_ids.shape
    _need(Bs == B_SUB and K == K_CLUSTERS, "only sub_spaces=16, num_clusters=256 is built")
    _need(tuple(cluster_key_counts.shape) == (bs, H, Bs, K) and tuple(codebook.shape[:3]) == (bs, H, Bs), "shape mismatch")
    _need(sorted_cluster_ids.stride(3) == 1 and cluster_key_counts.stride(3) == 1, "last dims must be contiguous")
    N = codebook.shape[3]
    cnt = torch.empty(bs, H, N, dtype=torch.int32, device=codebook.device)
    lut_ws = torch.empty(bs * H * B_SUB * K_CLUSTERS, dtype=torch.uint8, device=codebook.device)
    tc, nt = _tiers(tier_counts)
    si, ck, cb = sorted_cluster_ids, cluster_key_counts, codebook
    _lib.check(_lib.lib().pkv_update_cache_cnt(
        _p(si), si.stride(0), si.stride(1), si.stride(2), _p(ck), ck.stride(0), ck.stride(1), ck.stride(2),
        _p(cb), cb.stride(0), cb.stride(1), cb.stride(3), cb.stride(2), bs, H, N, tc, nt, _p(lut_ws), _p(cnt),
        _stream(cb)))
    return cnt


def update_cache_cnt_legacy(sorted_cluster_ids: torch.Tensor, topk_cluster_cnt: torch.Tensor,
                            codebook: torch.Tensor) -> torch.Tensor:
    """Single-tier vote on the legacy int32 tensors -> int32 [bs,H,N]."""
    _cuda(sorted_cluster_ids, topk_cluster_cnt, codebook)
    for t, name in ((sorted_cluster_ids, "sorted_cluster_ids"), (topk_cluster_cnt, "topk_cluster_cnt"), (codebook, "codebook")):
        _need(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be a contiguous int32 tensor")
    bs, H, Bs, K = sorted_cluster_ids.shape
    _need(Bs == B_SUB and K == K_CLUSTERS and tuple(topk_cluster_cnt.shape) == (bs, H, Bs) and
          tuple(codebook.shape[:3]) == (bs, H, Bs), "shape mismatch (sub_spaces=16, num_clusters=256 only)")
    N = codebook.shape[3]
    cnt = torch.empty(bs, H, N, dtype=torch.int32, device=codebook.device)
    lut_ws = torch.empty(bs * H * B_SUB * K_CLUSTERS, dtype=torch.uint8, device=codebook.device)
    _lib.check(_lib.lib().pkv_update_cache_cnt_legacy(_p(sorted_cluster_ids), _p(topk_cluster_cnt), _p(codebook), bs, H,
                                                      N, _p(lut_ws), _p(cnt), _stream(codebook)))
    return cnt


def pick_chunk_keys(rows: int, n_keys: int) -> int:
    chunk = 2048
    while chunk < 16384 and rows * ((n_keys + chunk - 1) // chunk) > 1024:
        chunk *= 2
    while chunk < 32768 and (n_keys + chunk - 1) // chunk > 512:
        chunk *= 2
    return chunk


def collision_scan(codebook: torch.Tensor, lut: torch.Tensor, out_dtype=torch.int32, want_hist: bool = False):
    """Votes per key from a ready table.  Returns (cnt [bs,H,N], (row_suf, chunk_suf) or None, chunk_keys);
    the suffix histograms count keys with a vote count >= t, per row and per chunk."""
    _cuda(codebook, lut)
    bs, H, Bs, N = codebook.shape
    _need(codebook.dtype == torch.uint8 and Bs == B_SUB, "codebook must be u8 [bs,H,16,N]")
    _need(lut.dtype == torch.uint8 and lut.is_contiguous() and lut.numel() == bs * H * B_SUB * K_CLUSTERS, "lut: u8 [bs,H,16,256]")
    cnt = torch.empty(bs, H, N, dtype=out_dtype, device=codebook.device)
    chunk = pick_chunk_keys(bs * H, N)
    hist = row_suf = None
    if want_hist:
        hist = torch.empty(bs * H, (N + chunk - 1) // chunk, 128, dtype=torch.int16, device=codebook.device)
        row_suf = torch.zeros(bs * H, 128, dtype=torch.int32, device=codebook.device)
    u8 = cnt if out_dtype == torch.uint8 else None
    i32 = cnt if out_dtype == torch.int32 else None
    _need(u8 is not None or i32 is not None, "out_dtype must be uint8 or int32")
    _lib.check(_lib.lib().pkv_collision_scan(_p(codebook), codebook.stride(0), codebook.stride(1), codebook.stride(3),
                                             codebook.stride(2), bs, H, N, _p(lut), _p(u8), _p(i32), _p(row_suf), _p(hist),
                                             chunk, _stream(codebook)))
    return cnt, ((row_suf, hist) if want_hist else None), chunk


# --------------------------------------------------------------- selections


def bucket_topk(x: torch.Tensor, k: int) -> torch.Tensor:
    """int32 [rows,L] values in [0,127] -> int64 [rows,k]."""
    _cuda(x)
    _need(x.dim() == 2, "input must be 2D [B, L]")
    if x.dtype != torch.int32:
        x = x.to(torch.int32)
    if x.stride(1) != 1:
        x = x.contiguous()
    rows, L = x.shape
    _need(k > 0, "k must be positive")
    _need(k <= L, "k cannot exceed sequence length")
    out = torch.empty(rows, k, dtype=torch.int64, device=x.device)
    nbytes = _lib.lib().pkv_bucket_topk_ws_bytes(rows, L)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    _lib.check(_lib.lib().pkv_bucket_topk(_p(x), x.stride(0), rows, L, k, _p(out), _p(ws), nbytes, _stream(x)))
    return out


def topk_f32(x: torch.Tensor, k: int, ids: Optional[torch.Tensor] = None, want_values: bool = False):
    """Exact top-k of fp32 [rows,L], descending; ties -> smaller ``ids`` (position when None)."""
    _cuda(x, ids)
    _need(x.dim() == 2, "input must be 2D [B, L]")
    if x.dtype != torch.float32:
        x = x.to(torch.float32)
    if x.stride(1) != 1:
        x = x.contiguous()
    rows, L = x.shape
    _need(k > 0, "k must be positive")
    _need(k <= L, "k cannot exceed sequence length")
    if ids is not None:
        _need(ids.dtype == torch.int64 and tuple(ids.shape) == (rows, L) and ids.stride(1) == 1, "ids: int64 [rows,L]")
    out = torch.empty(rows, k, dtype=torch.int64, device=x.device)
    vals = torch.empty(rows, k, dtype=torch.float32, device=x.device) if want_values else None
    nbytes = _lib.lib().pkv_topk_f32_ws_bytes(rows, L, k)   # 256 unless rows are wider than one workgroup sorts
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device) if nbytes > 256 else None
    _lib.check(_lib.lib().pkv_topk_f32(_p(x), x.stride(0), _p(ids), ids.stride(0) if ids is not None else 0, rows, L, k,
                                       _p(out), _p(vals), _p(ws), nbytes if ws is not None else 0, _stream(x)))
    return (out, vals) if want_values else out


def rerank4(coarse_indices: torch.Tensor, key_4bit: torch.Tensor, key_block_weight: torch.Tensor, qhat: torch.Tensor,
            qnorm: torch.Tensor, centers: torch.Tensor, want_v4b: bool = False):
    """fp32 scores [bs,H,C] of the candidates (and optionally the unpacked bf16 values)."""
    _cuda(coarse_indices, key_4bit, key_block_weight, qhat, qnorm, centers)
    _need(coarse_indices.dtype == torch.int64 and coarse_indices.is_contiguous(), "coarse_indices must be contiguous int64")
    _need(key_4bit.dtype == torch.uint8, "key_4bit must be byte tensor")
    _need(key_block_weight.dtype == torch.bfloat16, "key_block_weight must be bfloat16 tensor")
    bs, H, Bs, N, nb = key_4bit.shape
    _need(Bs == B_SUB and nb == 4, "only support B = 16, m = 8")
    _need(key_4bit.stride(-1) == 1, "key_4bit must be contiguous in the last dimension")
    _need(tuple(key_block_weight.shape) == (bs, H, Bs, N), "key_block_weight shape mismatch")
    Cn = coarse_indices.shape[-1]
    _need(tuple(coarse_indices.shape) == (bs, H, Cn), "coarse_indices must be [bs,H,C]")
    qhat = qhat.reshape(bs, H, HEAD_DIM)
    _need(qhat.dtype == torch.float32 and qhat.is_contiguous(), "qhat must be contiguous float32 [bs,H,128]")
    qnorm = qnorm.reshape(bs, H)
    _need(qnorm.dtype == torch.float32 and qnorm.is_contiguous(), "qnorm must be contiguous float32 [bs,H]")
    _need(centers.dtype == torch.float32 and centers.numel() == 8 and centers.is_contiguous(), "centers: float32[8]")
    scores = torch.empty(bs, H, Cn, dtype=torch.float32, device=key_4bit.device)
    v4b = torch.empty(bs, H, Bs, Cn, M_SUB, dtype=torch.bfloat16, device=key_4bit.device) if want_v4b else None
    k4, kw = key_4bit, key_block_weight
    _lib.check(_lib.lib().pkv_rerank4(
        _p(coarse_indices), bs, H, Cn, N, _p(k4), k4.stride(0), k4.stride(1), k4.stride(3), k4.stride(2),
        _p(kw), kw.stride(0), kw.stride(1), kw.stride(3), kw.stride(2), _p(qhat), _p(qnorm), _p(centers), _p(scores),
        _p(v4b), _stream(k4)))
    return scores, v4b


def adaptive_topk(sl_logits: torch.Tensor, sl_vnorm: torch.Tensor, cand_scores: torch.Tensor, cand_scale: float,
                  cand_ids: torch.Tensor, threshold: float, k_out: int, cand_vnorm: Optional[torch.Tensor] = None,
                  value_norm: Optional[torch.Tensor] = None, vn_offset: int = 0, k_min: int = 0, k_max: int = 0,
                  row_keys_base: Optional[int] = None):
    """Adaptive top-k by value-weighted attention mass.

    sl_logits / sl_vnorm fp32 [bs,H,sl] (last dim contiguous); cand_scores fp32 or bf16 [bs,H,C] contiguous
    (logit = score * cand_scale); cand_ids int64 [bs,H,C]; candidate value norms either ``cand_vnorm`` fp32 [bs,H,C]
    or gathered from ``value_norm`` fp32 [bs,H,cap] at ``cand_ids + vn_offset``.
    ``k_max > 0`` clamps k to [k_min, k_max] inside the kernel; ``row_keys_base`` asks for a third result,
    int32 [bs,H] = row_keys_base + k (the per-row key count of the attention that follows).
    Returns (adaptive_k int64 [bs,H], topk_ids int64 [bs,H,k_out])."""
    _cuda(sl_logits, sl_vnorm, cand_scores, cand_ids, cand_vnorm, value_norm)
    bs, H, Cn = cand_scores.shape
    rows = bs * H
    _need(cand_scores.is_contiguous() and cand_ids.is_contiguous() and cand_ids.dtype == torch.int64 and
          tuple(cand_ids.shape) == (bs, H, Cn), "cand_scores / cand_ids must be contiguous [bs,H,C]")
    sl = sl_logits.shape[-1]
    for t in (sl_logits, sl_vnorm):
        _need(t.dtype == torch.float32 and tuple(t.shape) == (bs, H, sl) and (sl == 0 or t.stride(2) == 1) and
              (H == 1 or t.stride(0) == H * t.stride(1)), "dense logits / value norms must be fp32 [bs,H,sl] with uniform row stride")
    _need(0 < k_out <= Cn, "topk_cap must be in (0, cand_len]")
    if cand_vnorm is not None:
        _need(cand_vnorm.dtype == torch.float32 and cand_vnorm.is_contiguous() and tuple(cand_vnorm.shape) == (bs, H, Cn),
              "cand_vnorm must be contiguous fp32 [bs,H,C]")
        vn_stride = vn_pos = 0
    else:
        _need(value_norm is not None and value_norm.dtype == torch.float32 and value_norm.dim() == 3 and
              tuple(value_norm.shape[:2]) == (bs, H) and value_norm.stride(2) >= 1 and
              value_norm.stride(1) == value_norm.shape[2] * value_norm.stride(2) and
              (bs == 1 or value_norm.stride(0) == H * value_norm.stride(1)),
              "value_norm must be fp32 [bs,H,cap] with one uniform position stride")
        vn_stride, vn_pos = value_norm.stride(1), value_norm.stride(2)
    dev = cand_scores.device
    ak = torch.empty(bs, H, dtype=torch.int64, device=dev)
    ids = torch.empty(bs, H, k_out, dtype=torch.int64, device=dev)
    row_keys = None if row_keys_base is None else torch.empty(bs, H, dtype=torch.int32, device=dev)
    nbytes = _lib.lib().pkv_adaptive_topk_ws_bytes(rows, Cn, k_out)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    row_stride = lambda t: t.stride(1) if H > 1 else (t.stride(0) if bs > 1 else max(1, sl))
    _lib.check(_lib.lib().pkv_adaptive_topk(
        _p(sl_logits), row_stride(sl_logits), _p(sl_vnorm), row_stride(sl_vnorm), sl, _p(cand_scores),
        _dt(cand_scores.dtype), float(cand_scale), _p(cand_vnorm), _p(value_norm), vn_stride, vn_offset, vn_pos,
        _p(cand_ids), Cn,
        float(threshold), k_out, rows, _p(ak), _p(ids), int(k_min), int(k_max), _p(row_keys),
        int(row_keys_base or 0), _p(ws), nbytes, _stream(cand_scores)))
    return (ak, ids) if row_keys is None else (ak, ids, row_keys)


def uniform_k(adaptive_k: torch.Tensor, row_keys_base: Optional[int] = None):
    """max over all (batch, kv-head) rows of ``adaptive_k`` (int64 [bs,H]) broadcast to every row, on the GPU: the
    ``global_k`` of cache_hub/polar_cache_atten_value_indices_adaptive_k.py:1585 without its host read.  Returns the
    int64 [bs,H] tensor, and with ``row_keys_base`` also int32 [bs,H] = base + max."""
    _cuda(adaptive_k)
    _need(adaptive_k.dtype == torch.int64 and adaptive_k.is_contiguous() and adaptive_k.numel() > 0,
          "adaptive_k: contiguous int64")
    out = torch.empty_like(adaptive_k)
    rk = None if row_keys_base is None else torch.empty(adaptive_k.shape, dtype=torch.int32, device=adaptive_k.device)
    _lib.check(_lib.lib().pkv_uniform_k(_p(adaptive_k), adaptive_k.numel(), _p(out), _p(rk), int(row_keys_base or 0),
                                        _stream(adaptive_k)))
    return out if rk is None else (out, rk)


def adaptive_topk_ws_bytes(rows: int, n_cand: int, k_out: int) -> int:
    return int(_lib.lib().pkv_adaptive_topk_ws_bytes(rows, n_cand, k_out))


def dense_logits(queries: torch.Tensor, keys: torch.Tensor, n_rows: int, scale: float,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Logits of the first ``n_rows`` rows of ``keys`` [bs,H,rows,128] (contiguous rows) against the mean of each KV
    head's query group: float32 [bs,H,n_rows] = dtype(mean_g(q) . k) * scale
    (cache_hub/polar_cache_adaptivek_varlen.py:1418-1419, :1731).  queries: contiguous [bs,1,H*G,128]."""
    _cuda(queries, keys)
    bs, H, rows, D = keys.shape
    _need(D == HEAD_DIM and keys.stride(3) == 1 and keys.stride(2) == D and 0 < n_rows <= rows and
          keys.dtype == queries.dtype, "keys: [bs,H,rows,128] with contiguous rows, dtype of the queries")
    _need(queries.is_contiguous() and queries.numel() % (bs * H * D) == 0, "queries must be contiguous [bs,1,Hq,128]")
    G = queries.numel() // (bs * H * D)
    if out is None:
        out = torch.empty(bs, H, n_rows, dtype=torch.float32, device=keys.device)
    _need(out.is_cuda and out.dtype == torch.float32 and tuple(out.shape[:2]) == (bs, H) and out.shape[2] >= n_rows and
          out.stride(2) == 1 and out.stride(1) >= n_rows and (bs == 1 or out.stride(0) == H * out.stride(1)),
          "out: fp32 [bs,H,>=n_rows] with contiguous rows at one uniform stride")
    _lib.check(_lib.lib().pkv_dense_logits(_p(queries), _dt(queries.dtype), bs, H, G, _p(keys), keys.stride(0),
                                           keys.stride(1), n_rows, float(scale), _p(out), out.stride(1), _stream(keys)))
    return out


# ------------------------------------------------------------------ gathers


def _gather(fn, src_k, src_v, idx, dst_k, dst_v, idx_offset, dst_row0, row_counts=None):
    """Shared checks and call of the gather entry points; ``row_counts`` only for the ragged one."""
    bs, H, src_len, D = src_k.shape
    _need(src_k.shape == src_v.shape and dst_k.shape == dst_v.shape, "K/V shape mismatch")
    _need(src_k.dtype == src_v.dtype == dst_k.dtype == dst_v.dtype, "K/V dtype mismatch")
    _need(idx.dtype == torch.int64 and idx.is_cuda and idx.is_contiguous() and tuple(idx.shape[:2]) == (bs, H),
          "selected_indices must be contiguous int64 [bs,H,K] on the GPU")
    for t in (src_k, src_v, dst_k, dst_v):
        _need(t.is_contiguous(), "K/V buffers must be contiguous")
    _need(dst_k.is_cuda and dst_v.is_cuda and tuple(dst_k.shape[:2]) == (bs, H) and dst_k.shape[3] == D, "dst shape mismatch")
    k = idx.shape[2]
    row_bytes = D * src_k.element_size()
    counts = () if row_counts is None else (_p(row_counts),)
    _lib.check(fn(_p(src_k), _p(src_v), src_len, _p(idx), k, *counts, idx_offset, _p(dst_k), _p(dst_v), dst_k.shape[2],
                  dst_row0, bs, H, row_bytes, _stream(dst_k)))


def gather_uva(src_k, src_v, idx, dst_k, dst_v, idx_offset: int = 0, dst_row0: int = 0) -> None:
    """dst[b,h,dst_row0+i,:] = src[b,h,idx[b,h,i]+idx_offset,:] with src in pinned host memory."""
    _need(src_k.is_cpu and src_v.is_cpu and src_k.is_pinned() and src_v.is_pinned(), "src must be pinned CPU tensors")
    _gather(_lib.lib().pkv_gather_uva, src_k, src_v, idx, dst_k, dst_v, idx_offset, dst_row0)


def gather_uva_ragged(src_k, src_v, idx, row_counts, dst_k, dst_v, idx_offset: int = 0, dst_row0: int = 0) -> None:
    """:func:`gather_uva` where row (b, h) moves only its first ``row_counts[b, h]`` indices (int64 [bs,H] on the GPU,
    values in [0, K]); the remaining dst rows are left as they are."""
    _need(src_k.is_cpu and src_v.is_cpu and src_k.is_pinned() and src_v.is_pinned(), "src must be pinned CPU tensors")
    _need(row_counts.is_cuda and row_counts.dtype == torch.int64 and row_counts.is_contiguous() and
          row_counts.numel() == idx.shape[0] * idx.shape[1], "row_counts: contiguous int64 [bs,H] on the GPU")
    _gather(_lib.lib().pkv_gather_uva_ragged, src_k, src_v, idx, dst_k, dst_v, idx_offset, dst_row0, row_counts=row_counts)


def gather_hbm(src_k, src_v, idx, dst_k, dst_v, idx_offset: int = 0, dst_row0: int = 0) -> None:
    _need(src_k.is_cuda and src_v.is_cuda, "src must be GPU tensors")
    _gather(_lib.lib().pkv_gather_hbm, src_k, src_v, idx, dst_k, dst_v, idx_offset, dst_row0)


def append_kv(key_states, value_states, dst_k, dst_v, slot: int, vnorm: Optional[torch.Tensor] = None) -> None:
    """dst_k[:, :, slot, :] = key_states[:, 0] and the same for values, in one launch
    (decode_update_kv_cache, cache_hub/polar_cache.py:848-856).  key_states/value_states [bs,1,Hkv,D];
    dst_k/dst_v [bs,Hkv,rows,D] with contiguous rows.  ``vnorm`` (fp32 [bs,Hkv,rows], last dim contiguous) also
    receives ``||value_states[b,0,h]||`` at ``[b,h,slot]``, computed in the K/V dtype
    (cache_hub/polar_cache_adaptivek_varlen.py:1179)."""
    bs, one, H, D = key_states.shape
    es = key_states.element_size()
    _need(one == 1 and value_states.shape == key_states.shape and key_states.stride(3) == 1 and
          value_states.stride(3) == 1, "key_states, value_states: [bs,1,Hkv,D] with contiguous rows")
    _need(dst_k.dtype == key_states.dtype and dst_v.dtype == key_states.dtype and value_states.dtype == key_states.dtype,
          "append: dtypes differ")
    _need(dst_k.shape == dst_v.shape and dst_k.stride() == dst_v.stride() and dst_k.stride(3) == 1 and
          dst_k.stride(2) == D and tuple(dst_k.shape[:2]) == (bs, H) and dst_k.shape[3] == D,
          "dst_k, dst_v: [bs,Hkv,rows,D] with contiguous rows")
    _need(key_states.is_cuda and dst_k.is_cuda, "append: tensors must be on the GPU")
    vn_b = vn_h = 0
    if vnorm is not None:
        _need(vnorm.is_cuda and vnorm.dtype == torch.float32 and tuple(vnorm.shape[:2]) == (bs, H) and
              vnorm.stride(2) == 1 and vnorm.shape[2] > slot, "vnorm: fp32 [bs,Hkv,rows] with contiguous rows")
        vn_b, vn_h = vnorm.stride(0), vnorm.stride(1)
    _lib.check(_lib.lib().pkv_append_kv(
        key_states.data_ptr(), key_states.stride(0) * es, key_states.stride(2) * es,
        value_states.data_ptr(), value_states.stride(0) * es, value_states.stride(2) * es, dst_k.data_ptr(),
        dst_v.data_ptr(), dst_k.stride(0) * es, dst_k.stride(1) * es, dst_k.shape[2], slot, bs, H, D * es,
        _p(vnorm), vn_b, vn_h, _stream(dst_k)))


OFFLOAD_ONE_COMMAND = 1


def offload_rows(src_k, src_v, dst_k_cpu, dst_v_cpu, dst_row0: int, stream=None, dma: bool = False, dma_flags: int = 0) -> None:
    """dst_cpu[:, :, dst_row0:dst_row0+n] = src for K and V on ``stream`` (default: the current one).
    src_k/src_v: GPU [bs,H,n,D] views with any batch / head / row strides (last dim contiguous); dst_*_cpu: pinned
    CPU [bs,H,rows,D] (a batch slice of a contiguous tensor is fine).  Asynchronous
    (cache_hub/polar_cache.py:457-471, :778-799).  ``dma=False``: one kernel that writes through the host store's
    device mapping; ``dma=True``: copy-engine commands, which leave the compute units to whatever runs beside."""
    bs, H, n, D = src_k.shape
    es = src_k.element_size()
    _need(src_k.is_cuda and src_v.is_cuda and src_v.shape == src_k.shape and src_v.stride() == src_k.stride() and
          src_k.stride(3) == 1 and src_v.dtype == src_k.dtype, "src_k, src_v: GPU [bs,H,n,D], same strides, contiguous rows")
    for t in (dst_k_cpu, dst_v_cpu):
        _need(t.is_cpu and t.is_pinned() and t.dtype == src_k.dtype and t.dim() == 4 and tuple(t.shape[:2]) == (bs, H) and
              t.shape[3] == D and t.stride(3) == 1 and t.stride(2) == D and t.stride(1) == t.shape[2] * D and
              (bs == 1 or t.stride(0) == H * t.stride(1)), "dst: pinned CPU [bs,H,rows,D], contiguous")
    s = stream if stream is not None else torch.cuda.current_stream(src_k.device)
    if dma:
        _lib.check(_lib.lib().pkv_offload_rows_dma(
            src_k.data_ptr(), src_v.data_ptr(), src_k.stride(0) * es, src_k.stride(1) * es, src_k.stride(2) * es,
            dst_k_cpu.data_ptr(), dst_v_cpu.data_ptr(), dst_k_cpu.shape[2], dst_row0, n, bs, H, D * es, dma_flags,
            C.c_void_p(s.cuda_stream)))
        return
    _lib.check(_lib.lib().pkv_offload_rows(
        src_k.data_ptr(), src_v.data_ptr(), src_k.stride(0) * es, src_k.stride(1) * es, src_k.stride(2) * es,
        dst_k_cpu.data_ptr(), dst_v_cpu.data_ptr(), dst_k_cpu.shape[2], dst_row0, n, bs, H, D * es,
        C.c_void_p(s.cuda_stream)))


def gather_uva_packed(src_k, src_v, k_packed, v_packed, indices_packed, cu_seqlens_topk, cu_seqlens_k,
                      sink_local_end: int, global_k: int) -> None:
    bs, H, src_len, D = src_k.shape
    _need(k_packed.is_cuda and v_packed.is_cuda and k_packed.is_contiguous() and v_packed.is_contiguous(), "packed dst on GPU")
    _need(indices_packed.dtype == torch.int64 and cu_seqlens_topk.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32,
          "indices int64, cu_seqlens int32")
    _need(cu_seqlens_topk.numel() == bs * H + 1 and cu_seqlens_k.numel() == bs * H + 1, "cu_seqlens must have V+1 entries")
    total_k = k_packed.shape[0]
    _lib.check(_lib.lib().pkv_gather_uva_packed(
        _p(src_k), _p(src_v), src_len, _p(indices_packed), _p(cu_seqlens_topk), _p(cu_seqlens_k), sink_local_end,
        max(1, global_k), _p(k_packed), _p(v_packed), total_k, bs, H, D * src_k.element_size(), _stream(k_packed)))


# --------------------------------------------------------- decode attention


class DecodeAttention:
    """softmax(q k^T * scale) v for one query token per sequence over up to four row segments of
    [bs, Hkv, rows, 128] K/V tensors, read in place (cache_hub/polar_cache.py:1084-1105)."""

    def __init__(self, bs: int, n_kv_heads: int, group: int, max_keys: int, device):
        self.bs, self.H, self.G = bs, n_kv_heads, group
        self.max_keys = max_keys
        nbytes = _lib.lib().pkv_decode_attention_ws_bytes(bs, n_kv_heads, group, max(1, max_keys))
        self.ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        self._segs = (_lib.AttnSegment * 4)()  # reused between calls: filling it is most of the host time

    def run(self, queries: torch.Tensor, segments, scale: float = None, out: torch.Tensor = None,
            row_keys: torch.Tensor = None) -> torch.Tensor:
        """queries [bs,1,Hq,128] (or [bs,Hq,128]); segments: list of (k, v, row0, n_rows) or (k, v, row0, n_rows, idx)
        with k, v [bs,Hkv,rows,128] tensors whose rows are contiguous.  Without ``idx`` a segment is rows
        row0 .. row0+n_rows-1; with ``idx`` (int64 [bs,Hkv,>=n_rows] on the GPU) it is rows row0 + idx[b,h,j], read in
        place (values outside the tensor are clamped).  row_keys: optional int32 [bs,Hkv] number of keys (in
        concatenated order) each row attends to.  Returns a tensor shaped like `queries`."""
        q = queries if queries.is_contiguous() else queries.contiguous()
        segs, out, scale = self._prepare(q, segments, scale, out, row_keys, self._segs)
        _lib.check(_lib.lib().pkv_decode_attention(_p(q), _dt(q.dtype), self.bs, self.H, self.G, segs, len(segments),
                                                   _p(row_keys), float(scale), _p(out), _p(self.ws), self.ws.numel(),
                                                   _stream(q)))
        return out

    def _prepare(self, q, segments, scale, out, row_keys, segs):
        """Validate and fill the C segment array `segs`; returns (segs, out, scale)."""
        _cuda(q)
        _need(q.shape[-1] == HEAD_DIM and q.numel() == self.bs * self.H * self.G * HEAD_DIM, "queries: [bs,1,Hq,128]")
        _need(1 <= len(segments) <= 4, "1..4 key segments")
        for i, seg in enumerate(segments):
            k, v, row0, n_rows = seg[:4]
            idx = seg[4] if len(seg) > 4 else None
            _cuda(k, v)
            _need(k.dtype == q.dtype and v.dtype == q.dtype, "q, k, v must share a dtype")
            _need(k.dim() == 4 and k.shape == v.shape and k.stride() == v.stride() and k.shape[3] == HEAD_DIM and
                  k.stride(3) == 1 and k.stride(2) == HEAD_DIM and tuple(k.shape[:2]) == (self.bs, self.H),
                  "k, v: [bs,Hkv,rows,128] with contiguous rows")
            segs[i].k, segs[i].v = _p(k), _p(v)
            segs[i].stride_b, segs[i].stride_h = k.stride(0), k.stride(1)
            segs[i].row0, segs[i].n_rows = row0, n_rows
            if idx is None:
                _need(0 <= row0 and row0 + n_rows <= k.shape[2], "segment rows out of range")
                segs[i].idx, segs[i].idx_stride, segs[i].idx_limit = None, 0, 0
            else:  # the segment's rows are row0 + idx[b, h, :n_rows], read where they lie
                _cuda(idx)
                _need(idx.dtype == torch.int64 and idx.is_contiguous() and idx.dim() == 3 and
                      tuple(idx.shape[:2]) == (self.bs, self.H) and idx.shape[2] >= n_rows and 0 <= row0 < k.shape[2],
                      "segment indices: contiguous int64 [bs,Hkv,>=n_rows]")
                segs[i].idx, segs[i].idx_stride, segs[i].idx_limit = _p(idx), idx.shape[2], k.shape[2] - row0
        if out is None:
            out = torch.empty_like(q)
        if scale is None:
            scale = 1.0 / math.sqrt(HEAD_DIM)
        if row_keys is not None:
            _cuda(row_keys)
            _need(row_keys.dtype == torch.int32 and row_keys.is_contiguous() and row_keys.numel() == self.bs * self.H,
                  "row_keys: contiguous int32 [bs,Hkv]")
        return segs, out, scale

    def c_args(self, q, segments, scale=None, out=None, row_keys=None):
        """(pkv_attn_args, out) for pkv_decode_step: the same call as :meth:`run`, deferred."""
        a = _lib.AttnArgs()
        _, out, scale = self._prepare(q, segments, scale, out, row_keys, a.segments)
        a.n_segments, a.row_keys, a.scale = len(segments), _p(row_keys), float(scale)
        a.out, a.ws, a.ws_bytes = _p(out), _p(self.ws), self.ws.numel()
        return a, out


def qk_norm_rope(qkv: torch.Tensor, n_q_heads: int, n_kv_heads: int, q_weight, k_weight, eps: float,
                 cos_row: torch.Tensor, sin_row: torch.Tensor, table_for=None, append=None):
    """Per-head RMSNorm of q and k plus rotary embedding for one decode token per sequence, one launch
    (model_hub/qwen.py:327-340, 410-431, 434-498).  qkv bf16 [bs,1,(Hq+2Hkv)*128] (last dim contiguous); cos_row /
    sin_row bf16 [64] of the token's position.  Returns (q [bs,1,Hq,128], k [bs,1,Hkv,128]).
    ``table_for``: a :class:`BoundStep` / :class:`BoundAdaptiveStep` whose retrieval will run on the returned q next:
    the same launch then also leaves the retrieval's rotated query and vote table in that step's workspace
    (pkv_qk_norm_rope_table) and the step's next launch skips its query-prep kernel.
    ``append`` (with ``table_for`` only): (dst_k, dst_v, slot) - the launch also writes the token's key (as returned) and
    value (as it stands in qkv) to row ``slot`` of the cache's dense bf16 K/V tensors [bs,Hkv,rows,128], which is
    what :func:`append_kv` does with them in a launch of its own."""
    bs = qkv.shape[0]
    _need(qkv.is_cuda and qkv.dtype == torch.bfloat16 and qkv.stride(-1) == 1 and qkv.numel() == bs * qkv.shape[-1] and
          qkv.shape[-1] >= (n_q_heads + 2 * n_kv_heads) * HEAD_DIM, "qkv: bf16 [bs,1,(Hq+2Hkv)*128]")
    for t in (cos_row, sin_row):
        _need(t.is_cuda and t.dtype == torch.bfloat16 and t.numel() == HEAD_DIM // 2 and t.is_contiguous(), "cos/sin: bf16 [64]")
    for t in (q_weight, k_weight):
        _need(t is None or (t.is_cuda and t.dtype == torch.bfloat16 and t.numel() == HEAD_DIM and t.is_contiguous()),
              "norm weights: bf16 [128]")
    q = torch.empty(bs, 1, n_q_heads, HEAD_DIM, dtype=torch.bfloat16, device=qkv.device)
    k = torch.empty(bs, 1, n_kv_heads, HEAD_DIM, dtype=torch.bfloat16, device=qkv.device)
    _need(append is None or table_for is not None, "append rides on the launch that builds the vote table")
    if table_for is not None:
        app = None
        if append is not None:
            dk, dv, slot = append
            _need(dk.is_cuda and dv.is_cuda and dk.dtype == torch.bfloat16 and dv.dtype == torch.bfloat16 and
                  dk.shape == dv.shape and dk.stride() == dv.stride() and dk.dim() == 4 and
                  tuple(dk.shape[:2]) == (bs, n_kv_heads) and dk.shape[3] == HEAD_DIM and dk.stride(3) == 1 and
                  dk.stride(2) == HEAD_DIM and 0 <= slot < dk.shape[2],
                  "append: dst_k, dst_v bf16 [bs,Hkv,rows,128] with contiguous rows, 0 <= slot < rows")
            ka = _lib.KvAppend(dk.data_ptr(), dv.data_ptr(), dk.stride(0), dk.stride(1), dk.shape[2], int(slot))
            app = C.byref(ka)
        _lib.check(_lib.lib().pkv_qk_norm_rope_table(_p(qkv), qkv.stride(0), n_q_heads, _p(q_weight), _p(k_weight), float(eps),
                                                     _p(cos_row), _p(sin_row), _p(q), _p(k), table_for._ra, table_for._ws,
                                                     table_for._ws_bytes, app, _stream(qkv)))
        table_for.a.table_ready = 1   # consumed (and reset) by the step's next launch
        return q, k
    _lib.check(_lib.lib().pkv_qk_norm_rope(_p(qkv), qkv.stride(0), bs, n_q_heads, n_kv_heads, _p(q_weight), _p(k_weight),
                                           float(eps), _p(cos_row), _p(sin_row), _p(q), _p(k), _stream(qkv)))
    return q, k


def add_rmsnorm(x: torch.Tensor, residual, weight: torch.Tensor, eps: float, want_sum: bool = True):
    """(x + residual, RMSNorm(x + residual) * weight) over the last dimension in one launch; ``residual`` may be None.
    bf16, contiguous (model_hub/LLM.py:186-193, qwen.py:395-407)."""
    width = x.shape[-1]
    rows = x.numel() // width
    _need(x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and weight.dtype == torch.bfloat16 and
          weight.numel() == width and weight.is_contiguous(), "x: contiguous bf16 [..., width]; weight bf16 [width]")
    _need(residual is None or (residual.shape == x.shape and residual.dtype == x.dtype and residual.is_contiguous()),
          "residual must match x")
    out_sum = torch.empty_like(x) if (want_sum and residual is not None) else None
    out_norm = torch.empty_like(x)
    _lib.check(_lib.lib().pkv_add_rmsnorm(_p(x), _p(residual), _p(weight), float(eps), rows, width, _p(out_sum), _p(out_norm),
                                          _stream(x)))
    return (out_sum if out_sum is not None else x), out_norm


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate_up[..., :n]) * gate_up[..., n:] with n = width / 2, bf16, one launch (model_hub/qwen.py:377-381)."""
    width = gate_up.shape[-1]
    inter = width // 2
    rows = gate_up.numel() // width
    _need(gate_up.is_cuda and gate_up.dtype == torch.bfloat16 and gate_up.is_contiguous() and width % 16 == 0,
          "gate_up: contiguous bf16 [..., 2n] with n a multiple of 8")
    out = torch.empty(*gate_up.shape[:-1], inter, dtype=gate_up.dtype, device=gate_up.device)
    _lib.check(_lib.lib().pkv_silu_mul(_p(gate_up), width, rows, inter, _p(out), _stream(gate_up)))
    return out


def alloc_pinned(shape, dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
    """Pinned, device-mapped host tensor of exactly the requested size, optionally zero-filled (``pkv_host_alloc_mapped`` =
    hipHostMalloc).  torch's own pinned allocator rounds every block up to a power of two, which nearly doubles the
    host footprint of an offloaded K/V store whose per-layer tensors are just over 1 GiB (72 x 1.07 GiB become
    144 GiB); these blocks are freed when the tensor and its views are gone."""
    import weakref

    import numpy as np

    n_elems = 1
    for d in shape:
        n_elems *= int(d)
    esz = torch.empty((), dtype=dtype).element_size()
    nbytes = max(1, n_elems * esz)
    ptr = C.c_void_p()
    _lib.check(_lib.lib().pkv_host_alloc_mapped(nbytes, C.byref(ptr)))
    buf = (C.c_uint8 * nbytes).from_address(ptr.value)
    arr = np.frombuffer(buf, dtype=np.uint8, count=nbytes)
    weakref.finalize(buf, _lib.lib().pkv_host_free, C.c_void_p(ptr.value))   # arr and every tensor view keep buf alive
    t = torch.from_numpy(arr)
    if zero:
        t.zero_()
    return t[:n_elems * esz].view(dtype).view(*shape)


def gather_cpu(src: torch.Tensor, index: torch.Tensor, out: torch.Tensor, n_threads: int = 1) -> None:
    """Host gather [B,H,N,D] -> [B,H,K,D] (cache_hub/gather/gather_cpu.cpp contract)."""
    _need(src.is_cpu and index.is_cpu and out.is_cpu, "src, index and out must be on CPU")
    _need(src.dim() == 4 and index.dim() == 3 and out.dim() == 4, "src [B,H,N,D], index [B,H,K], out [B,H,K,D]")
    _need(index.dtype == torch.int64 and index.is_contiguous(), "index must be contiguous int64")
    _need(src.dtype == out.dtype, "src/out dtype must match")
    Bn, H, N, D = src.shape
    K = index.shape[2]
    _need(tuple(index.shape[:2]) == (Bn, H) and tuple(out.shape) == (Bn, H, K, D), "shape mismatch")
    ss = (C.c_int64 * 4)(*src.stride())
    os_ = (C.c_int64 * 4)(*out.stride())
    _lib.check(_lib.lib().pkv_gather_cpu(_p(src), ss, _p(index), _p(out), os_, Bn, H, N, D, K, src.element_size(), n_threads))


# ------------------------------------------------------- fused decode step


class BoundStep:
    """The argument blocks of one layer's pkv_decode_step, validated once.  A launch patches only what moves with
    every token: the query and output pointers and, through ``a`` / ``segs``, the caller's row counts.  Filling and
    checking the blocks costs more host time than the seven launches themselves, which matters when the K/V live in
    HBM and the GPU side of a step is a few tens of microseconds."""

    __slots__ = ("a", "aa", "segs", "keep", "_ra", "_raa", "_ws", "_ws_bytes", "_fn", "_numel", "_dtype")

    def __init__(self, plan, a, aa, keep, q):
        self.a, self.aa, self.segs, self.keep = a, aa, aa.segments, keep
        self._ra, self._raa = C.byref(a), C.byref(aa)
        self._ws, self._ws_bytes = _p(plan.ws), plan.ws.numel()
        self._fn = _lib.lib().pkv_decode_step
        self._numel, self._dtype = q.numel(), q.dtype

    def launch(self, q: torch.Tensor) -> torch.Tensor:
        """q: contiguous [bs,1,Hq,128] of the bound dtype.  Returns the attention output, shaped like q."""
        _need(q.is_cuda and q.is_contiguous() and q.numel() == self._numel and q.dtype == self._dtype,
              "queries must be contiguous [bs,1,Hq,128] of the cache dtype")
        out = torch.empty_like(q)
        self.a.q, self.aa.out = q.data_ptr(), out.data_ptr()
        rc = self._fn(self._ra, self._ws, self._ws_bytes, self._raa, torch.cuda.current_stream(q.device).cuda_stream)
        self.a.table_ready = 0  # a table left by qk_norm_rope(table_for=self) serves one launch
        if rc != 0:
            _lib.check(rc)
        return out


class BoundAdaptiveStep:
    """:class:`BoundStep` for the adaptive-k step (pkv_adaptive_decode_step): three argument blocks, validated once.
    The caller patches what moves with every token (``ad.dense_rows``, ``ad.row_keys_base``, ``segs[0].n_rows``)."""

    __slots__ = ("a", "ad", "aa", "segs", "keep", "_ra", "_rad", "_raa", "_ws", "_ws_bytes", "_fn", "_numel", "_dtype")

    def __init__(self, plan, a, ad, aa, keep, q):
        self.a, self.ad, self.aa, self.segs, self.keep = a, ad, aa, aa.segments, keep
        self._ra, self._rad, self._raa = C.byref(a), C.byref(ad), C.byref(aa)
        self._ws, self._ws_bytes = _p(plan.ws), plan.ws.numel()
        self._fn = _lib.lib().pkv_adaptive_decode_step
        self._numel, self._dtype = q.numel(), q.dtype

    def launch(self, q: torch.Tensor) -> torch.Tensor:
        """q: contiguous [bs,1,Hq,128] of the bound dtype.  Returns the attention output, shaped like q."""
        _need(q.is_cuda and q.is_contiguous() and q.numel() == self._numel and q.dtype == self._dtype,
              "queries must be contiguous [bs,1,Hq,128] of the cache dtype")
        out = torch.empty_like(q)
        self.a.q, self.aa.out = q.data_ptr(), out.data_ptr()
        rc = self._fn(self._ra, self._ws, self._ws_bytes, self._rad, self._raa,
                      torch.cuda.current_stream(q.device).cuda_stream)
        self.a.table_ready = 0  # a table left by qk_norm_rope(table_for=self) serves one launch
        if rc != 0:
            _lib.check(rc)
        return out


def _retrieve_args(bs, H, group, cap, queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys,
                   tier_counts, n_cand, k, out_ids, out_scores, gather, candidates_only, any_order=False,
                   record_word_offset=0):
    """Validate one retrieval's operands (key-major storage of ``cap`` keys per row) and return its C argument block."""
    q = queries.reshape(bs, -1, HEAD_DIM)
    _need(q.is_contiguous() and q.shape[1] == H * group, "queries must be contiguous [bs,1,Hq,128]")
    a = _lib.RetrieveArgs()
    a.q, a.dtype, a.bs, a.n_kv_heads, a.group = q.data_ptr(), _dt(q.dtype), bs, H, group
    a.signs, a.centers, a.cluster_counts = signs.data_ptr(), centers.data_ptr(), cluster_counts.data_ptr()
    _need(cluster_counts.is_contiguous(), "cluster_counts must be contiguous")
    _need(codes_km.is_contiguous() and codes_km.shape[2] == cap, "codes must be contiguous [bs,H,cap,16]")
    for t in (nib_km, w_km):  # packed, or views into a wider per-key record
        _need(t.shape[2] == cap and t.stride(3) == 1 and t.stride(1) == cap * t.stride(2) and
              t.stride(0) == H * t.stride(1), "key-major nibbles / weights: [bs,H,cap,*] rows at one uniform key stride")
    a.codes, a.nib, a.weight = codes_km.data_ptr(), nib_km.data_ptr(), w_km.data_ptr()
    a.nib_key_stride, a.weight_key_stride = nib_km.stride(2), w_km.stride(2) * w_km.element_size()
    _need(record_word_offset == 0 or (record_word_offset % 4 == 0 and 64 <= record_word_offset <= nib_km.stride(2) - 4),
          "record_word_offset must name a 4-byte word of the key record outside its nibbles")
    a.record_word_offset = int(record_word_offset)
    a.cap, a.key0, a.n_keys = cap, key0, n_keys
    for i, t in enumerate(tier_counts):
        a.tier_counts[i] = int(t)
    a.n_tiers, a.n_cand, a.k = len(tier_counts), n_cand, k
    a.out_ids = None if candidates_only else out_ids.data_ptr()
    a.out_scores = out_scores.data_ptr() if out_scores is not None else None
    a.any_order = int(bool(any_order))
    if gather is not None:
        sk, sv, dk, dv = gather["src_k"], gather["src_v"], gather["dst_k"], gather["dst_v"]
        a.src_k, a.src_v, a.gather_from_host = sk.data_ptr(), sv.data_ptr(), int(bool(gather["from_host"]))
        a.src_len, a.idx_offset = sk.shape[2], int(gather.get("idx_offset", 0))
        a.dst_k, a.dst_v, a.dst_len, a.dst_row0 = dk.data_ptr(), dv.data_ptr(), dk.shape[2], int(gather.get("dst_row0", 0))
        a.row_bytes = sk.shape[3] * sk.element_size()
    return a


def retrieve_noalloc(queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, k,
                     out_ids, out_scores=None, gather=None, any_order=False, launch_plan=0):
    """One layer's retrieval through ``pkv_retrieve_noalloc``: the call of :meth:`RetrievePlan.run` for callers that may
    not allocate device memory.  The workspace is a fixed array inside the library (one per GPU, shared by every call
    on that GPU: overlapping calls race), so no plan is needed; ``out_ids`` int64 [bs,H,k] (and the optional
    ``out_scores`` / gather destinations) are the caller's.  Shapes beyond ``pkv_retrieve_noalloc_max_bytes()`` raise."""
    bs, H, cap = codes_km.shape[0], codes_km.shape[1], codes_km.shape[2]
    group = queries.numel() // (bs * H * HEAD_DIM)
    _cuda(queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, out_ids, out_scores)
    _need(out_ids.dtype == torch.int64 and out_ids.is_contiguous() and out_ids.numel() == bs * H * k,
          "out_ids: contiguous int64 [bs,H,k]")
    _need(out_scores is None or (out_scores.dtype == torch.float32 and out_scores.is_contiguous() and
                                 out_scores.numel() == bs * H * k), "out_scores: contiguous float32 [bs,H,k]")
    a = _retrieve_args(bs, H, group, cap, queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys,
                       tier_counts, n_cand, k, out_ids, out_scores, gather, False, any_order)
    a.launch_plan = int(launch_plan)
    _lib.check(_lib.lib().pkv_retrieve_noalloc(C.byref(a), _stream(codes_km)))
    return out_ids


class RetrievePlan:
    """Persistent workspace + argument block for :func:`pkv_retrieve` on key-major storage."""

    def __init__(self, bs: int, n_kv_heads: int, group: int, cap: int, device, max_keys: int, max_cand: int, max_k: int):
        self.bs, self.H, self.group, self.cap, self.device = bs, n_kv_heads, group, cap, device
        self.rows = bs * n_kv_heads
        nbytes = _lib.lib().pkv_retrieve_ws_bytes(self.rows, max_keys, max_cand, max_k)
        _need(nbytes > 0, "bad retrieval shape")
        # the layout depends on (n_keys, n_cand); size for the worst case of each segment
        self.ws = torch.empty(int(nbytes) + (1 << 16), dtype=torch.uint8, device=device)
        self.max = (max_keys, max_cand, max_k)
        # pkv_retrieve_args.launch_plan / skip_vote_counts of every argument block this plan fills: 0 = the stages
        # before the top-k as three launches, 1 = as one launch where the shape allows it; skip_vote_counts = the
        # u8 vote counts need not reach the workspace (callers that never look at the "cnt_u8" view)
        self.launch_plan = _lib.PLAN_SEPARATE
        self.skip_vote_counts = False

    def run_candidates(self, queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts,
                       n_cand):
        """Collision vote + candidate select + 4-bit rerank only.  Returns (cand int64 [bs,H,n_cand] in the select's
        fixed order, scores float32 [bs,H,n_cand]) as views of the workspace, valid until the next run."""
        self.run(queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, 1,
                 candidates_only=True)
        cand = self.view("cand", n_keys, n_cand, 1, torch.int64).view(self.bs, self.H, n_cand)
        scores = self.view("scores", n_keys, n_cand, 1, torch.float32).view(self.bs, self.H, n_cand)
        return cand, scores

    def _fill(self, queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, k,
              out_ids, out_scores, gather, candidates_only, any_order=False, record_word_offset=0):
        """Validate one retrieval's operands and return its C argument block (the workspace grows if it must)."""
        need = _lib.lib().pkv_retrieve_ws_bytes(self.rows, n_keys, n_cand, k)
        _need(need > 0, "need 0 < k <= n_cand <= n_keys")
        if need > self.ws.numel():
            self.ws = torch.empty(int(need), dtype=torch.uint8, device=self.device)
        a = _retrieve_args(self.bs, self.H, self.group, self.cap, queries, signs, centers, cluster_counts, codes_km,
                           nib_km, w_km, key0, n_keys, tier_counts, n_cand, k, out_ids, out_scores, gather,
                           candidates_only, any_order, record_word_offset)
        a.launch_plan, a.skip_vote_counts = int(self.launch_plan), int(bool(self.skip_vote_counts))
        return a

    def run(self, queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, k,
            out_ids=None, out_scores=None, gather=None, candidates_only=False, attention=None, any_order=False):
        """Returns out_ids int64 [bs,H,k] in descending score order, or, with ``any_order``, the same ids in an
        unspecified fixed order (the final sort is left out; enough for gather + attention).  ``gather`` = dict(src_k, src_v, from_host, idx_offset, dst_k, dst_v, dst_row0).
        ``attention`` = (DecodeAttention, segments, out or None): the attention over those segments is launched by the
        same C call, after the gather (pkv_decode_step); the output tensor is then in ``self.attn_out``."""
        lib = _lib.lib()
        if out_ids is None and not candidates_only:
            out_ids = torch.empty(self.bs, self.H, k, dtype=torch.int64, device=self.device)
        a = self._fill(queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, k,
                       out_ids, out_scores, gather, candidates_only, any_order)
        if attention is None:
            _lib.check(lib.pkv_retrieve(C.byref(a), _p(self.ws), self.ws.numel(), _stream(self.ws)))
        else:
            att, segments, att_out = attention
            _need(not candidates_only, "attention needs the final top-k")
            qq = queries if queries.is_contiguous() else queries.contiguous()
            aa, self.attn_out = att.c_args(qq, segments, out=att_out)
            _lib.check(lib.pkv_decode_step(C.byref(a), _p(self.ws), self.ws.numel(), C.byref(aa), _stream(self.ws)))
        return out_ids

    def bind(self, queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, k,
             out_ids, gather, att, segments, any_order=False):
        """Validate everything :meth:`run` would and keep the two argument blocks of pkv_decode_step for repeated
        launches with the same operands (one layer between two index refreshes): see :class:`BoundStep`."""
        a = self._fill(queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, k,
                       out_ids, None, gather, False, any_order)
        aa, _ = att.c_args(queries, segments, out=queries)  # out is patched at every launch
        keep = (signs, centers, cluster_counts, codes_km, nib_km, w_km, out_ids, gather, att, segments, self.ws)
        return BoundStep(self, a, aa, keep, queries)

    def bind_adaptive(self, queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts,
                      n_cand, adaptive: dict, att, segments):
        """The adaptive-k step of one layer as a :class:`BoundAdaptiveStep`.  ``adaptive``: dense_k [bs,H,rows,128],
        dense_rows, dense_vnorm fp32 [bs,H,rows], dense_logits fp32 [bs,H,>=rows] scratch, scale, value_norm fp32
        [bs,H,cap] (packed, or the :func:`record_value_norm_view` with ``record_word_offset`` = its byte offset: the
        rerank then hands the candidates' norms over and no second gather runs), vn_offset, threshold, k_out, k_min, k_max, adaptive_k int64 [bs,H], topk_ids int64 (>= bs*H*k_out
        elements), row_keys int32 [bs,H], row_keys_base, optional uniform_k int64 [bs,H] (then every row gathers and
        attends to max(adaptive_k) ids), ws uint8 (pkv_adaptive_topk_ws_bytes), src_k / src_v pinned
        CPU [bs,H,len,128], dst_k / dst_v GPU [bs,H,>=k_out,128].  ``segments`` are the attention's; its per-row key
        count is ``row_keys``."""
        d = adaptive
        a = self._fill(queries, signs, centers, cluster_counts, codes_km, nib_km, w_km, key0, n_keys, tier_counts, n_cand, 1,
                       None, None, None, True, record_word_offset=int(d.get("record_word_offset", 0)))
        bs, H = self.bs, self.H
        dk, dvn, dl, vn = d["dense_k"], d["dense_vnorm"], d["dense_logits"], d["value_norm"]
        ak, ids, rk, ws = d["adaptive_k"], d["topk_ids"], d["row_keys"], d["ws"]
        sk, sv, tk, tv = d["src_k"], d["src_v"], d["dst_k"], d["dst_v"]
        k_out = int(d["k_out"])
        _cuda(dk, dvn, dl, vn, ak, ids, rk, ws, tk, tv)
        _need(dk.dtype == queries.dtype and tuple(dk.shape[:2]) == (bs, H) and dk.shape[3] == HEAD_DIM and
              dk.stride(3) == 1 and dk.stride(2) == HEAD_DIM, "dense_k: [bs,H,rows,128] with contiguous rows")
        for t in (dvn, dl):
            _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape[:2]) == (bs, H),
                  "dense_vnorm / dense_logits: contiguous fp32 [bs,H,*]")
        _need(vn.dtype == torch.float32 and vn.dim() == 3 and tuple(vn.shape[:2]) == (bs, H) and vn.stride(2) >= 1 and
              vn.stride(1) == vn.shape[2] * vn.stride(2) and (bs == 1 or vn.stride(0) == H * vn.stride(1)),
              "value_norm: fp32 [bs,H,cap] with one uniform position stride")
        if d.get("record_word_offset", 0):  # the norms the rerank passes through must be the ones value_norm names
            _need(vn.data_ptr() == nib_km.data_ptr() + int(d["record_word_offset"]) and
                  vn.stride(2) * 4 == nib_km.stride(2) and int(d["vn_offset"]) == key0,
                  "record_word_offset: value_norm must be the view of that word of the key records")
        _need(0 < int(d["dense_rows"]) <= min(dl.shape[2], dvn.shape[2], dk.shape[2]),
              "dense_rows exceeds dense_k / dense_logits / dense_vnorm")
        _need(0 < k_out <= n_cand, "k_out must be in (0, n_cand]")
        _need(ak.dtype == torch.int64 and ak.is_contiguous() and ak.numel() == bs * H and ids.dtype == torch.int64 and
              ids.is_contiguous() and ids.numel() >= bs * H * k_out and rk.dtype == torch.int32 and rk.is_contiguous() and
              rk.numel() == bs * H, "adaptive_k / topk_ids / row_keys: contiguous int64 / int64 / int32 of the step's size")
        need = _lib.lib().pkv_adaptive_topk_ws_bytes(self.rows, n_cand, k_out)
        _need(ws.dtype == torch.uint8 and ws.is_contiguous() and ws.numel() >= need, "adaptive workspace too small")
        _need(sk.is_cpu and sv.is_cpu and sk.is_pinned() and sv.is_pinned() and sk.is_contiguous() and sv.is_contiguous() and
              sk.shape == sv.shape and tuple(sk.shape[:2]) == (bs, H) and sk.dtype == queries.dtype,
              "src_k / src_v: contiguous pinned CPU [bs,H,len,128] of the query dtype")
        _need(tk.is_contiguous() and tv.is_contiguous() and tk.shape == tv.shape and tuple(tk.shape[:2]) == (bs, H) and
              tk.shape[2] >= k_out and tk.dtype == queries.dtype, "dst_k / dst_v: contiguous GPU [bs,H,>=k_out,128]")
        ad = _lib.AdaptiveArgs()
        ad.dense_k, ad.dense_stride_b, ad.dense_stride_h, ad.dense_rows = dk.data_ptr(), dk.stride(0), dk.stride(1), int(d["dense_rows"])
        ad.dense_vnorm, ad.dense_vnorm_stride = dvn.data_ptr(), dvn.shape[2]
        ad.dense_logits, ad.dense_logits_stride = dl.data_ptr(), dl.shape[2]
        ad.scale, ad.value_norm, ad.vn_stride, ad.vn_offset = float(d["scale"]), vn.data_ptr(), vn.stride(1), int(d["vn_offset"])
        ad.vn_pos_stride = vn.stride(2)
        ad.threshold, ad.k_out, ad.k_min, ad.k_max = float(d["threshold"]), k_out, int(d["k_min"]), int(d["k_max"])
        ad.adaptive_k, ad.topk_ids, ad.row_keys, ad.row_keys_base = ak.data_ptr(), ids.data_ptr(), rk.data_ptr(), int(d["row_keys_base"])
        uk = d.get("uniform_k")
        if uk is not None:
            _cuda(uk)
            _need(uk.dtype == torch.int64 and uk.is_contiguous() and uk.numel() == bs * H, "uniform_k: contiguous int64 [bs,H]")
            ad.uniform_k = uk.data_ptr()
        ad.ws, ad.ws_bytes = ws.data_ptr(), ws.numel()
        ad.src_k, ad.src_v, ad.src_len, ad.idx_offset = sk.data_ptr(), sv.data_ptr(), sk.shape[2], int(d.get("idx_offset", 0))
        ad.dst_k, ad.dst_v, ad.dst_len, ad.dst_row0 = tk.data_ptr(), tv.data_ptr(), tk.shape[2], 0
        ad.row_bytes = HEAD_DIM * sk.element_size()
        aa, _ = att.c_args(queries, segments, out=queries, row_keys=rk)  # out is patched at every launch
        keep = (signs, centers, cluster_counts, codes_km, nib_km, w_km, d, att, segments, self.ws)
        return BoundAdaptiveStep(self, a, ad, aa, keep, queries)

    def view(self, name: str, n_keys: int, n_cand: int, k: int, dtype: torch.dtype) -> torch.Tensor:
        """An intermediate of the last :meth:`run` (qhat, qnorm, lut, cnt_u8, chunk_hist, cand, scores)."""
        ptr, nbytes = C.c_void_p(), C.c_size_t()
        _lib.check(_lib.lib().pkv_retrieve_ws_view(_p(self.ws), self.rows, n_keys, n_cand, k, name.encode(), C.byref(ptr),
                                                   C.byref(nbytes)))
        off = ptr.value - self.ws.data_ptr()
        return self.ws[off:off + nbytes.value].view(dtype)
