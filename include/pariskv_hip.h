/*
 * pariskv_hip.h -- C ABI of libpariskv_hip.so: ParisKV's per-decode-step KV
 * retrieval path as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - Every function returns 0 on success or a negative PKV_E* code;
 *     pkv_last_error() gives the message of the calling thread's last failure
 *     (the Python shims raise RuntimeError with it, like the reference's
 *     TORCH_CHECKs).
 *   - The caller owns every buffer, workspaces and outputs included; nothing
 *     is allocated or freed behind the caller's back (pkv_host_alloc_mapped /
 *     pkv_host_free excepted, which exist to allocate).
 *   - All device work is enqueued on `stream` (a hipStream_t passed as void*);
 *     no call synchronises, none touches the default stream on its own.
 *   - Strides are in ELEMENTS of the pointed-to type unless a name says bytes.
 *   - "row" means one (batch, kv-head) pair; R = bs * n_kv_heads.
 *   - Geometry is the reference's default codebook: head_dim 128 = 16 subspaces
 *     x 8 dims, 256 sign centroids per subspace
 *     (turboquant/codebooks/codebook_d128_m8_Kr1_Kw256_rabitq_sign.json).
 *
 * Each entry point cites the reference interface it replaces
 * (paths relative to the ParisKV checkout).
 */
#ifndef PARISKV_HIP_H
#define PARISKV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

#define PKV_OK 0
#define PKV_EINVAL (-22)   /* bad argument (shape, stride, alignment, range) */
#define PKV_ENOMEM (-12)   /* workspace too small / host allocation failed */
#define PKV_EHIP (-5)      /* a HIP runtime call failed */

#define PKV_DTYPE_F32 0
#define PKV_DTYPE_BF16 1

#define PKV_HEAD_DIM 128
#define PKV_SUBSPACES 16
#define PKV_SUBDIM 8
#define PKV_CLUSTERS 256
#define PKV_MAX_TIERS 8

int pkv_version(void);
const char *pkv_last_error(void);
/* sizeof of the argument structs as this library was compiled, for a binding to
 * compare with its own mirror: 0 pkv_attn_segment, 1 pkv_attn_args,
 * 2 pkv_retrieve_args, 3 pkv_adaptive_args (0 for any other number).
 * No counterpart in the reference. */
size_t pkv_struct_bytes(int which);

/* ------------------------------------------------------------------ append */

/* Replaces polar_cache.batch_encode + _count_cluster_keys
 * (cache_hub/polar_cache.py:924-978, 980-996; call sites :484-494, :768-775).
 * keys: [bs][h][n_keys][128] of `dtype` addressed with the given strides
 * (last dim contiguous).  signs: device float[128] of +-1 (SRHT diagonal).
 * For key i of row (b,h), subspace s:
 *   codes[b*cs_b + h*cs_h + i*cs_key + s*cs_sub]            (u8 sign code)
 *   nib  [b*ns_b + h*ns_h + i*ns_key + s*ns_sub + 0..3]     (u8 packed 4-bit)
 *   weight[b*ws_b + h*ws_h + i*ws_key + s*ws_sub]           (bf16 bits)
 * so both the reference's subspace-major tensors and key-major storage are
 * expressible.  cluster_counts (int32 [bs][h][16][256], strides cc_b, cc_h) is
 * incremented (+=, polar_cache.py:775) when non-NULL.  nib/weight may be NULL
 * (return_rabitq=False). */
int pkv_encode_append(const void *keys, int dtype, int bs, int n_kv_heads, int64_t n_keys,
                      int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_key,
                      const float *signs,
                      uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                      uint8_t *nib, int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub,
                      uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key, int64_t ws_sub,
                      int32_t *cluster_counts, int64_t cc_b, int64_t cc_h,
                      void *stream);

/* polar_cache._count_cluster_keys on its own (cache_hub/polar_cache.py:980-996):
 * cluster_counts[b][h][s][code] += 1 for every key and subspace. */
int pkv_count_cluster_keys(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                           int bs, int n_kv_heads, int64_t n_keys,
                           int32_t *cluster_counts, int64_t cc_b, int64_t cc_h, void *stream);

/* ------------------------------------------------------------- query side */

/* Replaces the query half of polar_cache.compute / _encode_query_blocks and the
 * centroid ranking of get_cache_cnt_fused, plus convert_to_bits
 * (cache_hub/polar_cache.py:1027-1031, 905-922, 1216-1222;
 *  cache_hub/collision_fused/collision.cu:71-151).
 * q: [bs][n_kv_heads*group][128] contiguous of `dtype` (the [bs,1,Hq,D] decode
 * query).  cluster_counts as above.  tier_counts: HOST array of n_tiers (1..8)
 * cumulative key thresholds.  Outputs (device): qhat float [R][128],
 * qnorm float [R], lut u8 [R][16][256] (votes a key gets per subspace for each
 * centroid), sorted_ids int64 [R][16][256] or NULL. */
int pkv_query_prep_lut(const void *q, int dtype, int bs, int n_kv_heads, int group,
                       const float *signs,
                       const int32_t *cluster_counts, int64_t cc_b, int64_t cc_h,
                       const uint32_t *tier_counts, int n_tiers,
                       float *qhat, float *qnorm, uint8_t *lut, int64_t *sorted_ids,
                       void *stream);

/* Replaces update_cache_cnt (cache_hub/collision_fused/collision.cu:250-411;
 * python: collison_interface.py:60-86 update_cache_cnt_cuda_interface).
 * sorted_ids int64 [bs][h][16][256] (strides si_b, si_h, si_sub; last dim
 * contiguous), cluster_counts likewise, codes u8 addressed as in
 * pkv_encode_append, tier_counts HOST array (n_tiers 1 or 6 in the reference;
 * 1..8 here).  lut_ws: device workspace of R*16*256 bytes.
 * cnt: int32 [bs][h][n_keys] contiguous. */
int pkv_update_cache_cnt(const int64_t *sorted_ids, int64_t si_b, int64_t si_h, int64_t si_sub,
                         const int32_t *cluster_counts, int64_t cc_b, int64_t cc_h, int64_t cc_sub,
                         const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                         int bs, int n_kv_heads, int64_t n_keys,
                         const uint32_t *tier_counts, int n_tiers,
                         uint8_t *lut_ws, int32_t *cnt, void *stream);

/* Legacy single-tier form: cache_hub/collision/collision.cu:146-276,
 * collision.py:87-98 (update_cache_cnt_cuda).  sorted_ids int32
 * [bs][h][16][256] contiguous, topk_cluster_cnt int32 [bs][h][16], codebook
 * int32 [bs][h][16][n_keys] contiguous.  A key scores 1 per subspace whose
 * code is among the first topk_cluster_cnt ranked clusters. */
int pkv_update_cache_cnt_legacy(const int32_t *sorted_ids, const int32_t *topk_cluster_cnt,
                                const int32_t *codebook, int bs, int n_kv_heads, int64_t n_keys,
                                uint8_t *lut_ws, int32_t *cnt, void *stream);

/* The scan stage of the fused pipeline: votes per key from a ready LUT
 * (the per-key loop of cache_hub/collision_fused/collision.cu:204-228).
 * cnt_u8 [R][n_keys] and/or cnt_i32 [R][n_keys] (either may be NULL, not both).
 * When chunk_suf is non-NULL the pass also leaves the histograms the candidate
 * select needs, in suffix form (suf[t] = number of keys with count >= t):
 * chunk_suf uint16 [R][n_chunks][128] for each `chunk_keys`-key chunk
 * (n_chunks = ceil(n_keys / chunk_keys)) and row_suf uint32 [R][128], which is
 * ADDED to with atomics and must be zero on entry.
 * chunk_keys must be a multiple of 2048 and at most 32768. */
int pkv_collision_scan(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                       int bs, int n_kv_heads, int64_t n_keys, const uint8_t *lut,
                       uint8_t *cnt_u8, int32_t *cnt_i32, uint32_t *row_suf, uint16_t *chunk_suf,
                       int chunk_keys, void *stream);

/* pkv_collision_scan (u8 counts, row stride cnt_u8_stride) as ONE launch whose
 * own begin/end timestamps are returned in *kernel_us: the call blocks until
 * the kernel has finished.  Measurement aid for the benchmark's roofline line;
 * no counterpart in the reference. */
int pkv_collision_scan_timed(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                             int bs, int n_kv_heads, int64_t n_keys, const uint8_t *lut,
                             uint8_t *cnt_u8, int64_t cnt_u8_stride, uint32_t *row_suf, uint16_t *chunk_suf,
                             int chunk_keys, float *kernel_us, void *stream);

/* ------------------------------------------------------------- selections */

/* Replaces bucket_topk / bucket_topk_3d and the integer use of radix_topk_3d
 * (cache_hub/topk/radix_topk.cu:39-120, 258-319; hot call
 * cache_hub/polar_cache.py:1241).  x: int32 [rows][len] (row stride x_stride),
 * values clamped to [0,127].  out: int64 [rows][k]: every index whose value is
 * above the k-th largest value (ascending index), then the smallest indices at
 * that value (ascending).  len == k gives 0..len-1.  ws: device workspace of
 * pkv_bucket_topk_ws_bytes(rows, len) bytes. */
size_t pkv_bucket_topk_ws_bytes(int rows, int64_t len);
int pkv_bucket_topk(const int32_t *x, int64_t x_stride, int rows, int64_t len, int64_t k,
                    int64_t *out, void *ws, size_t ws_bytes, void *stream);

/* Replaces radix_topk / radix_topk_3d on floats (radix_topk.cu:161-239,
 * 323-382) and torch.topk + gather at cache_hub/polar_cache.py:1300-1302.
 * Exact: the k largest of x[rows][len] in descending order, ties by smaller
 * ids[row][i] (by smaller position when ids == NULL).  out_ids int64 [rows][k]
 * = ids[..] (or positions); out_vals float [rows][k] or NULL.
 * ws: pkv_topk_f32_ws_bytes(rows, len, k) bytes. */
size_t pkv_topk_f32_ws_bytes(int rows, int64_t len, int64_t k);
int pkv_topk_f32(const float *x, int64_t x_stride, const int64_t *ids, int64_t ids_stride,
                 int rows, int64_t len, int64_t k, int64_t *out_ids, float *out_vals,
                 void *ws, size_t ws_bytes, void *stream);

/* Replaces partial_rerank (cache_hub/rerank/rerank.cu:141-219; python
 * rerank.py:214-263 partial_rerank_cuda).  cand int64 [bs][h][n_cand]
 * contiguous; nib / weight addressed as in pkv_encode_append with n_keys keys
 * per row; qhat float [R][128], qnorm float [R], centers float[8] (device).
 * scores float [R][n_cand].  v4b (bf16 bits [R][16][n_cand][8], the unpacked
 * values the reference also returns) is written when non-NULL.
 * Candidate indices outside [0,n_keys) score -inf instead of being read. */
int pkv_rerank4(const int64_t *cand, int bs, int n_kv_heads, int64_t n_cand, int64_t n_keys,
                const uint8_t *nib, int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub,
                const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key, int64_t ws_sub,
                const float *qhat, const float *qnorm, const float *centers,
                float *scores, uint16_t *v4b, void *stream);

/* ----------------------------------------------------------------- gathers */

/* Replaces h2d_gather_kv (cache_hub/gather_trans/trans_h2d.cu:79-121; python
 * trans_h2d.py:65-105).  src_k/src_v: pinned, device-mapped HOST memory
 * [bs][h][src_len][row_bytes/2 bf16]; idx int64 [bs][h][k] on the device;
 * dst_k/dst_v device [bs][h][dst_len][...].  Rows are row_bytes bytes
 * (multiple of 16; 256 for head_dim 128 bf16).  Out-of-range indices produce
 * zero rows.  idx_offset is added to every index before addressing src
 * (0 for the offload layout; retrieval_start for pkv_gather_hbm callers,
 * cache_hub/polar_cache.py:1090). */
int pkv_gather_uva(const void *src_k, const void *src_v, int64_t src_len,
                   const int64_t *idx, int64_t k, int64_t idx_offset,
                   void *dst_k, void *dst_v, int64_t dst_len, int64_t dst_row0,
                   int bs, int n_kv_heads, int row_bytes, void *stream);

/* Same contract with src in device memory: the no-offload branch
 * cache_hub/polar_cache.py:1089-1095 (torch.gather over the GPU KV). */
int pkv_gather_hbm(const void *src_k, const void *src_v, int64_t src_len,
                   const int64_t *idx, int64_t k, int64_t idx_offset,
                   void *dst_k, void *dst_v, int64_t dst_len, int64_t dst_row0,
                   int bs, int n_kv_heads, int row_bytes, void *stream);

/* One decode token per sequence written into the K/V stores: replaces the two
 * indexed assignments unified_keys_gpu[layer][:, :, pos, :] = key_states[:, 0]
 * (and values) of decode_update_kv_cache (cache_hub/polar_cache.py:848-856)
 * with one launch.  k_new/v_new: device rows of row_bytes bytes addressed
 * k_new + b*k_stride_b + h*k_stride_h (and likewise for v_new: the two often
 * are slices of one fused projection output with different strides);
 * dst_k/dst_v: device [bs][h][dst_len] rows addressed
 * dst + b*dst_stride_b + h*dst_stride_h + slot*row_bytes.
 * All strides in BYTES, multiples of 16.
 * vnorm (optional, device float, rows of 128 elements only: row_bytes 256 = bf16,
 * 512 = fp32): vnorm[b*vn_stride_b + h*vn_stride_h + slot] = ||v_new[b][h]||_2 in
 * the rows' dtype, widened - the value-norm bookkeeping of the adaptive-k cache
 * (cache_hub/polar_cache_adaptivek_varlen.py:1179) in the same launch; strides in
 * elements. */
int pkv_append_kv(const void *k_new, int64_t k_stride_b, int64_t k_stride_h,
                  const void *v_new, int64_t v_stride_b, int64_t v_stride_h,
                  void *dst_k, void *dst_v, int64_t dst_stride_b, int64_t dst_stride_h, int64_t dst_len,
                  int64_t slot, int bs, int n_kv_heads, int row_bytes,
                  float *vnorm, int64_t vn_stride_b, int64_t vn_stride_h, void *stream);

/* The oldest tokens of a layer leave the GPU: replaces the copy_() of staged
 * [bs][h][n][d] tensors into slices of the pinned host tensors on the side
 * stream (cache_hub/polar_cache.py:457-471 at prefill, :778-799 at an index
 * refresh), which torch executes as a strided device-to-host copy.  One
 * kernel writes the rows through the host store's device mapping:
 *   dst[(b,h)][dst_row0 + r] = src + b*src_stride_b + h*src_stride_h + r*src_stride_row
 * for r < n_rows, K and V.  src: device memory, strides in BYTES (multiples
 * of 16), so the model's [bs][seq][h][d] layout can be read in place;
 * dst_k_host/dst_v_host: pinned, device-mapped host memory
 * [bs][h][dst_len][row_bytes].  Asynchronous on `stream`; the host store is
 * complete when the stream reaches the caller's next event. */
int pkv_offload_rows(const void *src_k, const void *src_v, int64_t src_stride_b, int64_t src_stride_h,
                     int64_t src_stride_row, void *dst_k_host, void *dst_v_host, int64_t dst_len,
                     int64_t dst_row0, int64_t n_rows, int bs, int n_kv_heads, int row_bytes, void *stream);

/* pkv_offload_rows through the copy engines instead of a kernel: the same
 * move (cache_hub/polar_cache.py:457-471, :778-799, where torch issues the
 * copy on a side stream so that it overlaps the model's kernels), as
 * hipMemcpyAsync / hipMemcpy2DAsync commands on `stream`.  A kernel that
 * writes to host memory holds up every other kernel's stores while it runs;
 * the copy engines do not.  Source strides in BYTES, any values >= the
 * extents; dst_*_host: pinned host memory [bs][h][dst_len][row_bytes].
 * flags: PKV_OFFLOAD_ONE_COMMAND = issue one pitched copy per tensor when the
 * source's (b, h) blocks are contiguous and evenly spaced (otherwise, and
 * without the flag, one command per block). */
#define PKV_OFFLOAD_ONE_COMMAND 1
int pkv_offload_rows_dma(const void *src_k, const void *src_v, int64_t src_stride_b, int64_t src_stride_h,
                         int64_t src_stride_row, void *dst_k_host, void *dst_v_host, int64_t dst_len,
                         int64_t dst_row0, int64_t n_rows, int bs, int n_kv_heads, int row_bytes, int flags,
                         void *stream);

/* pkv_gather_uva with a per-row count: row (b, h) moves only its first
 * row_counts[b*h_count + h] selected rows (int64 on the device, values in
 * [0, k]); the other slots of dst are left untouched.  For the adaptive-k
 * cache (cache_hub/polar_cache_adaptivek_varlen.py:1597-1670), whose attention
 * takes the per-row key count: the ragged selection then needs neither the
 * packing of the indices nor a host read of the counts. */
int pkv_gather_uva_ragged(const void *src_k, const void *src_v, int64_t src_len,
                          const int64_t *idx, int64_t k, const int64_t *row_counts, int64_t idx_offset,
                          void *dst_k, void *dst_v, int64_t dst_len, int64_t dst_row0,
                          int bs, int n_kv_heads, int row_bytes, void *stream);

/* Ragged form used by the adaptive-k cache variant (kernel source absent from
 * the reference; contract from the call site
 * cache_hub/polar_cache_adaptivek_varlen.py:1634-1644, layout :1573-1586).
 * For virtual head v = b*h_count + h and slot s < cu_topk[v+1]-cu_topk[v]:
 *   dst row  = cu_k[v] + sink_local_end + s
 *   src row  = idx_packed[cu_topk[v] + s] of (b,h)
 * dst_k/dst_v: [total_k][row_bytes]; cu_* are int32 device arrays [V+1];
 * max_k bounds the per-head slot count (grid bound). */
int pkv_gather_uva_packed(const void *src_k, const void *src_v, int64_t src_len,
                          const int64_t *idx_packed, const int32_t *cu_topk, const int32_t *cu_k,
                          int64_t sink_local_end, int64_t max_k,
                          void *dst_k, void *dst_v, int64_t total_k,
                          int bs, int n_kv_heads, int row_bytes, void *stream);

/* Replaces gather_kv_out_cpu (cache_hub/gather/gather_cpu.cpp:116-170): host
 * gather [B][H][N][D] -> [B][H][K][D], element strides given, `elem_bytes` per
 * element.  Returns PKV_EINVAL if an index is out of range (bounds are checked
 * up front, like the reference's release build). */
int pkv_gather_cpu(const void *src, const int64_t *src_strides4, const int64_t *index,
                   void *out, const int64_t *out_strides4,
                   int64_t B, int64_t H, int64_t N, int64_t D, int64_t K, int elem_bytes,
                   int n_threads);

/* Streaming device copy of `bytes` (multiple of 16) bytes: the known-size kernel
 * against which the HBM traffic counters are calibrated.  No counterpart in the
 * reference. */
int pkv_copy_bytes(const void *src, void *dst, size_t bytes, void *stream);

/* Streaming read of `bytes` bytes with the collision scan's access pattern and
 * no other work (the words are xor-ed into a 256-byte device sink): what a
 * read-only kernel pulls out of HBM on the device at hand, the yardstick
 * beside the published peak.  No counterpart in the reference. */
int pkv_read_bytes(const void *src, size_t bytes, void *sink256, void *stream);

/* Pinned host memory that kernels can read in place (hipHostMalloc, mapped).
 * The reference relies on torch's pin_memory=True for the same purpose
 * (cache_hub/polar_cache.py:226-237). */
int pkv_host_alloc_mapped(size_t bytes, void **host_ptr);
int pkv_host_free(void *host_ptr);
/* Device-visible address of a pinned host pointer (PKV_EINVAL if not pinned). */
int pkv_host_device_pointer(const void *host_ptr, void **dev_ptr);

/* -------------------------------------------------------------- adaptive-k */

/* Replaces adaptive_topk (cache_hub/adaptive_k_fused/adaptive_topk.cu:272-309;
 * python adaptive_topk.py:331-405; semantics adaptive_topk_ref :255-313) and the
 * v2 form whose source is absent from the reference (call site
 * cache_hub/polar_cache_adaptivek_varlen.py:1741-1753).
 * sl_logits/sl_vnorm float [rows][sl] (row strides given) are the exact, already
 * scaled logits and value norms of the dense (sink/local/buffer) tokens.
 * Candidate logit = float(cand_scores[row][i]) * cand_scale with cand_scores
 * [rows][n_cand] of cand_dtype (PKV_DTYPE_F32 with cand_scale 1 for prescaled
 * logits; PKV_DTYPE_BF16 with the attention scale for raw rerank scores).
 * Candidate value norm = cand_vnorm[row][i], or, when cand_vnorm is NULL,
 * value_norm[row*vn_stride + (cand_ids[row][i] + vn_offset)*vn_pos_stride]
 * (vn_pos_stride 0 or 1: packed rows; larger when the norms sit inside wider
 * per-key records; a row then holds vn_stride / vn_pos_stride positions).
 * benefit = exp(logit - max) * ||v||; adaptive_k[row] = smallest k <= k_out with
 * dense_benefit + sum of the k largest candidate benefits >= threshold * total
 * (k_out if never, 1 if total <= 0); topk_ids int64 [rows][k_out] = cand_ids in
 * descending benefit order (ties: candidate position ascending).
 * k_max > 0: adaptive_k is clamped to [k_min, k_max] before it is written (the
 * caller's clamp, polar_cache_adaptivek_varlen.py:1759); row_keys (optional,
 * device int32 [rows]) receives row_keys_base + adaptive_k, the per-row key count
 * that pkv_decode_attention takes.
 * ws: pkv_adaptive_topk_ws_bytes(rows, n_cand, k_out) bytes. */
size_t pkv_adaptive_topk_ws_bytes(int rows, int64_t n_cand, int64_t k_out);
int pkv_adaptive_topk(const float *sl_logits, int64_t sl_stride, const float *sl_vnorm, int64_t slv_stride,
                      int64_t sl, const void *cand_scores, int cand_dtype, float cand_scale,
                      const float *cand_vnorm, const float *value_norm, int64_t vn_stride, int64_t vn_offset,
                      int64_t vn_pos_stride, const int64_t *cand_ids, int64_t n_cand, float threshold, int64_t k_out, int rows,
                      int64_t *adaptive_k, int64_t *topk_ids, int64_t k_min, int64_t k_max,
                      int32_t *row_keys, int64_t row_keys_base, void *ws, size_t ws_bytes, void *stream);

/* uniform_k[r] = max over the rows of adaptive_k (device int64 [rows] each);
 * row_keys (optional, device int32 [rows]) = row_keys_base + that maximum.  The
 * dense form of the adaptive step: every (batch, kv-head) row keeps as many ids
 * as the greediest one, which is how
 * cache_hub/polar_cache_atten_value_indices_adaptive_k.py:1585-1589, 1462-1499
 * sizes its gather and attention (global_k = adaptive_k.max().item()) - here
 * without the host read. */
int pkv_uniform_k(const int64_t *adaptive_k, int rows, int64_t *uniform_k, int32_t *row_keys,
                  int64_t row_keys_base, void *stream);

/* Logits of the dense (sink / local / update buffer) rows against the mean of
 * each KV head's query group: replaces query.mean over the group plus
 * torch.einsum("bhd,bhkd->bhk") .to(float32) * scale
 * (cache_hub/polar_cache_adaptivek_varlen.py:1418-1419, :1731) with one launch.
 * q [bs][1][n_kv_heads*group][128] contiguous, k rows of 128 elements addressed
 * k + b*k_stride_b + h*k_stride_h + r*128 (strides in elements), both of dtype;
 * out float [bs*n_kv_heads][out_stride], first n_rows of each row written.
 * bf16: the mean and the dot product are each rounded to bf16 (fp32 sums in a
 * fixed order), as the torch expressions round them. */
int pkv_dense_logits(const void *q, int dtype, int bs, int n_kv_heads, int group, const void *k,
                     int64_t k_stride_b, int64_t k_stride_h, int64_t n_rows, float scale, float *out,
                     int64_t out_stride, void *stream);

/* --------------------------------------------------------- decode attention */

#define PKV_ATTN_MAX_SEGMENTS 4

/* One run of K/V rows (head_dim 128, rows contiguous: 128 elements apart)
 * inside tensors laid out [bs][n_kv_heads][rows][128]; strides in elements.
 * idx == NULL: rows row0 .. row0+n_rows-1 of every (b, h) take part.
 * idx != NULL (device int64, [bs*n_kv_heads][idx_stride]): row (b, h) attends
 * to rows row0 + idx[(b*n_kv_heads+h)*idx_stride + j], j < n_rows - the
 * selected rows are read where they lie, which replaces the torch.gather of
 * the no-offload branch (cache_hub/polar_cache.py:1089-1095) altogether.
 * Index values are clamped to [0, idx_limit). */
typedef struct pkv_attn_segment {
  const void *k, *v;
  int64_t stride_b, stride_h;
  int64_t row0, n_rows;
  const int64_t *idx;
  int64_t idx_stride, idx_limit;
} pkv_attn_segment;

/* Replaces the torch.cat of sink / top-k / local K and V followed by
 * flash_attn_func (cache_hub/polar_cache.py:1084-1105): softmax(q k^T * scale) v
 * for one query token per sequence, non-causal, over the concatenation of up to
 * PKV_ATTN_MAX_SEGMENTS segments read in place.  q, out: [bs][n_kv_heads*group][128]
 * in `dtype` (query head h*group+g attends with KV head h); 1 <= group <= 8.
 * row_keys (device int32 [bs*n_kv_heads], or NULL): number of keys row (b, h)
 * attends to, counted in the concatenated order - at most the total of the
 * segments; lets the last segment be ragged (per-head adaptive k; the
 * reference packs such rows for flash_attn_varlen_func,
 * cache_hub/polar_cache_adaptivek_varlen.py:1597-1670).
 * ws: pkv_decode_attention_ws_bytes(...) bytes of device memory for the
 * per-split partial results.  fp32 accumulation; result rounded to `dtype`. */
size_t pkv_decode_attention_ws_bytes(int bs, int n_kv_heads, int group, int64_t total_keys);
int pkv_decode_attention(const void *q, int dtype, int bs, int n_kv_heads, int group,
                         const pkv_attn_segment *segments, int n_segments,
                         const int32_t *row_keys, float scale,
                         void *out, void *ws, size_t ws_bytes, void *stream);

/* ------------------------------------------------- decode glue (model side) */

/* One decode token per sequence between the fused QKV projection and the cache:
 * RMSNorm of every query and key head (weights bf16 [128], or both NULL for
 * models without q_norm / k_norm) followed by the rotary embedding in
 * rotate-half form with the position's cos / sin rows (bf16 [64] each).
 * Replaces the split + head_rmsnorm + apply_rotary_pos_emb sequence of the
 * reference's decode step (model_hub/qwen.py:327-340, 410-431, 434-498).
 * qkv: bf16 [bs][stride_b] with the q heads, then the k heads, then v;
 * q_out bf16 [bs][n_q_heads][128], k_out bf16 [bs][n_kv_heads][128].
 * head_dim 128, bf16 only; fp32 arithmetic, one rounding at the end. */
int pkv_qk_norm_rope(const void *qkv, int64_t stride_b, int bs, int n_q_heads, int n_kv_heads,
                     const void *q_weight, const void *k_weight, float eps,
                     const void *cos_row, const void *sin_row, void *q_out, void *k_out, void *stream);

/* out_sum = x + residual (bf16; residual may be NULL: out_sum = x) and
 * out_norm = RMSNorm(out_sum) * weight over the last dimension, one launch:
 * the residual add and the layer norm that follows it in the decode step
 * (model_hub/LLM.py:186-193, qwen.py:395-407).  x, residual, out_* bf16
 * [rows][width]; weight bf16 [width]; width % 8 == 0, at most 16384; out_sum may be NULL. */
int pkv_add_rmsnorm(const void *x, const void *residual, const void *weight, float eps, int rows, int width,
                    void *out_sum, void *out_norm, void *stream);

/* out[r][j] = silu(gate_up[r][j]) * gate_up[r][inter + j] (bf16): the gate of the
 * MLP (model_hub/qwen.py:377-381, flashinfer.activation.silu_and_mul there).
 * gate_up bf16 [rows][row_stride >= 2*inter]; out bf16 [rows][inter]. */
int pkv_silu_mul(const void *gate_up, int64_t row_stride, int rows, int inter, void *out, void *stream);

/* ------------------------------------------------------- fused decode step */

/* One layer's retrieval for one decode step, key-major storage:
 * query prep + LUT -> collision scan -> candidate select -> 4-bit rerank ->
 * exact top-k (-> optional gather).  Equivalent to
 * polar_cache.collision_based_topk_batch (cache_hub/polar_cache.py:1126-1162)
 * followed by the gather at :1075-1095.
 *   codes  u8   [R][cap][16]   (row stride = cap*16),   keys [key0, key0+n_keys)
 *   nib    u8   [R][cap][64]
 *   weight bf16 [R][cap][16]
 * out_ids int64 [R][k] (indices relative to key0, descending score).
 * If src_k != NULL the selected rows are gathered into dst_k/dst_v
 * (gather_from_host selects pkv_gather_uva vs pkv_gather_hbm semantics).
 * out_ids == NULL stops after the rerank (the adaptive-k caller,
 * cache_hub/polar_cache_adaptivek_varlen.py:1494-1496): the candidate ids
 * int64 [R][n_cand] and their scores float [R][n_cand] are then read from the
 * workspace segments "cand" and "scores" (pkv_retrieve_ws_view).
 * ws: pkv_retrieve_ws_bytes(R, n_keys, n_cand, k) bytes of device memory. */
typedef struct pkv_retrieve_args {
  const void *q;            /* [bs][n_kv_heads*group][128] */
  int dtype;                /* PKV_DTYPE_* of q */
  int bs, n_kv_heads, group;
  const float *signs;       /* device float[128] */
  const float *centers;     /* device float[8] */
  const int32_t *cluster_counts; /* [R][16][256] contiguous */
  const uint8_t *codes;
  const uint8_t *nib;
  const uint16_t *weight;
  int64_t cap;              /* keys per row in the three arrays above */
  int64_t key0;             /* first key of the retrieval zone */
  int64_t n_keys;           /* valid retrieval length N */
  uint32_t tier_counts[PKV_MAX_TIERS];
  int n_tiers;
  int64_t n_cand;           /* C */
  int64_t k;                /* K (<= C) */
  int64_t *out_ids;         /* [R][k], or NULL for candidates only */
  float *out_scores;        /* [R][k] or NULL */
  /* optional gather */
  const void *src_k, *src_v;
  int gather_from_host;
  int64_t src_len, idx_offset;
  void *dst_k, *dst_v;
  int64_t dst_len, dst_row0;
  int row_bytes;
  /* 0: out_ids in descending score order (torch.topk's order, cache_hub/polar_cache.py:1300-1302).
   * 1: the same k ids in an unspecified but fixed order (a function of the inputs only), for callers that
   *    use them as a set, as polar_cache.compute does (gather + attention): the final sort is left out. */
  int any_order;
  /* Bytes from one key's 64 nibble bytes (16 weights) to the next key's; 0 = packed arrays (64 / 32).  A key's
   * nibbles and weights are only ever read together (by the rerank, for candidates scattered over the zone) and
   * HBM is fetched in 128-byte lines, so keeping both in one 128-byte-aligned record per key (nib = record,
   * weight = record + 64, both strides 128) halves the traffic of that gather. */
  int64_t nib_key_stride, weight_key_stride;
  /* > 0: byte offset (multiple of 4, inside the nibble record, i.e. < nib_key_stride) of one fp32 word per key
   * that the fused select+rerank copies out for every candidate, into the workspace segment "cand_record_word"
   * ([R][n_cand] floats, same order as "cand").  The adaptive-k caches keep a key's value norm there, so that
   * it arrives with the candidate's HBM line instead of through a second scattered read
   * (cache_hub/polar_cache_adaptivek_varlen.py:1741-1753 gathers value_norm_gpu at cand_idx + sink). */
  int64_t record_word_offset;
  /* How the stages before the top-k are launched; the results are the same.
   * PKV_PLAN_SEPARATE (0, default): three launches (the reference's structure: collision kernel, top-k kernel,
   *   rerank kernel, cache_hub/polar_cache.py:1207-1298).
   * PKV_PLAN_ONE_LAUNCH (1): query prep, collision scan and select + rerank as ONE launch whose workgroups hand
   *   the row's vote table and histogram to each other through agent-scope stores, flags and bounded waits.
   *   Taken where the shape allows it (chunks of at most 8192 keys, at most 1024 workgroups, i.e. a grid that is
   *   resident as a whole) and `stream` is not being captured into a graph; otherwise the call proceeds as
   *   PKV_PLAN_SEPARATE.  Measured on MI355X it is within +-1 us of the three launches at 32 rows x 128K keys
   *   and 8 rows x 32K keys, up to 4 % faster at 8 rows x 1M keys: a hand-over between workgroups costs about
   *   what a launch boundary costs.  A workgroup that gives up a wait (2 s) counts itself in the workspace
   *   segment "handover_status" (0 after a good launch) and the results of that call are undefined. */
  int launch_plan;
  /* nonzero: the per-key vote counts need not be left in the workspace segment "cnt_u8" (the one-launch plan then
   * keeps them on chip). */
  int skip_vote_counts;
  /* nonzero: the workspace already holds this step's rotated query, its norm and the vote table, written by
   * pkv_qk_norm_rope_table for the queries `q` points to with these cluster counts and tier counts, and the words
   * the query-prep launch clears for the later stages are cleared: that launch is left out (PKV_PLAN_SEPARATE only). */
  int table_ready;
} pkv_retrieve_args;
#define PKV_PLAN_SEPARATE 0
#define PKV_PLAN_ONE_LAUNCH 1

size_t pkv_retrieve_ws_bytes(int rows, int64_t n_keys, int64_t n_cand, int64_t k);
int pkv_retrieve(const pkv_retrieve_args *args, void *ws, size_t ws_bytes, void *stream);

/* pkv_qk_norm_rope with the query side of the layer's retrieval in the same launch: besides q_out / k_out (as
 * pkv_qk_norm_rope writes them) the launch leaves in `ws` what the query-prep launch of pkv_retrieve(args, ws) would
 * compute from q_out - group mean, SRHT rotation, centroid ranking, vote table (cache_hub/polar_cache.py:1027-1031,
 * 905-922, 1216-1222) - so that the retrieval that follows, called with args->table_ready = 1 and args->q = q_out,
 * starts at the collision scan.  In the reference's decode step the two sit in different modules (model_hub/qwen.py:
 * 327-498 and cache_hub/polar_cache.py:1126-1162) with the cache update between them; nothing between them touches
 * the queries, the cluster sizes or the tier counts unless the update refreshes the index, after which the caller
 * must not set table_ready.  bf16 only; args->q is not read; n_q_heads = args->n_kv_heads * args->group. */
/* `append` (NULL: none): the token's rows of the cache in the same launch - the finished key (as k_out) and the
 * value head as it stands in qkv, behind the key heads, go to row `slot` of dst_k / dst_v [bs][kv_heads][rows][128]
 * (strides in elements): the two slot writes of decode_update_kv_cache (cache_hub/polar_cache.py:848-856), i.e.
 * what pkv_append_kv does with k_out and the value states in a launch of its own. */
typedef struct pkv_kv_append {
  void *dst_k, *dst_v;
  int64_t stride_b, stride_h, rows, slot;
} pkv_kv_append;
int pkv_qk_norm_rope_table(const void *qkv, int64_t stride_b, int n_q_heads, const void *q_weight, const void *k_weight,
                           float eps, const void *cos_row, const void *sin_row, void *q_out, void *k_out,
                           const pkv_retrieve_args *args, void *ws, size_t ws_bytes, const pkv_kv_append *append,
                           void *stream);

/* pkv_retrieve for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): the
 * same launches on `stream`, same results, but the workspace is a fixed
 * PKV_NOALLOC_SCRATCH_BYTES array inside the library's device code, one copy per
 * GPU, held until the process ends.  The call allocates and frees nothing.
 * No counterpart in the reference (its kernels allocate their outputs and
 * temporaries with torch::zeros on every call).
 *   - The GPU of `stream` must be the calling thread's current device (checked: PKV_EINVAL otherwise).
 *   - The first use of the array on a GPU looks its address up (hipGetSymbolAddress), which may make the HIP
 *     runtime load the library's code object there, and that allocates.  pkv_retrieve_noalloc_prepare() does the
 *     look-up for the current device ahead of time: call it once per GPU during set-up (before a graph capture,
 *     before the serving loop); afterwards pkv_retrieve_noalloc only reads the cached address.
 *   - Shapes whose workspace (pkv_retrieve_ws_bytes) exceeds the array are
 *     rejected with PKV_ENOMEM and a message naming both sizes;
 *     pkv_retrieve_noalloc_max_bytes() returns the array's size.
 *   - args->out_ids must be non-NULL (the candidates-only form returns its
 *     results in the workspace, which is not the caller's here).
 *   - All calls on one GPU share that GPU's array, which keeps the previous
 *     call's contents; every segment that must start at zero is cleared by the
 *     kernels themselves.  Calls that overlap in time on one GPU (two streams,
 *     two threads) race on it: serialise them, or use pkv_retrieve. */
#define PKV_NOALLOC_SCRATCH_BYTES (32u << 20)
size_t pkv_retrieve_noalloc_max_bytes(void);
int pkv_retrieve_noalloc_prepare(void);
int pkv_retrieve_noalloc(const pkv_retrieve_args *args, void *stream);

/* The whole decode step of one layer from one host call: pkv_retrieve (with its
 * gather) followed by pkv_decode_attention over the attended set, on the same
 * stream - polar_cache.compute (cache_hub/polar_cache.py:1002-1107) after the
 * dense-fallback test.  Queries, dtype and head counts are taken from
 * `retrieve`; the segments normally include the rows the gather just wrote. */
typedef struct pkv_attn_args {
  pkv_attn_segment segments[PKV_ATTN_MAX_SEGMENTS];
  int n_segments;
  const int32_t *row_keys;  /* or NULL */
  float scale;
  void *out;                /* [bs][n_kv_heads*group][128] in the query dtype */
  void *ws;
  size_t ws_bytes;          /* pkv_decode_attention_ws_bytes(...) */
} pkv_attn_args;

int pkv_decode_step(const pkv_retrieve_args *retrieve, void *ws, size_t ws_bytes,
                    const pkv_attn_args *attention, void *stream);

/* The adaptive-k decode step of one layer from one host call
 * (cache_hub/polar_cache_adaptivek_varlen.py:1391-1677 after the dense-fallback
 * test): pkv_retrieve in its candidates-only form (retrieve->out_ids == NULL,
 * retrieve->src_k == NULL) -> pkv_dense_logits over the first dense_rows rows of
 * the GPU K store -> pkv_adaptive_topk on the fp32 rerank scores (logit = score
 * times `scale`) with the value norms looked up by position ->
 * pkv_gather_uva_ragged of each row's own k rows from the pinned host store ->
 * pkv_decode_attention with row_keys = row_keys_base + k.  Every field has the
 * meaning of the same-named argument of those entry points. */
typedef struct pkv_adaptive_args {
  const void *dense_k;            /* GPU K store; rows 0 .. dense_rows-1 of each (b, h) are the dense tokens */
  int64_t dense_stride_b, dense_stride_h;  /* elements */
  int64_t dense_rows;
  const float *dense_vnorm;       /* [bs*n_kv_heads][dense_vnorm_stride] */
  int64_t dense_vnorm_stride;
  float *dense_logits;            /* scratch [bs*n_kv_heads][dense_logits_stride] */
  int64_t dense_logits_stride;
  float scale;                    /* attention scale: logits of dense rows and of candidates */
  const float *value_norm;        /* row r, position p at value_norm[r*vn_stride + p*vn_pos_stride]; p = candidate id + vn_offset */
  int64_t vn_stride, vn_offset, vn_pos_stride;  /* vn_pos_stride 0 or 1: packed rows */
  float threshold;
  int64_t k_out, k_min, k_max;
  int64_t *adaptive_k;            /* [bs*n_kv_heads] */
  int64_t *topk_ids;              /* [bs*n_kv_heads][k_out] */
  int32_t *row_keys;              /* [bs*n_kv_heads]; also passed to the attention */
  int64_t row_keys_base;
  int64_t *uniform_k;             /* NULL, or [bs*n_kv_heads]: pkv_uniform_k runs after the adaptive stage and the
                                     gather and row_keys use max(adaptive_k) for every row (the dense form) */
  void *ws;                       /* pkv_adaptive_topk_ws_bytes(rows, n_cand, k_out) */
  size_t ws_bytes;
  const void *src_k, *src_v;      /* pinned host K/V stores [bs][h][src_len] rows */
  int64_t src_len, idx_offset;
  void *dst_k, *dst_v;            /* GPU [bs][h][dst_len] rows; row (b, h) receives its k rows from dst_row0 on */
  int64_t dst_len, dst_row0;
  int row_bytes;
} pkv_adaptive_args;

int pkv_adaptive_decode_step(const pkv_retrieve_args *retrieve, void *ws, size_t ws_bytes,
                             const pkv_adaptive_args *adaptive, const pkv_attn_args *attention, void *stream);

/* Names and device pointers of the intermediates inside a pkv_retrieve
 * workspace (for tests and profiling): qhat, qnorm, lut, cnt_u8,
 * chunk_suffix_hist, row_suffix_hist, cand, scores, cand_record_word, handover_status.  Returns PKV_EINVAL for an
 * unknown name.  chunk_suffix_hist holds uint16 counts of the keys of a chunk with at least `bin` votes:
 * [row][chunk][128 bins] for rows scanned one chunk per workgroup, and [row][128 bins][chunk][4 pieces] where the
 * chunk size (the smallest power of two from 2048 that keeps a launch within 1024 workgroups) is 8192 keys or more and
 * a row has at most 128 chunks: a workgroup then scans four pieces of chunk_keys / 4 keys that lie n_chunks pieces
 * apart, and piece p of the row, in key order, is entry [p % n_chunks][p / n_chunks]. */
int pkv_retrieve_ws_view(void *ws, int rows, int64_t n_keys, int64_t n_cand, int64_t k,
                         const char *name, void **ptr, size_t *bytes);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif
