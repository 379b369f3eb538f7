/*
 * pkv_oracle.h -- CPU restatement (plain C) of ParisKV's per-decode-step KV
 * retrieval path.  TEST INFRASTRUCTURE ONLY: the checker that the HIP kernels
 * are compared against, and the timed "cpu_baseline" leg of the benchmark.
 * Nothing in the product package may include, link or call this.
 *
 * Every function cites the reference file:line whose arithmetic it restates
 * (paths relative to the ParisKV checkout).  Floating-point steps are evaluated
 * in one fixed, documented order with no fused multiply-add, so that integer
 * results derived from them (codes, nibbles, ranks, indices) can be compared
 * bit-for-bit with the GPU.
 *
 * "dtype" selects the rounding chain: PKV_O_F32 keeps every intermediate in
 * fp32; PKV_O_BF16 rounds to bfloat16 (round-to-nearest-even) at each point
 * where the reference's torch expression yields a bf16 tensor.
 *
 * PARITY UNPINNED (no reference fixture, library routine or closed form fixes
 * these; the oracle makes a documented choice inside the reference's contract):
 *   - pkv_o_fwht128: the butterfly order and internal rounding of the
 *     third-party fast_hadamard_transform kernel (not in the reference tree);
 *     pinned only as x * H_128 * scale with the natural-order Hadamard matrix;
 *   - pkv_o_rerank: the reference kernel rounds to bf16 after every operation;
 *     the oracle is the same expression in fp32 (agreement 1e-5 relative with
 *     the fp32 torch form, not with the bf16 kernel);
 *   - tie order of pkv_o_rank_centroids, pkv_o_select_candidates and
 *     pkv_o_topk_f32 where the reference's unstable argsort / atomic
 *     compaction leaves it open: the oracle picks (value desc, index asc);
 *   - summation orders of pkv_o_adaptive_topk and of the two numpy
 *     restatements that feed it (dense_logits, value_norm in pkv_oracle.py;
 *     the reference leaves all of them to torch): k agrees with the reference
 *     form within 1, logits and norms with torch's within one bf16 step.
 * Everything else, including the SRHT sign vector (a Philox4x32-10 draw,
 * checked against the generator's known-answer vectors and against torch's
 * device generator), is pinned by the tests named in tests/test_oracle_*.py.
 */
#ifndef PKV_ORACLE_H
#define PKV_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PKV_O_F32 0
#define PKV_O_BF16 1

#define PKV_O_D 128      /* head_dim */
#define PKV_O_B 16       /* subspaces (blocks) */
#define PKV_O_M 8        /* dims per block */
#define PKV_O_KW 256     /* sign centroids per subspace */

/* bf16 round-to-nearest-even of an fp32 value, returned as fp32. */
float pkv_o_bf16_round(float x);

/* Magnitude codebook constants, polar_cache.py:188-193 (bf16-rounded). */
void pkv_o_mag_constants(float thresholds[7], float centers[8]);

/* In-place natural-order Walsh-Hadamard transform of 128 fp32 values
 * (unnormalised).  Stands in for fast_hadamard_transform.hadamard_transform,
 * polar_cache.py:920,945. */
void pkv_o_fwht128(float *x);

/* polar_cache.py:924-978 (batch_encode) for n_keys keys of 128 dims.
 * keys: [n_keys][128] fp32 (bf16-representable values for the bf16 chain).
 * signs: SRHT diagonal, [128] of +-1.
 * Outputs are key-major: codes [n][16] u8, nib [n][16][4] u8,
 * weight [n][16] fp32 (bf16-representable), any may be NULL. */
void pkv_o_encode(const float *keys, int64_t n_keys, const float *signs,
                  int dtype, uint8_t *codes, uint8_t *nib, float *weight);

/* polar_cache.py:980-996 (_count_cluster_keys): counts[16][256] += histogram
 * of codes[n][16]. */
void pkv_o_count_cluster_keys(const uint8_t *codes, int64_t n_keys,
                              int32_t *counts);

/* polar_cache.py:1027-1031 + 905-922: group mean of G query heads, norm,
 * SRHT rotate.  q: [G][128].  Outputs qhat[128], *qnorm. */
void pkv_o_query_prep(const float *q, int G, const float *signs, int dtype,
                      float *qhat, float *qnorm);

/* polar_cache.py:1216-1217: centroid scores against the 256 sign patterns of
 * each subspace and their descending ranking (ties: smaller id first).
 * sorted_ids: [16][256]. */
void pkv_o_rank_centroids(const float *qhat, int dtype, int64_t *sorted_ids);

/* collision_fused/collision.cu:71-151 (convert_to_bits) restated as a weight
 * table: lut[s][c] = number of tiers whose bitset contains cluster c.
 * sorted_ids [n_sub][256], counts [n_sub][256], tier_counts[n_tiers]. */
void pkv_o_tier_lut(const int64_t *sorted_ids, const int32_t *counts,
                    int n_sub, const uint32_t *tier_counts, int n_tiers,
                    uint8_t *lut);

/* collision_fused/collision.cu:163-229 (update_cache_cnt_kernel):
 * cnt[i] = sum_s lut[s][code_s(i)].  codes addressed as
 * codes[i*stride_key + s*stride_sub]. */
void pkv_o_collision_count(const uint8_t *codes, int64_t n_keys,
                           int64_t stride_key, int64_t stride_sub, int n_sub,
                           const uint8_t *lut, int32_t *cnt);

/* topk/radix_topk.cu:39-120,161-239 selection rule with the build's tie rule:
 * all i with cnt[i] > theta (ascending i), then the smallest-index i with
 * cnt[i] == theta until k are chosen; n <= k gives 0..n-1 padded with 0.
 * Returns theta (or -1 for the identity case). */
int pkv_o_select_candidates(const int32_t *cnt, int64_t n, int64_t k,
                            int64_t *out);

/* rerank/rerank.cu:93-136 / polar_cache.py:1281-1298 in fp32, fixed order
 * (j = 0..7 inside a block, then blocks 0..15), no FMA.
 * nib addressed as nib[i*nib_stride_key + s*nib_stride_sub + byte],
 * weight as weight[i*w_stride_key + s*w_stride_sub]. */
void pkv_o_rerank(const int64_t *cand, int64_t n_cand, const uint8_t *nib,
                  int64_t nib_stride_key, int64_t nib_stride_sub,
                  const float *weight, int64_t w_stride_key,
                  int64_t w_stride_sub, const float *qhat, float qnorm,
                  const float *centers, float *scores);

/* polar_cache.py:1300-1302 (torch.topk + gather): the k best of n scores,
 * descending, ties broken by smaller ids[i] (position i when ids == NULL).
 * out_ids[k] receives ids[i] (or i); out_pos[k] (optional) the positions. */
void pkv_o_topk_f32(const float *scores, const int64_t *ids, int64_t n,
                    int64_t k, int64_t *out_ids, int64_t *out_pos);

/* gather_trans/trans_h2d.cu:38-74: dst[i][:] = src[idx[i]][:], rows of
 * row_bytes bytes. */
/* Dense attention of one KV head on the gathered key set, polar_cache.py:1084-1105
 * (flash_attn_func on the concatenated sink / top-k / local rows, non-causal,
 * softmax scale 1/sqrt(128) by default): out[g] = softmax(q[g] . K^T * scale) V
 * for the G query heads of the KV head.  q [G][128], k, v [S][128] fp32 (bf16
 * inputs are passed as their exact fp32 values); accumulated in double; out [G][128]
 * fp32, not rounded.  Pinned against torch's scaled_dot_product_attention. */
void pkv_o_attention(const float *q, int g_heads, const float *k, const float *v, int64_t s,
                     float scale, float *out);

void pkv_o_gather_rows(const void *src, const int64_t *idx, int64_t k,
                       int64_t row_bytes, void *dst);

/* The exponential used by adaptive-k: a fixed fp32 operation sequence shared
 * with the GPU so that exp() agrees to the bit. */
float pkv_o_expf(float x);

/* adaptive_k_fused/adaptive_topk.py:255-313 (adaptive_topk_ref), fp32.
 * Summation orders are fixed (the reference leaves them to torch): the two
 * benefit sums run over slices of 8192 elements (lane j mod 1024 in increasing
 * j, pairwise tree over the 1024 lanes, slice sums left to right); the
 * cumulative sum over the sorted benefits runs left to right inside blocks of
 * 64 and left to right over the block totals.
 * Returns adaptive k (before any min/max clamp by the caller);
 * out_ids[k_out] = candidate ids in descending benefit order
 * (ties: smaller candidate position first). */
int64_t pkv_o_adaptive_topk(const float *sl_logits, const float *sl_vnorm,
                            int64_t sl, const float *cand_logits,
                            const float *cand_vnorm, const int64_t *cand_ids,
                            int64_t n_cand, float threshold, int64_t k_out,
                            int64_t *out_ids);

/* One row of the whole retrieval (a4..a9): returns final ids in out_ids[K]. */
void pkv_o_retrieve_row(const float *q, int G, const float *signs, int dtype,
                        const uint8_t *codes, const uint8_t *nib,
                        const float *weight, const int32_t *cluster_counts,
                        int64_t n_keys, const uint32_t *tier_counts,
                        int n_tiers, int64_t n_cand, int64_t k,
                        int64_t *out_ids);

#ifdef __cplusplus
}
#endif
#endif
