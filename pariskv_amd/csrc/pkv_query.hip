// Query side of the retrieval: GQA group mean, normalise, SRHT rotate, rank the
// 256 sign centroids of every subspace, and turn the ranking plus the cluster
// sizes into a vote table lut[row][subspace][centroid] in [0, n_tiers].
//
// Reference: cache_hub/polar_cache.py:1027-1031, 905-922, 1216-1222 and
// cache_hub/collision_fused/collision.cu:71-151 (convert_to_bits).  The six
// nested tier bitsets of the reference collapse into one weight per centroid:
// weight = number of tiers whose key budget is not yet exhausted at the
// centroid's rank.
#include "pkv_common.h"
#include "pkv_lut.h"

namespace {

__device__ __forceinline__ int tier_weight_from_rank(int my_count, const PkvTiers &tiers, int *s_wave_tot) {
  return pkv_tier_weight_from_rank(my_count, tiers, s_wave_tot);
}

// grid (16 subspaces, R rows), 256 threads.
__global__ __launch_bounds__(256) void pkv_query_prep_lut_kernel(
    const void *__restrict__ q, int dtype, int n_kv_heads, int group, const float *__restrict__ signs,
    const int32_t *__restrict__ cc, int64_t cc_b, int64_t cc_h, PkvTiers tiers, float *__restrict__ qhat,
    float *__restrict__ qnorm, uint8_t *__restrict__ lut, int64_t *__restrict__ sorted_ids,
    uint32_t *__restrict__ row_suf_to_zero, uint32_t *__restrict__ zero_ptr, int64_t zero_words) {
  const int sub = blockIdx.x;
  const int row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;
  // words a later launch of the step accumulates into (the control blocks of a multi-workgroup top-k)
  for (int64_t i = ((int64_t)row * gridDim.x + sub) * 256 + tid; i < zero_words; i += (int64_t)gridDim.x * gridDim.y * 256)
    zero_ptr[i] = 0u;

  // the collision scan that follows accumulates the row's suffix histogram with atomics
  if (row_suf_to_zero && sub == 1 && tid < 128) row_suf_to_zero[(int64_t)row * 128 + tid] = 0u;

  __shared__ PkvLutSmem sm;
  pkv_lut_build_subspace(q, dtype, b, h, n_kv_heads, group, signs, cc + (int64_t)b * cc_b + (int64_t)h * cc_h + sub * 256,
                         tiers, sub, sm, lut + ((int64_t)row * 16 + sub) * 256,
                         sub == 0 ? qhat + (int64_t)row * 128 : nullptr, sub == 0 ? qnorm + row : nullptr,
                         sorted_ids ? sorted_ids + ((int64_t)row * 16 + sub) * 256 : nullptr);
}

// Ranking supplied by the caller (reference-shaped API).  grid (16, R), 256 threads.
template <typename IdT>
__global__ __launch_bounds__(256) void pkv_lut_from_sorted_kernel(
    const IdT *__restrict__ ids, int64_t si_b, int64_t si_h, int64_t si_sub, const int32_t *__restrict__ cc,
    int64_t cc_b, int64_t cc_h, int64_t cc_sub, const int32_t *__restrict__ topk_cluster_cnt, int n_kv_heads,
    PkvTiers tiers, uint8_t *__restrict__ lut) {
  const int sub = blockIdx.x;
  const int row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;
  __shared__ int s_wave_tot[4];
  __shared__ unsigned int s_lut[256];
  s_lut[tid] = 0;
  __syncthreads();
  const int id = (int)(ids[(int64_t)b * si_b + (int64_t)h * si_h + (int64_t)sub * si_sub + tid]) & 255;
  int w;
  if (topk_cluster_cnt) {
    // legacy single tier: the first topk_cluster_cnt ranked clusters vote once
    w = (tid < topk_cluster_cnt[(int64_t)row * 16 + sub]) ? 1 : 0;
  } else {
    const int cnt = cc[(int64_t)b * cc_b + (int64_t)h * cc_h + (int64_t)sub * cc_sub + id];
    w = tier_weight_from_rank(cnt, tiers, s_wave_tot);
  }
  atomicMax(&s_lut[id], (unsigned int)w);  // duplicates in `ids` keep the best-ranked occurrence
  __syncthreads();
  lut[((int64_t)row * 16 + sub) * 256 + tid] = (uint8_t)s_lut[tid];
}

}  // namespace

int pkv_launch_query_prep_lut(const void *q, int dtype, int bs, int n_kv_heads, int group, const float *signs,
                              const int32_t *cc, int64_t cc_b, int64_t cc_h, const PkvTiers &tiers, float *qhat,
                              float *qnorm, uint8_t *lut, int64_t *sorted_ids, uint32_t *row_suf_to_zero,
                              hipStream_t s, uint32_t *zero_ptr, int64_t zero_words) {
  dim3 grid(16, (unsigned)(bs * n_kv_heads));
  hipLaunchKernelGGL(pkv_query_prep_lut_kernel, grid, dim3(256), 0, s, q, dtype, n_kv_heads, group, signs, cc,
                     cc_b, cc_h, tiers, qhat, qnorm, lut, sorted_ids, row_suf_to_zero, zero_ptr, zero_ptr ? zero_words : 0);
  PKV_LAUNCH_CHECK("pkv_query_prep_lut_kernel");
  return PKV_OK;
}

static int make_tiers(const uint32_t *tier_counts, int n_tiers, PkvTiers &t) {
  PKV_REQUIRE(tier_counts != nullptr && n_tiers >= 1 && n_tiers <= PKV_MAX_TIERS,
              "n_tiers must be in [1,%d], got %d", PKV_MAX_TIERS, n_tiers);
  memset(&t, 0, sizeof t);
  t.n = n_tiers;
  for (int i = 0; i < n_tiers; ++i) t.t[i] = tier_counts[i];
  return PKV_OK;
}

extern "C" int pkv_query_prep_lut(const void *q, int dtype, int bs, int n_kv_heads, int group, const float *signs,
                                  const int32_t *cluster_counts, int64_t cc_b, int64_t cc_h,
                                  const uint32_t *tier_counts, int n_tiers, float *qhat, float *qnorm,
                                  uint8_t *lut, int64_t *sorted_ids, void *stream) {
  PKV_REQUIRE(q && signs && cluster_counts && qhat && qnorm && lut, "pkv_query_prep_lut: null pointer");
  PKV_REQUIRE(pkv_aligned(q, 16), "queries must be 16-byte aligned");
  PKV_REQUIRE(dtype == PKV_DTYPE_F32 || dtype == PKV_DTYPE_BF16, "unknown dtype %d", dtype);
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && group > 0 && (int64_t)bs * n_kv_heads <= 65535,
              "bad shape bs=%d kv_heads=%d group=%d", bs, n_kv_heads, group);
  PkvTiers t;
  int rc = make_tiers(tier_counts, n_tiers, t);
  if (rc) return rc;
  return pkv_launch_query_prep_lut(q, dtype, bs, n_kv_heads, group, signs, cluster_counts, cc_b, cc_h, t, qhat,
                                   qnorm, lut, sorted_ids, nullptr, (hipStream_t)stream);
}

extern "C" int pkv_update_cache_cnt(const int64_t *sorted_ids, int64_t si_b, int64_t si_h, int64_t si_sub,
                                    const int32_t *cluster_counts, int64_t cc_b, int64_t cc_h, int64_t cc_sub,
                                    const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key,
                                    int64_t cs_sub, int bs, int n_kv_heads, int64_t n_keys,
                                    const uint32_t *tier_counts, int n_tiers, uint8_t *lut_ws, int32_t *cnt,
                                    void *stream) {
  PKV_REQUIRE(sorted_ids && cluster_counts && codes && lut_ws && cnt, "pkv_update_cache_cnt: null pointer");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535 && n_keys > 0 &&
                  n_keys <= PKV_MAX_KEYS_PER_ROW,
              "bad shape bs=%d kv_heads=%d n_keys=%lld", bs, n_kv_heads, (long long)n_keys);
  PkvTiers t;
  int rc = make_tiers(tier_counts, n_tiers, t);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(16, (unsigned)(bs * n_kv_heads));
  hipLaunchKernelGGL(pkv_lut_from_sorted_kernel<int64_t>, grid, dim3(256), 0, s, sorted_ids, si_b, si_h, si_sub,
                     cluster_counts, cc_b, cc_h, cc_sub, (const int32_t *)nullptr, n_kv_heads, t, lut_ws);
  PKV_LAUNCH_CHECK("pkv_lut_from_sorted_kernel");
  return pkv_launch_scan(codes, cs_b, cs_h, cs_key, cs_sub, bs, n_kv_heads, n_keys, lut_ws, nullptr, 0, cnt,
                         nullptr, nullptr, pkv_pick_chunk_keys(bs * n_kv_heads, n_keys), s);
}

PKV_INTERNAL int pkv_launch_scan_i32_codes(const int32_t *codebook, int rows, int64_t n_keys, const uint8_t *lut,
                                           int32_t *cnt, hipStream_t s);

extern "C" int pkv_update_cache_cnt_legacy(const int32_t *sorted_ids, const int32_t *topk_cluster_cnt,
                                           const int32_t *codebook, int bs, int n_kv_heads, int64_t n_keys,
                                           uint8_t *lut_ws, int32_t *cnt, void *stream) {
  PKV_REQUIRE(sorted_ids && topk_cluster_cnt && codebook && lut_ws && cnt,
              "pkv_update_cache_cnt_legacy: null pointer");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535 && n_keys > 0,
              "bad shape bs=%d kv_heads=%d n_keys=%lld", bs, n_kv_heads, (long long)n_keys);
  hipStream_t s = (hipStream_t)stream;
  PkvTiers t;
  memset(&t, 0, sizeof t);
  dim3 grid(16, (unsigned)(bs * n_kv_heads));
  hipLaunchKernelGGL(pkv_lut_from_sorted_kernel<int32_t>, grid, dim3(256), 0, s, sorted_ids,
                     (int64_t)n_kv_heads * 16 * 256, (int64_t)16 * 256, (int64_t)256, (const int32_t *)nullptr,
                     (int64_t)0, (int64_t)0, (int64_t)0, topk_cluster_cnt, n_kv_heads, t, lut_ws);
  PKV_LAUNCH_CHECK("pkv_lut_from_sorted_kernel<int32>");
  return pkv_launch_scan_i32_codes(codebook, bs * n_kv_heads, n_keys, lut_ws, cnt, s);
}
