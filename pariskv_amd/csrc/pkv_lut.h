// Vote table of one (row, subspace) pair: GQA group mean of the query, normalise, SRHT rotate, rank the 256 sign
// centroids, turn the ranking plus the cluster sizes into votes per centroid.
//
// Reference: cache_hub/polar_cache.py:1027-1031, 905-922, 1216-1222 and
// cache_hub/collision_fused/collision.cu:71-151 (convert_to_bits).
//
// Shared by the query-prep kernel (one workgroup per (row, subspace)) and by the fused table + scan kernel.
#pragma once

#include "pkv_common.h"

#if defined(__HIPCC__)

struct PkvLutSmem {
  float y[128];
  __attribute__((aligned(16))) uint32_t key[256];
  int id[256];
  int cc[256];
  int part[128];
  int wave_tot[4];
};

// Exclusive prefix of the ranked cluster sizes -> tier weight, one thread per rank (256 threads).
__device__ __forceinline__ int pkv_tier_weight_from_rank(int my_count, const PkvTiers &tiers, int *s_wave_tot) {
  int total;
  int prefix = pkv_block_excl_scan<256>(my_count, s_wave_tot, total);
  int w = 0;
#pragma unroll
  for (int t = 0; t < PKV_MAX_TIERS; ++t)
    if (t < tiers.n && (uint32_t)prefix < tiers.t[t]) ++w;
  return w;
}

// Votes of one subspace from the rotated query in sm.y (all 128 dims, written and made visible by the caller:
// a barrier lies between that write and this call).  Called by all 256 threads of a workgroup; contains barriers.
//   cc_sub      cluster sizes of this (row, subspace): 256 ints in global memory
//   lut_out     256 bytes (global or LDS): votes per centroid id
//   sorted_out  int64[256] or null: centroid ids in ranked order
__device__ __forceinline__ void pkv_lut_rank_subspace(int dtype, const int32_t *__restrict__ cc_sub, const PkvTiers &tiers,
                                                      int sub, PkvLutSmem &sm, uint8_t *lut_out, int64_t *sorted_out);

// Called by all 256 threads of a workgroup (contains barriers; `sm` may be reused after the call once the
// caller has passed a barrier).  The rotation runs in the first wave only (two dims per lane, lane exchanges, no
// barriers); the 256 threads then score, rank and weigh the 256 centroids.
//   cc_sub      cluster sizes of this (row, subspace): 256 ints in global memory
//   lut_out     256 bytes (global or LDS): votes per centroid id
//   qhat_out    float[128] of the row or null; qnorm_out likewise (written when non-null)
//   sorted_out  int64[256] or null: centroid ids in ranked order
__device__ __forceinline__ void pkv_lut_build_subspace(const void *__restrict__ q, int dtype, int b, int h, int n_kv_heads,
                                                       int group, const float *__restrict__ signs,
                                                       const int32_t *__restrict__ cc_sub, const PkvTiers &tiers, int sub,
                                                       PkvLutSmem &sm, uint8_t *lut_out, float *qhat_out, float *qnorm_out,
                                                       int64_t *sorted_out) {
  const int tid = threadIdx.x;
  // cluster sizes by centroid id; issued first so that the latency overlaps the rotation
  const int my_cc = cc_sub[tid];

  if (tid < PKV_WAVE) {
    float y_lo, y_hi;
    const float n = pkv_query_mean_rotate_wave(q, dtype, b, h, n_kv_heads, group, signs, y_lo, y_hi);
    sm.y[tid] = y_lo, sm.y[tid + 64] = y_hi;
    if (qhat_out) qhat_out[tid] = y_lo, qhat_out[tid + 64] = y_hi;
    if (qnorm_out && tid == 0) *qnorm_out = n;
  }
  sm.cc[tid] = my_cc;
  __syncthreads();
  pkv_lut_rank_subspace(dtype, nullptr, tiers, sub, sm, lut_out, sorted_out);
}

__device__ __forceinline__ void pkv_lut_rank_subspace(int dtype, const int32_t *__restrict__ cc_sub, const PkvTiers &tiers,
                                                      int sub, PkvLutSmem &sm, uint8_t *lut_out, int64_t *sorted_out) {
  const int tid = threadIdx.x;
  if (cc_sub) sm.cc[tid] = cc_sub[tid];  // read again only after the barriers below

  // score of centroid c = tid: sum_j (+-) qhat_sub[j], sequential j
  {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = sm.y[8 * sub + j];
      const float t = ((tid >> j) & 1) ? v : -v;
      acc = (j == 0) ? t : acc + t;
    }
    acc = pkv_rdt(acc + 0.0f, dtype);
    uint32_t key = pkv_ordered_u32(acc);
    // bf16 scores occupy the top 16 bits: fold the tie rule (smaller id first) into one 32-bit key
    if (dtype == PKV_DTYPE_BF16) key = ((key >> 16) << 8) | (uint32_t)(255 - tid);
    sm.key[tid] = key;
  }
  __syncthreads();
  // rank = number of centroids ahead of this one under (score desc, id asc).  The sign codebook is
  // antipodal (score[255-c] == -score[c] exactly), hence rank[255-c] = 255 - rank[c]: thread t counts,
  // for centroid c = t & 127, over half (t >> 7) of the keys; the two partial counts are added.
  {
    const int c = tid & 127, half = tid >> 7;
    const uint32_t mine = sm.key[c];
    int part = 0;
    const pkv_u32x4 *k4 = (const pkv_u32x4 *)sm.key + half * 32;
    if (dtype == PKV_DTYPE_BF16) {
#pragma unroll 8
      for (int c4 = 0; c4 < 32; ++c4) {
        const pkv_u32x4 k = k4[c4];
        part += (k.x > mine) + (k.y > mine) + (k.z > mine) + (k.w > mine);
      }
    } else {
#pragma unroll 8
      for (int c4 = 0; c4 < 32; ++c4) {
        const pkv_u32x4 k = k4[c4];
        const int o = half * 128 + 4 * c4;
        part += (k.x > mine || (k.x == mine && o + 0 < c)) ? 1 : 0;
        part += (k.y > mine || (k.y == mine && o + 1 < c)) ? 1 : 0;
        part += (k.z > mine || (k.z == mine && o + 2 < c)) ? 1 : 0;
        part += (k.w > mine || (k.w == mine && o + 3 < c)) ? 1 : 0;
      }
    }
    if (half) sm.part[c] = part;
    __syncthreads();
    if (!half) {
      const int rank = part + sm.part[c];
      sm.id[rank] = c;
      sm.id[255 - rank] = 255 - c;
    }
  }
  __syncthreads();
  const int id = sm.id[tid];
  const int w = pkv_tier_weight_from_rank(sm.cc[id], tiers, sm.wave_tot);
  lut_out[id] = (uint8_t)w;
  if (sorted_out) sorted_out[tid] = id;
}

#endif  // __HIPCC__
