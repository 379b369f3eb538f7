/*
 * pkv_oracle.c -- CPU restatement of ParisKV's per-decode-step KV retrieval
 * path.  TEST INFRASTRUCTURE ONLY (see pkv_oracle.h).
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -shared -fPIC (see Makefile).
 * -ffp-contract=off matters: every a*b+c below is a rounded multiply followed
 * by a rounded add, which is what the GPU kernels are compiled to do as well.
 */
#include "pkv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ helpers */

static inline uint32_t f2u(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  return u;
}
static inline float u2f(uint32_t u) {
  float x;
  memcpy(&x, &u, 4);
  return x;
}

float pkv_o_bf16_round(float x) {
  uint32_t u = f2u(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return u2f((u | 0x00400000u) & 0xffff0000u); /* NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return u2f(u & 0xffff0000u);
}

static inline float rdt(float x, int dtype) {
  return dtype == PKV_O_BF16 ? pkv_o_bf16_round(x) : x;
}

/* Order-preserving map float -> uint32 (larger float <=> larger uint). */
static inline uint32_t ordered_u32(float x) {
  uint32_t b = f2u(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

void pkv_o_mag_constants(float thresholds[7], float centers[8]) {
  /* polar_cache.py:188-193: decimal literals stored as bf16 tensors. */
  static const double th[7] = {0.0843, 0.1698, 0.2578, 0.3499, 0.4487, 0.5585, 0.6901};
  static const double ce[8] = {0.0420, 0.1266, 0.2130, 0.3025, 0.3973, 0.5001, 0.6169, 0.7633};
  for (int i = 0; i < 7; ++i) thresholds[i] = pkv_o_bf16_round((float)th[i]);
  for (int i = 0; i < 8; ++i) centers[i] = pkv_o_bf16_round((float)ce[i]);
}

/* 1/sqrt(128) as the fp32 value of the Python double 1.0/math.sqrt(128)
 * (polar_cache.py:317). */
static const float kScale = 0.08838834764831845f;

void pkv_o_fwht128(float *x) {
  for (int h = 1; h < PKV_O_D; h <<= 1) {
    for (int i = 0; i < PKV_O_D; i += 2 * h) {
      for (int j = i; j < i + h; ++j) {
        float a = x[j], b = x[j + h];
        x[j] = a + b;
        x[j + h] = a - b;
      }
    }
  }
}

/* Sum of squares of 128 values: sequential inside each 8-wide block, then a
 * pairwise tree over the 16 block sums (stride 1, 2, 4, 8). */
static float sumsq128(const float *x) {
  float s[PKV_O_B];
  for (int b = 0; b < PKV_O_B; ++b) {
    float acc = x[8 * b] * x[8 * b];
    for (int j = 1; j < 8; ++j) acc = acc + x[8 * b + j] * x[8 * b + j];
    s[b] = acc;
  }
  for (int h = 1; h < PKV_O_B; h <<= 1)
    for (int i = 0; i < PKV_O_B; i += 2 * h) s[i] = s[i] + s[i + h];
  return s[0];
}

/* Normalise + SRHT rotate a 128-vector (polar_cache.py:938-945 / 915-920).
 * Returns the norm (rounded to dtype); y receives the rotated unit vector. */
static float normalize_rotate(const float *v, const float *signs, int dtype, float *y) {
  float n = rdt(sqrtf(sumsq128(v)), dtype);
  float den = n < 1e-8f ? 1e-8f : n;
  for (int i = 0; i < PKV_O_D; ++i) y[i] = rdt(v[i] / den, dtype) * signs[i];
  pkv_o_fwht128(y);
  for (int i = 0; i < PKV_O_D; ++i) y[i] = rdt(y[i] * kScale, dtype);
  return n;
}

/* ------------------------------------------------------------------- encode */

void pkv_o_encode(const float *keys, int64_t n_keys, const float *signs, int dtype,
                  uint8_t *codes, uint8_t *nib, float *weight) {
  float th[7], ce[8];
  pkv_o_mag_constants(th, ce);
  for (int64_t k = 0; k < n_keys; ++k) {
    float y[PKV_O_D];
    float n = normalize_rotate(keys + k * PKV_O_D, signs, dtype, y);
    for (int b = 0; b < PKV_O_B; ++b) {
      const float *yb = y + 8 * b;
      /* polar_cache.py:950-951: sign bit-pack, bit j <=> y_bj >= 0 */
      uint8_t code = 0;
      for (int j = 0; j < 8; ++j)
        if (yb[j] >= 0.0f) code |= (uint8_t)(1u << j);
      if (codes) codes[k * PKV_O_B + b] = code;
      if (!nib && !weight) continue;
      /* :958-960 block radius and direction */
      float acc = yb[0] * yb[0];
      for (int j = 1; j < 8; ++j) acc = acc + yb[j] * yb[j];
      float r = rdt(sqrtf(acc), dtype);
      float den = r < 1e-8f ? 1e-8f : r;
      uint8_t v4[8];
      float alpha = 0.0f;
      for (int j = 0; j < 8; ++j) {
        float u = rdt(yb[j] / den, dtype);
        float au = fabsf(u);
        /* :965 bucketize(right=False): number of thresholds strictly below */
        int t = 0;
        for (int i = 0; i < 7; ++i) t += (th[i] < au) ? 1 : 0;
        v4[j] = (uint8_t)(((yb[j] >= 0.0f) ? 8 : 0) | t);
        /* :972 alpha = sum(a[t] * |u|) with the product in the tensor dtype */
        float p = rdt(ce[t] * au, dtype);
        alpha = (j == 0) ? p : alpha + p;
      }
      if (alpha < 1e-6f) alpha = 1e-6f;
      if (nib) {
        /* :887-893 two values per byte, low nibble = even dim */
        for (int p = 0; p < 4; ++p)
          nib[(k * PKV_O_B + b) * 4 + p] = (uint8_t)((v4[2 * p + 1] << 4) | v4[2 * p]);
      }
      if (weight) {
        /* :975-976 weight = (r / alpha) * ||k||, stored bf16 in both chains */
        float w = (r / alpha) * n;
        weight[k * PKV_O_B + b] = pkv_o_bf16_round(w);
      }
    }
  }
}

void pkv_o_count_cluster_keys(const uint8_t *codes, int64_t n_keys, int32_t *counts) {
  for (int64_t k = 0; k < n_keys; ++k)
    for (int b = 0; b < PKV_O_B; ++b) counts[b * PKV_O_KW + codes[k * PKV_O_B + b]] += 1;
}

/* -------------------------------------------------------------- query side */

void pkv_o_query_prep(const float *q, int G, const float *signs, int dtype, float *qhat,
                      float *qnorm) {
  float m[PKV_O_D];
  for (int i = 0; i < PKV_O_D; ++i) {
    float acc = q[i];
    for (int g = 1; g < G; ++g) acc = acc + q[g * PKV_O_D + i];
    m[i] = rdt(acc / (float)G, dtype);
  }
  *qnorm = normalize_rotate(m, signs, dtype, qhat);
}

typedef struct {
  uint32_t key;
  int32_t id;
} rank_item;

static int rank_cmp(const void *a, const void *b) {
  const rank_item *x = (const rank_item *)a, *y = (const rank_item *)b;
  if (x->key != y->key) return x->key > y->key ? -1 : 1;
  return x->id < y->id ? -1 : (x->id > y->id ? 1 : 0);
}

void pkv_o_rank_centroids(const float *qhat, int dtype, int64_t *sorted_ids) {
  for (int b = 0; b < PKV_O_B; ++b) {
    rank_item it[PKV_O_KW];
    for (int c = 0; c < PKV_O_KW; ++c) {
      /* polar_cache.py:1216: scores = q_blocks @ V^T with V[c][j] = +-1 */
      float acc = 0.0f;
      for (int j = 0; j < 8; ++j) {
        float t = ((c >> j) & 1) ? qhat[8 * b + j] : -qhat[8 * b + j];
        acc = (j == 0) ? t : acc + t;
      }
      acc = rdt(acc + 0.0f, dtype);
      it[c].key = ordered_u32(acc);
      it[c].id = c;
    }
    qsort(it, PKV_O_KW, sizeof(rank_item), rank_cmp);
    for (int r = 0; r < PKV_O_KW; ++r) sorted_ids[b * PKV_O_KW + r] = it[r].id;
  }
}

void pkv_o_tier_lut(const int64_t *sorted_ids, const int32_t *counts, int n_sub,
                    const uint32_t *tier_counts, int n_tiers, uint8_t *lut) {
  memset(lut, 0, (size_t)n_sub * PKV_O_KW);
  for (int s = 0; s < n_sub; ++s) {
    int32_t prefix = 0; /* exclusive prefix of cluster sizes in ranked order */
    for (int r = 0; r < PKV_O_KW; ++r) {
      int c = (int)(sorted_ids[s * PKV_O_KW + r] & 255);
      int w = 0;
      for (int t = 0; t < n_tiers; ++t) w += ((uint32_t)prefix < tier_counts[t]) ? 1 : 0;
      if (w > lut[s * PKV_O_KW + c]) lut[s * PKV_O_KW + c] = (uint8_t)w;
      prefix += counts[s * PKV_O_KW + c];
    }
  }
}

void pkv_o_collision_count(const uint8_t *codes, int64_t n_keys, int64_t stride_key,
                           int64_t stride_sub, int n_sub, const uint8_t *lut, int32_t *cnt) {
  for (int64_t i = 0; i < n_keys; ++i) {
    int32_t c = 0;
    for (int s = 0; s < n_sub; ++s) c += lut[s * PKV_O_KW + codes[i * stride_key + s * stride_sub]];
    cnt[i] = c;
  }
}

/* ------------------------------------------------------------- selections */

int pkv_o_select_candidates(const int32_t *cnt, int64_t n, int64_t k, int64_t *out) {
  if (n <= k) {
    for (int64_t i = 0; i < k; ++i) out[i] = i < n ? i : 0;
    return -1;
  }
  int64_t hist[128];
  memset(hist, 0, sizeof hist);
  for (int64_t i = 0; i < n; ++i) {
    int v = cnt[i] < 0 ? 0 : (cnt[i] > 127 ? 127 : cnt[i]);
    hist[v] += 1;
  }
  int theta = 0;
  int64_t cum = 0;
  for (int b = 127; b >= 0; --b) {
    cum += hist[b];
    if (cum >= k) {
      theta = b;
      break;
    }
  }
  int64_t pos = 0;
  for (int64_t i = 0; i < n; ++i) {
    int v = cnt[i] < 0 ? 0 : (cnt[i] > 127 ? 127 : cnt[i]);
    if (v > theta) out[pos++] = i;
  }
  for (int64_t i = 0; i < n && pos < k; ++i) {
    int v = cnt[i] < 0 ? 0 : (cnt[i] > 127 ? 127 : cnt[i]);
    if (v == theta) out[pos++] = i;
  }
  return theta;
}

void pkv_o_rerank(const int64_t *cand, int64_t n_cand, const uint8_t *nib, int64_t nib_stride_key,
                  int64_t nib_stride_sub, const float *weight, int64_t w_stride_key,
                  int64_t w_stride_sub, const float *qhat, float qnorm, const float *centers,
                  float *scores) {
  for (int64_t i = 0; i < n_cand; ++i) {
    int64_t key = cand[i];
    float s = 0.0f;
    for (int b = 0; b < PKV_O_B; ++b) {
      const uint8_t *p = nib + key * nib_stride_key + b * nib_stride_sub;
      float t = 0.0f;
      for (int j = 0; j < 8; ++j) {
        uint8_t v = (j & 1) ? (uint8_t)(p[j >> 1] >> 4) : (uint8_t)(p[j >> 1] & 0x0f);
        float a = centers[v & 7];
        float val = (v & 8) ? a : -a; /* sign bit set = positive, rerank.cu:107-119 */
        float prod = qhat[8 * b + j] * val;
        t = (j == 0) ? prod : t + prod;
      }
      float tw = t * weight[key * w_stride_key + b * w_stride_sub];
      s = (b == 0) ? tw : s + tw;
    }
    scores[i] = s * qnorm;
  }
}

typedef struct {
  uint32_t key;
  int64_t id;
  int64_t pos;
} topk_item;

static int topk_cmp(const void *a, const void *b) {
  const topk_item *x = (const topk_item *)a, *y = (const topk_item *)b;
  if (x->key != y->key) return x->key > y->key ? -1 : 1;
  return x->id < y->id ? -1 : (x->id > y->id ? 1 : 0);
}

void pkv_o_topk_f32(const float *scores, const int64_t *ids, int64_t n, int64_t k,
                    int64_t *out_ids, int64_t *out_pos) {
  topk_item *it = (topk_item *)malloc((size_t)(n > 0 ? n : 1) * sizeof(topk_item));
  for (int64_t i = 0; i < n; ++i) {
    it[i].key = ordered_u32(scores[i]);
    it[i].id = ids ? ids[i] : i;
    it[i].pos = i;
  }
  qsort(it, (size_t)n, sizeof(topk_item), topk_cmp);
  for (int64_t i = 0; i < k; ++i) {
    if (out_ids) out_ids[i] = i < n ? it[i].id : 0;
    if (out_pos) out_pos[i] = i < n ? it[i].pos : 0;
  }
  free(it);
}

void pkv_o_gather_rows(const void *src, const int64_t *idx, int64_t k, int64_t row_bytes,
                       void *dst) {
  for (int64_t i = 0; i < k; ++i)
    memcpy((char *)dst + i * row_bytes, (const char *)src + idx[i] * row_bytes, (size_t)row_bytes);
}

/* --------------------------------------------------------- dense attention */

void pkv_o_attention(const float *q, int g_heads, const float *k, const float *v, int64_t s,
                     float scale, float *out) {
  double *logit = (double *)malloc(sizeof(double) * (size_t)(s > 0 ? s : 1));
  for (int g = 0; g < g_heads; ++g) {
    double mx = -INFINITY;
    for (int64_t i = 0; i < s; ++i) {
      double acc = 0.0;
      for (int d = 0; d < PKV_O_D; ++d) acc += (double)q[g * PKV_O_D + d] * (double)k[i * PKV_O_D + d];
      logit[i] = acc * (double)scale;
      if (logit[i] > mx) mx = logit[i];
    }
    double den = 0.0, o[PKV_O_D];
    for (int d = 0; d < PKV_O_D; ++d) o[d] = 0.0;
    for (int64_t i = 0; i < s; ++i) {
      const double p = exp(logit[i] - mx);
      den += p;
      for (int d = 0; d < PKV_O_D; ++d) o[d] += p * (double)v[i * PKV_O_D + d];
    }
    for (int d = 0; d < PKV_O_D; ++d) out[g * PKV_O_D + d] = (float)(o[d] / den);
  }
  free(logit);
}

/* --------------------------------------------------------------- adaptive-k */

float pkv_o_expf(float x) {
  if (!(x >= -87.0f)) return (x != x) ? x : 0.0f;
  if (x > 88.0f) return INFINITY;
  float n = rintf(x * 1.44269504f);
  float r = x - n * 0.693359375f;
  r = r - n * (-2.12194440e-4f);
  float p = 1.9875691500e-4f;
  p = p * r + 1.3981999507e-3f;
  p = p * r + 8.3334519073e-3f;
  p = p * r + 4.1665795894e-2f;
  p = p * r + 1.6666665459e-1f;
  p = p * r + 5.0000001201e-1f;
  float z = r * r;
  float y = p * z + r;
  y = y + 1.0f;
  int e = (int)n;
  return y * u2f((uint32_t)(e + 127) << 23);
}

/* Sum in a fixed parallel-friendly order.  The input is cut into slices of 8192
 * consecutive elements.  Inside a slice element j goes to lane j mod 1024,
 * accumulated in increasing j, then a pairwise tree runs over the 1024 lanes
 * (stride 1, 2, 4, ...).  The slice sums are added in slice order, the first
 * one taken as it is.  (Up to 8192 elements this is one slice.) */
#define PKV_O_SUM_LANES 1024
#define PKV_O_SUM_SLICE 8192
static float sum_slice(const float *x, int64_t n) {
  float lane[PKV_O_SUM_LANES];
  for (int t = 0; t < PKV_O_SUM_LANES; ++t) {
    float acc = 0.0f;
    for (int64_t i = t; i < n; i += PKV_O_SUM_LANES) acc = acc + x[i];
    lane[t] = acc;
  }
  for (int h = 1; h < PKV_O_SUM_LANES; h <<= 1)
    for (int i = 0; i < PKV_O_SUM_LANES; i += 2 * h) lane[i] = lane[i] + lane[i + h];
  return lane[0];
}

static float sum_lanes(const float *x, int64_t n) {
  float total = sum_slice(x, n < PKV_O_SUM_SLICE ? n : PKV_O_SUM_SLICE);
  for (int64_t s0 = PKV_O_SUM_SLICE; s0 < n; s0 += PKV_O_SUM_SLICE)
    total = total + sum_slice(x + s0, n - s0 < PKV_O_SUM_SLICE ? n - s0 : PKV_O_SUM_SLICE);
  return total;
}

int64_t pkv_o_adaptive_topk(const float *sl_logits, const float *sl_vnorm, int64_t sl,
                            const float *cand_logits, const float *cand_vnorm,
                            const int64_t *cand_ids, int64_t n_cand, float threshold,
                            int64_t k_out, int64_t *out_ids) {
  /* adaptive_topk.py:282-286 joint max */
  float g = -INFINITY;
  for (int64_t i = 0; i < sl; ++i) g = sl_logits[i] > g ? sl_logits[i] : g;
  for (int64_t i = 0; i < n_cand; ++i) g = cand_logits[i] > g ? cand_logits[i] : g;
  float *ben_sl = (float *)calloc((size_t)(sl > 0 ? sl : 1), sizeof(float));
  float *ben = (float *)malloc((size_t)(n_cand > 0 ? n_cand : 1) * sizeof(float));
  for (int64_t i = 0; i < sl; ++i) ben_sl[i] = pkv_o_expf(sl_logits[i] - g) * sl_vnorm[i];
  for (int64_t i = 0; i < n_cand; ++i) ben[i] = pkv_o_expf(cand_logits[i] - g) * cand_vnorm[i];
  float sl_benefit = sum_lanes(ben_sl, sl);        /* :289 */
  float total = sl_benefit + sum_lanes(ben, n_cand); /* :299 */
  /* :293-296 top-K_out by benefit, descending; ties by candidate position */
  int64_t *pos = (int64_t *)malloc((size_t)(k_out > 0 ? k_out : 1) * sizeof(int64_t));
  pkv_o_topk_f32(ben, NULL, n_cand, k_out, NULL, pos);
  int64_t k = k_out;
  if (total <= 0.0f) {
    k = 1; /* :304-306 */
  } else {
    /* :300-303 cumulative sum of the sorted benefits, in a fixed two-level order:
     * blocks of 64 consecutive elements are summed left to right (run), the block
     * totals are summed left to right (before), prefix = before + run. */
    float tgt = threshold * total, before = 0.0f, run = 0.0f;
    for (int64_t i = 0; i < k_out; ++i) {
      if (i % 64 == 0) {
        before = before + run; /* total of the previous block (0 at the start) */
        run = 0.0f;
      }
      run = run + ben[pos[i]];
      if (sl_benefit + (before + run) >= tgt) {
        k = i + 1;
        break;
      }
    }
  }
  for (int64_t i = 0; i < k_out; ++i) out_ids[i] = cand_ids[pos[i]];
  free(ben_sl);
  free(ben);
  free(pos);
  return k;
}

/* ------------------------------------------------------------ whole row */

void pkv_o_retrieve_row(const float *q, int G, const float *signs, int dtype,
                        const uint8_t *codes, const uint8_t *nib, const float *weight,
                        const int32_t *cluster_counts, int64_t n_keys,
                        const uint32_t *tier_counts, int n_tiers, int64_t n_cand, int64_t k,
                        int64_t *out_ids) {
  float qhat[PKV_O_D], qnorm, th[7], ce[8];
  int64_t sorted_ids[PKV_O_B * PKV_O_KW];
  uint8_t lut[PKV_O_B * PKV_O_KW];
  pkv_o_mag_constants(th, ce);
  pkv_o_query_prep(q, G, signs, dtype, qhat, &qnorm);
  pkv_o_rank_centroids(qhat, dtype, sorted_ids);
  pkv_o_tier_lut(sorted_ids, cluster_counts, PKV_O_B, tier_counts, n_tiers, lut);
  int32_t *cnt = (int32_t *)malloc((size_t)n_keys * sizeof(int32_t));
  pkv_o_collision_count(codes, n_keys, PKV_O_B, 1, PKV_O_B, lut, cnt);
  int64_t *cand = (int64_t *)malloc((size_t)n_cand * sizeof(int64_t));
  pkv_o_select_candidates(cnt, n_keys, n_cand, cand);
  float *scores = (float *)malloc((size_t)n_cand * sizeof(float));
  pkv_o_rerank(cand, n_cand, nib, 64, 4, weight, PKV_O_B, 1, qhat, qnorm, ce, scores);
  int64_t kk = k < n_cand ? k : n_cand;
  pkv_o_topk_f32(scores, cand, n_cand, kk, out_ids, NULL);
  free(cnt);
  free(cand);
  free(scores);
}
