// Shared device/host helpers for the ParisKV retrieval kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/pariskv_hip.h"

#define PKV_WAVE 64

// ---------------------------------------------------------------- host side

void pkv_set_error(const char *fmt, ...);

#define PKV_REQUIRE(cond, ...)        \
  do {                                \
    if (!(cond)) {                    \
      pkv_set_error(__VA_ARGS__);     \
      return PKV_EINVAL;              \
    }                                 \
  } while (0)

#define PKV_HIP(call)                                                         \
  do {                                                                        \
    hipError_t e_ = (call);                                                   \
    if (e_ != hipSuccess) {                                                   \
      pkv_set_error("%s failed: %s", #call, hipGetErrorString(e_));           \
      return PKV_EHIP;                                                        \
    }                                                                         \
  } while (0)

#define PKV_LAUNCH_CHECK(name)                                                \
  do {                                                                        \
    hipError_t e_ = hipGetLastError();                                        \
    if (e_ != hipSuccess) {                                                   \
      pkv_set_error("launch of %s failed: %s", name, hipGetErrorString(e_));  \
      return PKV_EHIP;                                                        \
    }                                                                         \
  } while (0)

static inline size_t pkv_align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
static inline bool pkv_aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

struct PkvTiers {
  uint32_t t[PKV_MAX_TIERS];
  int n;
};

// Keys per workgroup-chunk of the collision scan / candidate select, chosen so
// that rows * n_chunks is about a thousand workgroups (4 per CU, the measured
// optimum at 32 rows x 128K keys) while the per-row chunk histograms (uint16 [n_chunks][128]) stay small.  Always a
// multiple of 2048 and at most 32768 (a chunk's histogram bins are uint16).
static inline int pkv_pick_chunk_keys(int rows, int64_t n_keys) {
  int64_t chunk = 2048;
  while (chunk < 16384 && (int64_t)rows * ((n_keys + chunk - 1) / chunk) > 1024) chunk *= 2;
  while (chunk < 32768 && (n_keys + chunk - 1) / chunk > 512) chunk *= 2;
  return (int)chunk;
}
#define PKV_MAX_KEYS_PER_ROW ((int64_t)1 << 24)  // 512 chunks of 32768 keys

// Internal launchers shared between translation units (not exported).
#define PKV_INTERNAL __attribute__((visibility("hidden")))

PKV_INTERNAL int pkv_launch_query_prep_lut(const void *q, int dtype, int bs, int n_kv_heads, int group,
                                           const float *signs, const int32_t *cc, int64_t cc_b, int64_t cc_h,
                                           const PkvTiers &tiers, float *qhat, float *qnorm, uint8_t *lut,
                                           int64_t *sorted_ids, uint32_t *row_suf_to_zero, hipStream_t s,
                                           uint32_t *zero_ptr = nullptr, int64_t zero_words = 0);
PKV_INTERNAL int pkv_launch_scan(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                                 int bs, int n_kv_heads, int64_t n_keys, const uint8_t *lut, uint8_t *cnt_u8,
                                 int64_t cnt_u8_stride, int32_t *cnt_i32, uint32_t *row_suf, uint16_t *chunk_suf,
                                 int chunk_keys, hipStream_t s, int sub_blocks = 1);
// Pieces per chunk for the scan -> select + rerank pair of a retrieval: chunks of 8192 keys and more are cut into four
// pieces spread over the row (where the row's piece tables stay within what the select keeps in LDS), smaller
// chunks stay whole.
static inline int pkv_pick_sub_blocks(int chunk_keys, int64_t n_chunks) {
  return (chunk_keys >= 8192 && n_chunks * 4 <= 512) ? 4 : 1;
}
PKV_INTERNAL int pkv_launch_select(const uint8_t *cnt_u8, int64_t cnt_stride, const uint32_t *row_suf,
                                   const uint16_t *chunk_suf, int chunk_keys, int rows, int64_t n_keys, int64_t k,
                                   int64_t *out, hipStream_t s);
PKV_INTERNAL int pkv_launch_select_rerank(const uint8_t *cnt_u8, int64_t cnt_stride, const uint32_t *row_suf,
                                          const uint16_t *chunk_suf, int chunk_keys, int bs, int n_kv_heads, int64_t n_keys, int64_t k,
                                          const uint8_t *nib, int64_t ns_b, int64_t ns_h, int64_t ns_key,
                                          const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key,
                                          const float *qhat, const float *qnorm, const float *centers, int64_t *cand,
                                          float *scores, hipStream_t s, int64_t extra_off = 0,
                                          float *extra_out = nullptr, uint32_t *range_slots = nullptr,
                                          int64_t range_row_stride = 0, int sub_blocks = 1);
PKV_INTERNAL int pkv_launch_rerank(const int64_t *cand, int bs, int n_kv_heads, int64_t n_cand, int64_t n_keys,
                                   const uint8_t *nib, int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub,
                                   const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key,
                                   int64_t ws_sub, const float *qhat, const float *qnorm, const float *centers,
                                   float *scores, uint16_t *v4b, hipStream_t s);
PKV_INTERNAL size_t pkv_topk_ws_bytes_impl(int rows, int64_t len, int64_t k);
PKV_INTERNAL int64_t pkv_topk_ctl_words(int rows, int64_t len);
PKV_INTERNAL uint32_t *pkv_topk_range_slots(uint32_t *ctl, int64_t len, int64_t *row_stride);
PKV_INTERNAL int pkv_launch_topk_f32(const float *x, int64_t x_stride, const int64_t *ids, int64_t ids_stride,
                                     int rows, int64_t len, int64_t k, int64_t *out_ids, float *out_vals,
                                     void *ws, size_t ws_bytes, hipStream_t s, bool any_order = false,
                                     bool ctl_ready = false);
PKV_INTERNAL int pkv_launch_gather(const void *src_k, const void *src_v, int64_t src_len, const int64_t *idx,
                                   int64_t k, int64_t idx_offset, void *dst_k, void *dst_v, int64_t dst_len,
                                   int64_t dst_row0, int rows, int row_bytes, hipStream_t s, const int64_t *row_counts = nullptr);

// -------------------------------------------------------------- device side

#if defined(__HIPCC__)

typedef unsigned int pkv_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int pkv_u32x2 __attribute__((ext_vector_type(2)));

// Round to nearest even bf16 and widen again, in one instruction: the packed hardware conversion
// (v_cvt_pk_bf16_f32) of the pair (0, x) leaves bf16(x) in the upper half of the register and zero in the
// lower half, which is bf16(x) read as an fp32.
typedef __bf16 pkv_bf16x2 __attribute__((ext_vector_type(2)));
typedef float pkv_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float pkv_bf16_round(float x) {
  const pkv_f32x2 v = {0.0f, x};
  return __builtin_bit_cast(float, __builtin_convertvector(v, pkv_bf16x2));
}

__device__ __forceinline__ float pkv_rdt(float x, int dtype) {
  return dtype == PKV_DTYPE_BF16 ? pkv_bf16_round(x) : x;
}

__device__ __forceinline__ uint16_t pkv_f32_to_bf16_bits(float x) {
  return __builtin_bit_cast(uint16_t, (__bf16)x);
}

__device__ __forceinline__ float pkv_bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// Order-preserving map float -> uint32 (larger float <=> larger uint).
__device__ __forceinline__ uint32_t pkv_ordered_u32(float x) {
  uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ float pkv_from_ordered_u32(uint32_t k) {
  uint32_t b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(b);
}

// 1/sqrt(128) as the fp32 nearest to the double 1.0/sqrt(128.0).
#define PKV_HADAMARD_SCALE 0.08838834764831845f

__device__ __forceinline__ int pkv_lane() { return (int)(threadIdx.x & (PKV_WAVE - 1)); }

// Value of lane (lane ^ M).  M = 1, 2, 3, 4, 7, 8, 15 are data-parallel-primitive moves inside a row of 16 lanes
// (no trip through the LDS crossbar); 16 and 32 use the generic lane permute.
template <int M>
__device__ __forceinline__ uint32_t pkv_lane_xor(uint32_t v) {
  const int x = (int)v;
  if (M == 1) return (uint32_t)__builtin_amdgcn_mov_dpp(x, 0xB1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
  if (M == 2) return (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x4E, 0xf, 0xf, false);   // quad_perm [2,3,0,1]
  if (M == 3) return (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x1B, 0xf, 0xf, false);   // quad_perm [3,2,1,0]
  if (M == 7) return (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x141, 0xf, 0xf, false);  // row_half_mirror
  if (M == 15) return (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x140, 0xf, 0xf, false); // row_mirror
  if (M == 4) {
    int r = __builtin_amdgcn_update_dpp(x, x, 0x104, 0xf, 0x5, false);  // banks 0,2 read lane + 4 (row_shl:4)
    r = __builtin_amdgcn_update_dpp(r, x, 0x114, 0xf, 0xa, false);      // banks 1,3 read lane - 4 (row_shr:4)
    return (uint32_t)r;
  }
  if (M == 8) return (uint32_t)__builtin_amdgcn_mov_dpp(x, 0x128, 0xf, 0xf, false);  // row_ror:8
  return (uint32_t)__shfl_xor(x, M, PKV_WAVE);
}
template <int M>
__device__ __forceinline__ float pkv_lane_xor_f(float v) {
  return __uint_as_float(pkv_lane_xor<M>(__float_as_uint(v)));
}
template <int M>
__device__ __forceinline__ uint64_t pkv_lane_xor64(uint64_t v) {
  return ((uint64_t)pkv_lane_xor<M>((uint32_t)(v >> 32)) << 32) | pkv_lane_xor<M>((uint32_t)v);
}

// Inclusive scan over the 64 lanes of a wave: four row_shr steps inside each row of 16 lanes, then the
// row totals travel with row_bcast:15 (rows 1, 3) and row_bcast:31 (rows 2, 3).
__device__ __forceinline__ int pkv_wave_incl_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);
  return v;
}

// Normalise and SRHT-rotate one 128-vector spread over 16 lanes: the lane of block s holds
// dims 8s..8s+7 in x[] (and the matching SRHT signs in sg[]).  On return y[] holds the rotated unit
// vector's dims 8s..8s+7 and the norm is returned (both rounded to `dtype` where the reference's
// tensors are).  Operation order: sum of squares sequential inside the 8 dims, then a pairwise tree
// over the 16 blocks; natural-order Walsh-Hadamard butterflies h = 1..64 (three in-lane stages, four
// lane-xor stages); then * 1/sqrt(128).  All 16 lanes of the group must be active.
// M4 / M8: the lane distance (xor) to the block s ^ 4 / s ^ 8; blocks s ^ 1 and s ^ 2 sit at lane ^ 1 and lane ^ 2.
// The natural placement (block s in lane s) has M4 = 4, M8 = 8.
template <int M4 = 4, int M8 = 8>
__device__ __forceinline__ float pkv_normalize_rotate_16(const float (&x)[8], const float (&sg)[8], int s, int dtype,
                                                         float (&y)[8]) {
  float acc = x[0] * x[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) acc = acc + x[j] * x[j];
  acc = acc + pkv_lane_xor_f<1>(acc);
  acc = acc + pkv_lane_xor_f<2>(acc);
  acc = acc + pkv_lane_xor_f<M4>(acc);
  acc = acc + pkv_lane_xor_f<M8>(acc);
  const float n = pkv_rdt(sqrtf(acc), dtype);
  const float den = n < 1e-8f ? 1e-8f : n;
  float t[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) t[j] = pkv_rdt(x[j] / den, dtype) * sg[j];
#pragma unroll
  for (int hh = 1; hh < 8; hh <<= 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if ((i & hh) == 0) {
        const float a = t[i], c = t[i + hh];
        t[i] = a + c;
        t[i + hh] = a - c;
      }
    }
  }
#define PKV_FWHT_LANE_STAGE(BIT, M)                         \
  _Pragma("unroll") for (int j = 0; j < 8; ++j) {           \
    const float o = pkv_lane_xor_f<M>(t[j]);                \
    t[j] = (s & BIT) ? (o - t[j]) : (t[j] + o);             \
  }
  PKV_FWHT_LANE_STAGE(1, 1)
  PKV_FWHT_LANE_STAGE(2, 2)
  PKV_FWHT_LANE_STAGE(4, M4)
  PKV_FWHT_LANE_STAGE(8, M8)
#undef PKV_FWHT_LANE_STAGE
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = pkv_rdt(t[j] * PKV_HADAMARD_SCALE, dtype);
  return n;
}

// Mean of the G query heads of row (b, h) (polar_cache.py:1027): lane l of a wave gets dims 8(l & 15) .. +7
// in x[], rounded to the working dtype.  The G heads are added in order; their loads are all issued before
// the first add (4 at a time, with no branch between them, so that they are in flight together).
template <bool BF16>
__device__ __forceinline__ void pkv_query_group_mean_t(const void *__restrict__ q, int b, int h, int n_kv_heads,
                                                       int group, float (&x)[8]) {
  constexpr int dtype = BF16 ? PKV_DTYPE_BF16 : PKV_DTYPE_F32;
  const int s = pkv_lane() & 15;
  const int64_t base = ((int64_t)b * n_kv_heads * group + (int64_t)h * group) * 128 + 8 * s;
  float acc[8];
  constexpr int kHeadsInFlight = 4;
  for (int g0 = 0; g0 < group; g0 += kHeadsInFlight) {
    pkv_u32x4 raw[kHeadsInFlight][BF16 ? 1 : 2];
#pragma unroll
    for (int u = 0; u < kHeadsInFlight; ++u) {
      const int g = g0 + u < group ? g0 + u : group - 1;
      if (BF16) {
        raw[u][0] = *(const pkv_u32x4 *)((const uint16_t *)q + base + (int64_t)g * 128);
      } else {
        raw[u][0] = *(const pkv_u32x4 *)((const float *)q + base + (int64_t)g * 128);
        raw[u][BF16 ? 0 : 1] = *(const pkv_u32x4 *)((const float *)q + base + (int64_t)g * 128 + 4);
      }
    }
#pragma unroll
    for (int u = 0; u < kHeadsInFlight; ++u) {
      float v[8];
      if (BF16) {
        const uint32_t ww[4] = {raw[u][0].x, raw[u][0].y, raw[u][0].z, raw[u][0].w};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          v[2 * p] = __uint_as_float(ww[p] << 16);
          v[2 * p + 1] = __uint_as_float(ww[p] & 0xffff0000u);
        }
      } else {
        const pkv_u32x4 lo = raw[u][0], hi = raw[u][BF16 ? 0 : 1];
        v[0] = __uint_as_float(lo.x), v[1] = __uint_as_float(lo.y), v[2] = __uint_as_float(lo.z);
        v[3] = __uint_as_float(lo.w), v[4] = __uint_as_float(hi.x), v[5] = __uint_as_float(hi.y);
        v[6] = __uint_as_float(hi.z), v[7] = __uint_as_float(hi.w);
      }
      const bool first = g0 + u == 0, live = g0 + u < group;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = first ? v[j] : (live ? acc[j] + v[j] : acc[j]);
    }
  }
  if ((group & (group - 1)) == 0) {  // power of two: multiplying by the reciprocal is the same division, exactly
    const float inv = 1.0f / (float)group;
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = pkv_rdt(acc[j] * inv, dtype);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = pkv_rdt(acc[j] / (float)group, dtype);
  }
}

// The normalisation and rotation of pkv_normalize_rotate_16 with the 128-vector spread over the 64 lanes of ONE wave: lane l holds dims
// l and l + 64 (x_lo, x_hi).  Every value goes through the same sequence of fp32 operations as in
// pkv_normalize_rotate_16 (sum of squares: left to right inside each aligned block of 8 dims = 8 neighbouring lanes,
// then the pairwise tree over the 16 blocks; the butterflies h = 1 .. 64 in that order), so the results are
// bit-identical; what changes is the length of the dependent chain: two divisions and seven butterfly steps per
// lane instead of eight and fifty-six.  All 64 lanes must be active.  Returns the norm; y_lo / y_hi = rotated unit
// vector's dims l and l + 64.
__device__ __forceinline__ float pkv_normalize_rotate_64(float x_lo, float x_hi, float sg_lo, float sg_hi, int dtype,
                                                         float &y_lo, float &y_hi) {
  const int lane = pkv_lane();
  const bool first = (lane & 7) == 0;
  const float p_lo = x_lo * x_lo, p_hi = x_hi * x_hi;
  float r_lo = p_lo, r_hi = p_hi;
#pragma unroll
  for (int t = 1; t < 8; ++t) {  // after step t the lanes with (lane & 7) <= t hold p_0 + ... + p_(lane & 7), left to right
    const float below_lo = __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(r_lo), 0x111, 0xf, 0xf, true));
    const float below_hi = __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(r_hi), 0x111, 0xf, 0xf, true));
    r_lo = first ? p_lo : below_lo + p_lo;
    r_hi = first ? p_hi : below_hi + p_hi;
  }
  // block totals sit in the lanes with (lane & 7) == 7; tree over the block index: lane ^ 8, ^ 16, ^ 32, then the halves
  r_lo = r_lo + pkv_lane_xor_f<8>(r_lo);
  r_hi = r_hi + pkv_lane_xor_f<8>(r_hi);
  r_lo = r_lo + pkv_lane_xor_f<16>(r_lo);
  r_hi = r_hi + pkv_lane_xor_f<16>(r_hi);
  r_lo = r_lo + pkv_lane_xor_f<32>(r_lo);
  r_hi = r_hi + pkv_lane_xor_f<32>(r_hi);
  const float total = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(r_lo + r_hi), 7));
  const float n = pkv_rdt(sqrtf(total), dtype);
  const float den = n < 1e-8f ? 1e-8f : n;
  float t_lo = pkv_rdt(x_lo / den, dtype) * sg_lo;
  float t_hi = pkv_rdt(x_hi / den, dtype) * sg_hi;
#define PKV_FWHT_WAVE_STAGE(M)                         \
  {                                                    \
    const float o_lo = pkv_lane_xor_f<M>(t_lo);        \
    const float o_hi = pkv_lane_xor_f<M>(t_hi);        \
    t_lo = (lane & M) ? (o_lo - t_lo) : (t_lo + o_lo); \
    t_hi = (lane & M) ? (o_hi - t_hi) : (t_hi + o_hi); \
  }
  PKV_FWHT_WAVE_STAGE(1)
  PKV_FWHT_WAVE_STAGE(2)
  PKV_FWHT_WAVE_STAGE(4)
  PKV_FWHT_WAVE_STAGE(8)
  PKV_FWHT_WAVE_STAGE(16)
  PKV_FWHT_WAVE_STAGE(32)
#undef PKV_FWHT_WAVE_STAGE
  const float a = t_lo, c = t_hi;  // h = 64: the two halves of the lane
  y_lo = pkv_rdt((a + c) * PKV_HADAMARD_SCALE, dtype);
  y_hi = pkv_rdt((a - c) * PKV_HADAMARD_SCALE, dtype);
  return n;
}

// Group mean of the G query heads of row (b, h), dims l and l + 64 for lane l of one wave, rounded to the working
// dtype; the heads are added in order (polar_cache.py:1027).
template <bool BF16>
__device__ __forceinline__ void pkv_query_group_mean_wave_t(const void *__restrict__ q, int b, int h, int n_kv_heads,
                                                            int group, float &x_lo, float &x_hi) {
  constexpr int dtype = BF16 ? PKV_DTYPE_BF16 : PKV_DTYPE_F32;
  const int lane = pkv_lane();
  const int64_t base = ((int64_t)b * n_kv_heads * group + (int64_t)h * group) * 128 + lane;
  float a_lo = 0.f, a_hi = 0.f;
  constexpr int kHeadsInFlight = 4;
  for (int g0 = 0; g0 < group; g0 += kHeadsInFlight) {
    float v_lo[kHeadsInFlight], v_hi[kHeadsInFlight];
#pragma unroll
    for (int u = 0; u < kHeadsInFlight; ++u) {
      const int g = g0 + u < group ? g0 + u : group - 1;
      if (BF16) {
        v_lo[u] = pkv_bf16_bits_to_f32(((const uint16_t *)q)[base + (int64_t)g * 128]);
        v_hi[u] = pkv_bf16_bits_to_f32(((const uint16_t *)q)[base + (int64_t)g * 128 + 64]);
      } else {
        v_lo[u] = ((const float *)q)[base + (int64_t)g * 128];
        v_hi[u] = ((const float *)q)[base + (int64_t)g * 128 + 64];
      }
    }
#pragma unroll
    for (int u = 0; u < kHeadsInFlight; ++u) {
      const bool first = g0 + u == 0, live = g0 + u < group;
      a_lo = first ? v_lo[u] : (live ? a_lo + v_lo[u] : a_lo);
      a_hi = first ? v_hi[u] : (live ? a_hi + v_hi[u] : a_hi);
    }
  }
  if ((group & (group - 1)) == 0) {  // power of two: multiplying by the reciprocal is the same division, exactly
    const float inv = 1.0f / (float)group;
    x_lo = pkv_rdt(a_lo * inv, dtype), x_hi = pkv_rdt(a_hi * inv, dtype);
  } else {
    x_lo = pkv_rdt(a_lo / (float)group, dtype), x_hi = pkv_rdt(a_hi / (float)group, dtype);
  }
}

// Group mean, normalise, SRHT rotate by all 64 lanes of ONE wave: lane l gets dims l and l + 64 of the rotated unit
// vector and the norm of the mean as result (polar_cache.py:1027-1031, 905-922).
__device__ __forceinline__ float pkv_query_mean_rotate_wave(const void *__restrict__ q, int dtype, int b, int h,
                                                            int n_kv_heads, int group, const float *__restrict__ signs,
                                                            float &y_lo, float &y_hi) {
  const int lane = pkv_lane();
  const float sg_lo = signs[lane], sg_hi = signs[lane + 64];
  float x_lo, x_hi;
  if (dtype == PKV_DTYPE_BF16) pkv_query_group_mean_wave_t<true>(q, b, h, n_kv_heads, group, x_lo, x_hi);
  else pkv_query_group_mean_wave_t<false>(q, b, h, n_kv_heads, group, x_lo, x_hi);
  return pkv_normalize_rotate_64(x_lo, x_hi, sg_lo, sg_hi, dtype, y_lo, y_hi);
}

// ---- hand-overs between workgroups inside one launch ----
// The chip's eight dies have an L2 each and a launch's workgroups are dealt out over all of them, so plain stores
// of one workgroup (held in its die's write-back L2) and plain loads of another (served from its own die's L2 or the
// compute unit's L1) do not meet inside a launch.  Accesses that carry the agent-scope bit (sc1: what the compiler
// emits for relaxed atomic loads and stores at agent scope) do: such a store is written through to memory before it
// is acknowledged, such a load misses the L1 and is not served from a stale L2 line.  The protocol built on them:
// a producer writes its data with pkv_st_agent_*, every wave waits for its stores' acknowledgements
// (pkv_wait_vmem) before a workgroup barrier, then ONE lane publishes a flag with pkv_st_agent_u64; a consumer polls
// the flag with pkv_ld_agent_u64 and reads the data with pkv_ld_agent_* afterwards.  No cache write-back or
// invalidate instruction is involved.
__device__ __forceinline__ void pkv_wait_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void pkv_st_agent_u16(void *p, uint32_t v) {
  asm volatile("global_store_short %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void pkv_st_agent_u32(void *p, uint32_t v) {
  asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void pkv_st_agent_u64(void *p, uint64_t v) {
  asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void pkv_st_agent_x4(void *p, pkv_u32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
// Loads: the request and the wait for its data are ONE asm statement, so the compiler never sees the destination
// register before the data is in it (it may otherwise move or merge the register between a bare load and a later wait).
__device__ __forceinline__ uint32_t pkv_ld_agent_u32(const void *p) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ uint64_t pkv_ld_agent_u64(const void *p) {
  uint64_t v;
  asm volatile("global_load_dwordx2 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ pkv_u32x4 pkv_ld_agent_x4(const void *p) {
  pkv_u32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  return v;
}
// two half-words, both requests in flight together
__device__ __forceinline__ void pkv_ld_agent_u16_pair(const void *p0, const void *p1, uint32_t &a, uint32_t &b) {
  asm volatile("global_load_ushort %0, %2, off sc1\n\tglobal_load_ushort %1, %3, off sc1\n\ts_waitcnt vmcnt(0)"
               : "=&v"(a), "=&v"(b)
               : "v"(p0), "v"(p1)
               : "memory");
}

// Wait (lanes [0, n) of the calling wave, n <= 64, one flag each) until flags[lane] == epoch for all of them, for at
// most `ticks` of the 100 MHz wall clock.  All 64 lanes of the wave call it; returns false if it gave up.
__device__ __forceinline__ bool pkv_wait_flags(const uint64_t *flags, int n, uint64_t epoch, uint64_t ticks) {
  const int lane = pkv_lane();
  const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
  while (true) {
    const uint64_t f = lane < n ? pkv_ld_agent_u64(flags + lane) : epoch;
    if (__ballot(f != epoch) == 0ull) return true;
    __builtin_amdgcn_s_sleep(2);
    if (__builtin_amdgcn_s_memrealtime() - t0 > ticks) return false;
  }
}

// ---- 4-bit rerank core (shared by the stand-alone rerank and the fused select+rerank kernels) ----
// s_prod[d][v] = qhat[d] * value(v) for the 16 possible 4-bit codes v (bit 3 = sign, set = positive;
// bits 0-2 = magnitude centre): the product of the reference's expression is looked up instead of
// recomputed (same single rounding), one conflict-free LDS read per dim.
template <int NT>
__device__ __forceinline__ void pkv_build_prod_table(float *s_prod, const float *__restrict__ qhat_row,
                                                     const float *__restrict__ centers) {
#pragma unroll
  for (int u = 0; u < 128 * 16 / NT; ++u) {
    const int e = threadIdx.x + u * NT;
    const float a = centers[e & 7];
    s_prod[e] = qhat_row[e >> 4] * ((e & 8) ? a : -a);
  }
}

typedef const __attribute__((address_space(3))) float *pkv_lds_cfloat_ptr;

__device__ __forceinline__ float pkv_block_dot(const float *__restrict__ s_prod, int blk, uint32_t word) {
  // the table always lives in LDS: say so, or the 128 reads become flat loads with 64-bit addresses
  const pkv_lds_cfloat_ptr lp = (pkv_lds_cfloat_ptr)s_prod;
  float t = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float prod = lp[(8 * blk + j) * 16 + ((word >> (4 * j)) & 15u)];
    t = (j == 0) ? prod : t + prod;
  }
  return t;
}

// Score of one key stored key-major: 64 B of nibbles at np, 16 bf16 weights at wp (both 16-byte aligned; in the
// cache's layout the two sit in one 128-byte record, so a candidate costs one HBM line).
// Order: dims 0..7 inside a block, blocks 0..15, then * ||q||; multiply and add rounded separately.
// The four 16-byte groups are walked by a rolled loop that rotates the data registers, so that only one
// group's 32 table reads are in flight at a time (fully unrolled, the scheduler hoists all 128 reads and
// the kernel needs ~170 registers).
// LDS byte address base + 4 * (nibble of `word` at bit `shift`): a bit-field extract and a shift-and-add.  Written
// out because the compiler turns the same expression into shift, mask and add (three instructions, 128 times per key).
__device__ __forceinline__ uint32_t pkv_nibble_lds_addr(uint32_t word, int shift, uint32_t base) {
  uint32_t a;
  asm("v_bfe_u32 %0, %1, %2, 4\n\tv_lshl_add_u32 %0, %0, 2, %3" : "=&v"(a) : "v"(word), "s"(shift), "s"(base));
  return a;
}

__device__ __forceinline__ float pkv_rerank_keymajor(const float *__restrict__ s_prod, const pkv_u32x4 *__restrict__ np,
                                                     const pkv_u32x4 *__restrict__ wp, float qnorm) {
  pkv_u32x4 n0 = np[0], n1 = np[1], n2 = np[2], n3 = np[3];
  pkv_u32x4 w0 = wp[0], w1 = wp[1];
  const pkv_lds_cfloat_ptr lp = (pkv_lds_cfloat_ptr)s_prod;
  float s = 0.f;
#pragma unroll 1
  for (int u = 0; u < 4; ++u) {
    const uint32_t words[4] = {n0.x, n0.y, n0.z, n0.w};
    const uint32_t wpair[2] = {w0.x, w0.y};
    const uint32_t group_base = (uint32_t)(uintptr_t)(lp + 512 * u);  // LDS byte address of this group's 32 table rows
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float t = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float prod = ((pkv_lds_cfloat_ptr)(uintptr_t)pkv_nibble_lds_addr(words[i], 4 * j, group_base))[(8 * i + j) * 16];
        t = (j == 0) ? prod : t + prod;
      }
      const uint32_t wb = (i & 1) ? (wpair[i >> 1] >> 16) : (wpair[i >> 1] & 0xffffu);
      const float tw = t * pkv_bf16_bits_to_f32(wb);
      s = (u == 0 && i == 0) ? tw : s + tw;
    }
    n0 = n1, n1 = n2, n2 = n3;
    w0 = pkv_u32x4{w0.z, w0.w, w1.x, w1.y};
    w1 = pkv_u32x4{w1.z, w1.w, 0u, 0u};
  }
  return s * qnorm;
}

// Turn a 128-bin histogram in LDS (s_hist) into its suffix sums suf[t] = sum_{t' >= t} hist[t'],
// store them as the chunk's uint16 suffix histogram (bin t at chunk_suf[t * bin_stride]) and add them to the
// row's uint32 suffix totals (row_suf may be null).
// Called by all threads of a workgroup with >= 128 threads; contains barriers.  s_w0: one LDS word.
__device__ __forceinline__ void pkv_store_suffix_hist(const uint32_t *s_hist, uint32_t *s_w0,
                                                      uint32_t *__restrict__ row_suf, uint16_t *__restrict__ chunk_suf,
                                                      int64_t bin_stride = 1) {
  const int tid = threadIdx.x;
  int incl = 0;
  if (tid < 128) {  // thread t owns bin 127 - t: an inclusive scan over t is the suffix sum over bins
    incl = pkv_wave_incl_scan((int)s_hist[127 - tid]);
    if (tid == PKV_WAVE - 1) *s_w0 = (uint32_t)incl;
  }
  __syncthreads();
  if (tid < 128) {
    if (tid >= PKV_WAVE) incl += (int)*s_w0;
    chunk_suf[(int64_t)(127 - tid) * bin_stride] = (uint16_t)incl;  // bin_stride > 1: a bin-major table shared with other chunks
    if (row_suf && incl) atomicAdd(&row_suf[127 - tid], (uint32_t)incl);
  }
}

// Exclusive scan across a workgroup of NT threads (NT multiple of 64, <= 1024).
// `smem` must hold NT/64 ints and must not be reused before the next barrier by
// callers that loop (pass alternating buffers).  Returns the exclusive prefix;
// `total` receives the workgroup sum.
template <int NT>
__device__ __forceinline__ int pkv_block_excl_scan(int v, int *smem, int &total) {
  constexpr int NW = NT / PKV_WAVE;
  const int lane = pkv_lane();
  const int wave = (int)(threadIdx.x / PKV_WAVE);
  int incl = pkv_wave_incl_scan(v);
  if (lane == PKV_WAVE - 1) smem[wave] = incl;
  __syncthreads();
  int off = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    int t = smem[w];
    if (w < wave) off += t;
    tot += t;
  }
  total = tot;
  return off + incl - v;
}

#endif  // __HIPCC__
