// Shared device/host helpers for the ParisKV retrieval kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>
#include <stdio.h>
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
// that rows * n_chunks is about a thousand workgroups (4 per CU) while the
// per-row chunk histograms (uint16 [n_chunks][128]) stay small.  Always a
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
                                           int64_t *sorted_ids, hipStream_t s);
PKV_INTERNAL int pkv_launch_scan(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                                 int bs, int n_kv_heads, int64_t n_keys, const uint8_t *lut, uint8_t *cnt_u8,
                                 int64_t cnt_u8_stride, int32_t *cnt_i32, uint16_t *chunk_hist, int chunk_keys,
                                 hipStream_t s);
PKV_INTERNAL int pkv_launch_select(const uint8_t *cnt_u8, int64_t cnt_stride, const uint16_t *chunk_hist,
                                   int chunk_keys, int rows, int64_t n_keys, int64_t k, int64_t *out,
                                   hipStream_t s);
PKV_INTERNAL int pkv_launch_rerank(const int64_t *cand, int bs, int n_kv_heads, int64_t n_cand, int64_t n_keys,
                                   const uint8_t *nib, int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub,
                                   const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key,
                                   int64_t ws_sub, const float *qhat, const float *qnorm, const float *centers,
                                   float *scores, uint16_t *v4b, hipStream_t s);
PKV_INTERNAL size_t pkv_topk_ws_bytes_impl(int rows, int64_t len, int64_t k);
PKV_INTERNAL int pkv_launch_topk_f32(const float *x, int64_t x_stride, const int64_t *ids, int64_t ids_stride,
                                     int rows, int64_t len, int64_t k, int64_t *out_ids, float *out_vals,
                                     void *ws, size_t ws_bytes, hipStream_t s);
PKV_INTERNAL int pkv_launch_gather(const void *src_k, const void *src_v, int64_t src_len, const int64_t *idx,
                                   int64_t k, int64_t idx_offset, void *dst_k, void *dst_v, int64_t dst_len,
                                   int64_t dst_row0, int rows, int row_bytes, hipStream_t s);

// -------------------------------------------------------------- device side

#if defined(__HIPCC__)

typedef unsigned int pkv_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int pkv_u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float pkv_bf16_round(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return __uint_as_float((u | 0x00400000u) & 0xffff0000u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return __uint_as_float(u & 0xffff0000u);
}

__device__ __forceinline__ float pkv_rdt(float x, int dtype) {
  return dtype == PKV_DTYPE_BF16 ? pkv_bf16_round(x) : x;
}

__device__ __forceinline__ uint16_t pkv_f32_to_bf16_bits(float x) {
  return (uint16_t)(__float_as_uint(pkv_bf16_round(x)) >> 16);
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

// Inclusive scan over the 64 lanes of a wave.
__device__ __forceinline__ int pkv_wave_incl_scan(int v) {
  const int lane = pkv_lane();
#pragma unroll
  for (int d = 1; d < PKV_WAVE; d <<= 1) {
    int o = __shfl_up(v, d, PKV_WAVE);
    if (lane >= d) v += o;
  }
  return v;
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
