// Pieces of the candidate select shared by the stand-alone select kernels and the fused retrieval kernel:
// threshold masks over 16 packed vote counts, and the threshold / output offsets of one chunk from the suffix
// histograms of the collision scan.
//
// Reference: cache_hub/topk/radix_topk.cu:39-120 (bucket_topk_kernel), cache_hub/polar_cache.py:1237-1242.
#pragma once

#include "pkv_common.h"

#if defined(__HIPCC__)

constexpr int kSelThreads = 256;
constexpr int kSelKeysPerThread = 16;                             // one 128-bit load of counts
constexpr int kSelKeysPerIter = kSelThreads * kSelKeysPerThread;  // 4096

// 16 one-byte counts (all <= 127) against the threshold, four at a time: adding 127 - theta
// (128 - theta) to a byte sets its top bit exactly when the count is above (at or above) theta, and no
// byte overflows into its neighbour.  Bit 8b + 7 of gt[d] / eq[d] stands for key 4d + b; only the
// first n_valid keys count.
__device__ __forceinline__ void count_masks16(const pkv_u32x4 w, uint32_t theta, int64_t n_valid, uint32_t (&gt)[4],
                                              uint32_t (&eq)[4]) {
  const uint32_t kgt = (127u - theta) * 0x01010101u, kge = (128u - theta) * 0x01010101u;
  const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int64_t left = n_valid - 4 * d;
    const uint32_t vm = left >= 4 ? 0x80808080u : (left <= 0 ? 0u : (0x80808080u >> (8 * (4 - (int)left))));
    const uint32_t v7 = ww[d] & 0x7f7f7f7fu;
    const uint32_t g = (v7 + kgt) & vm;
    const uint32_t ge = (v7 + kge) & vm;
    gt[d] = g;
    eq[d] = ge & ~g;
  }
}

__device__ __forceinline__ int popc4(const uint32_t (&m)[4]) {
  return __popc(m[0]) + __popc(m[1]) + __popc(m[2]) + __popc(m[3]);
}

// Threshold and output offsets of one workgroup from the suffix histograms the collision scan leaves
// behind: row_suf[row][t] = keys of the row with count >= t (summed over chunks with atomics),
// chunk_suf[row][c][t] = the same for chunk c alone.  theta = largest t with row_suf[t] >= k;
// base_gt = keys above theta in earlier chunks; base_eq = (keys above theta in the row) + keys at
// theta in earlier chunks.  Two dependent loads, no loops over bins.
// rs_mine = row_suf[row][tid] for tid < 128, loaded by the caller as its first instruction so that the load is in
// flight while the caller sets up whatever else it needs before the threshold.
template <bool AGENT = false>
__device__ __forceinline__ void select_prologue(uint32_t rs_mine, const uint16_t *__restrict__ chunk_suf, int row,
                                                int chunk, int n_chunks, int64_t k, uint32_t &theta, int64_t &base_gt,
                                                int64_t &base_eq) {
  __shared__ uint32_t s_rs[129];
  __shared__ uint32_t s_theta, s_ngt;
  __shared__ uint32_t s_red[2][kSelThreads / PKV_WAVE];
  const int tid = threadIdx.x;
  if (tid < 128) s_rs[tid] = rs_mine;
  if (tid == 128) {
    s_rs[128] = 0;
    s_theta = 0;
    s_ngt = 0;
  }
  __syncthreads();
  if (tid < 128 && (int64_t)s_rs[tid] >= k && (int64_t)s_rs[tid + 1] < k) {
    s_theta = (uint32_t)tid;
    s_ngt = s_rs[tid + 1];
  }
  __syncthreads();
  theta = s_theta;
  uint32_t gt = 0, eq = 0;
  const uint16_t *cs = chunk_suf + (int64_t)row * n_chunks * 128;
  for (int c = tid; c < chunk; c += kSelThreads) {
    uint32_t ge, g;
    if (AGENT) {  // written by other workgroups of this launch
      pkv_ld_agent_u16_pair(cs + (int64_t)c * 128 + theta, cs + (int64_t)c * 128 + (theta < 127 ? theta + 1 : theta), ge, g);
      if (theta >= 127) g = 0u;
    } else {
      ge = cs[(int64_t)c * 128 + theta];
      g = theta < 127 ? cs[(int64_t)c * 128 + theta + 1] : 0u;
    }
    gt += g;
    eq += ge - g;
  }
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) {
    gt += __shfl_xor(gt, m, PKV_WAVE);
    eq += __shfl_xor(eq, m, PKV_WAVE);
  }
  if (pkv_lane() == 0) {
    s_red[0][tid / PKV_WAVE] = gt;
    s_red[1][tid / PKV_WAVE] = eq;
  }
  __syncthreads();
  gt = eq = 0;
#pragma unroll
  for (int w = 0; w < kSelThreads / PKV_WAVE; ++w) {
    gt += s_red[0][w];
    eq += s_red[1][w];
  }
  base_gt = gt;
  base_eq = (int64_t)s_ngt + eq;
}


#endif  // __HIPCC__
