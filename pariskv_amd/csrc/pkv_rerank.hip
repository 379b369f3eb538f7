// Fused 4-bit RaBitQ-style rerank of the candidate keys.
//
// Reference: cache_hub/rerank/rerank.cu:51-138 (partial_rerank_kernel) and the
// torch form cache_hub/polar_cache.py:1281-1298.  The reference gathers, per
// candidate, 16 x (4 B + 2 B) at stride kv_len (32 scattered sectors), rounds to
// bf16 after every operation and also stores the unpacked values.  With
// key-major storage a candidate is 64 B of nibbles + 32 B of weights, read with
// six 128-bit loads; the arithmetic is fp32 in a fixed order (dims 0..7 inside
// a block, blocks 0..15, then * ||q||) with separate multiply and add.
#include "pkv_common.h"

#include <math.h>

namespace {

constexpr int kRerankThreads = 256;

__device__ __forceinline__ void store_v4b(uint16_t *__restrict__ v4b, int64_t row, int64_t n_cand, int64_t i, int blk,
                                          const float *__restrict__ s_val, uint32_t word) {
  pkv_u32x4 o;
  uint32_t h[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) h[j] = __float_as_uint(s_val[(word >> (4 * j)) & 15u]) >> 16;
  o.x = h[0] | (h[1] << 16);
  o.y = h[2] | (h[3] << 16);
  o.z = h[4] | (h[5] << 16);
  o.w = h[6] | (h[7] << 16);
  *(pkv_u32x4 *)(v4b + (((row * 16 + blk) * n_cand) + i) * 8) = o;
}

// KEYMAJOR: 64 contiguous nibble bytes and 16 contiguous bf16 weights per key, both 16-byte aligned
// (key strides ns_key bytes / ws_key elements: 64 / 16 when packed, 128 / 64 inside a 128-byte record).
// Otherwise: nib addressed by (ns_key, ns_sub) in bytes (4-byte aligned words),
// weight by (ws_key, ws_sub) in elements.
template <bool KEYMAJOR, bool V4B>
__global__ __launch_bounds__(kRerankThreads) void pkv_rerank_kernel(
    const int64_t *__restrict__ cand, int n_kv_heads, int64_t n_cand, int64_t n_keys, const uint8_t *__restrict__ nib,
    int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub, const uint16_t *__restrict__ weight, int64_t ws_b,
    int64_t ws_h, int64_t ws_key, int64_t ws_sub, const float *__restrict__ qhat, const float *__restrict__ qnorm,
    const float *__restrict__ centers, float *__restrict__ scores, uint16_t *__restrict__ v4b) {
  const int row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;
  __shared__ float s_prod[128 * 16];
  __shared__ float s_val[16];
  if (tid < 16) {
    const float a = centers[tid & 7];
    s_val[tid] = (tid & 8) ? a : -a;  // sign bit set = positive (rerank.cu:107-119)
  }
  pkv_build_prod_table<kRerankThreads>(s_prod, qhat + (int64_t)row * 128, centers);
  __syncthreads();
  const int64_t i = (int64_t)blockIdx.x * kRerankThreads + tid;
  if (i >= n_cand) return;
  const int64_t key = cand[(int64_t)row * n_cand + i];
  float *out = scores + (int64_t)row * n_cand + i;
  if ((uint64_t)key >= (uint64_t)n_keys) {
    *out = -INFINITY;
    return;
  }
  const uint8_t *nrow = nib + (int64_t)b * ns_b + (int64_t)h * ns_h;
  const uint16_t *wrow = weight + (int64_t)b * ws_b + (int64_t)h * ws_h;
  float s = 0.f;
  if (KEYMAJOR) {
    const pkv_u32x4 *np = (const pkv_u32x4 *)(nrow + key * ns_key);
    const pkv_u32x4 *wp = (const pkv_u32x4 *)(wrow + key * ws_key);
    pkv_u32x4 nv[4], wv[2];
#pragma unroll
    for (int u = 0; u < 4; ++u) nv[u] = np[u];
    wv[0] = wp[0];
    wv[1] = wp[1];
    const uint32_t words[16] = {nv[0].x, nv[0].y, nv[0].z, nv[0].w, nv[1].x, nv[1].y, nv[1].z, nv[1].w,
                                nv[2].x, nv[2].y, nv[2].z, nv[2].w, nv[3].x, nv[3].y, nv[3].z, nv[3].w};
    const uint32_t wpair[8] = {wv[0].x, wv[0].y, wv[0].z, wv[0].w, wv[1].x, wv[1].y, wv[1].z, wv[1].w};
#pragma unroll
    for (int blk = 0; blk < 16; ++blk) {
      const float t = pkv_block_dot(s_prod, blk, words[blk]);
      const uint32_t wb = (blk & 1) ? (wpair[blk >> 1] >> 16) : (wpair[blk >> 1] & 0xffffu);
      const float tw = t * pkv_bf16_bits_to_f32(wb);
      s = (blk == 0) ? tw : s + tw;
      if (V4B) store_v4b(v4b, row, n_cand, i, blk, s_val, words[blk]);
    }
  } else {
#pragma unroll 4
    for (int blk = 0; blk < 16; ++blk) {
      const uint32_t word = *(const uint32_t *)(nrow + key * ns_key + (int64_t)blk * ns_sub);
      const float t = pkv_block_dot(s_prod, blk, word);
      const float tw = t * pkv_bf16_bits_to_f32(wrow[key * ws_key + (int64_t)blk * ws_sub]);
      s = (blk == 0) ? tw : s + tw;
      if (V4B) store_v4b(v4b, row, n_cand, i, blk, s_val, word);
    }
  }
  *out = s * qnorm[row];
}

}  // namespace

int pkv_launch_rerank(const int64_t *cand, int bs, int n_kv_heads, int64_t n_cand, int64_t n_keys, const uint8_t *nib,
                      int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub, const uint16_t *weight, int64_t ws_b,
                      int64_t ws_h, int64_t ws_key, int64_t ws_sub, const float *qhat, const float *qnorm,
                      const float *centers, float *scores, uint16_t *v4b, hipStream_t s) {
  PKV_REQUIRE(cand && nib && weight && qhat && qnorm && centers && scores, "pkv_rerank4: null pointer");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535 && n_cand > 0 && n_keys > 0,
              "bad shape bs=%d kv_heads=%d n_cand=%lld n_keys=%lld", bs, n_kv_heads, (long long)n_cand,
              (long long)n_keys);
  PKV_REQUIRE(!v4b || pkv_aligned(v4b, 16), "v4b must be 16-byte aligned");
  dim3 grid((unsigned)((n_cand + kRerankThreads - 1) / kRerankThreads), (unsigned)(bs * n_kv_heads));
  const bool keymajor = ns_sub == 4 && ns_key >= 64 && ns_key % 16 == 0 && ws_sub == 1 && ws_key >= 16 &&
                        ws_key % 8 == 0 && pkv_aligned(nib, 16) &&
                        pkv_aligned(weight, 16) && ns_b % 16 == 0 && ns_h % 16 == 0 && ws_b % 8 == 0 && ws_h % 8 == 0;
  if (!keymajor)
    PKV_REQUIRE(pkv_aligned(nib, 4) && ns_b % 4 == 0 && ns_h % 4 == 0 && ns_key % 4 == 0 && ns_sub % 4 == 0,
                "key_4bit blocks must be 4-byte aligned (strides %lld %lld %lld %lld)", (long long)ns_b,
                (long long)ns_h, (long long)ns_key, (long long)ns_sub);
#define PKV_RERANK_LAUNCH(KM, V)                                                                                     \
  hipLaunchKernelGGL((pkv_rerank_kernel<KM, V>), grid, dim3(kRerankThreads), 0, s, cand, n_kv_heads, n_cand, n_keys, \
                     nib, ns_b, ns_h, ns_key, ns_sub, weight, ws_b, ws_h, ws_key, ws_sub, qhat, qnorm, centers,      \
                     scores, v4b)
  if (keymajor) {
    if (v4b) PKV_RERANK_LAUNCH(true, true); else PKV_RERANK_LAUNCH(true, false);
  } else {
    if (v4b) PKV_RERANK_LAUNCH(false, true); else PKV_RERANK_LAUNCH(false, false);
  }
#undef PKV_RERANK_LAUNCH
  PKV_LAUNCH_CHECK("pkv_rerank_kernel");
  return PKV_OK;
}

extern "C" int pkv_rerank4(const int64_t *cand, int bs, int n_kv_heads, int64_t n_cand, int64_t n_keys,
                           const uint8_t *nib, int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub,
                           const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key, int64_t ws_sub,
                           const float *qhat, const float *qnorm, const float *centers, float *scores, uint16_t *v4b,
                           void *stream) {
  return pkv_launch_rerank(cand, bs, n_kv_heads, n_cand, n_keys, nib, ns_b, ns_h, ns_key, ns_sub, weight, ws_b, ws_h,
                           ws_key, ws_sub, qhat, qnorm, centers, scores, v4b, (hipStream_t)stream);
}
